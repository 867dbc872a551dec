// Per-opcode construction rules: output shape (ShapeParser), output dtype
// (TypeParser) and build-time elision (FuncOpt) of cfg/ops.yml, with the
// reference's error messages.  The generated code is a template per opcode;
// here the opcode is a run-time argument and the templates forward to it.
#ifndef TCH_OPRULES_HPP
#define TCH_OPRULES_HPP

#include "packattr.hpp"

namespace egen
{

/// cfg/ops.yml ShapeParser of `opcode` (default :26-43 = all shapes equal)
teq::Shape parse_shape (_GENERATED_OPCODE opcode, const marsh::Maps& attrs, const teq::ShapesT& shapes);

/// cfg/ops.yml TypeParser (default :52-62 = highest precision of the children)
_GENERATED_DTYPE parse_type (_GENERATED_OPCODE opcode, const marsh::Maps& attrs, const eigen::DTypesT& dtypes);

/// cfg/ops.yml FuncOpt: true when the node is redundant and its first child
/// stands in for it; `out_type` is the dtype the node would have
bool is_redundant (_GENERATED_OPCODE opcode, _GENERATED_DTYPE out_type,
	const marsh::Maps& attrs, const teq::TensptrsT& args);

template <_GENERATED_OPCODE OPCODE>
struct ShapeParser final
{
	teq::Shape operator() (const marsh::Maps& attrs, const teq::ShapesT& shapes) const
	{
		return parse_shape(OPCODE, attrs, shapes);
	}
};

template <_GENERATED_OPCODE OPCODE>
struct TypeParser final
{
	_GENERATED_DTYPE operator() (const marsh::Maps& attrs, const eigen::DTypesT& dtypes) const
	{
		return parse_type(OPCODE, attrs, dtypes);
	}
};

template <_GENERATED_OPCODE OPCODE>
struct FuncOpt final
{
	template <typename T>
	bool operator() (const marsh::Maps& attrs, const teq::TensptrsT& args) const
	{
		return is_redundant(OPCODE, get_type<T>(), attrs, args);
	}
};

}

#endif // TCH_OPRULES_HPP
