// Node types and node construction: Variable / Constant leaves, the Functor
// node, make_functor and friends with automatic CAST insertion, and the
// gradient rules.  Mirrors tenncor/eteq (variable.hpp, constant.hpp,
// functor.hpp, make.hpp, src/make.cpp, caster.hpp, backprop.hpp) so that graph
// building code written against those headers keeps working while every
// Functor evaluates on the GPU.
#ifndef TCH_ETEQ_HPP
#define TCH_ETEQ_HPP

#include <sstream>

#include "eigen_ops.hpp"
#include "oprules.hpp"

namespace eteq
{

// ---- leaves (tenncor/eteq/variable.hpp, constant.hpp) ----------------------

template <typename T>
struct Variable final : public eigen::iMutableLeaf
{
	static Variable<T>* get (const T* ptr, teq::Shape shape, std::string label = "",
		teq::Usage usage = teq::VARUSAGE)
	{
		return new Variable<T>(ptr, shape, label, usage);
	}

	/// New value from host data of any dtype; every dependant recomputes
	void assign (const void* input, egen::_GENERATED_DTYPE dtype, teq::Shape shape)
	{
		if (false == shape.compatible_after(shape_, 0))
		{
			global::fatalf("assigning data shaped %s to tensor %s",
				shape.to_string().c_str(), shape_.to_string().c_str());
		}
		size_t nelems = shape_.n_elems();
		std::vector<T> data(nelems);
		egen::type_convert(&data[0], input, dtype, nelems);
		upversion(global::last_version() + 1);
		ref_.assign(data.data(), nelems);
	}

	void assign (const T* input, teq::Shape shape) { assign(input, egen::get_type<T>(), shape); }

	teq::Shape shape (void) const override { return shape_; }
	teq::iDeviceRef& device (void) override { return ref_; }
	const teq::iDeviceRef& device (void) const override { return ref_; }
	const teq::iMetadata& get_meta (void) const override { return meta_; }
	std::string to_string (void) const override { return label_; }
	teq::Usage get_usage (void) const override { return usage_; }

	void upversion (size_t version) override
	{
		meta_.version_ = std::max(meta_.version_, version);
		global::note_version(meta_.version_);
	}

private:
	Variable (const T* data, teq::Shape shape, std::string label, teq::Usage usage) :
		ref_(data, shape), shape_(shape), meta_(1), label_(label), usage_(usage)
	{
		global::note_version(1);
	}

	eigen::SrcRef<T> ref_;
	teq::Shape shape_;
	eigen::EMetadata<T> meta_; // leaves start at version 1, variable.hpp:154
	std::string label_;
	teq::Usage usage_;
};

template <typename T>
using VarptrT = std::shared_ptr<Variable<T>>;

template <typename T>
struct Constant final : public teq::iLeaf
{
	static Constant<T>* get (const T* data, teq::Shape shape) { return new Constant<T>(data, shape); }

	teq::Shape shape (void) const override { return shape_; }
	teq::iDeviceRef& device (void) override { return ref_; }
	const teq::iDeviceRef& device (void) const override { return ref_; }
	const teq::iMetadata& get_meta (void) const override { return meta_; }
	teq::Usage get_usage (void) const override { return teq::IMMUTABLE; }

	/// The value when every element is equal, else the leading elements
	std::string to_string (void) const override
	{
		const T* data = (const T*) static_cast<const eigen::iEigen&>(ref_).data();
		size_t n = shape_.n_elems();
		// stream formatting, six significant digits: the labels the reference's
		// tests expect (tenncor/test/test_approx.cpp:85 "1.19209e-07", :462 "0.000999987")
		auto fmt = [](T v)
		{
			std::ostringstream s;
			s << v;
			return s.str();
		};
		if (std::all_of(data + 1, data + n, [&](const T& e) { return e == data[0]; })) { return fmt(data[0]); }
		std::string out = "[";
		for (size_t i = 0, m = std::min(n, (size_t) 5); i < m; ++i) { out += (i ? "\\" : "") + fmt(data[i]); }
		return out + (n > 5 ? "\\...]" : "]");
	}

	bool is_scalar (void) const
	{
		const T* data = (const T*) static_cast<const eigen::iEigen&>(ref_).data();
		size_t n = shape_.n_elems();
		return std::all_of(data + 1, data + n, [&](const T& e) { return e == data[0]; });
	}

private:
	Constant (const T* data, teq::Shape shape) : ref_(data, shape), shape_(shape), meta_(1) {}

	eigen::SrcRef<T> ref_;
	teq::Shape shape_;
	eigen::EMetadata<T> meta_;
};

// ---- the operator node (tenncor/eteq/functor.hpp) --------------------------

template <typename T>
struct Functor final : public eigen::Observable
{
	static Functor<T>* get (egen::_GENERATED_OPCODE opcode, teq::TensptrsT children, marsh::Maps&& attrs)
	{
		if (children.empty())
		{
			global::fatalf("cannot perform `%s` without arguments", egen::name_op(opcode).c_str());
		}
		teq::ShapesT shapes;
		shapes.reserve(children.size());
		for (auto& child : children) { shapes.push_back(child->shape()); }
		// CAST is the one node whose child has another dtype
		if (opcode != egen::CAST)
		{
			auto ctype = children.front()->get_meta().type_code();
			for (auto& child : children)
			{
				if (ctype != child->get_meta().type_code()) { global::fatal("children types are not all the same"); }
			}
		}
		teq::Shape outshape = egen::parse_shape(opcode, attrs, shapes);
		return new Functor<T>(opcode, outshape, children, std::move(attrs));
	}

	~Functor (void)
	{
		global::note_structure_change();
		for (teq::TensptrT child : args_)
		{
			if (auto f = dynamic_cast<eigen::Observable*>(child.get())) { f->unsubscribe(this); }
		}
	}

	Functor (const Functor<T>&) = delete;
	Functor<T>& operator = (const Functor<T>&) = delete;

	teq::Shape shape (void) const override { return shape_; }
	std::string to_string (void) const override { return opcode_.name_; }
	teq::Opcode get_opcode (void) const override { return opcode_; }
	teq::TensptrsT get_args (void) const override { return args_; }

	void update_child (teq::TensptrT arg, size_t index) override
	{
		if (index >= args_.size())
		{
			global::throw_errf("cannot replace argument %d when only there are only %d available",
				(int) index, (int) args_.size());
		}
		global::note_structure_change();
		uninitialize();
		teq::Shape nexshape = arg->shape();
		teq::Shape curshape = args_[index]->shape();
		if (false == nexshape.compatible_after(curshape, 0))
		{
			global::fatalf("cannot update child %d to argument with incompatible shape %s (requires shape %s)",
				(int) index, nexshape.to_string().c_str(), curshape.to_string().c_str());
		}
		auto nextype = arg->get_meta().type_label();
		auto curtype = args_[index]->get_meta().type_label();
		if (curtype != nextype)
		{
			global::fatalf("cannot update child %d to argument with different type %s (requires type %s)",
				(int) index, nextype.c_str(), curtype.c_str());
		}
		if (auto f = dynamic_cast<eigen::Observable*>(args_[index].get())) { f->unsubscribe(this); }
		args_[index] = arg;
		if (auto f = dynamic_cast<eigen::Observable*>(arg.get())) { f->subscribe(this); }
	}

	teq::iDeviceRef& device (void) override
	{
		if (false == has_data()) { must_initialize(); }
		return *ref_;
	}

	const teq::iDeviceRef& device (void) const override
	{
		if (false == has_data()) { global::fatal("cannot get device of uninitialized functor"); }
		return *ref_;
	}

	const teq::iMetadata& get_meta (void) const override { return meta_; }

	bool has_data (void) const override { return nullptr != ref_; }

	void uninitialize (void) override
	{
		if (has_data())
		{
			ref_ = nullptr;
			meta_.version_ = 0;
			for (auto& parent : this->subs_) { parent->uninitialize(); }
		}
	}

	/// Builds the launch closure once every operand has one
	bool initialize (void) override
	{
		if (std::all_of(args_.begin(), args_.end(), [](teq::TensptrT child)
			{
				if (auto f = dynamic_cast<eigen::Observable*>(child.get())) { return f->has_data(); }
				return true;
			}))
		{
			egen::typed_exec<T>((egen::_GENERATED_OPCODE) opcode_.code_, ref_, shape_, args_, *this);
			if (cache_data_) { ref_ = std::make_shared<eigen::CacheEigen>(ref_); }
		}
		return has_data();
	}

	void must_initialize (void) override
	{
		for (auto child : args_)
		{
			auto f = dynamic_cast<eigen::Observable*>(child.get());
			if (nullptr != f && false == f->has_data()) { f->must_initialize(); }
		}
		if (false == initialize()) { global::fatal("failed to initialize"); }
	}

	void cache_init (void) override
	{
		if (cache_data_) { return; }
		global::note_structure_change();
		cache_data_ = true;
		ref_ = nullptr;
		must_initialize();
	}

	/// Takes the newest operand version; true when that is news.  Operators
	/// that are not idempotent always move on (functor.hpp:246-269)
	bool prop_version (size_t max_version) override
	{
		size_t des_version = 0;
		for (auto& child : args_) { des_version = std::max(des_version, child->get_meta().state_version()); }
		size_t cur_version = meta_.version_;
		if (des_version <= cur_version &&
			false == egen::is_idempotent((egen::_GENERATED_OPCODE) opcode_.code_))
		{
			des_version = cur_version + 1;
		}
		des_version = std::min(des_version, max_version);
		bool propped = meta_.version_ < des_version;
		if (propped)
		{
			meta_.version_ = des_version;
			global::note_version(des_version);
		}
		return propped;
	}

private:
	Functor (egen::_GENERATED_OPCODE opcode, teq::Shape shape, teq::TensptrsT args, marsh::Maps&& attrs) :
		eigen::Observable(args, std::move(attrs)),
		opcode_(teq::Opcode{egen::name_op(opcode), opcode}), shape_(shape), args_(args) {}

	eigen::EigenptrT ref_ = nullptr;
	teq::Opcode opcode_;
	teq::Shape shape_;
	teq::TensptrsT args_;
	eigen::EMetadata<T> meta_; // functors start at version 0
	bool cache_data_ = false;
};

// ---- construction (tenncor/eteq/make.hpp, src/make.cpp, caster.hpp) --------

/// Children of another dtype get a CAST node in front (caster.hpp:11-46)
template <typename T>
teq::TensptrsT cast_children (egen::_GENERATED_OPCODE opcode, const teq::TensptrsT& children)
{
	if (opcode == egen::CAST) { return children; }
	auto type = egen::get_type<T>();
	teq::TensptrsT outs;
	outs.reserve(children.size());
	for (auto& child : children)
	{
		if (child->get_meta().type_code() != type)
		{
			marsh::Maps attrs;
			eigen::pack_attr(attrs, type);
			outs.push_back(teq::TensptrT(Functor<T>::get(egen::CAST, {child}, std::move(attrs))));
		}
		else { outs.push_back(child); }
	}
	return outs;
}

template <typename T>
teq::TensptrT make_tfuncattr (egen::_GENERATED_OPCODE opcode, teq::TensptrsT children, marsh::Maps& attrs)
{
	if (children.empty())
	{
		global::fatalf("cannot %s without arguments", egen::name_op(opcode).c_str());
	}
	if (egen::is_redundant(opcode, egen::get_type<T>(), attrs, children)) { return children.front(); }
	children = cast_children<T>(opcode, children);
	return teq::TensptrT(Functor<T>::get(opcode, children, std::move(attrs)));
}

/// dtype by the opcode's TypeParser, then the typed builder (src/make.cpp:14-29)
teq::TensptrT make_funcattr (egen::_GENERATED_OPCODE opcode, teq::TensptrsT children, marsh::Maps& attrs);

template <typename ...ARGS>
teq::TensptrT make_functor (egen::_GENERATED_OPCODE opcode, const teq::TensptrsT& children, ARGS... vargs)
{
	marsh::Maps attrs;
	eigen::pack_attr(attrs, vargs...);
	return make_funcattr(opcode, children, attrs);
}

template <typename T, typename ...ARGS>
teq::TensptrT make_tfunctor (egen::_GENERATED_OPCODE opcode, const teq::TensptrsT& children, ARGS... vargs)
{
	marsh::Maps attrs;
	eigen::pack_attr(attrs, vargs...);
	return make_tfuncattr<T>(opcode, children, attrs);
}

template <typename T>
VarptrT<T> make_variable (const T* data, teq::Shape shape, std::string label = "")
{
	return VarptrT<T>(Variable<T>::get(data, shape, label));
}

template <typename T>
VarptrT<T> make_variable_scalar (T scalar, teq::Shape shape, std::string label = "")
{
	std::vector<T> data(shape.n_elems(), scalar);
	return make_variable<T>(data.data(), shape, label.empty() ? std::to_string(scalar) : label);
}

template <typename T>
teq::TensptrT make_constant_tensor (const T* data, teq::Shape shape)
{
	return teq::TensptrT(Constant<T>::get(data, shape));
}

/// Constant of dtype `dtype` from data of type T
template <typename T>
teq::TensptrT make_constant_tensor (const T* data, teq::Shape shape, egen::_GENERATED_DTYPE dtype)
{
	if (egen::get_type<T>() == dtype) { return make_constant_tensor<T>(data, shape); }
	teq::TensptrT cst;
#define TCH_CSTTYPE(REALTYPE) {\
	std::vector<REALTYPE> tmp(data, data + shape.n_elems());\
	cst = make_constant_tensor<REALTYPE>(tmp.data(), shape); }
	TYPE_LOOKUP(TCH_CSTTYPE, dtype)
#undef TCH_CSTTYPE
	return cst;
}

template <typename T>
teq::TensptrT make_constant_scalar (T scalar, teq::Shape shape, egen::_GENERATED_DTYPE dtype = egen::get_type<T>())
{
	std::vector<T> data(shape.n_elems(), scalar);
	return make_constant_tensor<T>(data.data(), shape, dtype);
}

/// scalar Constant + EXTEND to the shape of `like` (make.hpp:168-183)
template <typename T>
teq::TensptrT make_constant_like (T scalar, teq::TensptrT like)
{
	auto like_type = (egen::_GENERATED_DTYPE) like->get_meta().type_code();
	teq::TensptrT cst = make_constant_scalar<T>(scalar, teq::Shape(), like_type);
	return make_functor(egen::EXTEND, teq::TensptrsT{cst}, (teq::TensptrT) like);
}

// ---- gradient rules (tenncor/eteq/backprop.hpp) ----------------------------

struct DerivativeFuncs final : public teq::iDerivativeFuncs
{
	teq::TensptrT lderive (teq::FuncptrT op, teq::TensptrT supgrad, size_t arg_idx) const override;
	teq::TensptrT get_const_one (teq::iTensor& reference) const override;
	teq::TensptrT get_const_zero (teq::iTensor& reference) const override;
	teq::TensptrT add (teq::TensptrsT elems) const override;
};

/// Evaluate `targets` with the registered evaluator on a GPU device
void run (const teq::TensptrsT& targets, const teq::TensptrsT& ignored = {});

// ---- typed handle (tenncor/eteq/etens.hpp:25-227) -------------------------
//
// What user code holds: a tensor plus the context whose evaluator and runtime
// memory evaluate it.  calc<T>() is the entry of the evaluation path
// (etens.hpp:152-162).  The reference also files every handle in a registry of
// tensor identities (for its remote-graph services); that bookkeeping has no
// part in evaluation and is not kept here.
struct ETensor
{
	ETensor (void) = default;

	ETensor (teq::TensptrT tens, const global::CfgMapptrT& ctx = global::context()) :
		tens_(nullptr != ctx ? tens : nullptr), ctx_(ctx) {}

	virtual ~ETensor (void) = default;

	friend bool operator == (const ETensor& l, const std::nullptr_t&) { return nullptr == l.get(); }
	friend bool operator == (const std::nullptr_t&, const ETensor& r) { return nullptr == r.get(); }
	friend bool operator != (const ETensor& l, const std::nullptr_t&) { return nullptr != l.get(); }
	friend bool operator != (const std::nullptr_t&, const ETensor& r) { return nullptr != r.get(); }

	operator teq::TensptrT() const { return tens_; }

	teq::iTensor& operator* () const { return *get(); }

	teq::iTensor* operator-> () const { return get(); }

	teq::iTensor* get (void) const { return tens_.get(); }

	/// nullptr once the context is gone: nothing can be evaluated then
	global::CfgMapptrT get_context (void) const { return ctx_.lock(); }

	/// Host pointer to the value the tensor holds now (nullptr if it holds none)
	template <typename T>
	T* data (void)
	{
		check_type<T>();
		return (T*) tens_->device().data();
	}

	/// The same, with the guard that counts as one read of the value
	template <typename T>
	teq::Once<T*> odata (void)
	{
		check_type<T>();
		auto held = tens_->device().odata();
		return teq::Once<T*>((T*) held.get(), std::move(held));
	}

	/// Evaluate with the context's evaluator and runtime memory, return the value
	template <typename T>
	T* calc (teq::TensSetT ignored = {}, size_t max_version = std::numeric_limits<size_t>::max())
	{
		auto ctx = get_context();
		if (nullptr == ctx || nullptr == tens_) { return nullptr; }
		eigen::Device device(eigen::get_runtime(ctx), max_version);
		teq::get_eval(ctx).evaluate(device, {get()}, ignored);
		return data<T>();
	}

	/// ... return the value with a guard: the caller's read is its last
	template <typename T>
	teq::Once<T*> calc_release (teq::TensSetT ignored = {}, size_t max_version = std::numeric_limits<size_t>::max())
	{
		auto ctx = get_context();
		if (nullptr == ctx || nullptr == tens_) { return teq::Once<T*>(nullptr); }
		eigen::Device device(eigen::get_runtime(ctx), max_version);
		teq::get_eval(ctx).evaluate(device, {get()}, ignored);
		return odata<T>();
	}

private:
	template <typename T>
	void check_type (void) const
	{
		if (nullptr == tens_) { global::fatal("cannot read the data of a null ETensor"); }
		if (tens_->get_meta().type_code() != egen::get_type<T>())
		{
			global::fatalf("cannot read %s as %s", tens_->get_meta().type_label().c_str(),
				egen::name_type(egen::get_type<T>()).c_str());
		}
	}

	teq::TensptrT tens_;
	global::CfgMaprefT ctx_;
};

using ETensorsT = std::vector<ETensor>;

teq::TensptrsT to_tensors (const ETensorsT& etensors);

/// Evaluate the targets together, in the context of the first
/// (tenncor/eteq/src/etens.cpp:46-62)
void run (const ETensorsT& targets, teq::TensSetT ignored = {},
	size_t max_version = std::numeric_limits<size_t>::max());

}

namespace tcr
{

/// d root / d target for every target (tenncor/src/eteq.cpp:40-76, local branch)
teq::TensptrsT derive (teq::TensptrT root, const teq::TensptrsT& targets);

}

#endif // TCH_ETEQ_HPP
