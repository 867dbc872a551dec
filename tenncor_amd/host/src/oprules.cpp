// Shape, type and elision rules of every opcode (cfg/ops.yml).
#include "oprules.hpp"

#include <cmath>

namespace egen
{

static const char* opnames[] = {
	"BAD_OP", "IDENTITY", "ABS", "NEG", "SIN", "COS", "TAN", "EXP", "LOG", "SQRT", "ROUND",
	"SIGMOID", "TANH", "SQUARE", "CUBE", "RAND_UNIF", "REVERSE", "REDUCE_SUM", "REDUCE_PROD",
	"REDUCE_MIN", "REDUCE_MAX", "ARGMAX", "PERMUTE", "EXTEND", "RESHAPE", "SLICE", "PAD",
	"STRIDE", "SCATTER", "POW", "ADD", "SUB", "MUL", "DIV", "MIN", "MAX", "EQ", "NEQ", "LT",
	"GT", "MATMUL", "CONTRACT", "CONV", "SELECT", "CONCAT", "ASSIGN", "ASSIGN_ADD",
	"ASSIGN_SUB", "ASSIGN_MUL", "ASSIGN_DIV", "CAST",
};

std::string name_op (_GENERATED_OPCODE code)
{
	if (code <= BAD_OP || code >= _N_GENERATED_OPCODES) { return "BAD_OP"; }
	return opnames[code];
}

_GENERATED_OPCODE get_op (const std::string& name)
{
	for (int i = 1; i < _N_GENERATED_OPCODES; ++i)
	{
		if (name == opnames[i]) { return (_GENERATED_OPCODE) i; }
	}
	return BAD_OP;
}

std::string name_type (_GENERATED_DTYPE type)
{
	switch (type)
	{
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) case ENUM: return #ENUM;
		EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
		default: return "BAD_TYPE";
	}
}

_GENERATED_DTYPE get_type (const std::string& name)
{
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) if (name == #ENUM) { return ENUM; }
	EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
	return BAD_TYPE;
}

static void need_args (const teq::ShapesT& shapes)
{
	if (shapes.empty()) { global::fatal(eigen::no_argument_err); }
}

// cfg/ops.yml:26-43
static teq::Shape same_shape (_GENERATED_OPCODE opcode, const teq::ShapesT& shapes)
{
	need_args(shapes);
	teq::Shape outshape = shapes.front();
	for (size_t i = 1, n = shapes.size(); i < n; ++i)
	{
		if (false == shapes[i].compatible_after(outshape, 0))
		{
			global::throw_errf("cannot %s with incompatible shapes %s and %s",
				name_op(opcode).c_str(), shapes[i].to_string().c_str(), outshape.to_string().c_str());
		}
	}
	return outshape;
}

teq::Shape parse_shape (_GENERATED_OPCODE opcode, const marsh::Maps& attrs, const teq::ShapesT& shapes)
{
	switch (opcode)
	{
		case IDENTITY: // :64-74
			need_args(shapes);
			return shapes.front();
		case REDUCE_SUM: case REDUCE_PROD: case REDUCE_MIN: case REDUCE_MAX: // :123-139
		{
			need_args(shapes);
			std::set<teq::RankT> ranks;
			eigen::Packer<std::set<teq::RankT>>().unpack(ranks, attrs);
			teq::DimsT slist(shapes.front().begin(), shapes.front().end());
			for (teq::RankT i : ranks)
			{
				if (i >= teq::rank_cap) { global::throw_errf("cannot access out of bounds index %d", (int) i); }
				slist[i] = 1;
			}
			return teq::Shape(slist);
		}
		case ARGMAX: // :169-186
		{
			need_args(shapes);
			teq::RankT return_dim;
			eigen::Packer<teq::RankT>().unpack(return_dim, attrs);
			if (return_dim >= teq::rank_cap) { return teq::Shape(); }
			teq::DimsT slist(shapes.front().begin(), shapes.front().end());
			slist[return_dim] = 1;
			return teq::Shape(slist);
		}
		case PERMUTE: // :207-238
		{
			need_args(shapes);
			teq::RanksT order;
			eigen::Packer<teq::RanksT>().unpack(order, attrs);
			bool visited[teq::rank_cap] = {false};
			for (size_t i = 0, n = std::min(order.size(), (size_t) teq::rank_cap); i < n; ++i)
			{
				if (order[i] >= teq::rank_cap) { global::throw_errf("cannot access out of bounds index %d", (int) order[i]); }
				if (visited[order[i]])
				{
					global::throw_errf("permute does not support repeated orders (order=%s)",
						eigen::range_to_string(order.begin(), order.end()).c_str());
				}
				visited[order[i]] = true;
			}
			if (order.size() > teq::rank_cap) { order.resize(teq::rank_cap); }
			for (teq::RankT i = 0; i < teq::rank_cap; ++i)
			{
				if (false == visited[i]) { order.push_back(i); }
			}
			teq::Shape shape = shapes.front();
			teq::DimsT slist(teq::rank_cap, 1);
			for (teq::RankT i = 0; i < teq::rank_cap; ++i) { slist[i] = shape.at(order[i]); }
			return teq::Shape(slist);
		}
		case EXTEND: // :256-283
		{
			need_args(shapes);
			teq::Shape shape = shapes.front();
			teq::DimsT bcast;
			if (auto bopt = eigen::unpack_extend(shape, attrs)) { bcast = *bopt; }
			if (std::any_of(bcast.begin(), bcast.end(), [](teq::DimT d) { return 0 == d; }))
			{
				global::throw_errf("cannot extend using zero dimensions %s",
					eigen::range_to_string(bcast.begin(), bcast.end()).c_str());
			}
			teq::DimsT slist(shape.begin(), shape.end());
			for (size_t i = 0, n = std::min(bcast.size(), (size_t) teq::rank_cap); i < n; ++i)
			{
				if (bcast[i] > 1 && shape.at(i) > 1)
				{
					global::throw_errf("cannot extend non-singular dimension %d of shape %s: bcast=%s",
						(int) i, shape.to_string().c_str(), eigen::range_to_string(bcast.begin(), bcast.end()).c_str());
				}
				slist[i] *= bcast[i];
			}
			return teq::Shape(slist);
		}
		case RESHAPE: // :299-318
		{
			need_args(shapes);
			teq::Shape outshape;
			eigen::Packer<teq::Shape>().unpack(outshape, attrs);
			if (shapes.front().n_elems() != outshape.n_elems())
			{
				global::throw_errf("cannot RESHAPE with shapes of different sizes %d (shape %s) and %d (shape %s)",
					(int) shapes.front().n_elems(), shapes.front().to_string().c_str(),
					(int) outshape.n_elems(), outshape.to_string().c_str());
			}
			return outshape;
		}
		case SLICE: // :350-371
		{
			need_args(shapes);
			eigen::PairVecT<teq::DimT> extents;
			eigen::Packer<eigen::PairVecT<teq::DimT>>().unpack(extents, attrs);
			teq::Shape shape = shapes.front();
			teq::DimsT slist(shape.begin(), shape.end());
			for (size_t i = 0, n = std::min(extents.size(), (size_t) teq::rank_cap); i < n; ++i)
			{
				teq::DimT offset = extents[i].first;
				if (offset < shape.at(i))
				{
					slist[i] = std::min(extents[i].second, (teq::DimT) (shape.at(i) - offset));
				}
			}
			return teq::Shape(slist);
		}
		case PAD: // :392-412
		{
			need_args(shapes);
			eigen::PairVecT<teq::DimT> paddings;
			eigen::Packer<eigen::PairVecT<teq::DimT>>().unpack(paddings, attrs);
			teq::DimsT slist(shapes.front().begin(), shapes.front().end());
			for (size_t i = 0, n = std::min(paddings.size(), (size_t) teq::rank_cap); i < n; ++i)
			{
				if (slist[i] > 0) { slist[i] += paddings[i].first + paddings[i].second; }
			}
			return teq::Shape(slist);
		}
		case STRIDE: // :415-438
		{
			need_args(shapes);
			teq::DimsT incrs;
			eigen::Packer<teq::DimsT>().unpack(incrs, attrs);
			teq::DimsT slist(shapes.front().begin(), shapes.front().end());
			for (size_t i = 0, n = std::min(incrs.size(), (size_t) teq::rank_cap); i < n; ++i)
			{
				slist[i] = (teq::DimT) std::round((double) slist[i] / incrs[i]);
			}
			return teq::Shape(slist);
		}
		case SCATTER: // :442-452
		{
			need_args(shapes);
			teq::Shape outshape;
			eigen::Packer<teq::Shape>().unpack(outshape, attrs);
			return outshape;
		}
		case MATMUL: // :496-514
		{
			if (shapes.size() < 2) { global::fatal(eigen::no_argument_err); }
			teq::Shape ashape = shapes[0], bshape = shapes[1];
			if (false == ashape.compatible_after(bshape, 2))
			{
				global::throw_errf("invalid shapes %s and %s do not match for dimensions 2+",
					ashape.to_string().c_str(), bshape.to_string().c_str());
			}
			if (ashape.at(0) != bshape.at(1))
			{
				global::throw_errf("invalid shapes %s and %s have mismatch common dimension 0,1",
					ashape.to_string().c_str(), bshape.to_string().c_str());
			}
			teq::DimsT outlist = {bshape.at(0), ashape.at(1)};
			outlist.insert(outlist.end(), ashape.begin() + 2, ashape.end());
			return teq::Shape(outlist);
		}
		case CONTRACT: // :517-565
		{
			if (shapes.size() < 2) { global::fatal(eigen::no_argument_err); }
			eigen::PairVecT<teq::RankT> ranks;
			eigen::Packer<eigen::PairVecT<teq::RankT>>().unpack(ranks, attrs);
			bool acommon[teq::rank_cap] = {false}, bcommon[teq::rank_cap] = {false};
			teq::Shape ashape = shapes[0], bshape = shapes[1];
			for (auto& coms : ranks)
			{
				if (ashape.at(coms.first) != bshape.at(coms.second))
				{
					global::throw_errf("invalid shapes %s and %s do not match common dimensions %s",
						ashape.to_string().c_str(), bshape.to_string().c_str(), eigen::to_string(ranks).c_str());
				}
				if (acommon[coms.first] || bcommon[coms.second])
				{
					global::throw_errf("contraction dimensions %s must be unique for each side",
						eigen::to_string(ranks).c_str());
				}
				acommon[coms.first] = bcommon[coms.second] = true;
			}
			teq::DimsT alist = teq::narrow_shape(ashape), blist = teq::narrow_shape(bshape), outlist;
			for (size_t i = 0; i < blist.size(); ++i) { if (!bcommon[i]) { outlist.push_back(blist[i]); } }
			for (size_t i = 0; i < alist.size(); ++i) { if (!acommon[i]) { outlist.push_back(alist[i]); } }
			return teq::Shape(outlist);
		}
		case CONV: // :568-607
		{
			if (shapes.size() < 2) { global::fatal(eigen::no_argument_err); }
			teq::RanksT ranks;
			eigen::Packer<teq::RanksT>().unpack(ranks, attrs);
			size_t n = std::min(ranks.size(), (size_t) teq::rank_cap);
			teq::Shape kernelshape = shapes[1];
			if (std::any_of(kernelshape.begin() + n, kernelshape.end(), [](teq::DimT d) { return d > 1; }))
			{
				global::throw_errf("cannot have ambiguous ranks not specified in kernelshape %s (ranks=%s)",
					kernelshape.to_string().c_str(), eigen::range_to_string(ranks.begin(), ranks.end()).c_str());
			}
			teq::Shape imgshape = shapes[0];
			teq::DimsT slist(imgshape.begin(), imgshape.end());
			for (size_t i = 0; i < n; ++i)
			{
				if (ranks[i] >= teq::rank_cap) { global::throw_errf("cannot access out of bounds index %d", (int) ranks[i]); }
				teq::DimT& sdim = slist[ranks[i]];
				teq::DimT kdim = kernelshape.at(i);
				if (0 == sdim || 0 == kdim) { sdim = 0; }
				else
				{
					if (kdim > sdim)
					{
						global::throw_errf("cannot convolve a kernel of shape %s against smaller image of shape %s "
							"at dimensions (shape:kernel=%d:%d)", kernelshape.to_string().c_str(),
							imgshape.to_string().c_str(), (int) ranks[i], (int) i);
					}
					sdim -= kdim - 1;
				}
			}
			return teq::Shape(slist);
		}
		case CONCAT: // :613-653
		{
			need_args(shapes);
			teq::RankT axis;
			eigen::Packer<teq::RankT>().unpack(axis, attrs);
			if (axis >= teq::rank_cap) { global::throw_errf("cannot access out of bounds index %d", (int) axis); }
			teq::Shape initshape = shapes.front();
			for (auto it = shapes.begin() + 1, et = shapes.end(); it != et; ++it)
			{
				if (false == initshape.compatible_before(*it, axis) ||
					(axis + 1 < teq::rank_cap && false == initshape.compatible_after(*it, axis + 1)))
				{
					global::throw_errf("cannot group concat incompatible shapes %s and %s along axis %d",
						initshape.to_string().c_str(), it->to_string().c_str(), (int) axis);
				}
			}
			teq::DimsT slist(initshape.begin(), initshape.end());
			if (shapes.size() > 2)
			{
				if (std::any_of(shapes.begin(), shapes.end(), [axis](teq::Shape shape) { return shape.at(axis) != 1; }))
				{
					global::throw_err("cannot group concat shapes with dimension that is not one");
				}
				slist[axis] = shapes.size();
				return teq::Shape(slist);
			}
			if (shapes.size() == 2)
			{
				teq::Shape backshape = shapes[1];
				if (slist[axis] == 0 || backshape.at(axis) == 0) { slist[axis] = 0; }
				else { slist[axis] += backshape.at(axis); }
			}
			return teq::Shape(slist);
		}
		case ASSIGN: case ASSIGN_ADD: case ASSIGN_SUB: case ASSIGN_MUL: case ASSIGN_DIV:
		default:
			return same_shape(opcode, shapes);
	}
}

_GENERATED_DTYPE parse_type (_GENERATED_OPCODE opcode, const marsh::Maps& attrs, const eigen::DTypesT& dtypes)
{
	if (dtypes.empty()) { global::fatal(eigen::no_argument_err); }
	switch (opcode)
	{
		case ASSIGN: case ASSIGN_ADD: case ASSIGN_SUB: case ASSIGN_MUL: case ASSIGN_DIV: // :656-664
			return dtypes.front();
		case CAST: // :696-710
			if (attrs.get_attr(eigen::Packer<_GENERATED_DTYPE>().get_key()))
			{
				_GENERATED_DTYPE out;
				eigen::Packer<_GENERATED_DTYPE>().unpack(out, attrs);
				return out;
			}
			return dtypes.front();
		default: // :52-62
			return *std::max_element(dtypes.begin(), dtypes.end(),
				[](_GENERATED_DTYPE lhs, _GENERATED_DTYPE rhs) { return type_precision(lhs) < type_precision(rhs); });
	}
}

bool is_redundant (_GENERATED_OPCODE opcode, _GENERATED_DTYPE out_type,
	const marsh::Maps& attrs, const teq::TensptrsT& args)
{
	switch (opcode)
	{
		case REDUCE_SUM: case REDUCE_PROD: case REDUCE_MIN: case REDUCE_MAX: // :108-122
		{
			std::set<teq::RankT> ranks;
			eigen::Packer<std::set<teq::RankT>>().unpack(ranks, attrs);
			return ranks.empty();
		}
		case ARGMAX: // :154-168
		{
			teq::RankT return_dim;
			eigen::Packer<teq::RankT>().unpack(return_dim, attrs);
			return return_dim < teq::rank_cap && args.front()->shape().at(return_dim) == 1;
		}
		case PERMUTE: // :189-206
		{
			teq::RanksT order;
			eigen::Packer<teq::RanksT>().unpack(order, attrs);
			bool redundant = order.empty() ? true : (order[0] == 0);
			for (size_t i = 1, n = std::min(order.size(), (size_t) teq::rank_cap); i < n && redundant; ++i)
			{
				redundant = redundant && (order[i] == (order[i - 1] + 1));
			}
			return redundant;
		}
		case EXTEND: // :241-255
		{
			auto bcast = eigen::unpack_extend(args.front()->shape(), attrs);
			bool uses_dims = nullptr != attrs.get_attr(eigen::Packer<teq::DimsT>().get_key());
			return false == bool(bcast) || (uses_dims && (bcast->empty() ||
				std::all_of(bcast->begin(), bcast->end(), [](teq::DimT d) { return 1 == d; })));
		}
		case RESHAPE: case SCATTER: // :286-298, :441
		{
			teq::Shape outshape;
			eigen::Packer<teq::Shape>().unpack(outshape, attrs);
			return outshape.compatible_after(args.front()->shape(), 0);
		}
		case SLICE: // :321-349
		{
			eigen::PairVecT<teq::DimT> extents;
			eigen::Packer<eigen::PairVecT<teq::DimT>>().unpack(extents, attrs);
			if (std::any_of(extents.begin(), extents.end(),
				[](std::pair<teq::DimT,teq::DimT> ext) { return ext.second == 0; }))
			{
				global::fatalf("cannot create slice with 0 dimensions (second value of extents) (extents=%s)",
					eigen::to_string(extents).c_str());
			}
			teq::Shape shape = args.front()->shape();
			bool redundant = true;
			for (size_t i = 0, n = std::min(extents.size(), (size_t) teq::rank_cap); i < n && redundant; ++i)
			{
				redundant = redundant && extents[i].first == 0 && extents[i].second > shape.at(i);
			}
			return redundant;
		}
		case PAD: // :374-391
		{
			eigen::PairVecT<teq::DimT> paddings;
			eigen::Packer<eigen::PairVecT<teq::DimT>>().unpack(paddings, attrs);
			return paddings.empty() || std::all_of(paddings.begin(), paddings.end(),
				[](std::pair<teq::DimT,teq::DimT> pad) { return pad.first == 0 && pad.second == 0; });
		}
		case ADD: case MUL: case CONCAT: // :457-468, :474, :612
			return args.size() < 2;
		case CAST: // :683-695
			return (_GENERATED_DTYPE) args.front()->get_meta().type_code() == out_type;
		default:
			return false;
	}
}

}
