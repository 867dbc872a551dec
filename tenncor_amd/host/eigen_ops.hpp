// Operator factories: one function per `stmt` of cfg/ops.yml with the names
// and argument lists of tenncor's internal/eigen/operator.hpp.  Where the
// reference returns a closure around an Eigen expression, these return a
// closure around one launch of the C ABI (include/tcg.h); attribute decoding
// (clamping, order completion, zero-copy slice detection) follows the
// reference line by line because it decides what the node computes.
#ifndef TCH_EIGEN_OPS_HPP
#define TCH_EIGEN_OPS_HPP

#include "eigen_device.hpp"

namespace eigen
{

using Shape8 = std::array<uint64_t,8>;

inline Shape8 shape8 (const teq::Shape& shape)
{
	Shape8 out;
	std::copy(shape.begin(), shape.end(), out.begin());
	return out;
}

inline bool is_2d (teq::Shape shape)
{
	return std::all_of(shape.begin() + 2, shape.end(), [](teq::DimT dim) { return 1 == dim; });
}

template <typename T>
EigenptrT make_op (const teq::Shape& outshape, const teq::CTensT& args, typename HipOp<T>::OpF op)
{
	return std::make_shared<HipOp<T>>(outshape, args, op);
}

// ---- elementwise (operator.hpp:377-987) ------------------------------------

template <typename T>
EigenptrT unary (int opcode, teq::Shape outshape, const teq::iTensor& in)
{
	uint64_t n = outshape.n_elems();
	return make_op<T>(outshape, {&in}, [opcode, n](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_ew_unary(ctx, opcode, egen::device_type<T>(), n, args[0], out));
	});
}

template <typename T>
EigenptrT binary (int opcode, teq::Shape outshape, const teq::iTensor& a, const teq::iTensor& b)
{
	uint64_t n = outshape.n_elems();
	return make_op<T>(outshape, {&a, &b}, [opcode, n](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_ew_binary(ctx, opcode, egen::device_type<T>(), n, args[0], args[1], out));
	});
}

template <typename T>
EigenptrT nnary (int opcode, teq::Shape outshape, const teq::TensptrsT& group)
{
	if (group.size() < 2) { global::fatal("n-ary operator needs at least two operands"); }
	uint64_t n = outshape.n_elems();
	teq::CTensT args;
	for (auto& g : group) { args.push_back(g.get()); }
	return make_op<T>(outshape, args, [opcode, n](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		if (args.size() == 2)
		{
			hip_check(tcg_ew_binary(ctx, opcode, egen::device_type<T>(), n, args[0], args[1], out));
		}
		else
		{
			hip_check(tcg_ew_nary(ctx, opcode, egen::device_type<T>(), n, (int) args.size(), args.data(), out));
		}
	});
}

#define TCH_UNARY(NAME, OPCODE) template <typename T>\
EigenptrT NAME (teq::Shape outshape, const teq::iTensor& in) { return unary<T>(OPCODE, outshape, in); }
TCH_UNARY(abs, TCG_ABS) TCH_UNARY(neg, TCG_NEG) TCH_UNARY(sin, TCG_SIN) TCH_UNARY(cos, TCG_COS)
TCH_UNARY(tan, TCG_TAN) TCH_UNARY(exp, TCG_EXP) TCH_UNARY(log, TCG_LOG) TCH_UNARY(sqrt, TCG_SQRT)
TCH_UNARY(round, TCG_ROUND) TCH_UNARY(sigmoid, TCG_SIGMOID) TCH_UNARY(tanh, TCG_TANH)
TCH_UNARY(square, TCG_SQUARE) TCH_UNARY(cube, TCG_CUBE)
#undef TCH_UNARY

#define TCH_BINARY(NAME, OPCODE) template <typename T>\
EigenptrT NAME (teq::Shape outshape, const teq::iTensor& a, const teq::iTensor& b) { return binary<T>(OPCODE, outshape, a, b); }
TCH_BINARY(pow, TCG_POW) TCH_BINARY(sub, TCG_SUB) TCH_BINARY(div, TCG_DIV) TCH_BINARY(eq, TCG_EQ)
TCH_BINARY(neq, TCG_NEQ) TCH_BINARY(lt, TCG_LT) TCH_BINARY(gt, TCG_GT) TCH_BINARY(min, TCG_MIN)
TCH_BINARY(max, TCG_MAX)
#undef TCH_BINARY

template <typename T>
EigenptrT add (teq::Shape outshape, const teq::TensptrsT& group) { return nnary<T>(TCG_ADD, outshape, group); }

template <typename T>
EigenptrT mul (teq::Shape outshape, const teq::TensptrsT& group) { return nnary<T>(TCG_MUL, outshape, group); }

/// operator.hpp:1050-1067
template <typename T>
EigenptrT select (teq::Shape outshape, const teq::iTensor& condition,
	const teq::iTensor& then, const teq::iTensor& otherwise)
{
	uint64_t n = outshape.n_elems();
	return make_op<T>(outshape, {&condition, &then, &otherwise},
	[n](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_ew_select(ctx, egen::device_type<T>(), n, args[0], args[1], args[2], out));
	});
}

/// operator.hpp:989-1044: uniform(a_i, b_i) per element from the seeded host
/// generator (integral: inclusive integer range)
template <typename T>
EigenptrT rand_uniform (teq::Shape outshape, const teq::iTensor& a, const teq::iTensor& b)
{
	if (global::device_random())
	{
		uint64_t n = outshape.n_elems();
		return make_op<T>(outshape, {&a, &b}, [n](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
		{
			hip_check(tcg_rand_uniform(ctx, egen::device_type<T>(), n, args[0], args[1], out));
		});
	}
	return std::make_shared<HostOp<T>>(outshape, teq::CTensT{&a, &b},
	[](T* out, const std::vector<const void*>& args, size_t n)
	{
		auto& gen = global::get_generator();
		const T* lo = (const T*) args[0];
		const T* hi = (const T*) args[1];
		for (size_t i = 0; i < n; ++i)
		{
			// drawn as int64_t / double whatever T is and narrowed afterwards
			// (internal/global/random.hpp:87-98): the same engine gives the same stream
			if constexpr (std::is_integral<T>::value)
			{
				out[i] = (T) std::uniform_int_distribution<int64_t>((int64_t) lo[i], (int64_t) hi[i])(gen);
			}
			else
			{
				out[i] = (T) std::uniform_real_distribution<double>((double) lo[i], (double) hi[i])(gen);
			}
		}
	});
}

// ---- reductions (operator.hpp:54-155) --------------------------------------

template <typename T>
EigenptrT reduce (int opcode, teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	std::set<teq::RankT> ranks;
	Packer<std::set<teq::RankT>>().unpack(ranks, attrib);
	if (ranks.empty()) { global::fatal("missing dimensions"); }
	unsigned mask = 0;
	for (teq::RankT r : ranks)
	{
		if (r < teq::rank_cap) { mask |= 1u << r; }
	}
	Shape8 inshape = shape8(in.shape());
	return make_op<T>(outshape, {&in}, [opcode, mask, inshape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_reduce(ctx, opcode, egen::device_type<T>(), inshape.data(), mask, args[0], out));
	});
}

template <typename T>
EigenptrT reduce_sum (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{ return reduce<T>(TCG_REDUCE_SUM, outshape, in, attrib); }

template <typename T>
EigenptrT reduce_prod (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{ return reduce<T>(TCG_REDUCE_PROD, outshape, in, attrib); }

template <typename T>
EigenptrT reduce_min (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{ return reduce<T>(TCG_REDUCE_MIN, outshape, in, attrib); }

template <typename T>
EigenptrT reduce_max (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{ return reduce<T>(TCG_REDUCE_MAX, outshape, in, attrib); }

template <typename T>
EigenptrT argmax (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	teq::RankT return_dim;
	Packer<teq::RankT>().unpack(return_dim, attrib);
	Shape8 inshape = shape8(in.shape());
	return make_op<T>(outshape, {&in}, [return_dim, inshape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_argmax(ctx, egen::device_type<T>(), inshape.data(), (int) return_dim, args[0], out));
	});
}

// ---- data movement (operator.hpp:157-368) ----------------------------------

template <typename T>
EigenptrT extend (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	auto inshape = in.shape();
	auto bopt = unpack_extend(inshape, attrib);
	if (!bopt) { global::fatal("cannot find extend attributes"); }
	Shape8 bcast;
	bcast.fill(1);
	for (size_t i = 0, n = std::min((size_t) teq::rank_cap, bopt->size()); i < n; ++i) { bcast[i] = (*bopt)[i]; }
	Shape8 ishape = shape8(inshape);
	return make_op<T>(outshape, {&in}, [bcast, ishape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_extend(ctx, egen::device_type<T>(), ishape.data(), bcast.data(), args[0], out));
	});
}

template <typename T>
EigenptrT permute (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	teq::RanksT order;
	Packer<teq::RanksT>().unpack(order, attrib);
	if (order.size() > teq::rank_cap) { order.resize(teq::rank_cap); }
	bool visited[teq::rank_cap] = {false};
	for (teq::RankT r : order) { visited[r] = true; }
	for (teq::RankT i = 0; i < teq::rank_cap; ++i)
	{
		if (false == visited[i]) { order.push_back(i); }
	}
	Shape8 reorder;
	std::copy(order.begin(), order.begin() + teq::rank_cap, reorder.begin());
	Shape8 ishape = shape8(in.shape());
	return make_op<T>(outshape, {&in}, [reorder, ishape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_permute(ctx, egen::device_type<T>(), ishape.data(), reorder.data(), args[0], out));
	});
}

template <typename T>
EigenptrT slice (teq::Shape outshape, const teq::TensptrT& in, const marsh::iAttributed& attrib)
{
	PairVecT<teq::DimT> encoding;
	Packer<PairVecT<teq::DimT>>().unpack(encoding, attrib);
	teq::Shape shape = in->shape();
	Shape8 offsets, extents = shape8(shape);
	offsets.fill(0);
	for (size_t i = 0, n = std::min(encoding.size(), (size_t) teq::rank_cap); i < n; ++i)
	{
		teq::DimT offset = std::min(encoding[i].first, (teq::DimT) (shape.at(i) - 1));
		offsets[i] = offset;
		extents[i] = std::min(encoding[i].second, (teq::DimT) (shape.at(i) - offset));
	}
	auto slist = teq::narrow_shape(shape);
	if (slist.size() > 0 && outshape.compatible_before(shape, slist.size() - 1))
	{
		// only the last significant dim is cut: the result is a contiguous run
		// of the input, aliased at an element offset (operator.hpp:231-248)
		teq::RankT lastdim = slist.size() - 1;
		teq::NElemT batchsize = shape.n_elems() / shape.at(lastdim);
		auto incr = offsets[lastdim] * batchsize;
		if (incr == 0) { return std::make_shared<TensRef>(*in); }
		return std::make_shared<UnsafeTensRef<T>>(*in, incr);
	}
	Shape8 ishape = shape8(shape);
	return make_op<T>(outshape, {in.get()}, [offsets, extents, ishape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_slice(ctx, egen::device_type<T>(), ishape.data(), offsets.data(), extents.data(), args[0], out));
	});
}

/// True when the value being launched for `self` is read by CONV nodes only,
/// each taking it as the image operand, and by no evaluation target
inline bool only_convolved (const Observable* self)
{
	if (nullptr == self || self->nsubs() == 0 || launch_scope().ttl != self->nsubs()) { return false; }
	for (Observable* sub : self->get_observables())
	{
		if (sub->get_opcode().code_ != egen::CONV) { return false; }
		auto args = sub->get_args();
		if (args.size() != 2 || args[0].get() != self || args[1].get() == self) { return false; }
	}
	return true;
}

template <typename T>
EigenptrT pad (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	PairVecT<teq::DimT> encoding;
	Packer<PairVecT<teq::DimT>>().unpack(encoding, attrib);
	Shape8 before, after;
	before.fill(0);
	after.fill(0);
	for (size_t i = 0, n = std::min((size_t) teq::rank_cap, encoding.size()); i < n; ++i)
	{
		before[i] = encoding[i].first;
		after[i] = encoding[i].second;
	}
	Shape8 ishape = shape8(in.shape());
	auto self = dynamic_cast<const Observable*>(&attrib);
	return make_op<T>(outshape, {&in}, [before, after, ishape, self](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		// convolutions read only the non-zero box of a padded image (see
		// nonzero_box): when they are the only readers the zero border is
		// never looked at and need not be written
		if (only_convolved(self))
		{
			launch_scope().partial = true;
			hip_check(tcg_pad_interior(ctx, egen::device_type<T>(), ishape.data(), before.data(), after.data(), args[0], out));
			return;
		}
		hip_check(tcg_pad(ctx, egen::device_type<T>(), ishape.data(), before.data(), after.data(), args[0], out));
	});
}

template <typename T>
EigenptrT stride (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	teq::DimsT c;
	Packer<teq::DimsT>().unpack(c, attrib);
	Shape8 incrs;
	incrs.fill(1);
	std::copy(c.begin(), c.begin() + std::min((size_t) teq::rank_cap, c.size()), incrs.begin());
	Shape8 ishape = shape8(in.shape()), oshape = shape8(outshape);
	return make_op<T>(outshape, {&in}, [incrs, ishape, oshape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_stride(ctx, egen::device_type<T>(), ishape.data(), incrs.data(), oshape.data(), args[0], out));
	});
}

template <typename T>
EigenptrT scatter (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	teq::DimsT dims;
	Packer<teq::DimsT>().unpack(dims, attrib);
	Shape8 incrs;
	incrs.fill(1);
	std::copy(dims.begin(), dims.begin() + std::min((size_t) teq::rank_cap, dims.size()), incrs.begin());
	Shape8 ishape = shape8(in.shape()), oshape = shape8(outshape);
	return make_op<T>(outshape, {&in}, [incrs, ishape, oshape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_scatter(ctx, egen::device_type<T>(), ishape.data(), incrs.data(), oshape.data(), args[0], out));
	});
}

template <typename T>
EigenptrT reverse (teq::Shape outshape, const teq::iTensor& in, const marsh::iAttributed& attrib)
{
	std::set<teq::RankT> dims;
	Packer<std::set<teq::RankT>>().unpack(dims, attrib);
	unsigned mask = 0;
	for (teq::RankT i : dims)
	{
		if (i < teq::rank_cap) { mask |= 1u << i; }
	}
	Shape8 shape = shape8(outshape);
	return make_op<T>(outshape, {&in}, [mask, shape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_reverse(ctx, egen::device_type<T>(), shape.data(), mask, args[0], out));
	});
}

template <typename T>
EigenptrT concat (teq::Shape outshape, const teq::TensptrsT& group, const marsh::iAttributed& attrib)
{
	if (group.size() < 2) { global::fatal("concat needs at least two operands"); }
	teq::RankT axis;
	Packer<teq::RankT>().unpack(axis, attrib);
	teq::CTensT args;
	std::vector<uint64_t> shapes;
	for (auto& g : group)
	{
		args.push_back(g.get());
		Shape8 s = shape8(g->shape());
		shapes.insert(shapes.end(), s.begin(), s.end());
	}
	return make_op<T>(outshape, args, [axis, shapes](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_concat(ctx, egen::device_type<T>(), (int) axis, (int) args.size(), shapes.data(), args.data(), out));
	});
}

/// operator.hpp:370-372 / src/operator.cpp:12-15: zero-copy alias
inline EigenptrT ref (const teq::TensptrT& in)
{
	return std::make_shared<TensRef>(*in);
}

// ---- contractions (operator.hpp:1069-1187) ---------------------------------

template <typename T>
EigenptrT contract (teq::Shape outshape, const teq::iTensor& a, const teq::iTensor& b, const marsh::iAttributed& attrib)
{
	PairVecT<teq::RankT> dims;
	Packer<PairVecT<teq::RankT>>().unpack(dims, attrib);
	if (dims.empty()) { global::fatal("missing dimensions"); }
	std::vector<uint64_t> pairs;
	for (auto& d : dims)
	{
		pairs.push_back(d.first);
		pairs.push_back(d.second);
	}
	Shape8 ashape = shape8(a.shape()), bshape = shape8(b.shape());
	return make_op<T>(outshape, {&a, &b}, [pairs, ashape, bshape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_contract(ctx, egen::device_type<T>(), ashape.data(), bshape.data(),
			(int) (pairs.size() / 2), pairs.data(), args[0], args[1], out));
	});
}

template <typename T>
EigenptrT matmul (teq::Shape outshape, const teq::iTensor& a, const teq::iTensor& b)
{
	Shape8 ashape = shape8(a.shape()), bshape = shape8(b.shape());
	return make_op<T>(outshape, {&a, &b}, [ashape, bshape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_matmul(ctx, egen::device_type<T>(), ashape.data(), bshape.data(), args[0], args[1], out));
	});
}

/// Where a node's value can be non-zero, known from how it was built: PAD
/// nodes (and IDENTITY aliases of them) shift and keep their operand's box
inline void nonzero_box (const teq::iTensor& tens, Shape8& lo, Shape8& hi)
{
	auto f = dynamic_cast<const teq::iFunctor*>(&tens);
	if (nullptr != f && f->get_opcode().code_ == egen::PAD)
	{
		auto arg = f->get_args().front();
		nonzero_box(*arg, lo, hi);
		PairVecT<teq::DimT> paddings;
		Packer<PairVecT<teq::DimT>>().unpack(paddings, *f);
		for (size_t i = 0, n = std::min((size_t) teq::rank_cap, paddings.size()); i < n; ++i)
		{
			lo[i] += paddings[i].first;
			hi[i] += paddings[i].first;
		}
		return;
	}
	if (nullptr != f && f->get_opcode().code_ == egen::IDENTITY)
	{
		nonzero_box(*f->get_args().front(), lo, hi);
		return;
	}
	lo.fill(0);
	hi = shape8(tens.shape());
}

/// The bounding box of the SLICEs reading `self`, false when anything else reads it
inline bool slices_window (const Observable* self, const teq::Shape& outshape, Shape8& lo, Shape8& hi)
{
	if (nullptr == self || self->nsubs() == 0) { return false; }
	bool first = true;
	for (Observable* sub : self->get_observables())
	{
		if (sub->get_opcode().code_ != egen::SLICE) { return false; }
		auto args = sub->get_args();
		if (args.size() != 1 || args[0].get() != self) { return false; }
		PairVecT<teq::DimT> encoding;
		Packer<PairVecT<teq::DimT>>().unpack(encoding, *sub);
		for (teq::RankT i = 0; i < teq::rank_cap; ++i)
		{
			uint64_t off = 0, ext = outshape.at(i);
			if (i < encoding.size())
			{
				off = std::min(encoding[i].first, (teq::DimT) (outshape.at(i) - 1));
				ext = std::min(encoding[i].second, (teq::DimT) (outshape.at(i) - off));
			}
			lo[i] = first ? off : std::min(lo[i], off);
			hi[i] = first ? off + ext : std::max(hi[i], off + ext);
		}
		first = false;
	}
	return true;
}

/// The part of `self`'s value its consumers read: when every consumer is a
/// SLICE of it and the node is no evaluation target, the bounding box of
/// those slices; otherwise everything (false)
inline bool consumed_window (const Observable* self, const teq::Shape& outshape, Shape8& lo, Shape8& hi)
{
	// a target is read in full
	if (nullptr == self || launch_scope().ttl != self->nsubs()) { return false; }
	return slices_window(self, outshape, lo, hi);
}

template <typename T>
EigenptrT convolution (teq::Shape outshape, const teq::iTensor& input,
	const teq::iTensor& kernel, const marsh::iAttributed& attrib)
{
	auto kshape = kernel.shape();
	teq::RanksT order;
	Packer<teq::RanksT>().unpack(order, attrib);
	bool visited[teq::rank_cap] = {false};
	size_t n = std::min(order.size(), (size_t) teq::rank_cap);
	for (size_t i = 0; i < n; ++i)
	{
		teq::RankT d = order[i];
		if (d >= teq::rank_cap || visited[d])
		{
			global::fatalf("convolution does not support repeated kernel dimensions: %s",
				range_to_string(order.begin(), order.end()).c_str());
		}
		visited[d] = true;
	}
	for (size_t i = n; i < teq::rank_cap; ++i)
	{
		if (kshape.at(i) > 1)
		{
			global::fatalf("given kernel shape %s, unspecified non-singular kernel dimension %d is undefined",
				kshape.to_string().c_str(), (int) i);
		}
	}
	std::vector<uint64_t> ranks(order.begin(), order.begin() + n);
	Shape8 ishape = shape8(input.shape()), ks = shape8(kshape);
	// padding the image operand carries is skipped, not multiplied
	Shape8 ilo, ihi;
	nonzero_box(input, ilo, ihi);
	auto self = dynamic_cast<const Observable*>(&attrib);
	return make_op<T>(outshape, {&input, &kernel},
	[ranks, ishape, ks, ilo, ihi, self, outshape](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		Shape8 olo, ohi;
		bool windowed = consumed_window(self, outshape, olo, ohi);
		launch_scope().partial = windowed;
		hip_check(tcg_conv_boxed(ctx, egen::device_type<T>(), ishape.data(), ks.data(), (int) ranks.size(),
			ranks.data(), ilo.data(), ihi.data(), windowed ? olo.data() : nullptr,
			windowed ? ohi.data() : nullptr, args[0], args[1], out));
	});
}

// ---- in-place updates and casts (operator.hpp:1189-1260) -------------------

template <typename T>
EigenptrT assign (teq::iTensor& target, const teq::iTensor& source)
{ return std::make_shared<TensAssign<T>>(target, source, TCG_ASSIGN); }

template <typename T>
EigenptrT assign_add (teq::iTensor& target, const teq::iTensor& source)
{ return std::make_shared<TensAssign<T>>(target, source, TCG_ASSIGN_ADD); }

template <typename T>
EigenptrT assign_sub (teq::iTensor& target, const teq::iTensor& source)
{ return std::make_shared<TensAssign<T>>(target, source, TCG_ASSIGN_SUB); }

template <typename T>
EigenptrT assign_mul (teq::iTensor& target, const teq::iTensor& source)
{ return std::make_shared<TensAssign<T>>(target, source, TCG_ASSIGN_MUL); }

template <typename T>
EigenptrT assign_div (teq::iTensor& target, const teq::iTensor& source)
{ return std::make_shared<TensAssign<T>>(target, source, TCG_ASSIGN_DIV); }

template <typename T>
EigenptrT cast (const teq::TensptrT& input)
{
	auto intype = (egen::_GENERATED_DTYPE) input->get_meta().type_code();
	if (egen::get_type<T>() == intype)
	{
		global::warnf("pointless to convert the same type %s", egen::name_type(intype).c_str());
		return std::make_shared<TensRef>(*input);
	}
	uint64_t n = input->shape().n_elems();
	return make_op<T>(input->shape(), {input.get()}, [intype, n](tcg_ctx* ctx, T* out, const std::vector<const void*>& args)
	{
		hip_check(tcg_cast(ctx, egen::device_type<T>(), egen::device_type(intype), n, args[0], out));
	});
}

}

namespace egen
{

/// The dispatcher tools/egen generates from cfg/ops.yml
/// (tools/egen/plugins/opcodes.py:36-46): one case per opcode running its stmt
template <typename T>
void typed_exec (_GENERATED_OPCODE opcode, eigen::EigenptrT& out, teq::Shape outshape,
	const teq::TensptrsT& in, const marsh::iAttributed& attrib)
{
	auto need = [&](size_t n)
	{
		if (in.size() < n)
		{
			global::fatalf("cannot %s with %d arguments", name_op(opcode).c_str(), (int) in.size());
		}
	};
	need(1);
	switch (opcode)
	{
		case IDENTITY: out = eigen::ref(in[0]); break;
		case ABS: out = eigen::abs<T>(outshape, *in[0]); break;
		case NEG: out = eigen::neg<T>(outshape, *in[0]); break;
		case SIN: out = eigen::sin<T>(outshape, *in[0]); break;
		case COS: out = eigen::cos<T>(outshape, *in[0]); break;
		case TAN: out = eigen::tan<T>(outshape, *in[0]); break;
		case EXP: out = eigen::exp<T>(outshape, *in[0]); break;
		case LOG: out = eigen::log<T>(outshape, *in[0]); break;
		case SQRT: out = eigen::sqrt<T>(outshape, *in[0]); break;
		case ROUND: out = eigen::round<T>(outshape, *in[0]); break;
		case SIGMOID: out = eigen::sigmoid<T>(outshape, *in[0]); break;
		case TANH: out = eigen::tanh<T>(outshape, *in[0]); break;
		case SQUARE: out = eigen::square<T>(outshape, *in[0]); break;
		case CUBE: out = eigen::cube<T>(outshape, *in[0]); break;
		case RAND_UNIF: need(2); out = eigen::rand_uniform<T>(outshape, *in[0], *in[1]); break;
		case REVERSE: out = eigen::reverse<T>(outshape, *in[0], attrib); break;
		case REDUCE_SUM: out = eigen::reduce_sum<T>(outshape, *in[0], attrib); break;
		case REDUCE_PROD: out = eigen::reduce_prod<T>(outshape, *in[0], attrib); break;
		case REDUCE_MIN: out = eigen::reduce_min<T>(outshape, *in[0], attrib); break;
		case REDUCE_MAX: out = eigen::reduce_max<T>(outshape, *in[0], attrib); break;
		case ARGMAX: out = eigen::argmax<T>(outshape, *in[0], attrib); break;
		case PERMUTE: out = eigen::permute<T>(outshape, *in[0], attrib); break;
		case EXTEND: out = eigen::extend<T>(outshape, *in[0], attrib); break;
		case RESHAPE: out = eigen::ref(in[0]); break;
		case SLICE: out = eigen::slice<T>(outshape, in[0], attrib); break;
		case PAD: out = eigen::pad<T>(outshape, *in[0], attrib); break;
		case STRIDE: out = eigen::stride<T>(outshape, *in[0], attrib); break;
		case SCATTER: out = eigen::scatter<T>(outshape, *in[0], attrib); break;
		case POW: need(2); out = eigen::pow<T>(outshape, *in[0], *in[1]); break;
		case ADD: out = eigen::add<T>(outshape, in); break;
		case SUB: need(2); out = eigen::sub<T>(outshape, *in[0], *in[1]); break;
		case MUL: out = eigen::mul<T>(outshape, in); break;
		case DIV: need(2); out = eigen::div<T>(outshape, *in[0], *in[1]); break;
		case MIN: need(2); out = eigen::min<T>(outshape, *in[0], *in[1]); break;
		case MAX: need(2); out = eigen::max<T>(outshape, *in[0], *in[1]); break;
		case EQ: need(2); out = eigen::eq<T>(outshape, *in[0], *in[1]); break;
		case NEQ: need(2); out = eigen::neq<T>(outshape, *in[0], *in[1]); break;
		case LT: need(2); out = eigen::lt<T>(outshape, *in[0], *in[1]); break;
		case GT: need(2); out = eigen::gt<T>(outshape, *in[0], *in[1]); break;
		case MATMUL: need(2); out = eigen::matmul<T>(outshape, *in[0], *in[1]); break;
		case CONTRACT: need(2); out = eigen::contract<T>(outshape, *in[0], *in[1], attrib); break;
		case CONV: need(2); out = eigen::convolution<T>(outshape, *in[0], *in[1], attrib); break;
		case SELECT: need(3); out = eigen::select<T>(outshape, *in[0], *in[1], *in[2]); break;
		case CONCAT: out = eigen::concat<T>(outshape, in, attrib); break;
		case ASSIGN: need(2); out = eigen::assign<T>(*in[0], *in[1]); break;
		case ASSIGN_ADD: need(2); out = eigen::assign_add<T>(*in[0], *in[1]); break;
		case ASSIGN_SUB: need(2); out = eigen::assign_sub<T>(*in[0], *in[1]); break;
		case ASSIGN_MUL: need(2); out = eigen::assign_mul<T>(*in[0], *in[1]); break;
		case ASSIGN_DIV: need(2); out = eigen::assign_div<T>(*in[0], *in[1]); break;
		case CAST: out = eigen::cast<T>(in[0]); break;
		default: global::fatal("unknown opcode");
	}
}

// Runs `MACRO(OPCODE)` with the opcode as a compile-time constant
// (OPCODE_LOOKUP of the generated opcode.hpp) -- kept for callers that pick a
// ShapeParser / FuncOpt template by opcode
#define TCH_OP_CASE(MACRO, OP) case egen::OP: MACRO(egen::OP) break;
#define OPCODE_LOOKUP(MACRO, OPCODE) switch (OPCODE) {\
	TCH_OP_CASE(MACRO, IDENTITY) TCH_OP_CASE(MACRO, ABS) TCH_OP_CASE(MACRO, NEG) TCH_OP_CASE(MACRO, SIN)\
	TCH_OP_CASE(MACRO, COS) TCH_OP_CASE(MACRO, TAN) TCH_OP_CASE(MACRO, EXP) TCH_OP_CASE(MACRO, LOG)\
	TCH_OP_CASE(MACRO, SQRT) TCH_OP_CASE(MACRO, ROUND) TCH_OP_CASE(MACRO, SIGMOID) TCH_OP_CASE(MACRO, TANH)\
	TCH_OP_CASE(MACRO, SQUARE) TCH_OP_CASE(MACRO, CUBE) TCH_OP_CASE(MACRO, RAND_UNIF) TCH_OP_CASE(MACRO, REVERSE)\
	TCH_OP_CASE(MACRO, REDUCE_SUM) TCH_OP_CASE(MACRO, REDUCE_PROD) TCH_OP_CASE(MACRO, REDUCE_MIN)\
	TCH_OP_CASE(MACRO, REDUCE_MAX) TCH_OP_CASE(MACRO, ARGMAX) TCH_OP_CASE(MACRO, PERMUTE) TCH_OP_CASE(MACRO, EXTEND)\
	TCH_OP_CASE(MACRO, RESHAPE) TCH_OP_CASE(MACRO, SLICE) TCH_OP_CASE(MACRO, PAD) TCH_OP_CASE(MACRO, STRIDE)\
	TCH_OP_CASE(MACRO, SCATTER) TCH_OP_CASE(MACRO, POW) TCH_OP_CASE(MACRO, ADD) TCH_OP_CASE(MACRO, SUB)\
	TCH_OP_CASE(MACRO, MUL) TCH_OP_CASE(MACRO, DIV) TCH_OP_CASE(MACRO, MIN) TCH_OP_CASE(MACRO, MAX)\
	TCH_OP_CASE(MACRO, EQ) TCH_OP_CASE(MACRO, NEQ) TCH_OP_CASE(MACRO, LT) TCH_OP_CASE(MACRO, GT)\
	TCH_OP_CASE(MACRO, MATMUL) TCH_OP_CASE(MACRO, CONTRACT) TCH_OP_CASE(MACRO, CONV) TCH_OP_CASE(MACRO, SELECT)\
	TCH_OP_CASE(MACRO, CONCAT) TCH_OP_CASE(MACRO, ASSIGN) TCH_OP_CASE(MACRO, ASSIGN_ADD)\
	TCH_OP_CASE(MACRO, ASSIGN_SUB) TCH_OP_CASE(MACRO, ASSIGN_MUL) TCH_OP_CASE(MACRO, ASSIGN_DIV)\
	TCH_OP_CASE(MACRO, CAST) default: global::fatal("executing bad op"); }

}

#endif // TCH_EIGEN_OPS_HPP
