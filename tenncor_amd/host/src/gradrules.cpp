// The gradient builder's operator rules: for a functor f, an operand index k
// and the gradient `up` that arrives at f, the graph of d(loss)/d(operand k).
// What each rule must build is fixed by the reference (tenncor/eteq/
// backprop.hpp:58-576; its expected graphs, tenncor/eteq/test/
// test_backprop.cpp:68-773, are compared line by line in the tests), because
// every node a rule emits is a node the evaluation backend then runs.
//
// Layout: one small function per rule, looked up by opcode in a table; the
// functions share a handful of graph-building helpers and, for the index
// bookkeeping of CONTRACT and PERMUTE, `RankSplit` and `undo_order` below.
#include "eteq.hpp"

#include <numeric>

namespace eteq
{

namespace
{

using Node = teq::TensptrT;
using RankPairs = eigen::PairVecT<teq::RankT>;
using DimPairs = eigen::PairVecT<teq::DimT>;

/// The place a rule is applied at
struct Site final
{
	teq::FuncptrT f;      ///< functor being differentiated
	teq::TensptrsT in;    ///< its operands
	Node up;              ///< gradient arriving at f
	size_t k;             ///< operand the gradient is taken for

	const Node& x (void) const { return in.front(); }
	Node y (void) const { return f; }

	template <typename T>
	T attr (void) const
	{
		T out;
		eigen::Packer<T>().unpack(out, *f);
		return out;
	}
};

template <typename ...ATTRS>
Node make (egen::_GENERATED_OPCODE code, teq::TensptrsT operands, ATTRS... attrs)
{
	return make_functor(code, operands, attrs...);
}

/// `value` in the dtype of `like`, extended to its shape
Node filled (float value, Node like)
{
	auto dtype = (egen::_GENERATED_DTYPE) like->get_meta().type_code();
	Node scalar = make_constant_tensor(&value, teq::Shape(), dtype);
	return make(egen::EXTEND, {scalar}, like);
}

Node times (Node a, Node b) { return make(egen::MUL, {a, b}); }

Node over (Node a, Node b) { return make(egen::DIV, {a, b}); }

/// d f / d operand, elementwise, chained with what arrives
Node chained (Node local, const Site& s) { return times(local, s.up); }

/// `t` (shaped like f) spread back over the dims a reduction f took away
Node unreduced (Node t, const Site& s)
{
	teq::Shape full = s.x()->shape();
	teq::DimsT factors(teq::rank_cap, 1);
	for (teq::RankT d : s.attr<std::set<teq::RankT>>())
	{
		if (d < teq::rank_cap) { factors[d] = full.at(d); }
	}
	return make(egen::EXTEND, {t}, factors);
}

/// The order that puts back what PERMUTE with `order` moved: a full
/// permutation p is completed from `order` (dims it does not name follow in
/// ascending order) and inverted
teq::RanksT undo_order (const teq::RanksT& order)
{
	teq::RanksT full;
	std::vector<bool> named(teq::rank_cap, false);
	for (size_t i = 0; i < order.size() && i < teq::rank_cap; ++i)
	{
		full.push_back(order[i]);
		named[order[i]] = true;
	}
	for (teq::RankT d = 0; d < teq::rank_cap; ++d)
	{
		if (false == named[d]) { full.push_back(d); }
	}
	teq::RanksT inverse(teq::rank_cap, 0);
	for (teq::RankT at = 0; at < teq::rank_cap; ++at) { inverse[full[at]] = at; }
	return inverse;
}

/// One operand of a CONTRACT: which of its significant dims are summed (in
/// the order the pairs list them) and which survive (ascending)
struct RankSplit final
{
	RankSplit (const RankPairs& pairs, bool second, const teq::Shape& shape)
	{
		std::vector<bool> taken(teq::rank_cap, false);
		for (auto& pr : pairs)
		{
			teq::RankT d = second ? pr.second : pr.first;
			summed.push_back(d);
			taken[d] = true;
		}
		teq::RankT significant = teq::narrow_shape(shape).size();
		for (teq::RankT d = 0; d < significant; ++d)
		{
			if (false == taken[d]) { kept.push_back(d); }
		}
	}

	teq::RanksT summed, kept;
};

// ---- the rules -----------------------------------------------------------

Node pass_through (const Site& s) { return s.up; }

Node rule_neg (const Site& s) { return make(egen::NEG, {s.up}); }

Node rule_tan (const Site& s) // up / cos(x)^2
{
	return over(s.up, make(egen::SQUARE, {make(egen::COS, {s.x()})}));
}

Node rule_log (const Site& s) { return over(s.up, s.x()); }

Node rule_sqrt (const Site& s) // up / (2 sqrt(x))
{
	return over(s.up, times(filled(2.f, s.y()), s.y()));
}

Node rule_abs (const Site& s) { return chained(over(s.x(), s.y()), s); }

Node rule_sin (const Site& s) { return chained(make(egen::COS, {s.x()}), s); }

Node rule_cos (const Site& s) { return chained(make(egen::NEG, {make(egen::SIN, {s.x()})}), s); }

Node rule_exp (const Site& s) { return chained(s.y(), s); }

Node rule_square (const Site& s) { return chained(times(filled(2.f, s.x()), s.x()), s); }

Node rule_cube (const Site& s) { return chained(times(filled(3.f, s.x()), make(egen::SQUARE, {s.x()})), s); }

Node rule_sigmoid (const Site& s) // y (1 - y)
{
	return chained(times(s.y(), make(egen::SUB, {filled(1.f, s.y()), s.y()})), s);
}

Node rule_tanh (const Site& s) // 1 - y^2
{
	return chained(make(egen::SUB, {filled(1.f, s.y()), make(egen::SQUARE, {s.y()})}), s);
}

Node rule_pow (const Site& s)
{
	const Node& base = s.in[0];
	const Node& exponent = s.in[1];
	if (0 == s.k) // e b^(e-1)
	{
		Node lowered = make(egen::POW, {base, make(egen::SUB, {exponent, filled(1.f, exponent)})});
		return chained(times(exponent, lowered), s);
	}
	return chained(times(make(egen::LOG, {base}), s.y()), s); // ln(b) b^e
}

Node rule_mul (const Site& s) // the product of the other factors
{
	teq::TensptrsT others;
	for (size_t i = 0; i < s.in.size(); ++i)
	{
		if (i != s.k) { others.push_back(s.in[i]); }
	}
	return chained(make(egen::MUL, others), s);
}

Node rule_extremum (const Site& s) // 1 where this operand is the one picked
{
	return chained(make(egen::EQ, {s.y(), s.in.at(s.k)}), s);
}

Node rule_sub (const Site& s) { return 0 == s.k ? s.up : make(egen::NEG, {s.up}); }

Node rule_div (const Site& s)
{
	const Node& num = s.in[0];
	const Node& den = s.in[1];
	if (0 == s.k) { return over(s.up, den); }
	return over(over(times(make(egen::NEG, {s.up}), num), den), den); // -up n / d / d
}

Node rule_reduce_sum (const Site& s) { return unreduced(s.up, s); }

Node rule_reduce_prod (const Site& s) // up * (y / x), both spread back
{
	return times(unreduced(s.up, s), over(unreduced(s.y(), s), s.x()));
}

Node rule_reduce_extremum (const Site& s) // EQ(y spread back, x * up spread back)
{
	return make(egen::EQ, {unreduced(s.y(), s), times(s.x(), unreduced(s.up, s))});
}

Node rule_extend (const Site& s) // sum over the dims that were repeated
{
	auto factors = eigen::unpack_extend(s.x()->shape(), *s.f);
	if (false == (bool) factors) { global::fatal("cannot find extend attributes"); }
	std::set<teq::RankT> repeated;
	for (teq::RankT d = 0; d < teq::rank_cap && d < factors->size(); ++d)
	{
		if ((*factors)[d] > 1) { repeated.emplace(d); }
	}
	return make(egen::REDUCE_SUM, {s.up}, repeated);
}

Node rule_permute (const Site& s)
{
	return make(egen::PERMUTE, {s.up}, undo_order(s.attr<teq::RanksT>()));
}

Node rule_reshape (const Site& s) { return make(egen::RESHAPE, {s.up}, s.x()->shape()); }

Node rule_matmul (const Site& s) // up . b^T  and  a^T . up
{
	teq::RanksT swap{1, 0};
	if (0 == s.k) { return make(egen::MATMUL, {s.up, make(egen::PERMUTE, {s.in[1]}, swap)}); }
	return make(egen::MATMUL, {make(egen::PERMUTE, {s.in[0]}, swap), s.up});
}

// f = CONTRACT(a, b, pairs) has the dims [kept dims of b..., kept dims of a...].
// The gradient for one operand is `up` contracted with the OTHER operand over
// that operand's kept dims.  The result of that inner CONTRACT(up, other) has
// the dims [other's remaining dims = the summed ones, in the other's dim
// order..., up's remaining dims = this operand's kept ones...]; read through
// the pairs, that is this operand's [summed..., kept...], and a PERMUTE puts
// every dim where the operand has it.
Node rule_contract (const Site& s)
{
	RankPairs pairs = s.attr<RankPairs>();
	RankSplit a(pairs, false, s.in[0]->shape()), b(pairs, true, s.in[1]->shape());
	const bool for_a = 0 == s.k;
	const RankSplit& mine = for_a ? a : b;
	const RankSplit& theirs = for_a ? b : a;
	Node other = s.in[for_a ? 1 : 0];
	// where the other operand's kept dims sit inside `up`: b's come first
	teq::RankT first = for_a ? 0 : (teq::RankT) b.kept.size();
	RankPairs sum_over;
	for (teq::RankT i = 0; i < theirs.kept.size(); ++i)
	{
		sum_over.push_back({(teq::RankT) (first + i), theirs.kept[i]});
	}
	if (sum_over.empty())
	{
		// nothing to sum: an outer product, spelled as a contraction over the
		// first singleton dim past both operands
		sum_over.push_back({(teq::RankT) teq::narrow_shape(s.up->shape()).size(),
			(teq::RankT) teq::narrow_shape(other->shape()).size()});
	}
	teq::RanksT arrives = mine.summed; // the order the inner result has this operand's dims in
	arrives.insert(arrives.end(), mine.kept.begin(), mine.kept.end());
	return make(egen::PERMUTE, {make(egen::CONTRACT, {s.up, other}, sum_over)}, undo_order(arrives));
}

Node rule_conv (const Site& s)
{
	teq::RanksT listed = s.attr<teq::RanksT>();
	teq::RanksT slides; // image dim each kernel dim slides along
	for (size_t i = 0; i < listed.size() && i < teq::rank_cap && listed[i] < teq::rank_cap; ++i)
	{
		slides.push_back(listed[i]);
	}
	if (0 == s.k)
	{
		// image: `up` padded by kernel extent - 1 on both sides of every dim a
		// kernel dim slides along, correlated with the kernel flipped in all
		// of its listed dims
		teq::Shape kshape = s.in[1]->shape();
		DimPairs border(teq::rank_cap, {0, 0});
		std::set<teq::RankT> flipped;
		for (teq::RankT i = 0; i < slides.size(); ++i)
		{
			teq::DimT reach = kshape.at(i) - 1;
			border[slides[i]] = {reach, reach};
			flipped.emplace(i);
		}
		return make(egen::CONV, {make(egen::PAD, {s.up}, border), make(egen::REVERSE, {s.in[1]}, flipped)}, slides);
	}
	// kernel: the image correlated with `up` dim for dim, moved to the kernel's dims
	teq::RanksT straight(teq::rank_cap);
	std::iota(straight.begin(), straight.end(), 0);
	return make(egen::PERMUTE, {make(egen::CONV, {s.in[0], s.up}, straight)}, slides);
}

Node rule_slice (const Site& s) // zeros around `up`, back to the operand's shape
{
	DimPairs cut = s.attr<DimPairs>();
	teq::Shape full = s.x()->shape();
	DimPairs border;
	for (teq::RankT d = 0; d < cut.size() && d < teq::rank_cap; ++d)
	{
		teq::DimT size = full.at(d);
		teq::DimT from = std::min<teq::DimT>(cut[d].first, size - 1);
		teq::DimT count = std::min<teq::DimT>(cut[d].second, size - from);
		border.push_back({from, (teq::DimT) (size - from - count)});
	}
	return make(egen::PAD, {s.up}, border);
}

Node rule_pad (const Site& s) // the part of `up` that is not border
{
	DimPairs border = s.attr<DimPairs>();
	teq::Shape padded = s.f->shape();
	DimPairs cut;
	for (teq::RankT d = 0; d < border.size() && d < teq::rank_cap; ++d)
	{
		cut.push_back({border[d].first, (teq::DimT) (padded.at(d) - border[d].first - border[d].second)});
	}
	return make(egen::SLICE, {s.up}, cut);
}

Node rule_concat (const Site& s) // this operand's stretch of `up` along the axis
{
	teq::RankT axis = s.attr<teq::RankT>();
	DimPairs cut(std::max<size_t>(teq::rank_cap, axis), {0, std::numeric_limits<teq::DimT>::max()});
	if (s.in.size() > 2) { cut[axis] = {(teq::DimT) s.k, 1}; } // many operands: one index each
	else
	{
		teq::DimT from = 0 == s.k ? 0 : s.in[0]->shape().at(axis);
		cut[axis] = {from, s.in[s.k]->shape().at(axis)};
	}
	return make(egen::SLICE, {s.up}, cut);
}

Node rule_stride (const Site& s)
{
	return make(egen::SCATTER, {s.up}, s.x()->shape(), s.attr<teq::DimsT>());
}

Node rule_scatter (const Site& s)
{
	teq::DimsT steps = s.attr<teq::DimsT>();
	if (steps.size() > teq::rank_cap) { steps.resize(teq::rank_cap); }
	return make(egen::STRIDE, {s.up}, steps);
}

Node rule_reverse (const Site& s) { return make(egen::REVERSE, {s.up}, s.attr<std::set<teq::RankT>>()); }

Node rule_select (const Site& s)
{
	if (0 == s.k) { return filled(0.f, s.x()); } // nothing flows into the condition
	Node nothing = filled(0.f, s.y());
	return 1 == s.k ? make(egen::SELECT, {s.in[0], s.up, nothing}) : make(egen::SELECT, {s.in[0], nothing, s.up});
}

Node rule_zero (const Site& s) { return filled(0.f, s.x()); }

Node rule_refused (const Site& s)
{
	global::fatalf("cannot derive %s", s.f->get_opcode().name_.c_str());
}

using Rule = Node (*) (const Site&);

const std::vector<Rule>& rule_table (void)
{
	static const std::vector<Rule> table = []
	{
		std::vector<Rule> t(egen::_N_GENERATED_OPCODES, nullptr);
		for (auto code : {egen::IDENTITY, egen::CAST, egen::ROUND, egen::ADD}) { t[code] = pass_through; }
		t[egen::NEG] = rule_neg;
		t[egen::TAN] = rule_tan;
		t[egen::LOG] = rule_log;
		t[egen::SQRT] = rule_sqrt;
		t[egen::ABS] = rule_abs;
		t[egen::SIN] = rule_sin;
		t[egen::COS] = rule_cos;
		t[egen::EXP] = rule_exp;
		t[egen::SQUARE] = rule_square;
		t[egen::CUBE] = rule_cube;
		t[egen::SIGMOID] = rule_sigmoid;
		t[egen::TANH] = rule_tanh;
		t[egen::POW] = rule_pow;
		t[egen::MUL] = rule_mul;
		t[egen::MAX] = t[egen::MIN] = rule_extremum;
		t[egen::SUB] = rule_sub;
		t[egen::DIV] = rule_div;
		t[egen::REDUCE_SUM] = rule_reduce_sum;
		t[egen::REDUCE_PROD] = rule_reduce_prod;
		t[egen::REDUCE_MAX] = t[egen::REDUCE_MIN] = rule_reduce_extremum;
		t[egen::EXTEND] = rule_extend;
		t[egen::PERMUTE] = rule_permute;
		t[egen::RESHAPE] = rule_reshape;
		t[egen::MATMUL] = rule_matmul;
		t[egen::CONTRACT] = rule_contract;
		t[egen::CONV] = rule_conv;
		t[egen::SLICE] = rule_slice;
		t[egen::PAD] = rule_pad;
		t[egen::CONCAT] = rule_concat;
		t[egen::STRIDE] = rule_stride;
		t[egen::SCATTER] = rule_scatter;
		t[egen::REVERSE] = rule_reverse;
		t[egen::SELECT] = rule_select;
		for (auto code : {egen::RAND_UNIF, egen::EQ, egen::NEQ, egen::GT, egen::LT}) { t[code] = rule_zero; }
		for (auto code : {egen::ASSIGN, egen::ASSIGN_ADD, egen::ASSIGN_SUB, egen::ASSIGN_MUL, egen::ASSIGN_DIV,
			egen::ARGMAX}) { t[code] = rule_refused; }
		return t;
	}();
	return table;
}

/// A leaf of the dtype and shape of `reference` holding `value` everywhere
Node constant_shaped_like (float value, teq::iTensor& reference)
{
	auto dtype = (egen::_GENERATED_DTYPE) reference.get_meta().type_code();
	teq::Shape shape = reference.shape();
	std::vector<float> data(shape.n_elems(), value);
	return make_constant_tensor(data.data(), shape, dtype);
}

}

teq::TensptrT DerivativeFuncs::lderive (teq::FuncptrT op, teq::TensptrT supgrad, size_t arg_idx) const
{
	teq::Opcode opcode = op->get_opcode();
	auto& table = rule_table();
	Rule rule = opcode.code_ < table.size() ? table[opcode.code_] : nullptr;
	if (nullptr == rule) { global::fatalf("Unknown op %s", opcode.name_.c_str()); }
	Site site{op, op->get_args(), supgrad, arg_idx};
	return rule(site);
}

teq::TensptrT DerivativeFuncs::get_const_one (teq::iTensor& reference) const
{
	return constant_shaped_like(1.f, reference);
}

teq::TensptrT DerivativeFuncs::get_const_zero (teq::iTensor& reference) const
{
	return constant_shaped_like(0.f, reference);
}

teq::TensptrT DerivativeFuncs::add (teq::TensptrsT elems) const
{
	if (elems.empty()) { global::fatal("cannot add nothing"); }
	return make_functor(egen::ADD, elems);
}

}
