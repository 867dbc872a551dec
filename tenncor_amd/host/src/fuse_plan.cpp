// Which functors of an evaluation pass share a launch (see fuse_plan.hpp).
#include "fuse_plan.hpp"

#include <limits>
#include <type_traits>
#include <algorithm>
#include <functional>
#include <map>
#include <set>

#include "eigen_ops.hpp"

namespace eigen
{

namespace
{

enum Kind { OTHER = 0, EW, VIEW };

constexpr size_t max_members = 48;
constexpr int far_behind = 32;  // positions in the pass between a launch and a node that could still join it

struct View final
{
	teq::iTensor* base = nullptr;
	int64_t off = 0;
	int64_t stride[8];
	uint64_t lo[8];
	uint64_t hi[8];

	bool operator < (const View& o) const
	{
		if (base != o.base) { return base < o.base; }
		if (off != o.off) { return off < o.off; }
		int c = memcmp(stride, o.stride, sizeof(stride));
		if (c != 0) { return c < 0; }
		c = memcmp(lo, o.lo, sizeof(lo));
		if (c != 0) { return c < 0; }
		return memcmp(hi, o.hi, sizeof(hi)) < 0;
	}
};

struct Node final
{
	Observable* f = nullptr;
	Kind kind = OTHER;
	int op = 0;
	int dtype = 0;
	bool target = false;
	bool absorbed = false;      // a VIEW no launch of its own computes
	int swapped_from = -1;      // PERMUTE launched as the swapped product of this CONTRACT node
	int conv_from = -1;         // this node receives the result of that CONV node, launched over views (itself, or the end of a chain behind it)
	bool through_conv = false;  // PAD / PERMUTE / REVERSE that only such convolutions read through, or
	                            // a node between such a CONV and the node that receives its result
	bool parts_folded = false;  // CONCAT / ADD of PADs that only products read, part by part
	int part_products = -1;     // CONTRACT, or ADD over CONTRACT terms, launched as products over parts (index into part_calls_)
	bool ranged = false;        // such a product that leaves its K ranges for the groups that read it: never laid out
	bool summed = false;        // ADD launched as one sum of the products it adds
	bool summed_term = false;   // CONTRACT / PERMUTE that is a term of such a sum
	std::vector<int> args;      // index of the functor operand, -1 for a leaf
	teq::TensptrsT arg_tens;
	std::vector<int> consumers; // functors of this pass reading the node
	// args with folded single-operand IDENTITY nodes looked through (an alias
	// of an elementwise node must not keep that node out of its reader's
	// group), and the aliases skipped on the way
	std::vector<int> direct;
	std::vector<std::vector<int>> aliases;
	Shape8 shape;
};

bool is_unary (int op)
{
	return op >= egen::ABS && op <= egen::CUBE;
}

bool is_binary (int op)
{
	return op >= egen::POW && op <= egen::GT;
}

bool is_assign (int op)
{
	return op >= egen::ASSIGN && op <= egen::ASSIGN_DIV;
}

/// Nodes whose value is their first operand's buffer (TensRef / UnsafeTensRef):
/// reading them reads whatever that buffer holds at the time of the read
bool is_buffer_alias (int op)
{
	return op == egen::IDENTITY || op == egen::RESHAPE || op == egen::SLICE;
}

View dense_view (teq::iTensor* tens, const Shape8& shape)
{
	View v;
	v.base = tens;
	int64_t s = 1;
	for (int d = 0; d < 8; ++d)
	{
		v.stride[d] = s;
		s *= (int64_t) shape[d];
		v.lo[d] = 0;
		v.hi[d] = shape[d];
	}
	return v;
}

bool scalar_constant (const teq::iTensor* tens, double& value)
{
	auto leaf = dynamic_cast<const teq::iLeaf*>(tens);
	if (nullptr == leaf || leaf->get_usage() != teq::IMMUTABLE || leaf->shape().n_elems() != 1)
	{
		return false;
	}
	const void* data = leaf->device().data();
	switch (leaf->get_meta().type_code())
	{
		// a double carries every value of a type of at most 32 bits; a 64-bit
		// integer only below 2^53, beyond which the constant stays an operand
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) case egen::ENUM:\
			value = (double) *(const CTYPE*) data;\
			return sizeof(CTYPE) < 8 || std::is_floating_point<CTYPE>::value ||\
				(value > -0x1p53 && value < 0x1p53);
		EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
		default: return false;
	}
}

struct Planner final
{
	Planner (const std::vector<Observable*>& funcs, const teq::TensSetT& targets)
	{
		nodes_.resize(funcs.size());
		for (size_t i = 0; i < funcs.size(); ++i) { index_.emplace(funcs[i], (int) i); }
		for (size_t i = 0; i < funcs.size(); ++i)
		{
			Node& n = nodes_[i];
			n.f = funcs[i];
			n.op = (int) n.f->get_opcode().code_;
			n.dtype = (int) n.f->get_meta().type_code();
			n.target = targets.count(n.f) > 0;
			n.shape = shape8(n.f->shape());
			n.arg_tens = n.f->get_args();
			for (auto& arg : n.arg_tens)
			{
				auto it = index_.find(arg.get());
				int a = it == index_.end() ? -1 : it->second;
				n.args.push_back(a);
				if (a >= 0 && (nodes_[a].consumers.empty() || nodes_[a].consumers.back() != (int) i))
				{
					nodes_[a].consumers.push_back((int) i);
				}
			}
			n.kind = classify(n);
		}
		find_written();
		// PERMUTE{1,0} of a matrix-valued CONTRACT nothing else reads: launch the
		// swapped product instead; the CONTRACT node is looked through like a view
		for (size_t i = 0; i < nodes_.size(); ++i)
		{
			Node& n = nodes_[i];
			if (n.op != egen::PERMUTE || n.args.size() != 1 || n.args[0] < 0) { continue; }
			Node& c = nodes_[n.args[0]];
			if (c.op != egen::CONTRACT || c.target || c.consumers.size() != 1 || c.args.size() != 2) { continue; }
			teq::RanksT order;
			Packer<teq::RanksT>().unpack(order, *n.f);
			bool swaps = order.size() >= 2 && order[0] == 1 && order[1] == 0;
			for (size_t d = 2; d < order.size() && swaps; ++d) { swaps = order[d] == d; }
			for (int d = 2; d < 8 && swaps; ++d) { swaps = c.shape[d] == 1; }
			if (false == swaps || c.shape[0] == 1 || c.shape[1] == 1) { continue; }
			// one surviving dim from each operand: only then is the transpose
			// of the result the product with the operands exchanged
			PairVecT<teq::RankT> dims;
			Packer<PairVecT<teq::RankT>>().unpack(dims, *c.f);
			size_t free_dims[2] = {0, 0};
			for (size_t k = 0; k < 2; ++k)
			{
				Shape8 shape = shape8(c.arg_tens[k]->shape());
				for (teq::RankT d = 0; d < 8; ++d)
				{
					bool contracted = std::any_of(dims.begin(), dims.end(), [&](const std::pair<teq::RankT,teq::RankT>& pr)
					{
						return (k == 0 ? pr.first : pr.second) == d;
					});
					free_dims[k] += shape[d] > 1 && false == contracted;
				}
			}
			if (free_dims[0] != 1 || free_dims[1] != 1) { continue; }
			// the product would read its operands where the PERMUTE stands
			if (written_between(n.args[0], {0, 1}, n.args[0], (int) i)) { continue; }
			n.kind = OTHER;
			n.swapped_from = n.args[0];
			c.kind = VIEW;
			c.absorbed = true;
		}
		find_viewed_convs();
		find_summed_products();
		// a view is folded away when everything that reads it can read through it
		std::vector<int> last_reader(nodes_.size(), 0); // position of the last launch reading through a folded view
		for (size_t i = nodes_.size(); i-- > 0;)
		{
			Node& n = nodes_[i];
			if (n.kind != VIEW || n.target || n.consumers.empty() || n.op == egen::CONTRACT || n.through_conv || n.summed_term) { continue; }
			n.absorbed = std::all_of(n.consumers.begin(), n.consumers.end(), [&](int c)
			{
				// (a CONTRACT that is launched as the swapped product of the PERMUTE behind it, or
				// as a term of a sum of products, is marked like a view but reads its operands
				// from memory)
				return nodes_[c].kind == EW || (nodes_[c].kind == VIEW && nodes_[c].absorbed && false == nodes_[c].through_conv &&
					nodes_[c].op != egen::CONTRACT && false == nodes_[c].summed_term);
			});
			if (false == n.absorbed) { continue; }
			for (int c : n.consumers)
			{
				last_reader[i] = std::max(last_reader[i], nodes_[c].kind == EW ? c : last_reader[c]);
			}
			// a materialised view holds the operand's value from where it stands
			// in the pass: it cannot be folded into a launch that runs after an
			// assignment to that operand (IDENTITY holds nothing: it is the
			// operand's buffer, whoever reads it)
			if (n.op != egen::IDENTITY && written_between((int) i, {0}, (int) i, last_reader[i]))
			{
				n.absorbed = false;
			}
		}
		find_part_products();
		for (Node& n : nodes_)
		{
			for (int a : n.args)
			{
				std::vector<int> skipped;
				while (a >= 0 && is_alias(a))
				{
					skipped.push_back(a);
					a = nodes_[a].args[0];
				}
				n.direct.push_back(a);
				n.aliases.push_back(skipped);
			}
		}
		uf_.resize(nodes_.size());
		for (size_t i = 0; i < uf_.size(); ++i) { uf_[i] = (int) i; }
		minpos_.resize(nodes_.size());
		maxpos_.resize(nodes_.size());
		members_.resize(nodes_.size());
		deps_.resize(nodes_.size());
		vdeps_.resize(nodes_.size());
		stamp_.assign(nodes_.size(), 0);
	}

	/// Node a has a buffer of its own when its launch has run (whose reads are counted)
	bool holds_value (int a) const
	{
		const Node& n = nodes_[a];
		return false == (n.kind == VIEW && n.absorbed) && false == n.ranged;
	}

	/// Operand k of a node is the first occurrence of that tensor among its operands:
	/// a node is one consumer of a tensor however often it names it (MUL(x, x))
	static bool first_occurrence (const Node& n, size_t k)
	{
		for (size_t j = 0; j < k; ++j)
		{
			if (n.arg_tens[j] == n.arg_tens[k]) { return false; }
		}
		return true;
	}

	bool is_alias (int i) const
	{
		const Node& n = nodes_[i];
		return n.kind == VIEW && n.absorbed && n.op == egen::IDENTITY;
	}

	// ---- convolutions over views ----

	struct ConvFold final
	{
		std::vector<int> image, kernel; // folded nodes from the CONV's operand down to (excluding) the tensor that is read
		std::vector<int> result;        // nodes behind the CONV up to (including) the one that receives the result
	};

	static bool is_layout (const Node& n)
	{
		return (n.op == egen::PERMUTE || n.op == egen::REVERSE) && n.args.size() == 1;
	}

	bool is_plain_conv (int i) const
	{
		const Node& n = nodes_[i];
		return n.op == egen::CONV && n.kind == OTHER && n.args.size() == 2 &&
			(int) n.arg_tens[0]->get_meta().type_code() == n.dtype &&
			(int) n.arg_tens[1]->get_meta().type_code() == n.dtype;
	}

	/// Position of the last convolution that would read through node v
	int last_conv_reader (int v) const
	{
		int last = -1;
		for (int c : nodes_[v].consumers)
		{
			last = std::max(last, nodes_[c].op == egen::CONV ? c : last_conv_reader(c));
		}
		return last;
	}

	/// PAD node whose only readers are convolutions taking it as their image
	bool pad_feeds_convs (int v) const
	{
		const Node& n = nodes_[v];
		if (n.op != egen::PAD || n.kind != VIEW || n.target || n.consumers.empty()) { return false; }
		for (int c : n.consumers)
		{
			if (false == is_plain_conv(c) || nodes_[c].args[0] != v || nodes_[c].args[1] == v) { return false; }
		}
		// the convolutions read the operand where they stand, not where the PAD does
		return false == written_between(v, {0}, v, last_conv_reader(v) + 1);
	}

	/// PERMUTE / REVERSE node that only convolutions read, directly, through
	/// such a PAD or through further nodes of this kind
	bool layout_feeds_convs (int v)
	{
		auto memo = feeds_convs_.find(v);
		if (memo != feeds_convs_.end()) { return memo->second; }
		const Node& n = nodes_[v];
		bool ok = is_layout(n) && false == n.target && false == n.consumers.empty() &&
			n.swapped_from < 0 && false == n.summed_term;
		for (size_t k = 0; k < n.consumers.size() && ok; ++k)
		{
			int c = n.consumers[k];
			if (nodes_[c].op == egen::CONV) { ok = is_plain_conv(c); }
			else if (nodes_[c].op == egen::PAD) { ok = pad_feeds_convs(c); }
			else { ok = is_layout(nodes_[c]) && nodes_[c].args[0] == v && layout_feeds_convs(c); }
		}
		ok = ok && false == written_between(v, {0}, v, last_conv_reader(v) + 1);
		feeds_convs_[v] = ok;
		return ok;
	}

	void find_viewed_convs (void)
	{
		for (size_t i = 0; i < nodes_.size(); ++i)
		{
			if (false == is_plain_conv((int) i)) { continue; }
			ConvFold fold;
			int cur = nodes_[i].args[0];
			if (cur >= 0 && cur != nodes_[i].args[1] && pad_feeds_convs(cur))
			{
				fold.image.push_back(cur);
				cur = nodes_[cur].args[0];
			}
			while (cur >= 0 && layout_feeds_convs(cur))
			{
				fold.image.push_back(cur);
				cur = nodes_[cur].args[0];
			}
			cur = nodes_[i].args[1];
			while (cur >= 0 && layout_feeds_convs(cur))
			{
				fold.kernel.push_back(cur);
				cur = nodes_[cur].args[0];
			}
			// behind the convolution: one reader at a time, each only moving data,
			// standing where nothing rewrites the operands in between
			cur = (int) i;
			while (false == nodes_[cur].target && nodes_[cur].consumers.size() == 1)
			{
				int next = nodes_[cur].consumers[0];
				const Node& m = nodes_[next];
				if (false == is_layout(m) || m.args[0] != cur || m.swapped_from >= 0 || m.summed_term ||
					m.dtype != nodes_[i].dtype) { break; }
				fold.result.push_back(next);
				cur = next;
			}
			if (false == fold.result.empty())
			{
				// the launch stands where the last of them does
				bool rewritten = written_between((int) i, {0, 1}, (int) i, fold.result.back());
				for (const std::vector<int>* chain : {&fold.image, &fold.kernel})
				{
					for (int v : *chain) { rewritten = rewritten || written_between(v, {0}, (int) i, fold.result.back()); }
				}
				if (rewritten) { fold.result.clear(); }
			}
			if (fold.image.empty() && fold.kernel.empty() && fold.result.empty()) { continue; }
			folds_.emplace((int) i, fold);
		}
		// marks are set once every decision has been taken on the graph as built
		for (auto& kv : folds_)
		{
			const ConvFold& fold = kv.second;
			for (const std::vector<int>* chain : {&fold.image, &fold.kernel})
			{
				for (int v : *chain)
				{
					nodes_[v].kind = VIEW;
					nodes_[v].absorbed = true;
					nodes_[v].through_conv = true;
				}
			}
			int last = fold.result.empty() ? kv.first : fold.result.back();
			if (false == fold.result.empty())
			{
				nodes_[kv.first].kind = VIEW;
				nodes_[kv.first].absorbed = true;
				nodes_[kv.first].through_conv = true;
				for (int v : fold.result)
				{
					if (v == last) { break; }
					nodes_[v].kind = VIEW;
					nodes_[v].absorbed = true;
					nodes_[v].through_conv = true;
				}
				nodes_[last].kind = OTHER;
			}
			nodes_[last].conv_from = kv.first;
		}
	}

	// ---- products over the parts of concatenations ----

	struct Part final
	{
		uint64_t start = 0, extent = 0; // along the axis of the concatenation
		View view;                      // of the part, in its own coordinates
	};

	struct Parts final
	{
		int axis = 0;
		std::vector<Part> parts;
	};

	/// A matrix seen in a view: element (f, k) at base[off + f * sf + k * sk]
	struct Mat final
	{
		teq::iTensor* base = nullptr;
		int64_t off = 0, sf = 0, sk = 0;
		uint64_t F = 1, K = 1;
	};

	/// Node z as a concatenation of views along one dim: a CONCAT, or an ADD of
	/// PADs (each read by the ADD alone) that tile one dim without overlap
	bool concat_parts (int z, Parts& out)
	{
		const Node& n = nodes_[z];
		if (n.kind != EW || n.target || n.args.size() < 2 || n.consumers.empty()) { return false; }
		out.parts.clear();
		if (n.op == egen::CONCAT)
		{
			teq::RankT axis = 0;
			Packer<teq::RankT>().unpack(axis, *n.f);
			if (axis >= 8) { return false; }
			out.axis = axis;
			uint64_t at = 0;
			for (size_t k = 0; k < n.args.size(); ++k)
			{
				Part part;
				part.start = at;
				part.extent = shape8(n.arg_tens[k]->shape())[axis];
				part.view = view_of_arg(z, k);
				at += part.extent;
				out.parts.push_back(part);
			}
		}
		else if (n.op == egen::ADD)
		{
			int axis = -1;
			for (size_t k = 0; k < n.args.size(); ++k)
			{
				int a = n.args[k];
				if (a < 0) { return false; }
				const Node& pad = nodes_[a];
				if (pad.op != egen::PAD || pad.kind != VIEW || false == pad.absorbed || pad.consumers.size() != 1) { return false; }
				PairVecT<teq::DimT> encoding;
				Packer<PairVecT<teq::DimT>>().unpack(encoding, *pad.f);
				Part part;
				int padded = -1;
				for (size_t d = 0, m = std::min(encoding.size(), (size_t) 8); d < m; ++d)
				{
					if (encoding[d].first == 0 && encoding[d].second == 0) { continue; }
					if (padded >= 0) { return false; }
					padded = (int) d;
					part.start = encoding[d].first;
				}
				if (padded < 0 || (axis >= 0 && padded != axis)) { return false; }
				axis = padded;
				part.extent = shape8(pad.arg_tens[0]->shape())[axis];
				part.view = view_of_arg(a, 0);
				out.parts.push_back(part);
			}
			out.axis = axis;
			std::sort(out.parts.begin(), out.parts.end(), [](const Part& x, const Part& y) { return x.start < y.start; });
			uint64_t at = 0;
			for (const Part& part : out.parts)
			{
				if (part.start != at) { return false; }
				at += part.extent;
			}
			if (at != n.shape[axis]) { return false; }
		}
		else { return false; }
		// the views beneath are counted as read with the products: nothing else may read through them
		for (int a : n.args)
		{
			if (a >= 0 && false == sole_chain(a)) { return false; }
		}
		// parts that are whole values: no zero border inside them
		for (const Part& part : out.parts)
		{
			Shape8 pshape = n.shape;
			pshape[out.axis] = part.extent;
			for (int d = 0; d < 8; ++d)
			{
				if (part.view.lo[d] != 0 || part.view.hi[d] != pshape[d]) { return false; }
			}
		}
		return true;
	}

	/// Folded views from node a down, each with one reader
	bool sole_chain (int a) const
	{
		const Node& n = nodes_[a];
		if (false == (n.kind == VIEW && n.absorbed)) { return true; }
		if (n.consumers.size() != 1 || n.target || n.op == egen::REVERSE) { return false; }
		for (int b : n.args)
		{
			if (b >= 0 && false == sole_chain(b)) { return false; }
		}
		return true;
	}

	/// A view of extents `shape` with contracted dim `cdim` as a matrix; false
	/// when more than one other dim is significant
	static bool as_matrix (const View& v, const Shape8& shape, int cdim, Mat& out)
	{
		out = Mat();
		out.base = v.base;
		out.off = v.off;
		out.K = shape[cdim];
		out.sk = v.stride[cdim];
		int fdim = -1;
		for (int d = 0; d < 8; ++d)
		{
			if (d == cdim || shape[d] == 1) { continue; }
			if (fdim >= 0) { return false; }
			fdim = d;
		}
		if (fdim >= 0)
		{
			out.F = shape[fdim];
			out.sf = v.stride[fdim];
		}
		return true;
	}

	/// One side of a product: the operand as one matrix, or as the matrices of
	/// its parts when it is a concatenation that is being folded
	struct Side final
	{
		int cdim = 0;
		int z = -1;              // folded concatenation, -1: a plain operand
		bool along_k = false;    // the parts split the contracted dim (else the surviving one)
		std::vector<Mat> mats;   // one per part (one in all for a plain operand)
		std::vector<uint64_t> starts;
	};

	bool make_side (int c, size_t k, int cdim, const std::set<int>& folded, Side& out)
	{
		const Node& n = nodes_[c];
		out = Side();
		out.cdim = cdim;
		int a = n.args[k];
		Shape8 shape = shape8(n.arg_tens[k]->shape());
		if (a >= 0 && folded.count(a))
		{
			const Parts& parts = part_lists_.at(a);
			out.z = a;
			out.along_k = parts.axis == cdim;
			for (const Part& part : parts.parts)
			{
				Shape8 pshape = shape;
				pshape[parts.axis] = part.extent;
				Mat m;
				if (false == as_matrix(part.view, pshape, cdim, m)) { return false; }
				// the axis must be the contracted dim or the one that survives
				if (false == out.along_k && (shape[parts.axis] == 1)) { return false; }
				out.mats.push_back(m);
				out.starts.push_back(part.start);
			}
			if (false == out.along_k)
			{
				// the surviving dim must be the axis
				int fdim = -1;
				for (int d = 0; d < 8; ++d)
				{
					if (d != cdim && shape[d] > 1) { fdim = d; }
				}
				if (fdim != parts.axis) { return false; }
			}
			return true;
		}
		if (a >= 0 && nodes_[a].kind == VIEW && nodes_[a].absorbed) { return false; }
		Mat m;
		if (false == as_matrix(dense_view(n.arg_tens[k].get(), shape), shape, cdim, m)) { return false; }
		out.mats.push_back(m);
		out.starts.push_back(0);
		return true;
	}

	static uint64_t gcd64 (uint64_t x, uint64_t y)
	{
		while (y)
		{
			uint64_t r = x % y;
			x = y;
			y = r;
		}
		return x;
	}

	/// Layout flags and leading dims of one term; false when the matrices do not
	/// lie the way the product kernels read them
	static bool term_layout (const Mat& a, const Mat& b, bool& trans_a, bool& trans_b, PartProducts::Term& term)
	{
		term.a = a.base;
		term.b = b.base;
		term.a_off = a.off;
		term.b_off = b.off;
		// A(m, k) at m * sf + k * sk; B(k, n) at k * sk + n * sf
		if (a.sk == 1 && (a.F == 1 || a.sf >= (int64_t) a.K)) { trans_a = false; term.lda = a.F == 1 ? a.K : (uint64_t) a.sf; }
		else if (a.sf == 1 && a.sk >= (int64_t) a.F) { trans_a = true; term.lda = (uint64_t) a.sk; }
		else { return false; }
		if (b.sf == 1 && b.sk >= (int64_t) b.F) { trans_b = false; term.ldb = (uint64_t) b.sk; }
		else if (b.sk == 1 && (b.F == 1 || b.sf >= (int64_t) b.K)) { trans_b = true; term.ldb = b.F == 1 ? b.K : (uint64_t) b.sf; }
		else { return false; }
		return true;
	}

	/// Whether the matrix cores take the product (else the terms would be launched one by one)
	static bool fast_shape (const PartProducts::Product& p)
	{
		bool ok = p.terms.size() >= 1 && p.terms.size() <= 128 && p.M >= 32 && p.N >= 32 && p.K >= 16 && p.K % 16 == 0 &&
			(p.trans_a ? p.M : p.K) % 4 == 0 && (p.trans_b ? p.K : p.N) % 4 == 0 && p.c_off % 4 == 0 && p.ldc % 4 == 0;
		for (const PartProducts::Term& t : p.terms)
		{
			ok = ok && t.a_off % 4 == 0 && t.b_off % 4 == 0 && t.lda % 4 == 0 && t.ldb % 4 == 0;
		}
		return ok;
	}

	/// The contraction dims of CONTRACT node c when it is a product of two
	/// matrices over one pair of dims
	bool single_pair (int c, int& adim, int& bdim) const
	{
		const Node& n = nodes_[c];
		if ((n.op != egen::CONTRACT && n.op != egen::MATMUL) || n.args.size() != 2) { return false; }
		PairVecT<teq::RankT> dims;
		if (n.op == egen::MATMUL) { dims.push_back({0, 1}); } // cfg/ops.yml:507-513: dim 0 of a meets dim 1 of b
		else { Packer<PairVecT<teq::RankT>>().unpack(dims, *n.f); }
		// pairs of dims of extent 1 change nothing
		Shape8 ashape = shape8(n.arg_tens[0]->shape()), bshape = shape8(n.arg_tens[1]->shape());
		int found = 0;
		for (auto& pr : dims)
		{
			if (pr.first >= 8 || pr.second >= 8) { return false; }
			if (ashape[pr.first] == 1 && bshape[pr.second] == 1) { continue; }
			adim = pr.first;
			bdim = pr.second;
			++found;
		}
		return found == 1;
	}

	/// CONTRACT node c (launched on its own) over the parts of its operands
	bool terms_of_contract (int c, const std::set<int>& folded, PartProducts& out)
	{
		const Node& n = nodes_[c];
		int adim = 0, bdim = 0;
		if (n.kind != OTHER || n.dtype != egen::FLOAT || false == single_pair(c, adim, bdim)) { return false; }
		if (n.f->shape().n_elems() <= 4096) { return false; }
		Side sa, sb;
		if (false == make_side(c, 0, adim, folded, sa) || false == make_side(c, 1, bdim, folded, sb)) { return false; }
		// exactly one side split along the contracted dim, the other one whole
		const bool a_parts = sa.z >= 0, b_parts = sb.z >= 0;
		if (a_parts == b_parts) { return false; }
		const Side& split = a_parts ? sa : sb;
		const Side& whole = a_parts ? sb : sa;
		if (false == split.along_k) { return false; }
		uint64_t chunk = 0;
		for (const Mat& m : split.mats) { chunk = gcd64(chunk, m.K); }
		if (chunk == 0) { return false; }
		PartProducts::Product prod;
		const Mat& w = whole.mats[0];
		prod.M = sa.mats[0].F;
		prod.N = sb.mats[0].F;
		prod.K = chunk;
		prod.ldc = prod.N;
		// the columns (rows) the SLICEs that are all that read the result look at
		uint64_t m0 = 0, n0 = 0;
		Shape8 olo, ohi;
		out.partial = false == n.target && slices_window(n.f, n.f->shape(), olo, ohi);
		// the result holds b's surviving dim before a's (cfg/ops.yml:547-565)
		int sig[2] = {-1, -1}, nsig = 0;
		for (int d = 0; d < 8; ++d)
		{
			if (n.shape[d] > 1)
			{
				if (nsig < 2) { sig[nsig] = d; }
				++nsig;
			}
		}
		if (nsig != 2 || n.shape[sig[0]] != prod.N || n.shape[sig[1]] != prod.M) { return false; }
		if (out.partial)
		{
			n0 = olo[sig[0]];
			m0 = olo[sig[1]];
			prod.N = ohi[sig[0]] - n0;
			prod.M = ohi[sig[1]] - m0;
			out.partial = prod.N < n.shape[sig[0]] || prod.M < n.shape[sig[1]];
		}
		prod.c_off = (int64_t) (m0 * prod.ldc + n0);
		bool first = true;
		for (size_t p = 0; p < split.mats.size(); ++p)
		{
			for (uint64_t k0 = 0; k0 < split.mats[p].K; k0 += chunk)
			{
				Mat ma = a_parts ? split.mats[p] : w, mb = a_parts ? w : split.mats[p];
				Mat& part = a_parts ? ma : mb;
				Mat& other = a_parts ? mb : ma;
				part.off += (int64_t) k0 * part.sk;
				other.off += (int64_t) (split.starts[p] + k0) * other.sk;
				ma.K = mb.K = chunk;
				ma.off += (int64_t) m0 * ma.sf;
				mb.off += (int64_t) n0 * mb.sf;
				ma.F = prod.M;
				mb.F = prod.N;
				PartProducts::Term term;
				bool ta = false, tb = false;
				if (false == term_layout(ma, mb, ta, tb, term)) { return false; }
				if (false == first && (ta != prod.trans_a || tb != prod.trans_b)) { return false; }
				prod.trans_a = ta;
				prod.trans_b = tb;
				first = false;
				prod.terms.push_back(term);
			}
		}
		if (false == fast_shape(prod)) { return false; }
		out.node = n.f;
		out.dtype = n.dtype;
		out.products = {prod};
		out.label = "parts " + nodes_[split.z].f->get_opcode().name_ + "+" + n.f->get_opcode().name_ + " x" + std::to_string(prod.terms.size()) +
			(out.partial ? "+SLICE" : "");
		return true;
	}

	/// ADD node s launched as one sum of products (find_summed_products) whose
	/// terms' operands are concatenations along the dims that survive: one sum
	/// of products per block of the result
	bool blocks_of_sum (int s, const std::set<int>& folded, PartProducts& out)
	{
		const Node& n = nodes_[s];
		if (false == n.summed || n.dtype != egen::FLOAT) { return false; }
		PartProducts::Product proto;
		std::vector<std::vector<PartProducts::Product>> blocks; // [part of a][part of b]
		bool any_parts = false;
		for (size_t t = 0; t < n.args.size(); ++t)
		{
			int arg = n.args[t];
			const bool swapped = nodes_[arg].op == egen::PERMUTE;
			int c = swapped ? nodes_[arg].args[0] : arg;
			int adim = 0, bdim = 0;
			if (false == single_pair(c, adim, bdim)) { return false; }
			Side s0, s1;
			if (false == make_side(c, 0, adim, folded, s0) || false == make_side(c, 1, bdim, folded, s1)) { return false; }
			// the product as launched: operands exchanged under a PERMUTE{1,0}
			const Side& sa = swapped ? s1 : s0;
			const Side& sb = swapped ? s0 : s1;
			if ((sa.z >= 0 && sa.along_k) || (sb.z >= 0 && sb.along_k)) { return false; }
			any_parts = any_parts || sa.z >= 0 || sb.z >= 0;
			if (t == 0)
			{
				blocks.assign(sa.mats.size(), std::vector<PartProducts::Product>(sb.mats.size()));
				uint64_t nfull = 0;
				for (const Mat& m : sb.mats) { nfull += m.F; }
				for (size_t i = 0; i < sa.mats.size(); ++i)
				{
					for (size_t j = 0; j < sb.mats.size(); ++j)
					{
						PartProducts::Product& p = blocks[i][j];
						p.M = sa.mats[i].F;
						p.N = sb.mats[j].F;
						p.K = sa.mats[i].K;
						p.ldc = nfull;
						p.c_off = (int64_t) (sa.starts[i] * nfull + sb.starts[j]);
					}
				}
			}
			if (blocks.size() != sa.mats.size() || blocks[0].size() != sb.mats.size()) { return false; }
			for (size_t i = 0; i < sa.mats.size(); ++i)
			{
				for (size_t j = 0; j < sb.mats.size(); ++j)
				{
					PartProducts::Product& p = blocks[i][j];
					if (p.M != sa.mats[i].F || p.N != sb.mats[j].F || p.K != sa.mats[i].K || p.K != sb.mats[j].K) { return false; }
					PartProducts::Term term;
					bool ta = false, tb = false;
					if (false == term_layout(sa.mats[i], sb.mats[j], ta, tb, term)) { return false; }
					if (t > 0 && (ta != p.trans_a || tb != p.trans_b)) { return false; }
					p.trans_a = ta;
					p.trans_b = tb;
					p.terms.push_back(term);
				}
			}
		}
		if (false == any_parts) { return false; }
		out.node = n.f;
		out.dtype = n.dtype;
		out.partial = false;
		out.products.clear();
		for (auto& row : blocks)
		{
			for (auto& p : row)
			{
				if (false == fast_shape(p)) { return false; }
				out.products.push_back(p);
			}
		}
		out.label = "blocks CONTRACT x" + std::to_string(n.args.size()) + " " + std::to_string(blocks.size()) + "x" +
			std::to_string(blocks[0].size());
		// one launch for all of them when every part keeps one leading dim over the terms
		bool uniform = true;
		for (auto& row : blocks)
		{
			for (auto& p : row)
			{
				for (const PartProducts::Term& t : p.terms)
				{
					uniform = uniform && t.lda == p.terms[0].lda && t.ldb == p.terms[0].ldb;
				}
				uniform = uniform && p.trans_a == blocks[0][0].trans_a && p.trans_b == blocks[0][0].trans_b &&
					p.K == blocks[0][0].K && p.terms.size() == blocks[0][0].terms.size();
			}
		}
		if (uniform)
		{
			out.grid_m = (uint32_t) blocks.size();
			out.grid_n = (uint32_t) blocks[0].size();
		}
		return true;
	}

	/// The product that reads concatenation z through consumer c: c itself, or
	/// the sum c is a term of; -1 when c is neither
	int product_reading (int c) const
	{
		const Node& n = nodes_[c];
		if (n.op != egen::CONTRACT && n.op != egen::MATMUL) { return -1; }
		if (false == n.summed_term) { return n.kind == OTHER ? c : -1; }
		// a term of a sum: the CONTRACT itself or the PERMUTE over it is an operand of the ADD
		int up = c;
		for (int hop = 0; hop < 2; ++hop)
		{
			if (nodes_[up].consumers.size() != 1) { return -1; }
			up = nodes_[up].consumers[0];
			if (nodes_[up].summed) { return up; }
		}
		return -1;
	}

	void find_part_products (void)
	{
		std::set<int> folded;
		for (size_t z = 0; z < nodes_.size(); ++z)
		{
			Parts parts;
			if (concat_parts((int) z, parts))
			{
				part_lists_.emplace((int) z, parts);
				folded.insert((int) z);
			}
		}
		// a concatenation is folded when every reader is a product that takes it
		// part by part; dropping one may undo products that leaned on it as well
		std::map<int,PartProducts> calls;
		for (bool changed = true; changed;)
		{
			changed = false;
			calls.clear();
			if (folded.empty()) { break; }
			std::set<int> failed;
			std::set<int> products;
			for (int z : folded)
			{
				for (int c : nodes_[z].consumers)
				{
					int p = product_reading(c);
					if (p < 0) { failed.insert(z); }
					else { products.insert(p); }
				}
			}
			for (int p : products)
			{
				PartProducts call;
				bool ok = nodes_[p].summed ? blocks_of_sum(p, folded, call) : terms_of_contract(p, folded, call);
				// the launch stands where the product does: nothing may rewrite what the parts show in between
				if (ok) { calls.emplace(p, call); }
			}
			for (int z : folded)
			{
				for (int c : nodes_[z].consumers)
				{
					int p = product_reading(c);
					if (p < 0 || 0 == calls.count(p)) { failed.insert(z); continue; }
					std::vector<size_t> all(nodes_[z].args.size());
					bool rewritten = false;
					for (size_t k = 0; k < nodes_[z].args.size(); ++k)
					{
						rewritten = rewritten || written_between(z, {k}, (int) z, p);
					}
					if (rewritten) { failed.insert(z); }
				}
			}
			for (int z : failed)
			{
				folded.erase(z);
				changed = true;
			}
		}
		for (int z : folded)
		{
			Node& n = nodes_[z];
			n.kind = VIEW;
			n.absorbed = true;
			n.parts_folded = true;
		}
		for (auto& kv : calls)
		{
			nodes_[kv.first].part_products = (int) part_calls_.size();
			choose_ranges(kv.first, kv.second);
			part_calls_.push_back(kv.second);
		}
	}

	/// Do only elementwise groups read node v, and only through SLICE / PAD /
	/// IDENTITY nodes folded into them (views that still walk the result row by row)?
	bool only_groups_read_through (int v, bool top = true) const
	{
		const Node& n = nodes_[v];
		if (n.target || n.consumers.empty()) { return false; }
		for (int c : n.consumers)
		{
			const Node& m = nodes_[c];
			if (m.kind == EW && false == top) { continue; }
			bool folded_view = m.kind == VIEW && m.absorbed && false == m.through_conv && false == m.parts_folded &&
				false == m.summed_term && (m.op == egen::SLICE || m.op == egen::PAD || m.op == egen::IDENTITY);
			if (false == folded_view || false == only_groups_read_through(c, false)) { return false; }
		}
		return true;
	}

	/// A product with few results under a long K runs as K ranges on separate
	/// workgroups, and a launch of its own would add them up.  When elementwise
	/// groups reading through SLICEs are all that reads the node, the ranges
	/// stay side by side and those groups add them while they load.
	void choose_ranges (int c, PartProducts& call)
	{
		const Node& n = nodes_[c];
		if (n.summed || call.products.size() != 1 || n.dtype != egen::FLOAT) { return; }
		const PartProducts::Product& p = call.products[0];
		const uint64_t depth = p.K * p.terms.size();
		const uint64_t cus = 256;
		if (false == only_groups_read_through(c)) { return; }
		// few results that elementwise nodes are all that reads (a time step of a recurrent
		// cell): the product may take the launch of those nodes as its epilogue, which
		// finish() decides when it knows the launches.  Until then, and when it decides
		// otherwise, the result waits for them in temporary memory like K ranges do
		const uint64_t tiles128 = ((p.M + 127) / 128) * ((p.N + 127) / 128);
		const bool few = tiles128 < 2 * cus;
		call.epilogue = few && false == p.trans_a && p.terms.size() <= 8 && epilogues_enabled();
		// the shapes the product kernels split: a transposed operand (row-major
		// operands with enough 32 x 32 blocks share K between the waves of a workgroup)
		uint32_t ranges = 1;
		if ((p.trans_a || p.trans_b) && tiles128 * std::min<uint64_t>(32, depth / 256) < cus)
		{
			uint64_t tiles = ((p.M + 63) / 64) * ((p.N + 63) / 64);
			uint64_t want = std::min<uint64_t>({32, 2 * cus / tiles, depth / 128});
			while (2 * ranges <= want && depth % (2 * ranges * 16) == 0) { ranges *= 2; }
			// every reader adds the ranges up again: worth it for one or two
			size_t readers = 0;
			for (int v : n.consumers) { readers += nodes_[v].consumers.size(); }
			if (readers > 2) { ranges = 1; }
		}
		if (ranges < 2 && false == call.epilogue) { return; }
		// ... and the groups must see the product's dtype (a view changes none)
		call.ranges = ranges;
		call.label += " ranges=" + std::to_string(ranges);
		nodes_[c].ranged = true;
	}

	/// TCR_EPILOGUES=0 keeps every product and the group that reads it apart (two
	/// launches, as the check of the single one)
	static bool epilogues_enabled (void)
	{
		static const bool on = []
		{
			const char* env = getenv("TCR_EPILOGUES");
			return !(env && env[0] == '0');
		}();
		return on;
	}

	/// The elementwise nodes that read node v through folded views
	void readers_through (int v, std::vector<int>& out) const
	{
		for (int c : nodes_[v].consumers)
		{
			if (nodes_[c].kind == EW) { out.push_back(c); }
			else { readers_through(c, out); }
		}
	}

	// ---- sums of products ----

	/// The CONTRACT behind operand `i` of an ADD when it can be a term of a sum
	/// of products: a CONTRACT node, or the PERMUTE that is launched as a
	/// swapped product, read by nothing else; -1 otherwise
	int product_term (int i) const
	{
		if (i < 0) { return -1; }
		const Node& n = nodes_[i];
		if (n.target || n.consumers.size() != 1) { return -1; }
		if (n.op == egen::PERMUTE && n.swapped_from >= 0) { return n.swapped_from; }
		if (n.op == egen::CONTRACT && n.kind == OTHER && n.args.size() == 2) { return i; }
		return -1;
	}

	/// fp32 ADD nodes all of whose operands are such products of one pair of
	/// shapes, pairs and form: one launch over the concatenated summed index
	void find_summed_products (void)
	{
		for (size_t i = 0; i < nodes_.size(); ++i)
		{
			Node& n = nodes_[i];
			if (n.op != egen::ADD || n.dtype != egen::FLOAT || n.args.size() < 4 || n.args.size() > 128) { continue; }
			// results of a few thousand elements gain nothing (and their passes are
			// recorded as the steps of one kernel, which this launch is not)
			if (n.f->shape().n_elems() <= 4096) { continue; }
			std::vector<int> seen(n.args.begin(), n.args.end());
			std::sort(seen.begin(), seen.end());
			if (std::adjacent_find(seen.begin(), seen.end()) != seen.end()) { continue; } // x + x: two reads of one node
			int first = product_term(n.args[0]);
			if (first < 0) { continue; }
			const Node& proto = nodes_[first];
			bool swapped = nodes_[n.args[0]].op == egen::PERMUTE;
			PairVecT<teq::RankT> dims;
			Packer<PairVecT<teq::RankT>>().unpack(dims, *proto.f);
			Shape8 ashape = shape8(proto.arg_tens[0]->shape()), bshape = shape8(proto.arg_tens[1]->shape());
			bool all = true;
			int earliest = (int) i;
			for (int a : n.args)
			{
				int c = product_term(a);
				all = c >= 0 && (nodes_[a].op == egen::PERMUTE) == swapped && nodes_[c].dtype == n.dtype;
				if (false == all) { break; }
				const Node& term = nodes_[c];
				PairVecT<teq::RankT> tdims;
				Packer<PairVecT<teq::RankT>>().unpack(tdims, *term.f);
				all = tdims == dims && shape8(term.arg_tens[0]->shape()) == ashape && shape8(term.arg_tens[1]->shape()) == bshape;
				if (false == all) { break; }
				earliest = std::min(earliest, c);
			}
			if (false == all) { continue; }
			// the products would read their operands where the ADD stands
			bool rewritten = false;
			for (int a : n.args)
			{
				int c = product_term(a);
				rewritten = rewritten || written_between(c, {0, 1}, earliest, (int) i);
			}
			if (rewritten) { continue; }
			n.kind = OTHER;
			n.summed = true;
			for (int a : n.args)
			{
				int c = product_term(a);
				for (int t : {a, c})
				{
					nodes_[t].kind = VIEW;
					nodes_[t].absorbed = true;
					nodes_[t].summed_term = true;
					nodes_[t].swapped_from = -1;
				}
			}
		}
	}

	// ---- buffers that ASSIGN* nodes of the pass rewrite ----
	//
	// The walk runs node by node, so a node that reads a variable before an
	// ASSIGN* to it in the walk's order sees the old value and one after it
	// the new one (internal/eigen/device.hpp:508-544 updates the target's
	// buffer in place).  Launches are reordered and merged here, so every read
	// of such a buffer is pinned to its side of every write to it.

	/// The tensor whose buffer an ASSIGN* node (or a chain of aliases) rewrites
	teq::iTensor* written_base (int i) const
	{
		const Node& n = nodes_[i];
		if (n.args[0] < 0) { return n.arg_tens[0].get(); }
		const Node& a = nodes_[n.args[0]];
		if (is_assign(a.op) || is_buffer_alias(a.op)) { return written_base(n.args[0]); }
		return a.f;
	}

	void find_written (void)
	{
		writes_.assign(nodes_.size(), -1);
		for (size_t i = 0; i < nodes_.size(); ++i)
		{
			if (false == is_assign(nodes_[i].op) || nodes_[i].args.empty()) { continue; }
			teq::iTensor* base = written_base((int) i);
			auto it = resource_.emplace(base, (int) write_pos_.size()).first;
			if (it->second == (int) write_pos_.size()) { write_pos_.emplace_back(); }
			write_pos_[it->second].push_back((int) i);
			writes_[i] = it->second;
		}
	}

	/// Rewritten buffers that are read when operand k of node i is read.
	/// `folded`: look through every node that can be folded into its reader
	/// (while that is being decided) instead of those that have been.
	void touched_by_arg (int i, size_t k, bool folded, std::set<int>& out) const
	{
		const Node& n = nodes_[i];
		int a = n.args[k];
		auto it = resource_.find(a < 0 ? n.arg_tens[k].get() : (teq::iTensor*) nodes_[a].f);
		if (it != resource_.end()) { out.insert(it->second); }
		if (a < 0) { return; }
		const Node& arg = nodes_[a];
		if (is_assign(arg.op)) { out.insert(writes_[a]); }
		else if (is_buffer_alias(arg.op)) { touched_by_arg(a, 0, folded, out); }
		else if (arg.kind == VIEW && (folded || arg.absorbed))
		{
			for (size_t j = 0; j < arg.args.size(); ++j) { touched_by_arg(a, j, folded, out); }
		}
	}

	/// Is a buffer that operands `ks` of node i read rewritten after position
	/// `from` and before position `to`?
	bool written_between (int i, std::initializer_list<size_t> ks, int from, int to) const
	{
		if (resource_.empty()) { return false; }
		std::set<int> touched;
		for (size_t k : ks) { touched_by_arg(i, k, true, touched); }
		for (int r : touched)
		{
			for (int w : write_pos_[r])
			{
				if (from < w && w < to) { return true; }
			}
		}
		return false;
	}

	/// Dependence edges that keep launch i on its side of the writes: called
	/// for every launch in the order of the pass
	void order_around_writes (int i)
	{
		if (resource_.empty()) { return; }
		const Node& n = nodes_[i];
		std::set<int> touched;
		for (size_t k = is_assign(n.op) ? 1 : 0; k < n.args.size(); ++k) { touched_by_arg(i, k, false, touched); }
		for (int r : touched)
		{
			if (last_write_[r] >= 0) { deps_[i].insert(last_write_[r]); }
			readers_[r].push_back(i);
		}
		int w = writes_[i];
		if (w < 0) { return; }
		for (int reader : readers_[w])
		{
			if (find(reader) != i) { deps_[i].insert(find(reader)); }
		}
		if (last_write_[w] >= 0) { deps_[i].insert(last_write_[w]); }
		readers_[w].clear();
		last_write_[w] = i;
	}

	/// Does anything other than the launch described by `inside` read node i?
	template <typename F>
	bool read_elsewhere (int i, F inside) const
	{
		for (int c : nodes_[i].consumers)
		{
			if (is_alias(c) ? read_elsewhere(c, inside) : false == inside(c)) { return true; }
		}
		return false;
	}

	template <typename F>
	bool read_by (int i, F inside) const
	{
		for (int c : nodes_[i].consumers)
		{
			if (is_alias(c) ? read_by(c, inside) : inside(c)) { return true; }
		}
		return false;
	}

	Kind classify (const Node& n) const
	{
		size_t nargs = n.args.size();
		bool ew = (is_unary(n.op) && nargs == 1) ||
			(is_binary(n.op) && (nargs == 2 || ((n.op == egen::ADD || n.op == egen::MUL) && nargs > 2))) ||
			(n.op == egen::SELECT && nargs == 3);
		if (n.op == egen::CONCAT)
		{
			// every element comes from exactly one operand: the operands become
			// zero-bordered leaves whose boxes tile the output, OR-ed together
			if (nargs < 2 || nargs > TCG_FX_MAX_LEAVES) { return OTHER; }
			for (auto& arg : n.arg_tens)
			{
				if ((int) arg->get_meta().type_code() != n.dtype) { return OTHER; }
			}
			return EW;
		}
		if (ew)
		{
			if (nargs > TCG_FX_MAX_LEAVES) { return OTHER; }
			for (auto& arg : n.arg_tens)
			{
				if (shape8(arg->shape()) != n.shape || (int) arg->get_meta().type_code() != n.dtype) { return OTHER; }
			}
			return EW;
		}
		if (nargs != 1) { return OTHER; }
		switch (n.op)
		{
			case egen::IDENTITY: case egen::EXTEND: case egen::SLICE: case egen::PAD:
				return VIEW;
			case egen::PERMUTE:
			{
				// reading through a permutation that moves the fastest dim is
				// uncoalesced: worth it only while the tensor is small
				teq::RanksT order;
				Packer<teq::RanksT>().unpack(order, *n.f);
				bool keeps_dim0 = order.empty() || order[0] == 0;
				return keeps_dim0 || n.f->shape().n_elems() <= (1u << 16) ? VIEW : OTHER;
			}
			default: return OTHER;
		}
	}

	// ---- views ----

	/// How consumer `c` sees its operand `argpos`, in c's operand coordinates
	View view_of_arg (int c, size_t argpos, std::vector<int>* through = nullptr)
	{
		int a = nodes_[c].args[argpos];
		if (a >= 0 && nodes_[a].kind == VIEW && nodes_[a].absorbed)
		{
			return view_through(a, through);
		}
		teq::iTensor* tens = nodes_[c].arg_tens[argpos].get();
		return dense_view(tens, shape8(tens->shape()));
	}

	View view_through (int v, std::vector<int>* through)
	{
		if (through) { through->push_back(v); }
		const Node& n = nodes_[v];
		View in = view_of_arg(v, 0, through);
		Shape8 inshape = shape8(n.arg_tens[0]->shape());
		View out = in;
		switch (n.op)
		{
			case egen::IDENTITY: break;
			case egen::EXTEND:
			{
				auto bopt = unpack_extend(n.arg_tens[0]->shape(), *n.f);
				if (!bopt) { global::fatal("cannot find extend attributes"); }
				for (size_t d = 0, m = std::min((size_t) 8, bopt->size()); d < m; ++d)
				{
					if ((*bopt)[d] > 1)
					{
						out.stride[d] = 0;
						bool whole = in.lo[d] == 0 && in.hi[d] >= 1;
						out.lo[d] = 0;
						out.hi[d] = whole ? n.shape[d] : 0;
					}
				}
			}
				break;
			case egen::SLICE:
			{
				PairVecT<teq::DimT> encoding;
				Packer<PairVecT<teq::DimT>>().unpack(encoding, *n.f);
				for (size_t d = 0, m = std::min(encoding.size(), (size_t) 8); d < m; ++d)
				{
					uint64_t offset = std::min<uint64_t>(encoding[d].first, inshape[d] - 1);
					uint64_t extent = std::min<uint64_t>(encoding[d].second, inshape[d] - offset);
					out.off += (int64_t) offset * in.stride[d];
					out.lo[d] = in.lo[d] > offset ? in.lo[d] - offset : 0;
					out.hi[d] = in.hi[d] > offset ? std::min(in.hi[d] - offset, extent) : 0;
				}
			}
				break;
			case egen::PAD:
			{
				PairVecT<teq::DimT> encoding;
				Packer<PairVecT<teq::DimT>>().unpack(encoding, *n.f);
				for (size_t d = 0, m = std::min(encoding.size(), (size_t) 8); d < m; ++d)
				{
					uint64_t before = encoding[d].first;
					out.off -= (int64_t) before * in.stride[d];
					out.lo[d] = in.lo[d] + before;
					out.hi[d] = in.hi[d] + before;
				}
			}
				break;
			case egen::PERMUTE:
			{
				teq::RanksT order;
				Packer<teq::RanksT>().unpack(order, *n.f);
				if (order.size() > 8) { order.resize(8); }
				bool visited[8] = {false};
				for (teq::RankT r : order) { visited[r] = true; }
				for (teq::RankT d = 0; d < 8; ++d)
				{
					if (false == visited[d]) { order.push_back(d); }
				}
				for (int d = 0; d < 8; ++d)
				{
					out.stride[d] = in.stride[order[d]];
					out.lo[d] = in.lo[order[d]];
					out.hi[d] = in.hi[order[d]];
				}
			}
				break;
			case egen::REVERSE:
			{
				// only for the operands of convolutions: elementwise launches do not walk backwards
				std::set<teq::RankT> dims;
				Packer<std::set<teq::RankT>>().unpack(dims, *n.f);
				for (teq::RankT d : dims)
				{
					if (d >= 8) { continue; }
					out.off += (int64_t) (inshape[d] - 1) * in.stride[d];
					out.stride[d] = -in.stride[d];
					out.lo[d] = inshape[d] - in.hi[d];
					out.hi[d] = inshape[d] - in.lo[d];
				}
			}
				break;
			default: global::fatal("not a view");
		}
		return out;
	}

	/// The launch of the convolution whose result node u receives
	ViewedConv viewed_conv (int u, int step, FusionPlan& plan, std::map<int,int>& last_conv)
	{
		const int ci = nodes_[u].conv_from;
		const Node& c = nodes_[ci];
		const ConvFold& fold = folds_.at(ci);
		ViewedConv call;
		call.node = nodes_[u].f;
		call.dtype = c.dtype;
		call.imgshape = shape8(c.arg_tens[0]->shape());
		call.kshape = shape8(c.arg_tens[1]->shape());
		teq::RanksT order;
		Packer<teq::RanksT>().unpack(order, *c.f);
		for (size_t k = 0; k < std::min(order.size(), (size_t) teq::rank_cap); ++k) { call.ranks.push_back(order[k]); }
		// operands: the views the folded nodes add up to
		View image = view_of_arg(ci, 0), kernel = view_of_arg(ci, 1);
		call.image = image.base;
		call.kernel = kernel.base;
		call.image_off = image.off;
		call.kernel_off = kernel.off;
		for (int d = 0; d < 8; ++d)
		{
			call.image_stride[d] = image.stride[d];
			call.kernel_stride[d] = kernel.stride[d];
			call.ilo[d] = image.lo[d];
			call.ihi[d] = image.hi[d];
			if (kernel.lo[d] != 0 || kernel.hi[d] != call.kshape[d]) { global::fatal("a kernel read through a border"); }
		}
		for (const std::vector<int>* chain : {&fold.image, &fold.kernel})
		{
			for (int v : *chain) { last_conv[v] = step; }
		}
		// the operands the CONV node itself would have counted as read
		for (size_t k = 0; k < 2; ++k)
		{
			int a = c.args[k];
			if (a >= 0 && holds_value(a) && first_occurrence(c, k))
			{
				call.reads.push_back(c.arg_tens[k].get());
			}
		}
		// the result: which output dim each dim of the receiving node is, and in which direction
		Shape8 oshape = c.shape;
		call.windowed = fold.result.empty() && false == c.target && slices_window(c.f, c.f->shape(), call.olo, call.ohi);
		if (false == call.windowed)
		{
			for (int d = 0; d < 8; ++d)
			{
				call.olo[d] = 0;
				call.ohi[d] = oshape[d];
			}
		}
		int from[8];          // dim of the receiving node -> output dim of the convolution
		bool backwards[8];
		for (int d = 0; d < 8; ++d)
		{
			from[d] = d;
			backwards[d] = false;
		}
		for (int v : fold.result)
		{
			const Node& m = nodes_[v];
			if (m.op == egen::PERMUTE)
			{
				teq::RanksT perm;
				Packer<teq::RanksT>().unpack(perm, *m.f);
				if (perm.size() > 8) { perm.resize(8); }
				bool visited[8] = {false};
				for (teq::RankT r : perm) { visited[r] = true; }
				for (teq::RankT d = 0; d < 8; ++d)
				{
					if (false == visited[d]) { perm.push_back(d); }
				}
				int was[8];
				bool wasback[8];
				std::copy(from, from + 8, was);
				std::copy(backwards, backwards + 8, wasback);
				for (int d = 0; d < 8; ++d)
				{
					from[d] = was[perm[d]];
					backwards[d] = wasback[perm[d]];
				}
			}
			else
			{
				std::set<teq::RankT> dims;
				Packer<std::set<teq::RankT>>().unpack(dims, *m.f);
				for (teq::RankT d : dims)
				{
					if (d < 8) { backwards[d] = !backwards[d]; }
				}
			}
			if (v != u) { plan.absorbed.push_back(m.f); }
		}
		if (false == fold.result.empty()) { plan.absorbed.push_back(c.f); }
		Shape8 rshape = nodes_[u].shape;
		int64_t run = 1;
		call.out_off = 0;
		for (int d = 0; d < 8; ++d)
		{
			// dim d of the receiving node walks output dim from[d]
			call.out_stride[from[d]] = backwards[d] ? -run : run;
			if (backwards[d]) { call.out_off += (int64_t) (rshape[d] - 1) * run; }
			run *= (int64_t) rshape[d];
		}
		// label: image side, kernel side, CONV, result side
		std::string label;
		for (auto it = fold.image.rbegin(); it != fold.image.rend(); ++it) { label += nodes_[*it].f->get_opcode().name_ + "+"; }
		for (auto it = fold.kernel.rbegin(); it != fold.kernel.rend(); ++it) { label += nodes_[*it].f->get_opcode().name_ + "+"; }
		label += "CONV";
		for (int v : fold.result) { label += "+" + nodes_[v].f->get_opcode().name_; }
		if (call.windowed) { label += "+SLICE"; }
		call.label = label;
		return call;
	}

	// ---- units: what is launched as one thing ----

	int find (int i)
	{
		while (uf_[i] != i)
		{
			uf_[i] = uf_[uf_[i]];
			i = uf_[i];
		}
		return i;
	}

	/// Units whose results node i reads (through folded views)
	void inputs_of (int i, std::vector<int>& out)
	{
		for (int a : nodes_[i].args)
		{
			if (a < 0) { continue; }
			if (nodes_[a].kind == VIEW && nodes_[a].absorbed) { inputs_of(a, out); }
			else { out.push_back(find(a)); }
		}
	}

	/// Does unit u depend, directly or not, on unit g?
	bool reaches (int u, int g)
	{
		++clock_;
		return reaches_rec(find(u), find(g));
	}

	bool reaches_rec (int u, int g)
	{
		if (u == g) { return true; }
		if (maxpos_[u] < minpos_[g] || stamp_[u] == clock_) { return false; }
		stamp_[u] = clock_;
		for (int d : deps_[u])
		{
			if (reaches_rec(find(d), g)) { return true; }
		}
		return false;
	}

	void group_all (void)
	{
		last_write_.assign(write_pos_.size(), -1);
		readers_.assign(write_pos_.size(), {});
		for (size_t i = 0; i < nodes_.size(); ++i)
		{
			Node& n = nodes_[i];
			minpos_[i] = maxpos_[i] = (int) i;
			if (n.kind == VIEW && n.absorbed) { continue; }
			std::vector<int> ins;
			inputs_of((int) i, ins);
			deps_[i].insert(ins.begin(), ins.end());
			// what the node reads through a folded view it reads from memory, at other
			// coordinates than its own: that value must come from an earlier launch
			for (int a : n.args)
			{
				while (a >= 0 && is_alias(a)) { a = nodes_[a].args[0]; }
				if (a >= 0 && nodes_[a].kind == VIEW && nodes_[a].absorbed)
				{
					std::vector<int> through;
					inputs_of(a, through);
					vdeps_[i].insert(through.begin(), through.end());
				}
			}
			order_around_writes((int) i);
			if (n.kind != EW) { continue; }
			members_[i].push_back((int) i);
			std::vector<int> cands;
			for (int a : n.direct)
			{
				if (a >= 0 && nodes_[a].kind == EW && nodes_[a].shape == n.shape && n.op != egen::CONCAT)
				{
					cands.push_back(find(a));
				}
			}
			std::sort(cands.begin(), cands.end(), [&](int x, int y) { return maxpos_[x] > maxpos_[y]; });
			cands.erase(std::unique(cands.begin(), cands.end()), cands.end());
			// A node that stands far behind the launch its operands come from, and that only
			// elementwise nodes of its shape read, waits for those readers instead: the factors
			// the gradient builder derives from a forward value (1 - s, s (1 - s) of a gate,
			// tenncor/eteq/backprop.hpp:58-560) stand with the backward pass.  Computed in the
			// forward launch each is one more tensor stored there and loaded again much later;
			// computed where it is read it costs an instruction and the forward value is
			// stored once for all of them.
			if (n.consumers.size() > 0 && std::all_of(n.consumers.begin(), n.consumers.end(), [&](int c)
				{ return nodes_[c].kind == EW && nodes_[c].shape == n.shape && nodes_[c].op != egen::CONCAT; }))
			{
				cands.erase(std::remove_if(cands.begin(), cands.end(), [&](int cand)
				{
					return (int) i - maxpos_[find(cand)] > far_behind;
				}), cands.end());
			}
			int self = (int) i;
			for (int cand : cands)
			{
				cand = find(cand);
				self = find(self);
				if (cand == self || members_[self].size() + members_[cand].size() > max_members) { continue; }
				if (mergeable(self, cand)) { self = merge(self, cand); }
			}
		}
	}

	/// No launch outside the two units may sit between them
	bool mergeable (int g, int cand)
	{
		for (int d : vdeps_[g]) { if (find(d) == cand) { return false; } }
		for (int d : vdeps_[cand]) { if (find(d) == g) { return false; } }
		for (int d : deps_[g])
		{
			d = find(d);
			if (d != cand && d != g && reaches(d, cand)) { return false; }
		}
		for (int d : deps_[cand])
		{
			d = find(d);
			if (d != cand && d != g && reaches(d, g)) { return false; }
		}
		return true;
	}

	int merge (int g, int cand)
	{
		// the earlier unit stays the root: positions order the members
		int root = std::min(g, cand), other = std::max(g, cand);
		uf_[other] = root;
		std::vector<int> merged;
		std::merge(members_[root].begin(), members_[root].end(),
			members_[other].begin(), members_[other].end(), std::back_inserter(merged));
		members_[root] = merged;
		members_[other].clear();
		std::set<int> deps;
		for (int d : deps_[root]) { if (find(d) != root) { deps.insert(find(d)); } }
		for (int d : deps_[other]) { if (find(d) != root) { deps.insert(find(d)); } }
		deps_[root] = deps;
		deps_[other].clear();
		vdeps_[root].insert(vdeps_[other].begin(), vdeps_[other].end());
		vdeps_[other].clear();
		minpos_[root] = std::min(minpos_[root], minpos_[other]);
		maxpos_[root] = std::max(maxpos_[root], maxpos_[other]);
		return root;
	}

	// ---- emission ----

	/// members [lo, hi) of unit g as one launch; false when it does not fit
	bool build (const std::vector<int>& members, size_t lo, size_t hi, FusedGroup& out, std::vector<int>& views)
	{
		out = FusedGroup();
		views.clear();
		const Node& first = nodes_[members[lo]];
		out.dtype = first.dtype;
		out.shape = first.shape;
		std::map<int,size_t> pos; // member -> position in the launch
		for (size_t p = lo; p < hi; ++p) { pos.emplace(members[p], p - lo); }
		auto inside = [&](int a) { return a >= 0 && pos.count(a) > 0; };
		std::vector<size_t> last_use(hi - lo, 0);
		std::vector<bool> stored(hi - lo, false);
		for (size_t p = lo; p < hi; ++p)
		{
			const Node& n = nodes_[members[p]];
			for (int a : n.direct)
			{
				if (inside(a)) { last_use[pos[a]] = p - lo; }
			}
			stored[p - lo] = n.target || read_elsewhere(members[p], inside);
		}
		std::map<View,int> leaf_of;
		std::vector<int> reg_of(hi - lo, -1);
		std::vector<bool> busy(TCG_FX_MAX_REGS, false);
		auto take_reg = [&]() -> int
		{
			for (int r = 0; r < TCG_FX_MAX_REGS; ++r)
			{
				if (false == busy[r])
				{
					busy[r] = true;
					return r;
				}
			}
			return -1;
		};
		for (size_t p = lo; p < hi; ++p)
		{
			const Node& n = nodes_[members[p]];
			size_t here = p - lo;
			// operands: a register of this launch, an immediate or a leaf
			bool fold = n.args.size() > 2 && n.op != egen::SELECT;
			const bool concat = n.op == egen::CONCAT;
			teq::RankT axis = 0;
			uint64_t before = 0; // extent of the operands already placed along `axis`
			if (concat) { Packer<teq::RankT>().unpack(axis, *n.f); }
			std::vector<uint8_t> codes;
			std::vector<double> vals;
			for (size_t k = 0; k < n.args.size(); ++k)
			{
				int a = n.direct[k];
				if (false == concat && inside(a))
				{
					codes.push_back((uint8_t) (TCG_FX_REG0 + reg_of[pos[a]]));
					vals.push_back(0);
					views.insert(views.end(), n.aliases[k].begin(), n.aliases[k].end());
					continue;
				}
				View v = view_of_arg(members[p], k, &views);
				if (concat)
				{
					// operand k occupies [before, before + extent) of the axis
					// and reads as zero elsewhere, like a PAD of it would
					uint64_t extent = shape8(n.arg_tens[k]->shape())[axis];
					v.off -= (int64_t) before * v.stride[axis];
					v.lo[axis] += before;
					v.hi[axis] += before;
					before += extent;
				}
				double value;
				if (false == concat && scalar_constant(v.base, value))
				{
					// an instruction carries one immediate: operands sharing an
					// instruction (all of them unless the node is an n-ary fold,
					// where only the first two do) must agree on it
					bool clash = false;
					for (size_t j = fold ? (k == 1 ? 0 : k) : 0; j < k; ++j)
					{
						clash = clash || (codes[j] == TCG_FX_IMM && vals[j] != value);
					}
					if (false == clash)
					{
						codes.push_back(TCG_FX_IMM);
						vals.push_back(value);
						continue;
					}
				}
				// an operand whose launch left K ranges: the window lies there as a dense matrix
				int ranges_of = -1;
				uint32_t nsum = 0;
				int64_t sum_stride = 0;
				auto producer = index_.find(v.base);
				if (producer != index_.end() && nodes_[producer->second].ranged)
				{
					ranges_of = nodes_[producer->second].part_products;
					const PartProducts& call = part_calls_[ranges_of];
					const PartProducts::Product& prod = call.products[0];
					// from the first element the view reads: steps along a row stay steps
					// of one, steps from row to row become steps of the window's width
					const int64_t ld = (int64_t) prod.ldc, m0 = prod.c_off / ld, n0 = prod.c_off % ld;
					int64_t first = v.off;
					for (int d = 0; d < 8; ++d) { first += (int64_t) v.lo[d] * v.stride[d]; }
					if (first < 0 || first / ld < m0 || first % ld < n0) { return false; }
					int64_t at = (first / ld - m0) * (int64_t) prod.N + (first % ld - n0);
					for (int d = 0; d < 8; ++d)
					{
						if (v.stride[d] < 0 || (v.stride[d] >= ld && v.stride[d] % ld != 0)) { return false; }
						v.stride[d] = (v.stride[d] / ld) * (int64_t) prod.N + v.stride[d] % ld;
						at -= (int64_t) v.lo[d] * v.stride[d];
					}
					v.off = at;
					nsum = call.ranges;
					sum_stride = (int64_t) (prod.M * prod.N);
				}
				auto it = leaf_of.find(v);
				if (it == leaf_of.end())
				{
					if (out.leaves.size() >= TCG_FX_MAX_LEAVES) { return false; }
					FusedGroup::Leaf leaf;
					leaf.base = v.base;
					leaf.ranges_of = ranges_of;
					leaf.view.nsum = nsum;
					leaf.view.sum_stride = sum_stride;
					leaf.view.ptr = nullptr;
					leaf.view.offset = v.off;
					std::copy(v.stride, v.stride + 8, leaf.view.stride);
					std::copy(v.lo, v.lo + 8, leaf.view.lo);
					std::copy(v.hi, v.hi + 8, leaf.view.hi);
					it = leaf_of.emplace(v, (int) out.leaves.size()).first;
					out.leaves.push_back(leaf);
				}
				codes.push_back((uint8_t) (TCG_FX_LEAF0 + it->second));
				vals.push_back(0);
			}
			auto imm_of = [&](size_t j, size_t k)
			{
				return codes[j] == TCG_FX_IMM ? vals[j] : codes[k] == TCG_FX_IMM ? vals[k] : 0.0;
			};
			// registers: a one-instruction node may overwrite an operand that
			// dies here; a fold keeps its accumulator apart from its operands
			auto release_dead = [&]()
			{
				for (int a : n.direct)
				{
					if (inside(a) && last_use[pos[a]] == here) { busy[reg_of[pos[a]]] = false; }
				}
			};
			if (false == fold) { release_dead(); }
			int dst = take_reg();
			if (dst < 0) { return false; }
			reg_of[here] = dst;
			tcg_fx_instr ins;
			memset(&ins, 0, sizeof(ins));
			ins.dst = (uint8_t) (TCG_FX_REG0 + dst);
			ins.opcode = (uint8_t) (concat ? TCG_FX_BITOR : n.op);
			if (fold)
			{
				// ((a0 op a1) op a2) ... like the n-ary kernel
				ins.a = codes[0];
				ins.b = codes[1];
				ins.imm = imm_of(0, 1);
				out.program.push_back(ins);
				for (size_t k = 2; k < codes.size(); ++k)
				{
					ins.a = (uint8_t) (TCG_FX_REG0 + dst);
					ins.b = codes[k];
					ins.imm = imm_of(k, k);
					out.program.push_back(ins);
				}
				release_dead();
			}
			else
			{
				ins.a = codes[0];
				ins.b = codes.size() > 1 ? codes[1] : (uint8_t) TCG_FX_NONE;
				ins.c = codes.size() > 2 ? codes[2] : (uint8_t) TCG_FX_NONE;
				for (size_t k = 0; k < codes.size(); ++k)
				{
					if (codes[k] == TCG_FX_IMM) { ins.imm = vals[k]; }
				}
				out.program.push_back(ins);
			}
			if (stored[here])
			{
				if (out.outputs.size() >= TCG_FX_MAX_OUTS) { return false; }
				tcg_fx_instr st;
				memset(&st, 0, sizeof(st));
				st.opcode = TCG_FX_STORE;
				st.a = (uint8_t) (TCG_FX_REG0 + dst);
				st.dst = (uint8_t) out.outputs.size();
				out.program.push_back(st);
				out.outputs.push_back(n.f);
			}
			if (false == read_by(members[p], inside))
			{
				busy[dst] = false; // nothing in this launch reads it
			}
			if (out.program.size() > TCG_FX_MAX_INSTRS) { return false; }
			out.members.push_back(n.f);
			// reads the plain pass would have counted
			for (size_t k = 0; k < n.args.size(); ++k)
			{
				int a = n.args[k];
				if (a < 0) { continue; }
				bool materialised = inside(a) ? stored[pos[a]] : holds_value(a);
				if (materialised && first_occurrence(n, k)) { out.reads.push_back(n.arg_tens[k].get()); }
			}
		}
		return true;
	}

	FusionPlan finish (void)
	{
		FusionPlan plan;
		std::vector<bool> done(nodes_.size(), false);
		std::map<int,int> last_user; // folded view -> last group reading through it
		std::map<int,int> last_conv; // PAD read in place -> last convolution of its operand
		std::map<int,int> last_parts; // folded concatenation, or view beneath it -> last products over its parts
		std::map<int,int> last_ranges; // product that leaves K ranges (index into plan.part_products) -> last group adding them up
		std::function<void(int)> visit = [&](int u)
		{
			u = find(u);
			if (done[u]) { return; }
			done[u] = true;
			std::vector<int> deps;
			for (int d : deps_[u]) { deps.push_back(find(d)); }
			std::sort(deps.begin(), deps.end(), [&](int x, int y) { return minpos_[x] < minpos_[y]; });
			for (int d : deps)
			{
				if (d != u) { visit(d); }
			}
			if (nodes_[u].part_products >= 0)
			{
				const Node& n = nodes_[u];
				PartProducts call = part_calls_[n.part_products];
				FusionPlan::Step step;
				step.parts = (int) plan.part_products.size();
				// the products under the node, and their operands: folded
				// concatenations are counted when the last product through them is out
				std::vector<int> products;
				if (n.summed)
				{
					for (int arg : n.args)
					{
						int c = nodes_[arg].op == egen::PERMUTE ? nodes_[arg].args[0] : arg;
						plan.absorbed.push_back(nodes_[c].f);
						if (c != arg) { plan.absorbed.push_back(nodes_[arg].f); }
						products.push_back(c);
					}
				}
				else { products.push_back(u); }
				for (int c : products)
				{
					for (size_t k = 0; k < 2; ++k)
					{
						int a = nodes_[c].args[k];
						if (a < 0) { continue; }
						if (nodes_[a].parts_folded) { mark_parts_user(a, step.parts, last_parts); }
						else if (holds_value(a) && first_occurrence(nodes_[c], k))
						{
							call.reads.push_back(nodes_[c].arg_tens[k].get());
						}
					}
				}
				if (call.ranges > 0) { plan.absorbed.push_back(n.f); }
				emitted_parts_[n.part_products] = step.parts;
				plan.part_products.push_back(call);
				plan.steps.push_back(step);
				return;
			}
			if (nodes_[u].kind != EW && nodes_[u].swapped_from >= 0)
			{
				const Node& c = nodes_[nodes_[u].swapped_from];
				SwappedContract call;
				call.node = nodes_[u].f;
				call.dtype = c.dtype;
				call.a = c.arg_tens[1].get();
				call.b = c.arg_tens[0].get();
				call.ashape = shape8(call.a->shape());
				call.bshape = shape8(call.b->shape());
				PairVecT<teq::RankT> dims;
				Packer<PairVecT<teq::RankT>>().unpack(dims, *c.f);
				for (auto& d : dims)
				{
					call.pairs.push_back(d.second);
					call.pairs.push_back(d.first);
				}
				// the reads the two nodes would have counted: the product's operands
				for (size_t k = 0; k < 2; ++k)
				{
					int a = c.args[k];
					if (a >= 0 && holds_value(a) && first_occurrence(c, k))
					{
						call.reads.push_back(c.arg_tens[k].get());
					}
				}
				FusionPlan::Step step;
				step.contract = (int) plan.contracts.size();
				plan.contracts.push_back(call);
				plan.absorbed.push_back(c.f);
				plan.steps.push_back(step);
				return;
			}
			if (nodes_[u].summed)
			{
				const Node& n = nodes_[u];
				SummedContracts call;
				call.node = n.f;
				call.dtype = n.dtype;
				for (size_t k = 0; k < n.args.size(); ++k)
				{
					int arg = n.args[k];
					bool swapped = nodes_[arg].op == egen::PERMUTE;
					const Node& c = nodes_[swapped ? nodes_[arg].args[0] : arg];
					// a swapped product is launched with its operands exchanged
					int ia = swapped ? 1 : 0, ib = swapped ? 0 : 1;
					call.a.push_back(c.arg_tens[ia].get());
					call.b.push_back(c.arg_tens[ib].get());
					if (0 == k)
					{
						call.ashape = shape8(c.arg_tens[ia]->shape());
						call.bshape = shape8(c.arg_tens[ib]->shape());
						PairVecT<teq::RankT> dims;
						Packer<PairVecT<teq::RankT>>().unpack(dims, *c.f);
						for (auto& d : dims)
						{
							call.pairs.push_back(swapped ? d.second : d.first);
							call.pairs.push_back(swapped ? d.first : d.second);
						}
					}
					// the reads the term's nodes would have counted: the product's operands
					for (size_t j = 0; j < 2; ++j)
					{
						int operand = c.args[j];
						if (operand >= 0 && holds_value(operand) && first_occurrence(c, j))
						{
							call.reads.push_back(c.arg_tens[j].get());
						}
					}
					plan.absorbed.push_back(c.f);
					if (swapped) { plan.absorbed.push_back(nodes_[arg].f); }
				}
				FusionPlan::Step step;
				step.sum = (int) plan.sums.size();
				plan.sums.push_back(call);
				plan.steps.push_back(step);
				return;
			}
			if (nodes_[u].kind != EW && nodes_[u].conv_from >= 0)
			{
				FusionPlan::Step step;
				step.conv = (int) plan.convs.size();
				plan.convs.push_back(viewed_conv(u, step.conv, plan, last_conv));
				plan.steps.push_back(step);
				return;
			}
			if (nodes_[u].kind != EW)
			{
				FusionPlan::Step step;
				step.node = nodes_[u].f;
				plan.steps.push_back(step);
				return;
			}
			const std::vector<int>& members = members_[u];
			for (size_t lo = 0; lo < members.size();)
			{
				FusedGroup group, next;
				std::vector<int> views, next_views;
				size_t hi = lo + 1;
				if (false == build(members, lo, hi, group, views))
				{
					global::fatalf("cannot plan a launch for %s", nodes_[members[lo]].f->to_string().c_str());
				}
				while (hi < members.size() && build(members, lo, hi + 1, next, next_views))
				{
					group = next;
					views = next_views;
					++hi;
				}
				FusionPlan::Step step;
				if (hi == lo + 1 && views.empty() && false == uses_immediate(group) &&
					nodes_[members[lo]].op != egen::CONCAT)
				{
					step.node = nodes_[members[lo]].f; // nothing to gain: its own kernel
				}
				else
				{
					step.group = (int) plan.groups.size();
					for (int v : views) { last_user[v] = step.group; }
					const int producer = epilogue_producer(members, lo, hi, group);
					for (FusedGroup::Leaf& leaf : group.leaves)
					{
						if (leaf.ranges_of < 0) { continue; }
						leaf.ranges_of = emitted_parts_.at(leaf.ranges_of);
						last_ranges[leaf.ranges_of] = step.group;
					}
					if (producer >= 0)
					{
						// the product moves from where it stood to this launch
						const int at = emitted_parts_.at(producer);
						auto old = std::find_if(plan.steps.begin(), plan.steps.end(), [&](const FusionPlan::Step& st)
						{
							return st.parts == at && st.group < 0;
						});
						if (old != plan.steps.end())
						{
							plan.steps.erase(old);
							step.parts = at;
						}
					}
					for (size_t p = lo; p < hi; ++p)
					{
						const Node& n = nodes_[members[p]];
						if (std::find(group.outputs.begin(), group.outputs.end(), n.f) == group.outputs.end())
						{
							plan.absorbed.push_back(n.f);
						}
					}
					plan.groups.push_back(group);
				}
				plan.steps.push_back(step);
				lo = hi;
			}
		};
		for (size_t i = 0; i < nodes_.size(); ++i)
		{
			if (nodes_[i].target) { visit((int) i); }
		}
		// a folded view counts one read of its operand, when the last launch
		// that looks through it has been enqueued
		// a node folded into convolutions counts one read of its operand, when
		// the last of them has been enqueued
		for (auto& kv : last_conv)
		{
			const Node& v = nodes_[kv.first];
			plan.absorbed.push_back(v.f);
			int a = v.args[0];
			if (a >= 0 && holds_value(a))
			{
				plan.convs[kv.second].reads.push_back(v.arg_tens[0].get());
			}
		}
		for (auto& kv : last_ranges) { plan.groups[kv.second].frees.push_back(kv.first); }
		for (auto& kv : last_parts)
		{
			const Node& v = nodes_[kv.first];
			plan.absorbed.push_back(v.f);
			for (size_t k = 0; k < v.args.size(); ++k)
			{
				int a = v.args[k];
				if (a >= 0 && holds_value(a))
				{
					plan.part_products[kv.second].reads.push_back(v.arg_tens[k].get());
				}
			}
		}
		for (auto& kv : last_user)
		{
			const Node& v = nodes_[kv.first];
			plan.absorbed.push_back(v.f);
			int a = v.args[0];
			if (a >= 0 && holds_value(a))
			{
				plan.groups[kv.second].reads.push_back(v.arg_tens[0].get());
			}
		}
		pad_shared_operands(plan);
		return plan;
	}

	/// TCR_PADDED_OPERANDS=0 leaves every operand where it lies
	static bool padding_enabled (void)
	{
		static const bool on = []
		{
			const char* env = getenv("TCR_PADDED_OPERANDS");
			return !(env && env[0] == '0');
		}();
		return on;
	}

	/// See FusionPlan::PaddedOperand: leaves that eight and more products with an
	/// epilogue read as a K-contiguous B operand whose rows are a multiple of 32
	/// elements long, and that nothing in the pass assigns to
	void pad_shared_operands (FusionPlan& plan) const
	{
		if (false == padding_enabled()) { return; }
		std::set<const teq::iTensor*> assigned;
		for (const Node& n : nodes_)
		{
			if (nullptr != n.f && is_assign((int) n.f->get_opcode().code_)) { assigned.insert(n.f->get_args().front().get()); }
		}
		std::map<teq::iTensor*,size_t> uses;
		auto candidate = [&](const FusionPlan::Step& step, const PartProducts::Term& term) -> bool
		{
			if (step.parts < 0 || step.group < 0) { return false; }
			const PartProducts& call = plan.part_products[step.parts];
			const PartProducts::Product& p = call.products.at(0);
			if (false == p.trans_b || call.dtype != (int) egen::FLOAT || nullptr == dynamic_cast<teq::iLeaf*>(term.b)) { return false; }
			teq::Shape shape = term.b->shape();
			return term.ldb == shape.at(0) && term.ldb % 32 == 0 && term.ldb >= 256 && shape.n_elems() % term.ldb == 0 &&
				0 == assigned.count(term.b);
		};
		for (const FusionPlan::Step& step : plan.steps)
		{
			if (step.parts < 0 || step.group < 0) { continue; }
			std::set<teq::iTensor*> seen;
			for (const PartProducts::Term& term : plan.part_products[step.parts].products.at(0).terms)
			{
				if (candidate(step, term) && seen.insert(term.b).second) { ++uses[term.b]; }
			}
		}
		std::map<teq::iTensor*,int> index;
		for (const FusionPlan::Step& step : plan.steps)
		{
			if (step.parts < 0 || step.group < 0) { continue; }
			PartProducts& call = plan.part_products[step.parts];
			for (PartProducts::Term& term : call.products.at(0).terms)
			{
				if (false == candidate(step, term) || uses[term.b] < 8) { continue; }
				auto it = index.find(term.b);
				if (it == index.end())
				{
					FusionPlan::PaddedOperand op;
					op.tensor = term.b;
					op.ld = term.ldb;
					op.rows = term.b->shape().n_elems() / term.ldb;
					op.pad = 16;
					op.dtype = call.dtype;
					it = index.emplace(term.b, (int) plan.padded.size()).first;
					plan.padded.push_back(op);
				}
				term.b_padded = it->second;
			}
		}
	}

	/// The product (index into part_calls_) that can take the launch of members
	/// [lo, hi) as its epilogue: the only product whose result the launch reads in
	/// place of a tensor, read by nothing outside the launch, with nothing
	/// rewriting its operands between where it stands and where the launch does;
	/// -1 when there is none
	int epilogue_producer (const std::vector<int>& members, size_t lo, size_t hi, const FusedGroup& group) const
	{
		int producer = -1;
		for (const FusedGroup::Leaf& leaf : group.leaves)
		{
			if (leaf.ranges_of < 0) { continue; }
			if (producer >= 0 && producer != leaf.ranges_of) { return -1; }
			producer = leaf.ranges_of;
		}
		if (producer < 0 || false == part_calls_[producer].epilogue) { return -1; }
		int c = -1;
		for (size_t i = 0; i < nodes_.size() && c < 0; ++i)
		{
			if (nodes_[i].part_products == producer) { c = (int) i; }
		}
		if (c < 0) { return -1; }
		std::vector<int> readers;
		readers_through(c, readers);
		for (int r : readers)
		{
			if (std::find(members.begin() + lo, members.begin() + hi, r) == members.begin() + hi) { return -1; }
		}
		// the product would read its operands where the launch stands
		const int last = members[hi - 1];
		for (size_t k = 0; k < nodes_[c].args.size(); ++k)
		{
			int a = nodes_[c].args[k];
			if (written_between(c, {k}, c, last)) { return -1; }
			if (a >= 0 && nodes_[a].parts_folded)
			{
				for (size_t j = 0; j < nodes_[a].args.size(); ++j)
				{
					if (written_between(a, {j}, a, last)) { return -1; }
				}
			}
		}
		return producer;
	}

	/// Folded concatenation z and the views beneath it are read by products `step`
	void mark_parts_user (int z, int step, std::map<int,int>& last_parts) const
	{
		last_parts[z] = step;
		for (int a : nodes_[z].args)
		{
			if (a >= 0 && nodes_[a].kind == VIEW && nodes_[a].absorbed) { mark_parts_user(a, step, last_parts); }
		}
	}

	static bool uses_immediate (const FusedGroup& group)
	{
		return std::any_of(group.program.begin(), group.program.end(), [](const tcg_fx_instr& ins)
		{
			return ins.a == TCG_FX_IMM || ins.b == TCG_FX_IMM || ins.c == TCG_FX_IMM;
		});
	}

	std::vector<Node> nodes_;
	std::map<int,Parts> part_lists_;     // CONCAT / ADD of PADs -> its parts
	std::vector<PartProducts> part_calls_;
	std::map<int,int> emitted_parts_;    // index into part_calls_ -> index into the plan's part_products
	std::map<int,ConvFold> folds_;       // CONV node -> what is folded into its launch
	std::map<int,bool> feeds_convs_;     // memo of layout_feeds_convs
	std::unordered_map<teq::iTensor*,int> index_;
	std::vector<int> uf_, minpos_, maxpos_;
	std::vector<std::vector<int>> members_;
	std::vector<std::set<int>> deps_;
	std::vector<std::set<int>> vdeps_;   // unit -> units whose results it reads through folded views
	std::vector<size_t> stamp_;
	size_t clock_ = 0;
	// buffers rewritten by ASSIGN* nodes of the pass
	std::unordered_map<teq::iTensor*,int> resource_; // tensor owning the buffer -> id
	std::vector<std::vector<int>> write_pos_;        // id -> positions of the ASSIGN* nodes, ascending
	std::vector<int> writes_;                        // node -> id it rewrites, -1 for none
	std::vector<int> last_write_;                    // while grouping: id -> latest ASSIGN* seen
	std::vector<std::vector<int>> readers_;          // while grouping: id -> launches reading it since
};

}

/// The tensors in the order their functors were made (leaves last): the targets
/// of a pass come as an unordered set, and which launches share a kernel depends
/// on the order in which the functors under them are met
std::vector<teq::iTensor*> birth_order (std::vector<teq::iTensor*> tensors)
{
	auto born = [](teq::iTensor* t)
	{
		auto f = dynamic_cast<Observable*>(t);
		return nullptr == f ? std::numeric_limits<uint64_t>::max() : f->born();
	};
	std::stable_sort(tensors.begin(), tensors.end(), [&](teq::iTensor* a, teq::iTensor* b) { return born(a) < born(b); });
	return tensors;
}

FusionPlan plan_fusion (const std::vector<Observable*>& funcs, const teq::TensSetT& targets)
{
	Planner planner(funcs, targets);
	planner.group_all();
	return planner.finish();
}

std::string describe_step (const FusionPlan& plan, const FusionPlan::Step& step)
{
	if (nullptr != step.node) { return "node " + step.node->get_opcode().name_; }
	if (step.contract >= 0) { return "swapped CONTRACT+PERMUTE"; }
	if (step.sum >= 0) { return "summed CONTRACT x" + std::to_string(plan.sums[step.sum].a.size()); }
	if (step.parts >= 0 && step.group < 0) { return plan.part_products[step.parts].label; }
	if (step.conv >= 0) { return "viewed " + plan.convs[step.conv].label; }
	const FusedGroup& group = plan.groups[step.group];
	std::string out;
	if (step.parts >= 0) { out = plan.part_products[step.parts].label + " with epilogue "; }
	out += "group ";
	for (size_t i = 0; i < group.members.size(); ++i) { out += (i ? "+" : "") + group.members[i]->get_opcode().name_; }
	return out + " leaves=" + std::to_string(group.leaves.size()) + " stores=" + std::to_string(group.outputs.size()) +
		" instrs=" + std::to_string(group.program.size());
}

bool step_batchable (const FusionPlan& plan, const FusionPlan::Step& step)
{
	// a few iterations per lane of one workgroup: more is declined by the launch anyway
	constexpr size_t most = (size_t) 1 << 14;
	if (nullptr != step.node)
	{
		int op = (int) step.node->get_opcode().code_;
		bool known = is_unary(op) || is_binary(op) || op == egen::CONTRACT || op == egen::MATMUL ||
			op == egen::REDUCE_SUM || op == egen::REDUCE_PROD || op == egen::REDUCE_MIN || op == egen::REDUCE_MAX;
		if (false == known || step.node->shape().n_elems() > most) { return false; }
		for (auto& arg : step.node->get_args())
		{
			if (arg->shape().n_elems() > most) { return false; }
		}
		return true;
	}
	if (step.group >= 0 && step.parts < 0)
	{
		size_t n = 1;
		for (uint64_t extent : plan.groups[step.group].shape) { n *= (size_t) extent; }
		return n <= most;
	}
	if (step.contract >= 0)
	{
		const SwappedContract& c = plan.contracts[step.contract];
		return c.node->shape().n_elems() <= most && c.a->shape().n_elems() <= most && c.b->shape().n_elems() <= most;
	}
	return false;
}

static bool batches_enabled (void)
{
	static const bool on = []
	{
		const char* env = getenv("TCR_BATCHES");
		return !(env && env[0] == '0');
	}();
	return on;
}

std::vector<LaunchUnit> launch_units (const FusionPlan& plan, bool batches)
{
	std::vector<LaunchUnit> units;
	batches = batches && batches_enabled();
	for (size_t i = 0, n = plan.steps.size(); i < n;)
	{
		size_t end = i + 1;
		if (batches && step_batchable(plan, plan.steps[i]))
		{
			while (end < n && step_batchable(plan, plan.steps[end])) { ++end; }
		}
		units.push_back({i, end});
		i = end;
	}
	return units;
}

std::string describe_unit (const FusionPlan& plan, const LaunchUnit& unit)
{
	if (unit.second - unit.first < 2) { return describe_step(plan, plan.steps[unit.first]); }
	std::string out = "batch of " + std::to_string(unit.second - unit.first) + ":";
	for (size_t i = unit.first; i < unit.second; ++i)
	{
		const FusionPlan::Step& step = plan.steps[i];
		out += " ";
		if (nullptr != step.node) { out += step.node->get_opcode().name_; }
		else if (step.contract >= 0) { out += "CONTRACT+PERMUTE"; }
		else
		{
			auto& members = plan.groups[step.group].members;
			out += "(";
			for (size_t k = 0; k < members.size(); ++k) { out += (k ? "+" : "") + members[k]->get_opcode().name_; }
			out += ")";
		}
	}
	return out;
}

void launch_unit (const FusionPlan& plan, const LaunchUnit& unit, Device& device, const teq::TensSetT& targets,
	RangeTempsT& temps)
{
	if (unit.second - unit.first < 2)
	{
		launch_step(plan, plan.steps[unit.first], device, targets, temps);
		return;
	}
	// small steps in a row: held back and sent out as one launch where the launch
	// takes them (a step it does not take goes out by itself, in its place)
	tcg_ctx* ctx = hip_context();
	try
	{
		for (size_t i = unit.first; i < unit.second; ++i)
		{
			hip_check(tcg_batch_begin(ctx));
			launch_step(plan, plan.steps[i], device, targets, temps);
		}
	}
	catch (...)
	{
		(void) tcg_batch_end(ctx);
		throw;
	}
	hip_check(tcg_batch_end(ctx));
}

/// Off unless TCR_FORKS=1: on the two gradients of a 5x5 convolution over
/// 128 x 20 x 20 x 64 outputs the launches did overlap, and each ran as much
/// slower as the other took (0.413 ms per pass with the second stream, 0.401
/// without): neither leaves the compute units idle for the other to use
static bool forks_enabled (void)
{
	static const bool on = []
	{
		const char* env = getenv("TCR_FORKS");
		return env && env[0] == '1';
	}();
	return on;
}

/// Whether `tens` is `node` or shares its buffer (IDENTITY / RESHAPE / SLICE of it)
static bool same_buffer (const teq::iTensor* tens, const teq::iTensor* node)
{
	while (nullptr != tens)
	{
		if (tens == node) { return true; }
		auto f = dynamic_cast<const teq::iFunctor*>(tens);
		if (nullptr == f || false == is_buffer_alias((int) f->get_opcode().code_)) { return false; }
		tens = f->get_args().front().get();
	}
	return false;
}

/// Whether the step reads (or may write over) the value of `node`
static bool step_touches (const FusionPlan& plan, const FusionPlan::Step& step, const teq::iTensor* node)
{
	auto any = [node](const std::vector<teq::iTensor*>& reads)
	{
		return std::any_of(reads.begin(), reads.end(), [node](const teq::iTensor* t) { return same_buffer(t, node); });
	};
	if (nullptr != step.node)
	{
		if (is_assign((int) step.node->get_opcode().code_)) { return true; } // may rewrite a leaf the node's launch reads
		for (auto& arg : step.node->get_args())
		{
			if (same_buffer(arg.get(), node)) { return true; }
		}
		return false;
	}
	bool hit = false;
	if (step.conv >= 0)
	{
		const ViewedConv& c = plan.convs[step.conv];
		hit = any(c.reads) || same_buffer(c.image, node) || same_buffer(c.kernel, node);
	}
	if (step.contract >= 0)
	{
		const SwappedContract& c = plan.contracts[step.contract];
		hit = hit || any(c.reads) || same_buffer(c.a, node) || same_buffer(c.b, node);
	}
	if (step.sum >= 0) { hit = hit || any(plan.sums[step.sum].reads) || any(plan.sums[step.sum].a) || any(plan.sums[step.sum].b); }
	if (step.parts >= 0)
	{
		const PartProducts& p = plan.part_products[step.parts];
		hit = hit || any(p.reads);
		for (auto& product : p.products)
		{
			for (auto& term : product.terms) { hit = hit || same_buffer(term.a, node) || same_buffer(term.b, node); }
		}
	}
	if (step.group >= 0)
	{
		const FusedGroup& g = plan.groups[step.group];
		hit = hit || any(g.reads);
		for (auto& leaf : g.leaves) { hit = hit || (nullptr != leaf.base && same_buffer(leaf.base, node)); }
	}
	return hit;
}

static bool heavy_step (const FusionPlan::Step& step)
{
	if (nullptr != step.node)
	{
		int op = (int) step.node->get_opcode().code_;
		return op == egen::CONV || op == egen::CONTRACT || op == egen::MATMUL;
	}
	return step.conv >= 0 || step.contract >= 0 || step.sum >= 0 || step.parts >= 0;
}

void launch_pass (const FusionPlan& plan, Device& device, const teq::TensSetT& targets, RangeTempsT& temps,
	bool batches, bool forks)
{
	forks = forks && forks_enabled();
	tcg_ctx* ctx = hip_context();
	const std::vector<LaunchUnit> units = launch_units(plan, batches);
	const teq::iTensor* forked = nullptr;     // the node whose launch runs on the second stream
	std::vector<teq::iTensor*> forked_reads;  // what it reads: counted as read when it has been waited for
	auto join = [&]
	{
		hip_check(tcg_join(ctx));
		for (teq::iTensor* tens : forked_reads) { eigen_ref(*tens).odevice(); }
		forked_reads.clear();
		forked = nullptr;
	};
	try
	{
		for (size_t u = 0; u < units.size(); ++u)
		{
			const LaunchUnit& unit = units[u];
			if (nullptr != forked)
			{
				bool touches = false;
				for (size_t i = unit.first; i < unit.second && false == touches; ++i) { touches = step_touches(plan, plan.steps[i], forked); }
				if (touches) { join(); }
			}
			const FusionPlan::Step& step = plan.steps[unit.first];
			if (forks && nullptr == forked && unit.second - unit.first == 1 && step.conv >= 0)
			{
				// a convolution whose result nothing reads before another product has been
				// launched: the two run side by side
				const teq::iTensor* node = plan.convs[step.conv].node;
				bool beside = false;
				for (size_t i = unit.second; i < plan.steps.size() && false == step_touches(plan, plan.steps[i], node); ++i)
				{
					beside = beside || heavy_step(plan.steps[i]);
				}
				if (beside)
				{
					hip_check(tcg_fork(ctx));
					forked = node;
					launch_conv(plan.convs[step.conv], targets, device.memory(), &forked_reads);
					hip_check(tcg_fork_end(ctx));
					continue;
				}
			}
			launch_unit(plan, unit, device, targets, temps);
		}
		if (nullptr != forked) { join(); }
	}
	catch (...)
	{
		(void) tcg_join(ctx);
		throw;
	}
}

void launch_step (const FusionPlan& plan, const FusionPlan::Step& step, Device& device, const teq::TensSetT& targets,
	RangeTempsT& temps)
{
	if (nullptr != step.node) { device.calc_forced(*step.node, (size_t) (targets.count(step.node) > 0)); }
	else if (step.conv >= 0) { launch_conv(plan.convs[step.conv], targets, device.memory()); }
	else if (step.contract >= 0) { launch_contract(plan.contracts[step.contract], targets, device.memory()); }
	else if (step.sum >= 0) { launch_sum(plan.sums[step.sum], targets, device.memory()); }
	else if (step.parts >= 0 && step.group >= 0)
	{
		launch_group(plan.groups[step.group], targets, device.memory(), temps, &plan.part_products[step.parts], step.parts, &plan);
	}
	else if (step.parts >= 0) { launch_parts(plan.part_products[step.parts], targets, device.memory(), temps[step.parts]); }
	else { launch_group(plan.groups[step.group], targets, device.memory(), temps); }
}

void launch_contract (const SwappedContract& call, const teq::TensSetT& targets, RTMemptrT& memory)
{
	Observable* out = call.node;
	size_t ttl = std::max<size_t>(1, out->nsubs() + (size_t) (targets.count(out) > 0));
	void* dst = static_cast<iEigen&>(out->device()).borrow_output(ttl, memory);
	if (nullptr == dst) { global::fatalf("%s cannot take a product", out->to_string().c_str()); }
	const void* a = eigen_ref(*call.a).device_data();
	const void* b = eigen_ref(*call.b).device_data();
	if (nullptr == a || nullptr == b)
	{
		global::fatalf("operand %s of the matrix product behind %s has no data",
			(nullptr == a ? call.a : call.b)->to_string().c_str(), out->to_string().c_str());
	}
	try
	{
		hip_check(tcg_contract(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype), call.ashape.data(), call.bshape.data(),
			(int) (call.pairs.size() / 2), call.pairs.data(), a, b, dst));
	}
	catch (...)
	{
		static_cast<iEigen&>(out->device()).drop(); // an unfilled buffer must not read as a value
		throw;
	}
	for (teq::iTensor* tens : call.reads) { eigen_ref(*tens).odevice(); }
}

void launch_sum (const SummedContracts& call, const teq::TensSetT& targets, RTMemptrT& memory)
{
	Observable* out = call.node;
	size_t ttl = std::max<size_t>(1, out->nsubs() + (size_t) (targets.count(out) > 0));
	auto& ref = static_cast<iEigen&>(out->device());
	void* dst = ref.borrow_output(ttl, memory);
	if (nullptr == dst) { global::fatalf("%s cannot take a sum of products", out->to_string().c_str()); }
	std::vector<const void*> a, b;
	for (size_t t = 0; t < call.a.size(); ++t)
	{
		a.push_back(eigen_ref(*call.a[t]).device_data());
		b.push_back(eigen_ref(*call.b[t]).device_data());
		if (nullptr == a.back() || nullptr == b.back())
		{
			global::fatalf("operand %s of term %d of the sum of products %s has no data",
				(nullptr == a.back() ? call.a[t] : call.b[t])->to_string().c_str(), (int) t, out->to_string().c_str());
		}
	}
	try
	{
		hip_check(tcg_contract_sum(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype), call.ashape.data(), call.bshape.data(),
			(int) (call.pairs.size() / 2), call.pairs.data(), (int) a.size(), a.data(), b.data(), dst));
	}
	catch (...)
	{
		ref.drop();
		throw;
	}
	for (teq::iTensor* tens : call.reads) { eigen_ref(*tens).odevice(); }
}

void launch_parts (const PartProducts& call, const teq::TensSetT& targets, RTMemptrT& memory, std::pair<void*,size_t>& temp)
{
	Observable* out = call.node;
	const int64_t esz = (int64_t) egen::type_size((egen::_GENERATED_DTYPE) call.dtype);
	if (call.ranges > 0)
	{
		// the node gets no buffer: its K ranges wait in `temp` for the groups that add them up
		const PartProducts::Product& p = call.products.at(0);
		std::vector<const void*> a, b;
		std::vector<uint64_t> lda, ldb;
		for (const PartProducts::Term& term : p.terms)
		{
			const char* pa = (const char*) eigen_ref(*term.a).device_data();
			const char* pb = (const char*) eigen_ref(*term.b).device_data();
			if (nullptr == pa || nullptr == pb)
			{
				global::fatalf("operand %s of the products over parts %s has no data",
					(nullptr == pa ? term.a : term.b)->to_string().c_str(), call.label.c_str());
			}
			a.push_back(pa + esz * term.a_off);
			b.push_back(pb + esz * term.b_off);
			lda.push_back(term.lda);
			ldb.push_back(term.ldb);
		}
		if (nullptr == memory) { global::fatal("cannot borrow from null memory"); }
		temp.second = (size_t) esz * call.ranges * p.M * p.N;
		temp.first = memory->allocate(temp.second);
		if (call.ranges == 1)
		{
			// (a product that waited for a launch it could have been the epilogue of)
			hip_check(tcg_gemm_terms(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype), p.M, p.N, p.K,
				(int) p.terms.size(), a.data(), lda.data(), p.trans_a, b.data(), ldb.data(), p.trans_b, temp.first, p.N));
		}
		else
		{
			hip_check(tcg_gemm_terms_ranges(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype), p.M, p.N, p.K,
				(int) p.terms.size(), a.data(), lda.data(), p.trans_a, b.data(), ldb.data(), p.trans_b,
				(int) call.ranges, temp.first));
		}
		for (teq::iTensor* tens : call.reads) { eigen_ref(*tens).odevice(); }
		return;
	}
	size_t ttl = std::max<size_t>(1, out->nsubs() + (size_t) (targets.count(out) > 0));
	auto& ref = static_cast<iEigen&>(out->device());
	char* dst = (char*) ref.borrow_output(ttl, memory);
	if (nullptr == dst) { global::fatalf("%s cannot take products over parts", out->to_string().c_str()); }
	if (call.partial) { ref.mark_partial(); }
	if (call.grid_m > 0)
	{
		// the blocks of one result: row i brings the A operands, column j the B operands
		const size_t nterms = call.products.at(0).terms.size();
		std::vector<uint64_t> mp, np, lda, ldb;
		std::vector<const void*> a, b;
		auto address = [&](teq::iTensor* tens, int64_t off)
		{
			const char* base = (const char*) eigen_ref(*tens).device_data();
			if (nullptr == base) { global::fatalf("operand %s of the blocks %s has no data", tens->to_string().c_str(), call.label.c_str()); }
			return (const void*) (base + esz * off);
		};
		for (uint32_t i = 0; i < call.grid_m; ++i)
		{
			const PartProducts::Product& p = call.products.at((size_t) i * call.grid_n);
			mp.push_back(p.M);
			lda.push_back(p.terms[0].lda);
			for (const PartProducts::Term& term : p.terms) { a.push_back(address(term.a, term.a_off)); }
		}
		for (uint32_t j = 0; j < call.grid_n; ++j)
		{
			const PartProducts::Product& p = call.products.at(j);
			np.push_back(p.N);
			ldb.push_back(p.terms[0].ldb);
			for (const PartProducts::Term& term : p.terms) { b.push_back(address(term.b, term.b_off)); }
		}
		const PartProducts::Product& first = call.products[0];
		try
		{
			hip_check(tcg_gemm_terms_grid(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype),
				(int) call.grid_m, mp.data(), (int) call.grid_n, np.data(), first.K, (int) nterms,
				a.data(), lda.data(), first.trans_a, b.data(), ldb.data(), first.trans_b,
				dst + esz * first.c_off, first.ldc));
		}
		catch (...)
		{
			ref.drop();
			throw;
		}
		for (teq::iTensor* tens : call.reads) { eigen_ref(*tens).odevice(); }
		return;
	}
	try
	{
		for (const PartProducts::Product& p : call.products)
		{
			std::vector<const void*> a, b;
			std::vector<uint64_t> lda, ldb;
			for (const PartProducts::Term& term : p.terms)
			{
				const char* pa = (const char*) eigen_ref(*term.a).device_data();
				const char* pb = (const char*) eigen_ref(*term.b).device_data();
				if (nullptr == pa || nullptr == pb)
			{
				global::fatalf("operand %s of the products over parts %s has no data",
					(nullptr == pa ? term.a : term.b)->to_string().c_str(), call.label.c_str());
			}
				a.push_back(pa + esz * term.a_off);
				b.push_back(pb + esz * term.b_off);
				lda.push_back(term.lda);
				ldb.push_back(term.ldb);
			}
			hip_check(tcg_gemm_terms(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype), p.M, p.N, p.K,
				(int) p.terms.size(), a.data(), lda.data(), p.trans_a, b.data(), ldb.data(), p.trans_b,
				dst + esz * p.c_off, p.ldc));
		}
	}
	catch (...)
	{
		ref.drop();
		throw;
	}
	for (teq::iTensor* tens : call.reads) { eigen_ref(*tens).odevice(); }
}

void launch_conv (const ViewedConv& call, const teq::TensSetT& targets, RTMemptrT& memory,
	std::vector<teq::iTensor*>* later_reads)
{
	Observable* out = call.node;
	size_t ttl = std::max<size_t>(1, out->nsubs() + (size_t) (targets.count(out) > 0));
	auto& ref = static_cast<iEigen&>(out->device());
	void* dst = ref.borrow_output(ttl, memory);
	if (nullptr == dst) { global::fatalf("%s cannot take a convolution", out->to_string().c_str()); }
	const void* image = eigen_ref(*call.image).device_data();
	const void* kernel = eigen_ref(*call.kernel).device_data();
	if (nullptr == image || nullptr == kernel) { global::fatal("operand of a convolution has no data"); }
	if (call.windowed) { ref.mark_partial(); }
	// addresses of the first image element inside the box, of kernel element 0
	// and of the first output of the window
	const int64_t esz = (int64_t) egen::type_size((egen::_GENERATED_DTYPE) call.dtype);
	int64_t first_image = call.image_off, first_out = call.out_off;
	for (int d = 0; d < 8; ++d)
	{
		first_image += (int64_t) call.ilo[d] * call.image_stride[d];
		first_out += (int64_t) call.olo[d] * call.out_stride[d];
	}
	try
	{
		hip_check(tcg_conv_views(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype),
			call.imgshape.data(), call.kshape.data(), (int) call.ranks.size(), call.ranks.data(),
			call.ilo.data(), call.ihi.data(), call.olo.data(), call.ohi.data(),
			(const char*) image + esz * first_image, call.image_stride.data(),
			(const char*) kernel + esz * call.kernel_off, call.kernel_stride.data(),
			(char*) dst + esz * first_out, call.out_stride.data()));
	}
	catch (...)
	{
		ref.drop();
		throw;
	}
	if (nullptr != later_reads) { later_reads->insert(later_reads->end(), call.reads.begin(), call.reads.end()); }
	else { for (teq::iTensor* tens : call.reads) { eigen_ref(*tens).odevice(); } }
}

/// The product of `call` with `group` as its epilogue, one launch; false when
/// the kernel does not take the shapes (nothing has been launched then)
/// The copy of a padded operand (FusionPlan::padded) for this pass: made by the
/// first launch that asks for it, given back with the pass's temporaries
static const char* padded_copy (const FusionPlan& plan, int index, RTMemptrT& memory, RangeTempsT& temps)
{
	const FusionPlan::PaddedOperand& op = plan.padded.at(index);
	std::pair<void*,size_t>& slot = temps.at(plan.part_products.size() + (size_t) index);
	if (nullptr == slot.first)
	{
		const void* src = eigen_ref(*op.tensor).device_data();
		if (nullptr == src) { global::fatalf("operand %s has no data", op.tensor->to_string().c_str()); }
		size_t bytes = (size_t) (op.rows * (op.ld + op.pad)) * egen::type_size((egen::_GENERATED_DTYPE) op.dtype);
		void* dst = memory->allocate(bytes);
		if (nullptr == dst) { global::fatal("no memory for the copy of an operand"); }
		slot = {dst, bytes};
		const uint64_t shape[8] = {op.ld, op.rows, 1, 1, 1, 1, 1, 1};
		const uint64_t before[8] = {0, 0, 0, 0, 0, 0, 0, 0};
		const uint64_t after[8] = {op.pad, 0, 0, 0, 0, 0, 0, 0};
		hip_check(tcg_pad(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) op.dtype), shape, before, after, src, dst));
	}
	return (const char*) slot.first;
}

static bool launch_with_epilogue (const PartProducts& call, const FusedGroup& group, int producer_index,
	const std::vector<void*>& outs, const FusionPlan* plan, RTMemptrT& memory, RangeTempsT& temps)
{
	const PartProducts::Product& p = call.products.at(0);
	const int64_t esz = (int64_t) egen::type_size((egen::_GENERATED_DTYPE) call.dtype);
	std::vector<const void*> a, b;
	std::vector<uint64_t> lda, ldb;
	for (const PartProducts::Term& term : p.terms)
	{
		const char* pa = (const char*) eigen_ref(*term.a).device_data();
		const char* pb = (const char*) eigen_ref(*term.b).device_data();
		if (nullptr == pa || nullptr == pb)
		{
			global::fatalf("operand %s of the products over parts %s has no data",
				(nullptr == pa ? term.a : term.b)->to_string().c_str(), call.label.c_str());
		}
		a.push_back(pa + esz * term.a_off);
		lda.push_back(term.lda);
		if (term.b_padded >= 0 && nullptr != plan)
		{
			// the same element of the copy: rows are `pad` elements further apart there
			const FusionPlan::PaddedOperand& op = plan->padded.at(term.b_padded);
			const int64_t row = term.b_off / (int64_t) op.ld, col = term.b_off % (int64_t) op.ld;
			b.push_back(padded_copy(*plan, term.b_padded, memory, temps) + esz * (row * (int64_t) (op.ld + op.pad) + col));
			ldb.push_back(op.ld + op.pad);
		}
		else
		{
			b.push_back(pb + esz * term.b_off);
			ldb.push_back(term.ldb);
		}
	}
	std::vector<tcg_fx_leaf> leaves;
	for (auto& leaf : group.leaves)
	{
		tcg_fx_leaf view = leaf.view;
		if (leaf.ranges_of == producer_index)
		{
			// the view over the dense window, as the kernel's own result
			view.ptr = nullptr;
			view.from_product = 1;
			view.nsum = 0;
			view.sum_stride = 0;
		}
		else
		{
			view.ptr = eigen_ref(*leaf.base).device_data();
			if (nullptr == view.ptr) { global::fatalf("operand %s has no data", leaf.base->to_string().c_str()); }
		}
		leaves.push_back(view);
	}
	int rc = tcg_gemm_terms_fx(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) call.dtype), p.M, p.N, p.K,
		(int) p.terms.size(), a.data(), lda.data(), p.trans_a, b.data(), ldb.data(), p.trans_b,
		group.shape.data(), (int) leaves.size(), leaves.data(), (int) group.program.size(), group.program.data(),
		(int) outs.size(), outs.data());
	if (TCG_ERR_UNSUPPORTED == rc) { return false; }
	hip_check(rc);
	return true;
}

void launch_group (const FusedGroup& group, const teq::TensSetT& targets, RTMemptrT& memory, RangeTempsT& temps,
	const PartProducts* producer, int producer_index, const FusionPlan* plan)
{
	std::vector<void*> outs;
	for (Observable* out : group.outputs)
	{
		size_t ttl = std::max<size_t>(1, out->nsubs() + (size_t) (targets.count(out) > 0));
		void* ptr = static_cast<iEigen&>(out->device()).borrow_output(ttl, memory);
		if (nullptr == ptr) { global::fatalf("%s cannot take a fused result", out->to_string().c_str()); }
		outs.push_back(ptr);
	}
	try
	{
		bool done = false;
		if (nullptr != producer)
		{
			done = launch_with_epilogue(*producer, group, producer_index, outs, plan, memory, temps);
			if (false == done)
			{
				// two launches after all: the product into temporary memory first
				launch_parts(*producer, targets, memory, temps.at(producer_index));
			}
			else
			{
				for (teq::iTensor* tens : producer->reads) { eigen_ref(*tens).odevice(); }
			}
		}
		if (false == done)
		{
			std::vector<tcg_fx_leaf> leaves;
			for (auto& leaf : group.leaves)
			{
				tcg_fx_leaf view = leaf.view;
				view.ptr = leaf.ranges_of >= 0 ? temps.at(leaf.ranges_of).first : eigen_ref(*leaf.base).device_data();
				if (nullptr == view.ptr) { global::fatalf("operand %s has no data", leaf.base->to_string().c_str()); }
				leaves.push_back(view);
			}
			hip_check(tcg_ew_fusedx(hip_context(), egen::device_type((egen::_GENERATED_DTYPE) group.dtype), group.shape.data(), (int) leaves.size(), leaves.data(),
				(int) group.program.size(), group.program.data(), (int) outs.size(), outs.data()));
		}
	}
	catch (...)
	{
		for (Observable* out : group.outputs) { static_cast<iEigen&>(out->device()).drop(); }
		throw;
	}
	for (teq::iTensor* tens : group.reads) { eigen_ref(*tens).odevice(); }
	for (int done : group.frees)
	{
		// after this launch in stream order
		std::pair<void*,size_t>& temp = temps.at(done);
		if (nullptr != temp.first) { memory->deallocate(temp.first, temp.second); }
		temp = {nullptr, 0};
	}
}

}
