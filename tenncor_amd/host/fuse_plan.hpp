// Grouping of elementwise functors for the replaying evaluator: which nodes
// of an evaluation pass are computed together in one tcg_ew_fusedx launch,
// which EXTEND / SLICE / PAD / PERMUTE / IDENTITY nodes are never materialised
// because elementwise groups read straight through them, which PAD / PERMUTE /
// REVERSE nodes round a convolution become strides of its launch, and in which
// order the remaining launches run.  The reference evaluates one node at a time
// (internal/teq/evaluator.hpp:33-45 calling internal/eigen/device.hpp:555-570);
// Eigen fuses only inside one node's expression.
#ifndef TCH_FUSE_PLAN_HPP
#define TCH_FUSE_PLAN_HPP

#include "eigen_device.hpp"

namespace eigen
{

/// One launch computing several elementwise nodes
struct FusedGroup final
{
	struct Leaf final
	{
		teq::iTensor* base = nullptr; ///< materialised tensor the view starts from
		tcg_fx_leaf view = {};        ///< ptr is filled in at launch
		/// >= 0: the operand is the sum of the K ranges that product
		/// (FusionPlan::part_products) left side by side instead of a tensor's value
		int ranges_of = -1;
	};

	int dtype = 0;
	std::array<uint64_t,8> shape;
	std::vector<Observable*> members;  ///< in evaluation order
	std::vector<Observable*> outputs;  ///< members whose value is stored, by output index
	std::vector<Leaf> leaves;
	std::vector<tcg_fx_instr> program;
	/// materialised tensors that count one read when this group has launched:
	/// what the members and the views folded into them would have read
	std::vector<teq::iTensor*> reads;
	/// products (FusionPlan::part_products) whose K ranges nothing reads after this group
	std::vector<int> frees;
};

/// PERMUTE{1,0}(CONTRACT(a, b)) with a matrix result is CONTRACT(b, a) with
/// the pairs swapped: one product written straight into the PERMUTE node's
/// buffer, no transposition pass (the shape every matrix-product gradient
/// takes, tenncor/eteq/backprop.hpp:269-359)
struct SwappedContract final
{
	Observable* node = nullptr;      ///< the PERMUTE node that receives the result
	teq::iTensor* a = nullptr;       ///< first operand of the product that is launched
	teq::iTensor* b = nullptr;
	std::array<uint64_t,8> ashape, bshape;
	std::vector<uint64_t> pairs;     ///< flattened (dim of a, dim of b)
	int dtype = 0;
	std::vector<teq::iTensor*> reads;
};

/// ADD over CONTRACT nodes of one pair of shapes (or over their PERMUTE{1,0}
/// forms, see SwappedContract), each read by the ADD alone: the sum of products
/// the gradient builder makes for a weight that many nodes read
/// (tenncor/eteq/backprop.hpp:563-567 over :269-359 -- one term per step of an
/// unrolled recurrent layer).  Launched as one tcg_contract_sum into the ADD
/// node's buffer; the terms never hold values of their own.
struct SummedContracts final
{
	Observable* node = nullptr;      ///< the ADD node that receives the result
	std::vector<teq::iTensor*> a, b; ///< operands of the products as launched, in term order
	std::array<uint64_t,8> ashape, bshape;
	std::vector<uint64_t> pairs;     ///< flattened (dim of a, dim of b)
	int dtype = 0;
	std::vector<teq::iTensor*> reads;
};

/// A CONV node computed from the tensors its operands are layouts of, into the
/// tensor its result is a layout of.  tenncor surrounds every convolution with
/// nodes that only move data: conv2d reverses the kernel, pads a singleton axis
/// of the image and permutes the result (cfg/tenncor/nn.yml:88-93); its
/// gradients permute and pad the upstream gradient in front of the correlation
/// and permute and reverse what comes out (tenncor/eteq/backprop.hpp:372-439).
/// Where convolutions are all that read such a PAD / PERMUTE / REVERSE node,
/// and where one PERMUTE / REVERSE is all that reads the result, none of these
/// is laid out: the correlation reads and writes through element strides
/// (tcg_conv_views), and the padded image exists only as the box in which the
/// operand sits inside the zero border.
struct ViewedConv final
{
	Observable* node = nullptr;      ///< receives the result: the CONV node, or the last PERMUTE / REVERSE behind it
	teq::iTensor* image = nullptr;   ///< materialised tensor the image is read from
	teq::iTensor* kernel = nullptr;  ///< materialised tensor the kernel is read from
	std::array<uint64_t,8> imgshape, kshape; ///< of the CONV node's operands as it sees them
	std::array<uint64_t,8> ilo, ihi; ///< where the image is not zero border
	/// image element c (inside the box) is element image_off + sum c[d] * image_stride[d] of `image`
	int64_t image_off = 0;
	std::array<int64_t,8> image_stride;
	/// kernel element w is element kernel_off + sum w[i] * kernel_stride[i] of `kernel`
	int64_t kernel_off = 0;
	std::array<int64_t,8> kernel_stride;
	bool windowed = false;           ///< only SLICEs read the result:
	std::array<uint64_t,8> olo, ohi; ///< their bounding box (else the whole result)
	/// output element c is element out_off + sum c[d] * out_stride[d] of `node`'s buffer
	int64_t out_off = 0;
	std::array<int64_t,8> out_stride;
	std::vector<uint64_t> ranks;
	int dtype = 0;
	std::vector<teq::iTensor*> reads;
	std::string label;               ///< the nodes this launch stands for, for printing
};

/// Matrix products over operands that are parts of tensors, launched as
/// tcg_gemm_terms calls into one node's buffer.  A contraction over a dim
/// along which an operand is a concatenation -- a CONCAT (the input and the
/// hidden state in front of the gate product of a recurrent cell,
/// cfg/tenncor/layer.yml:716-768) or an ADD of PADs that tile the dim (the
/// gradient of the SLICEs that cut the gates back out,
/// tenncor/eteq/backprop.hpp:402-421) -- is the sum of the products of the
/// parts with the rows of the other operand they meet; a sum of products
/// whose operands are concatenations along a dim that survives (the weight
/// gradient of such a cell) falls into blocks of the result, one sum of
/// products per pair of parts.  Where products are all that read such a
/// concatenation it is never laid out.
struct PartProducts final
{
	struct Term final
	{
		teq::iTensor* a = nullptr;  ///< materialised tensors the operands are read from,
		teq::iTensor* b = nullptr;
		int64_t a_off = 0, b_off = 0; ///< element offsets of A_t(0, 0) and B_t(0, 0) in them
		uint64_t lda = 0, ldb = 0;
		/// >= 0: B_t is read from that copy of `b` with a longer leading dim
		/// (FusionPlan::padded) by the launch that has the epilogue
		int b_padded = -1;
	};

	/// C[c_off + m * ldc + n] = sum_t sum_k A_t(m, k) B_t(k, n), flags as tcg_gemm
	struct Product final
	{
		uint64_t M = 0, N = 0, K = 0;
		bool trans_a = false, trans_b = false;
		std::vector<Term> terms;
		int64_t c_off = 0;
		uint64_t ldc = 0;
	};

	Observable* node = nullptr;      ///< receives the results
	int dtype = 0;
	std::vector<Product> products;
	bool partial = false;            ///< only the window its SLICE readers look at is computed
	/// > 0: the node is never laid out; the product leaves that many K ranges of
	/// its window side by side in temporary memory ([range][M][N]) and the
	/// elementwise groups that read the node add them up while they load
	uint32_t ranges = 0;
	/// With `ranges` > 0: when one launch of elementwise nodes is all that reads
	/// the node, the product may run as one launch with that group as its
	/// epilogue (tcg_gemm_terms_fx) instead of leaving anything in memory
	bool epilogue = false;
	/// > 0: `products` are the grid_m x grid_n blocks (row by row) of one result
	/// whose operands are concatenated along the dims that survive, every block
	/// (i, j) with the A operands of row i and the B operands of column j and
	/// one leading dim per part: launched as one tcg_gemm_terms_grid
	uint32_t grid_m = 0, grid_n = 0;
	std::vector<teq::iTensor*> reads;
	std::string label;
};

struct FusionPlan final
{
	struct Step final
	{
		Observable* node = nullptr; ///< launched through its own closure, or
		int group = -1;             ///< index into groups, or
		int contract = -1;          ///< index into contracts, or
		int conv = -1;              ///< index into convs, or
		int sum = -1;               ///< index into sums, or
		int parts = -1;             ///< index into part_products
		/// parts and group both >= 0: the product with the group that reads it as
		/// its epilogue, one launch where the kernel takes the shapes, else the two
	};

	std::vector<FusedGroup> groups;
	std::vector<SwappedContract> contracts;
	std::vector<ViewedConv> convs;
	std::vector<SummedContracts> sums;
	std::vector<PartProducts> part_products;
	/// A leaf that many products with an epilogue read as their K-contiguous B
	/// operand under a leading dim that is a multiple of 32 elements (the
	/// transposed weight of every backward step of an unrolled recurrent layer):
	/// such a product loads its operands straight into registers in the layout
	/// of the matrix instruction, sixteen rows a power of two apart per load, and
	/// runs a quarter faster when the rows are `pad` elements further apart
	/// (measured: 12.3 -> 9.2 us per step with 16).  The pass makes one copy with
	/// the longer leading dim in front of the first product that reads it
	/// (`rows` x `ld` elements, one tcg_pad) and gives it back at its end; it lives
	/// in the pass's temporaries behind those of part_products.
	struct PaddedOperand final
	{
		teq::iTensor* tensor = nullptr;
		uint64_t rows = 0, ld = 0, pad = 0;
		int dtype = 0;
	};
	std::vector<PaddedOperand> padded;
	std::vector<Step> steps;
	/// functors that are computed inside a group or folded into operand views
	/// and therefore never hold a value of their own
	std::vector<Observable*> absorbed;
};

/// The tensors in the order their functors were made (leaves last): the targets
/// of a pass come as an unordered set, and which launches share a kernel depends
/// on the order in which the functors under them are met, so they are walked in
/// this order rather than in the order of their addresses
std::vector<teq::iTensor*> birth_order (std::vector<teq::iTensor*> tensors);

/// `funcs`: every functor under the targets, children first
FusionPlan plan_fusion (const std::vector<Observable*>& funcs, const teq::TensSetT& targets);

/// Enqueue one group: borrows the outputs' buffers (lifetimes as
/// eigen::Device::calc gives them), launches, counts the reads
/// Temporary memory of the products that leave K ranges, by index into
/// FusionPlan::part_products: {address, bytes}, held from the product's
/// launch to the last group that reads it
using RangeTempsT = std::vector<std::pair<void*,size_t>>;

/// An empty set of temporaries for one pass over `plan`: one slot per product
/// that may leave K ranges, then one per padded operand
inline RangeTempsT pass_temps (const FusionPlan& plan)
{
	return RangeTempsT(plan.part_products.size() + plan.padded.size(), {nullptr, 0});
}

/// `producer` (with its index into the plan's part_products): the product whose
/// result only this group reads, launched with it (see FusionPlan::Step)
/// `plan`: where the padded operands of the producer's terms are described
void launch_group (const FusedGroup& group, const teq::TensSetT& targets, RTMemptrT& memory, RangeTempsT& temps,
	const PartProducts* producer = nullptr, int producer_index = -1, const FusionPlan* plan = nullptr);

void launch_contract (const SwappedContract& call, const teq::TensSetT& targets, RTMemptrT& memory);

/// later_reads: the operands are not counted as read now but appended there, for
/// a launch that runs beside the launches that follow it (the caller counts them
/// when it has waited for the launch)
void launch_conv (const ViewedConv& call, const teq::TensSetT& targets, RTMemptrT& memory,
	std::vector<teq::iTensor*>* later_reads = nullptr);

void launch_sum (const SummedContracts& call, const teq::TensSetT& targets, RTMemptrT& memory);

void launch_parts (const PartProducts& call, const teq::TensSetT& targets, RTMemptrT& memory, std::pair<void*,size_t>& temp);

/// One line for a step: what is launched (tcr_launch_plan prints these)
std::string describe_step (const FusionPlan& plan, const FusionPlan::Step& step);

/// Enqueues the launches of one step, whatever its kind
void launch_step (const FusionPlan& plan, const FusionPlan::Step& step, Device& device, const teq::TensSetT& targets,
	RangeTempsT& temps);

/// What goes out together: one step, or a run [first, second) of steps over a
/// few thousand elements each (elementwise groups, reductions, contractions),
/// which are handed over between tcg_batch_begin and tcg_batch_end and run as
/// the steps of one kernel.  TCR_BATCHES=0 makes every step a unit of its own.
using LaunchUnit = std::pair<size_t,size_t>;

std::vector<LaunchUnit> launch_units (const FusionPlan& plan, bool batches = true);

std::string describe_unit (const FusionPlan& plan, const LaunchUnit& unit);

void launch_unit (const FusionPlan& plan, const LaunchUnit& unit, Device& device, const teq::TensSetT& targets,
	RangeTempsT& temps);

/// The whole pass, unit by unit.  forks: a convolution whose result nothing
/// reads before another convolution or product has been launched goes to the
/// context's second stream (tcg_fork) and runs beside what follows, up to the
/// first launch that reads it, rewrites a leaf, or the end of the pass; its
/// operands stay allocated until then.  Only with TCR_FORKS=1 in the environment
/// (measured without gain on the gradients of a convolutional layer).
void launch_pass (const FusionPlan& plan, Device& device, const teq::TensSetT& targets, RangeTempsT& temps,
	bool batches, bool forks);

}

#endif // TCH_FUSE_PLAN_HPP
