// An evaluator for graphs that are evaluated again and again with new leaf
// values (training and inference loops such as tenncor/bm/benchmark.cpp:
// 334-393): the launches of one full pass of teq::Evaluator
// (internal/teq/evaluator.hpp:11-61) are recorded into a device-side launch
// sequence the first time a set of targets comes back, and later passes
// enqueue that sequence as a whole instead of walking the graph node by node.
// Installed like any other evaluator, through teq::set_eval (the precedent
// for swapping evaluators is dbg/peval/plugin_eval.hpp:21-42).
//
// What a replay guarantees is what the plain evaluator guarantees: after
// evaluate() every target holds the value of its expression over the current
// leaf values, every node has the version the plain pass would have given it,
// and intermediate buffers have been read out and handed back.  What differs:
// a replay recomputes every functor under the targets (the plain pass skips
// a functor whose operands did not move and whose value is still held), and
// the buffers the recorded launches write stay reserved for the recording.
#ifndef TCH_REPLAY_EVAL_HPP
#define TCH_REPLAY_EVAL_HPP

#include <map>
#include <memory>
#include <string>

#include "eigen_device.hpp"

namespace eigen
{

struct ReplayEvaluator final : public teq::iEvaluator
{
	struct Stats final
	{
		size_t plain = 0;     ///< passes handed to the node-by-node evaluator
		size_t recorded = 0;  ///< recordings made
		size_t replayed = 0;  ///< passes served by a recording
		size_t skipped = 0;   ///< passes with nothing to do
		size_t launches = 0;  ///< device launches in the most recent recording
		size_t reserved_bytes = 0; ///< device memory held by live recordings
		size_t record_failures = 0; ///< target sets whose pass could not be recorded
		/// What the most recent recording cost on the host: milliseconds from
		/// planning to the finished launch sequence, of which `jit_ms` went into
		/// `jit_compiled` kernels compiled at run time and `jit_from_disk`
		/// kernels an earlier process had left on disk
		double record_ms = 0.0, jit_ms = 0.0;
		size_t jit_compiled = 0, jit_from_disk = 0;
		/// why the latest of them could not ("" when none): the message of the
		/// failure raised while recording; the set is walked node by node instead
		std::string record_error;
	};

	/// A set of targets is recorded when it is asked for the
	/// (`warm_passes` + 1)-th time; at most `max_plans` recordings are kept
	/// With `fuse`, elementwise functors that feed one another are computed
	/// in shared launches (fuse_plan.hpp); with `small_passes` as well, the
	/// pass over a graph of small tensors is recorded as the steps of one
	/// kernel (sums then run in index order: equal to the walk within the
	/// tolerance of reductions and contractions, not bit for bit)
	ReplayEvaluator (size_t warm_passes = 1, size_t max_plans = 16, bool fuse = true, bool small_passes = true);

	~ReplayEvaluator (void);

	void evaluate (teq::iDevice& device, const teq::TensSetT& targets,
		const teq::TensSetT& ignored = {}) override;

	/// Forget every recording (their memory returns to the pool)
	void clear (void);

	const Stats& stats (void) const { return stats_; }

private:
	struct Plan;

	struct Slot final
	{
		size_t seen = 0;
		bool unplannable = false;
		size_t last_used = 0;
		std::unique_ptr<Plan> plan;
	};

	using KeyT = std::vector<teq::iTensor*>;

	void plain (teq::iDevice& device, const teq::TensSetT& targets, const teq::TensSetT& ignored);

	std::unique_ptr<Plan> record (Device& device, const KeyT& key, const teq::TensSetT& targets);

	bool replay (Device& device, Plan& plan);

	void evict (void);

	static void release (Plan& plan);

	std::map<KeyT,Slot> slots_;
	teq::Evaluator plain_;
	Stats stats_;
	size_t warm_passes_;
	size_t max_plans_;
	bool fuse_;
	bool small_passes_ = true;
	size_t epoch_ = 0;
	size_t clock_ = 0;
};

}

#endif // TCH_REPLAY_EVAL_HPP
