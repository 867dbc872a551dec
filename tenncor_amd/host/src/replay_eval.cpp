// Recording and replaying whole evaluation passes (see replay_eval.hpp).
#include "replay_eval.hpp"

#include <limits>
#include <unordered_map>
#include "fuse_plan.hpp"

#include <algorithm>
#include <chrono>
#include <cstdlib>

namespace eigen
{

namespace
{

/// Functors under the targets in the order the plain evaluator computes them
/// (children first, internal/teq/evaluator.hpp:33-45), and the leaves
struct Collector final : public teq::iOnceTraveler
{
	std::vector<Observable*> funcs_;
	std::vector<teq::iLeaf*> leaves_;

private:
	void visit_leaf (teq::iLeaf& leaf) override { leaves_.push_back(&leaf); }

	void visit_func (teq::iFunctor& func) override
	{
		auto dependencies = func.get_args();
		teq::multi_visit(*this, dependencies);
		funcs_.push_back(static_cast<Observable*>(&func));
	}
};

}

namespace
{

// a context without an evaluator of its own gets this one (teq::get_eval)
[[maybe_unused]] const bool default_registered = []
{
	teq::set_default_eval_factory([]() -> teq::iEvaluator* { return new ReplayEvaluator(); });
	return true;
}();

}

struct ReplayEvaluator::Plan final
{
	std::vector<Observable*> funcs;
	std::vector<iEigen*> devs;
	std::vector<iEigen::LifeState> after;
	std::vector<iEigen*> effects; // launches with host-side effects (ASSIGN*)
	bool plain_assigns = false;   // the pass holds a plain ASSIGN, which the walk may skip
	std::vector<iEigen*> targets;
	std::vector<teq::iLeaf*> leaves;
	std::vector<const void*> leaf_ptrs;
	std::vector<size_t> leaf_versions;
	std::vector<size_t> leaf_fed; // bytes the launch carries for the leaf (0: read from device memory)
	tcg_graph* graph = nullptr;
	uint64_t bytes = 0;
	bool fresh = true;
};

ReplayEvaluator::ReplayEvaluator (size_t warm_passes, size_t max_plans, bool fuse, bool small_passes) :
	warm_passes_(warm_passes), max_plans_(std::max<size_t>(1, max_plans)), fuse_(fuse),
	small_passes_(fuse && small_passes), epoch_(global::structure_epoch()) {}

ReplayEvaluator::~ReplayEvaluator (void)
{
	clear();
}

void ReplayEvaluator::release (Plan& plan)
{
	if (nullptr != plan.graph && false == global::process_exiting())
	{
		tcg_graph_destroy(hip_context(), plan.graph);
	}
	plan.graph = nullptr;
}

void ReplayEvaluator::clear (void)
{
	for (auto& kv : slots_)
	{
		if (kv.second.plan) { release(*kv.second.plan); }
	}
	slots_.clear();
	stats_.reserved_bytes = 0;
}

void ReplayEvaluator::plain (teq::iDevice& device, const teq::TensSetT& targets, const teq::TensSetT& ignored)
{
	++stats_.plain;
	plain_.evaluate(device, targets, ignored);
}

void ReplayEvaluator::evict (void)
{
	size_t live = 0;
	for (auto& kv : slots_) { live += (nullptr != kv.second.plan); }
	while (live > max_plans_)
	{
		Slot* oldest = nullptr;
		for (auto& kv : slots_)
		{
			if (kv.second.plan && (nullptr == oldest || kv.second.last_used < oldest->last_used))
			{
				oldest = &kv.second;
			}
		}
		stats_.reserved_bytes -= oldest->plan->bytes;
		release(*oldest->plan);
		oldest->plan = nullptr;
		oldest->seen = 0;
		--live;
	}
}

/// Would the walk skip a plain ASSIGN among `funcs` (children first) at this
/// pass?  It runs a node whose operands are newer than the node
/// (tenncor/eteq/functor.hpp:246-268); an ASSIGN leaves its target at least one
/// version past its source (eteq/variable.hpp:129-132), so with two writers of
/// one variable, or a target that was fed after the source last moved, an
/// ASSIGN can find nothing newer than itself and keep out of a pass in which
/// another writer of its target runs.  A recording runs every node, so such a
/// pass must be walked.  Versions are carried forward as the walk would.
static bool walk_skips_an_assign (const std::vector<Observable*>& funcs, size_t max_version)
{
	std::unordered_map<const teq::iTensor*,size_t> moved;
	auto version_of = [&](const teq::iTensor* tens)
	{
		auto it = moved.find(tens);
		return it == moved.end() ? tens->get_meta().state_version() : it->second;
	};
	for (Observable* f : funcs)
	{
		auto op = (egen::_GENERATED_OPCODE) f->get_opcode().code_;
		auto args = f->get_args();
		size_t wanted = 0;
		for (auto& arg : args) { wanted = std::max(wanted, version_of(arg.get())); }
		const size_t held = f->get_meta().state_version();
		if (wanted <= held && false == egen::is_idempotent(op)) { wanted = held + 1; }
		wanted = std::min(wanted, max_version);
		const bool runs = held < wanted;
		if (runs) { moved[f] = wanted; }
		if (op < egen::ASSIGN || op > egen::ASSIGN_DIV) { continue; }
		if (false == runs)
		{
			if (op == egen::ASSIGN) { return true; }
			continue;
		}
		// the target: through the nodes that stand for their operand's buffer
		const teq::iTensor* target = args.front().get();
		while (auto inner = dynamic_cast<const teq::iFunctor*>(target))
		{
			auto code = (egen::_GENERATED_OPCODE) inner->get_opcode().code_;
			bool alias = (code >= egen::ASSIGN && code <= egen::ASSIGN_DIV) || code == egen::IDENTITY ||
				code == egen::RESHAPE || code == egen::SLICE;
			if (false == alias) { break; }
			target = inner->get_args().front().get();
		}
		moved[target] = std::max(version_of(target), version_of(args.back().get()) + 1);
	}
	return false;
}

void ReplayEvaluator::evaluate (teq::iDevice& device, const teq::TensSetT& targets, const teq::TensSetT& ignored)
{
	auto gpu = dynamic_cast<Device*>(&device);
	// a caller's own runtime memory is asked for every buffer of every pass
	// (internal/eigen/memory.hpp:14-22); the buffers of a recording stay with the
	// recording, so such a device is walked
	if (nullptr == gpu || false == ignored.empty() || targets.empty() ||
		nullptr == std::dynamic_pointer_cast<RuntimeMemory>(gpu->memory()))
	{
		plain(device, targets, ignored);
		return;
	}
	if (epoch_ != global::structure_epoch())
	{
		// some node went away or was rewired: remembered pointers may dangle
		clear();
		epoch_ = global::structure_epoch();
	}
	KeyT key;
	key.reserve(targets.size());
	for (teq::iTensor* t : targets)
	{
		if (nullptr != t) { key.push_back(t); }
	}
	std::sort(key.begin(), key.end());
	Slot& slot = slots_[key];
	slot.last_used = ++clock_;
	if (slot.unplannable)
	{
		plain(device, targets, ignored);
		return;
	}
	bool checked = false;
	if (nullptr == slot.plan)
	{
		if (slot.seen++ < warm_passes_)
		{
			plain(device, targets, ignored);
			return;
		}
		slot.plan = record(*gpu, key, targets);
		checked = true; // record() looks before it moves any version
		if (nullptr == slot.plan)
		{
			slot.unplannable = true;
			plain(device, targets, ignored);
			return;
		}
		stats_.reserved_bytes += slot.plan->bytes;
		evict();
	}
	bool walk = false == checked && slot.plan->plain_assigns && walk_skips_an_assign(slot.plan->funcs, gpu->max_version_);
	if (walk || false == replay(*gpu, *slot.plan))
	{
		stats_.reserved_bytes -= slot.plan->bytes;
		release(*slot.plan);
		slot.plan = nullptr;
		slot.unplannable = true;
		plain(device, targets, ignored);
	}
}

std::unique_ptr<ReplayEvaluator::Plan> ReplayEvaluator::record (Device& device, const KeyT& key, const teq::TensSetT& targets)
{
	const auto begun = std::chrono::steady_clock::now();
	uint64_t compiled0 = 0, disk0 = 0;
	double jit0 = 0.0;
	tcg_jit_stats(hip_context(), &compiled0, &disk0, &jit0);
	Collector collector;
	teq::multi_visit(collector, birth_order(key));
	if (collector.funcs_.empty()) { return nullptr; }
	auto plan = std::make_unique<Plan>();
	plan->funcs = collector.funcs_;
	plan->leaves = collector.leaves_;
	if (walk_skips_an_assign(plan->funcs, device.max_version_)) { return nullptr; }
	for (Observable* f : plan->funcs)
	{
		// device() builds the launch closure of a functor that has none yet
		auto dev = &static_cast<iEigen&>(f->device());
		if (false == dev->replayable()) { return nullptr; }
		plan->devs.push_back(dev);
		// nodes that run at every pass of the walk: the non-idempotent ones, and
		// plain ASSIGN too, which leaves its target newer than itself
		// (tenncor/eteq/functor.hpp:246-268 compares the operands' versions with
		// the node's; internal/eigen/device.hpp:508-544 bumps the target's)
		auto op = (egen::_GENERATED_OPCODE) f->get_opcode().code_;
		if (false == egen::is_idempotent(op) || op == egen::ASSIGN)
		{
			plan->effects.push_back(dev);
		}
		plan->plain_assigns = plan->plain_assigns || op == egen::ASSIGN;
		if (targets.count(f)) { plan->targets.push_back(dev); }
	}
	// leaves reach the device before recording starts: uploads are not recorded
	for (teq::iLeaf* leaf : plan->leaves)
	{
		plan->leaf_ptrs.push_back(eigen_ref(*leaf).device_data());
		plan->leaf_versions.push_back(leaf->get_meta().state_version());
	}
	// which launches the pass needs: elementwise nodes share launches and read
	// through the views in front of them
	FusionPlan fusion;
	if (fuse_) { fusion = plan_fusion(plan->funcs, targets); }
	else
	{
		for (Observable* f : plan->funcs)
		{
			FusionPlan::Step step;
			step.node = f;
			fusion.steps.push_back(step);
		}
	}
	// every value under the targets is recomputed into memory of the recording
	tcg_ctx* ctx = hip_context();
	std::string failure;
	auto attempt = [&](bool as_one_kernel)
	{
		for (iEigen* dev : plan->devs) { dev->drop(); }
		for (Observable* f : plan->funcs) { f->prop_version(device.max_version_); }
		hip_check(as_one_kernel ? tcg_capture_begin_small(ctx) : tcg_capture_begin(ctx));
		bool ok = true;
		RangeTempsT temps = pass_temps(fusion);
		try
		{
			if (as_one_kernel)
			{
				for (auto& step : fusion.steps) { launch_step(fusion, step, device, targets, temps); }
			}
			else
			{
				launch_pass(fusion, device, targets, temps, small_passes_, small_passes_);
			}
		}
		catch (const std::exception& err)
		{
			// kept: the node-by-node pass that follows may not hit it again
			failure = err.what();
			ok = false;
		}
		catch (...)
		{
			failure = "a failure that is not a std::exception";
			ok = false;
		}
		for (auto& temp : temps)
		{
			// a pass that failed half way: what its products borrowed goes back
			if (nullptr != temp.first) { device.memory()->deallocate(temp.first, temp.second); }
		}
		plan->leaf_fed.assign(plan->leaves.size(), 0);
		if (ok && as_one_kernel)
		{
			// small leaves that no node of the pass updates in place travel with
			// the launch: a new value costs no copy launch of its own
			teq::TensSetT updated;
			for (Observable* f : plan->funcs)
			{
				auto op = (egen::_GENERATED_OPCODE) f->get_opcode().code_;
				if (op >= egen::ASSIGN && op <= egen::ASSIGN_DIV) { updated.emplace(f->get_args().front().get()); }
			}
			size_t total = 0;
			for (size_t i = 0, n = plan->leaves.size(); i < n && ok; ++i)
			{
				teq::iLeaf* leaf = plan->leaves[i];
				size_t bytes = leaf->shape().n_elems() * leaf->get_meta().type_size();
				if (teq::IMMUTABLE == leaf->get_usage() || updated.count(leaf) || bytes > 256 || total + bytes > 960) { continue; }
				const void* host = static_cast<const teq::iTensor*>(leaf)->device().data();
				ok = TCG_OK == tcg_capture_feed(ctx, plan->leaf_ptrs[i], bytes, host);
				if (false == ok) { failure = tcg_last_error(ctx); }
				plan->leaf_fed[i] = bytes;
				total += (bytes + 15) & ~(size_t) 15;
			}
		}
		if (ok)
		{
			ok = TCG_OK == tcg_capture_end(ctx, &plan->graph);
			if (false == ok) { failure = tcg_last_error(ctx); }
		}
		else
		{
			tcg_capture_abort(ctx);
		}
		return ok;
	};
	// a graph of small tensors costs what its launches cost: its pass is
	// recorded as the steps of one kernel when every launch can be a step
	bool small = fuse_ && small_passes_ && plan->funcs.size() <= 256 &&
		std::all_of(plan->funcs.begin(), plan->funcs.end(), [](Observable* f) { return f->shape().n_elems() <= 4096; });
	bool ok = small && attempt(true);
	if (false == ok) { ok = attempt(false); }
	if (false == ok)
	{
		for (iEigen* dev : plan->devs) { dev->drop(); }
		++stats_.record_failures;
		stats_.record_error = failure;
		global::warnf("pass over %d functors not recorded, walked node by node instead: %s",
			(int) plan->funcs.size(), failure.c_str());
		return nullptr;
	}
	plan->after.reserve(plan->devs.size());
	for (iEigen* dev : plan->devs) { plan->after.push_back(dev->save_life()); }
	uint64_t launches = 0;
	tcg_graph_stats(plan->graph, &launches, &plan->bytes);
	++stats_.recorded;
	stats_.launches = launches;
	uint64_t compiled1 = 0, disk1 = 0;
	double jit1 = 0.0;
	tcg_jit_stats(ctx, &compiled1, &disk1, &jit1);
	stats_.record_ms = std::chrono::duration<double,std::milli>(std::chrono::steady_clock::now() - begun).count();
	stats_.jit_ms = jit1 - jit0;
	stats_.jit_compiled = (size_t) (compiled1 - compiled0);
	stats_.jit_from_disk = (size_t) (disk1 - disk0);
	return plan;
}

bool ReplayEvaluator::replay (Device& device, Plan& plan)
{
	bool stale = plan.fresh || false == plan.effects.empty();
	for (size_t i = 0, n = plan.leaves.size(); i < n; ++i)
	{
		size_t version = plan.leaves[i]->get_meta().state_version();
		bool moved = version != plan.leaf_versions[i];
		if (plan.leaf_fed[i] > 0)
		{
			// the launch carries the value: the device copy stays as it is
			if (eigen_ref(*plan.leaves[i]).device_address() != plan.leaf_ptrs[i]) { return false; }
			if (moved)
			{
				const void* host = static_cast<const teq::iTensor*>(plan.leaves[i])->device().data();
				hip_check(tcg_graph_feed(hip_context(), plan.graph, plan.leaf_ptrs[i], host, plan.leaf_fed[i]));
			}
		}
		// uploads a leaf whose host copy moved on
		else if (eigen_ref(*plan.leaves[i]).device_data() != plan.leaf_ptrs[i]) { return false; }
		if (moved)
		{
			plan.leaf_versions[i] = version;
			stale = true;
		}
	}
	for (size_t i = 0, n = plan.targets.size(); i < n && false == stale; ++i)
	{
		stale = nullptr == plan.targets[i]->device_data();
	}
	if (false == stale)
	{
		++stats_.skipped;
		return true;
	}
	for (Observable* f : plan.funcs) { f->prop_version(device.max_version_); }
	hip_check(tcg_graph_launch(hip_context(), plan.graph));
	for (size_t i = 0, n = plan.devs.size(); i < n; ++i)
	{
		plan.devs[i]->restore_life(plan.after[i], device.memory(), plan.graph);
	}
	for (iEigen* dev : plan.effects) { dev->replayed(); }
	plan.fresh = false;
	++stats_.replayed;
	return true;
}

}
