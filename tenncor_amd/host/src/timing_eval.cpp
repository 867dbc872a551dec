// Per-launch device times of a pass (see timing_eval.hpp).
#include "timing_eval.hpp"

#include <algorithm>
#include <sstream>

#include "fuse_plan.hpp"

namespace eigen
{

namespace
{

struct Collector final : public teq::iOnceTraveler
{
	std::vector<Observable*> funcs_;

private:
	void visit_leaf (teq::iLeaf&) override {}

	void visit_func (teq::iFunctor& func) override
	{
		auto dependencies = func.get_args();
		teq::multi_visit(*this, dependencies);
		funcs_.push_back(static_cast<Observable*>(&func));
	}
};

}

void TimingEvaluator::evaluate (teq::iDevice& device, const teq::TensSetT& targets, const teq::TensSetT& ignored)
{
	auto gpu = dynamic_cast<Device*>(&device);
	if (nullptr == gpu || false == ignored.empty() || targets.empty())
	{
		++walked_;
		plain_.evaluate(device, targets, ignored);
		return;
	}
	std::vector<teq::iTensor*> key(targets.begin(), targets.end());
	key.erase(std::remove(key.begin(), key.end(), nullptr), key.end());
	std::sort(key.begin(), key.end());
	Collector collector;
	teq::multi_visit(collector, birth_order(key));
	bool launchable = false == collector.funcs_.empty();
	for (Observable* f : collector.funcs_)
	{
		// host operators and custom devices are walked, as under the replaying evaluator
		launchable = launchable && static_cast<iEigen&>(f->device()).replayable();
	}
	if (false == launchable)
	{
		++walked_;
		plain_.evaluate(device, targets, ignored);
		return;
	}
	// leaves reach the device first, so that no upload falls between two events
	struct Leaves final : public teq::iOnceTraveler
	{
		void visit_leaf (teq::iLeaf& leaf) override { eigen_ref(leaf).device_data(); }
		void visit_func (teq::iFunctor& func) override
		{
			auto dependencies = func.get_args();
			teq::multi_visit(*this, dependencies);
		}
	} leaves;
	teq::multi_visit(leaves, key);
	FusionPlan plan = plan_fusion(collector.funcs_, targets);
	for (Observable* f : collector.funcs_)
	{
		static_cast<iEigen&>(f->device()).drop();
		f->prop_version(gpu->max_version_);
	}
	tcg_ctx* ctx = hip_context();
	std::vector<LaunchUnit> units = launch_units(plan);
	std::vector<void*> events(units.size() + 1, nullptr);
	for (void*& ev : events) { hip_check(tcg_event_create(ctx, &ev)); }
	RangeTempsT temps = pass_temps(plan);
	auto give_back = [&]
	{
		for (auto& temp : temps)
		{
			if (nullptr != temp.first) { gpu->memory()->deallocate(temp.first, temp.second); }
		}
		for (void* ev : events) { tcg_event_destroy(ctx, ev); }
	};
	try
	{
		// the stream is held while the pass is enqueued (kernels compiled at run time
		// included) and runs it back to back at the release: the events see the
		// device's pace, the gap in front of a launch counted with it
		hip_check(tcg_hold(ctx));
		try
		{
			hip_check(tcg_event_record(ctx, events[0]));
			for (size_t i = 0; i < units.size(); ++i)
			{
				launch_unit(plan, units[i], *gpu, targets, temps);
				hip_check(tcg_event_record(ctx, events[i + 1]));
			}
		}
		catch (...)
		{
			tcg_release(ctx);
			throw;
		}
		hip_check(tcg_release(ctx));
		for (size_t i = 0; i < units.size(); ++i)
		{
			float ms = 0.0f;
			hip_check(tcg_event_elapsed(ctx, events[i], events[i + 1], &ms));
			Row& row = table_[describe_unit(plan, units[i])];
			++row.launches;
			row.us += 1e3 * (double) ms;
		}
	}
	catch (...)
	{
		give_back();
		throw;
	}
	give_back();
	++passes_;
	launches_ = units.size();
}

std::vector<TimingEvaluator::Row> TimingEvaluator::rows (void) const
{
	std::vector<Row> out;
	for (auto& kv : table_)
	{
		Row row = kv.second;
		row.what = kv.first;
		out.push_back(row);
	}
	std::sort(out.begin(), out.end(), [](const Row& a, const Row& b) { return a.us > b.us; });
	return out;
}

std::string TimingEvaluator::report (void) const
{
	std::ostringstream ss;
	double total = 0.0;
	for (auto& kv : table_) { total += kv.second.us; }
	ss << passes_ << " passes timed launch by launch (" << launches_ << " launches in the latest), " << walked_
		<< " walked node by node; " << total << " us between events in all\n";
	char line[64];
	for (const Row& row : rows())
	{
		snprintf(line, sizeof(line), "%8zu x %9.2f us = %11.1f us  ", row.launches, row.us / (double) row.launches, row.us);
		ss << line << row.what << "\n";
	}
	return ss.str();
}

}
