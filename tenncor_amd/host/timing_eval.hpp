// An evaluator that says where the time of a pass goes: it runs the launches the
// replaying evaluator would record -- elementwise groups, products over parts,
// products with epilogues, convolutions over views -- one after the other on
// the device's stream without recording them, with a HIP event in front of and
// behind every launch, and keeps the microseconds per kind of launch.
// Installed through teq::set_eval like the reference's debugging evaluator
// (dbg/peval/plugin_eval.hpp:21-42, which walks and then hands the visited
// nodes to its plugins); the values it leaves in the nodes are those of the
// launches it timed.
#ifndef TCH_TIMING_EVAL_HPP
#define TCH_TIMING_EVAL_HPP

#include <map>
#include <string>
#include <vector>

#include "eigen_device.hpp"

namespace eigen
{

struct TimingEvaluator final : public teq::iEvaluator
{
	struct Row final
	{
		std::string what;    ///< the launch as tcr_launch_plan names it
		size_t launches = 0; ///< over all passes
		double us = 0.0;     ///< device time between the two events, summed
	};

	void evaluate (teq::iDevice& device, const teq::TensSetT& targets,
		const teq::TensSetT& ignored = {}) override;

	/// Kinds of launches by time spent, the largest first
	std::vector<Row> rows (void) const;

	/// The same as text: a header with the passes and launches per pass, a line per kind
	std::string report (void) const;

	void clear (void)
	{
		table_.clear();
		passes_ = walked_ = launches_ = 0;
	}

private:
	teq::Evaluator plain_;
	std::map<std::string,Row> table_;
	size_t passes_ = 0, walked_ = 0, launches_ = 0;
};

}

#endif // TCH_TIMING_EVAL_HPP
