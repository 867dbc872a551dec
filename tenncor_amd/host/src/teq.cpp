// Evaluator slot and reverse-mode derivation (internal/teq/src/evaluator.cpp,
// internal/teq/src/derive.cpp).
#include "teq.hpp"

#include <cstdlib>
#include <list>

namespace global
{

LogSinkF& log_sink (void)
{
	static LogSinkF sink;
	return sink;
}

size_t& last_version (void)
{
	static size_t version = 0;
	return version;
}

size_t& structure_epoch (void)
{
	static size_t epoch = 0;
	return epoch;
}

bool& process_exiting (void)
{
	static bool exiting = false;
	return exiting;
}

CfgMapptrT context (void)
{
	static CfgMapptrT ctx = std::make_shared<ConfigMap>();
	// registered after the map exists, so it runs before the map (and the
	// services it owns) is destroyed
	static bool registered = (std::atexit([] { process_exiting() = true; }), true);
	(void) registered;
	return ctx;
}

RandEngineT& get_generator (void)
{
	static RandEngineT engine;
	return engine;
}

void seed (size_t s)
{
	get_generator().seed(s);
}

bool& device_random (void)
{
	static bool on_device = false;
	return on_device;
}

}

namespace teq
{

TravEvaluator::TravEvaluator (iDevice& device, const TensSetT& targets, const TensSetT& ignored) :
	ignored_(ignored), device_(&device), targets_(targets)
{
	for (auto ig : ignored)
	{
		if (nullptr != ig && nullptr == ig->device().data())
		{
			global::throw_errf("cannot ignore tensor %s without existing data", ig->to_string().c_str());
		}
	}
}

// internal/teq/src/evaluator.cpp:9-30
const std::string eval_key = "evaluater";

void set_eval (iEvaluator* eval, global::CfgMapptrT ctx)
{
	if (nullptr == ctx) { global::fatal("cannot register an evaluator in a null context"); }
	ctx->rm_entry(eval_key);
	if (nullptr != eval)
	{
		ctx->add_entry<iEvaluator>(eval_key, [eval] { return eval; });
	}
}

static EvalFactoryT& default_eval_factory (void)
{
	static EvalFactoryT factory = nullptr;
	return factory;
}

void set_default_eval_factory (EvalFactoryT factory)
{
	default_eval_factory() = factory;
}

iEvaluator& get_eval (const global::CfgMapptrT& ctx)
{
	if (nullptr == ctx) { global::fatal("cannot look an evaluator up in a null context"); }
	auto eval = static_cast<iEvaluator*>(ctx->get_obj(eval_key));
	if (nullptr == eval)
	{
		const char* plain = getenv("TCR_EVAL_PLAIN");
		EvalFactoryT factory = default_eval_factory();
		eval = (nullptr != factory && false == (plain && plain[0] == '1')) ? factory() : new Evaluator();
		set_eval(eval, ctx);
	}
	return *eval;
}

namespace
{

// Which children of each functor lead to a target; a target functor is not
// descended into (internal/teq/traveler.hpp:199-290)
struct PathFinder final : public iOnceTraveler
{
	PathFinder (const TensSetT& targets) : targets_(targets) {}

	TensMapT<std::vector<size_t>> roadmap_;

private:
	void visit_leaf (iLeaf&) override {}

	void visit_func (iFunctor& func) override
	{
		if (targets_.count(&func)) { return; }
		auto args = func.get_args();
		multi_visit(*this, args);
		std::vector<size_t> nexts;
		for (size_t i = 0, n = args.size(); i < n; ++i)
		{
			iTensor* tens = args[i].get();
			if (targets_.count(tens) || roadmap_.count(tens)) { nexts.push_back(i); }
		}
		if (false == nexts.empty()) { roadmap_.emplace(&func, nexts); }
	}

	TensSetT targets_;
};

// Longest distance to a leaf, and first-visit order, of every node
struct GraphStat final : public iOnceTraveler
{
	TensMapT<size_t> height_;
	TensMapT<size_t> index_;

private:
	void visit_leaf (iLeaf& leaf) override
	{
		height_[&leaf] = 0;
		index_.emplace(&leaf, index_.size());
	}

	void visit_func (iFunctor& func) override
	{
		index_.emplace(&func, index_.size());
		auto args = func.get_args();
		multi_visit(*this, args);
		size_t h = 0;
		for (auto& arg : args) { h = std::max(h, height_[arg.get()]); }
		height_[&func] = h + 1;
	}
};

// shared_ptr of every functor reachable from the roots
struct OwnerTracker final : public iOnceTraveler
{
	TensMapT<TensptrT> owners_;

private:
	void visit_leaf (iLeaf&) override {}

	void visit_func (iFunctor& func) override
	{
		for (auto& arg : func.get_args())
		{
			owners_.emplace(arg.get(), arg);
			arg->accept(*this);
		}
	}
};

}

TensptrsT derive (TensptrT root, const TensptrsT& targets, const iDerivativeFuncs& funcs)
{
	TensptrsT out;
	out.reserve(targets.size());
	if (root == nullptr)
	{
		for (auto& target : targets) { out.push_back(funcs.get_const_zero(*target)); }
		return out;
	}

	TensMapT<TensptrsT> grads = {{root.get(), {funcs.get_const_one(*root)}}};
	TensSetT targset;
	for (auto& target : targets)
	{
		if (nullptr != target && target != root) { targset.emplace(target.get()); }
	}
	PathFinder pfinder(targset);
	root->accept(pfinder);
	if (false == pfinder.roadmap_.empty())
	{
		GraphStat stat;
		root->accept(stat);
		OwnerTracker owners;
		owners.owners_.emplace(root.get(), root);
		root->accept(owners);

		// parents before children: descending height; ties by label, then by
		// visit order, so that the traversal is deterministic
		std::list<iFunctor*> tovisits;
		for (auto& road : pfinder.roadmap_) { tovisits.push_back(static_cast<iFunctor*>(road.first)); }
		tovisits.sort([&](iFunctor* a, iFunctor* b)
		{
			size_t aheight = stat.height_[a], bheight = stat.height_[b];
			if (aheight == bheight)
			{
				std::string astr = a->to_string(), bstr = b->to_string();
				if (astr == bstr) { return stat.index_[a] > stat.index_[b]; }
				return astr > bstr;
			}
			return aheight > bheight;
		});

		for (iFunctor* tens : tovisits)
		{
			auto it = grads.find(tens);
			if (it == grads.end() || it->second.empty())
			{
				global::fatalf("failed to find existing grads for %s", tens->to_string().c_str());
			}
			TensptrsT prevs = it->second;
			TensptrT bwd = prevs.size() > 1 ? funcs.add(prevs) : prevs.front();
			auto visitable = std::static_pointer_cast<iFunctor>(owners.owners_[tens]);
			TensptrsT children = tens->get_args();
			for (size_t i : pfinder.roadmap_[tens])
			{
				grads[children[i].get()].push_back(funcs.lderive(visitable, bwd, i));
			}
		}
	}

	for (auto& target : targets)
	{
		TensptrT tens;
		if (nullptr == target) { tens = funcs.get_const_zero(*root); }
		else
		{
			auto it = grads.find(target.get());
			if (it != grads.end() && it->second.size() > 0)
			{
				tens = it->second.size() == 1 ? it->second.front() : funcs.add(it->second);
			}
			else { tens = funcs.get_const_zero(*target); }
		}
		out.push_back(tens);
	}
	return out;
}

}
