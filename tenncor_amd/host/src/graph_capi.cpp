// Flat C binding of the host graph layer (include/tcgraph.h).
#include "tcgraph.h"

#include <algorithm>
#include <cstring>
#include <sstream>

#include "eteq.hpp"
#include "replay_eval.hpp"
#include "timing_eval.hpp"
#include "fuse_plan.hpp"
#include "hone.hpp"

struct tcr_graph
{
	std::vector<teq::TensptrT> nodes;
	std::unordered_map<teq::iTensor*,int> ids;

	int add (teq::TensptrT tens)
	{
		auto it = ids.find(tens.get());
		if (it != ids.end()) { return it->second; }
		int id = (int) nodes.size();
		nodes.push_back(tens);
		ids.emplace(tens.get(), id);
		return id;
	}

	teq::TensptrT at (int id) const
	{
		if (id < 0 || (size_t) id >= nodes.size()) { global::fatalf("unknown node %d", id); }
		return nodes[id];
	}
};

static thread_local std::string g_error;

template <typename F>
static int guarded (F fn)
{
	try
	{
		fn();
		return 0;
	}
	catch (const std::exception& e)
	{
		g_error = e.what();
		return 1;
	}
}

static teq::Shape to_shape (const uint64_t shape[8])
{
	teq::DimsT dims;
	for (int i = 0; i < 8; ++i)
	{
		if (shape[i] > 65535) { global::fatalf("dimension %d of extent %llu exceeds 65535", i, (unsigned long long) shape[i]); }
		dims.push_back((teq::DimT) shape[i]);
	}
	return teq::Shape(dims);
}

// One node per line, children indented under their parent with "`--" branches
// and "|" rails for parents that still have children to come
static void print_tree (std::ostringstream& out, const teq::TensptrT& node,
	const std::string& prefix, bool root, bool last)
{
	if (!root) { out << "\n" << prefix << "`--"; }
	out << "(";
	auto f = dynamic_cast<teq::iFunctor*>(node.get());
	auto leaf = dynamic_cast<teq::iLeaf*>(node.get());
	if (leaf && leaf->get_usage() == teq::IMMUTABLE) { out << "constant:"; }
	else if (leaf) { out << "variable:"; }
	out << node->to_string() << "<" << node->get_meta().type_label() << ">" << node->shape().to_string() << ")";
	if (f)
	{
		std::string child_prefix = root ? "_" : prefix + (last ? "____" : "|___");
		auto args = f->get_args();
		for (size_t i = 0; i < args.size(); ++i)
		{
			print_tree(out, args[i], child_prefix, false, i + 1 == args.size());
		}
	}
}

// The flat API numbers element types like the device library (enum tcg_dtype)
// in every type configuration; the C++ layer numbers them like the
// reference's generated enum, which differs between configurations
static egen::_GENERATED_DTYPE host_dtype (int64_t wire)
{
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) if (wire == DEVICE) { return egen::ENUM; }
	EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
	global::fatalf("element type %d is not part of this build's type configuration", (int) wire);
}

extern "C" {

const char* tcr_last_error (void) { return g_error.c_str(); }

int tcr_graph_create (tcr_graph** out)
{
	return guarded([&] { *out = new tcr_graph(); });
}

int tcr_graph_destroy (tcr_graph* g)
{
	return guarded([&] { delete g; });
}

int tcr_variable (tcr_graph* g, int dtype, const uint64_t shape[8], const void* data, const char* label, int* node)
{
	return guarded([&]
	{
		teq::Shape s = to_shape(shape);
		std::string lbl = label ? label : "";
		teq::TensptrT out;
#define TCH_VAR(T) out = eteq::make_variable<T>((const T*) data, s, lbl);
		TYPE_LOOKUP(TCH_VAR, host_dtype(dtype))
#undef TCH_VAR
		*node = g->add(out);
	});
}

int tcr_constant (tcr_graph* g, int dtype, const uint64_t shape[8], const void* data, int* node)
{
	return guarded([&]
	{
		teq::Shape s = to_shape(shape);
		teq::TensptrT out;
#define TCH_CST(T) out = eteq::make_constant_tensor<T>((const T*) data, s);
		TYPE_LOOKUP(TCH_CST, host_dtype(dtype))
#undef TCH_CST
		*node = g->add(out);
	});
}

int tcr_assign (tcr_graph* g, int variable, const void* data)
{
	return guarded([&]
	{
		teq::TensptrT tens = g->at(variable);
		auto dtype = (egen::_GENERATED_DTYPE) tens->get_meta().type_code();
#define TCH_ASSIGN(T) {\
		auto var = dynamic_cast<eteq::Variable<T>*>(tens.get());\
		if (nullptr == var) { global::fatalf("node %d is not a variable", variable); }\
		var->assign((const T*) data, tens->shape()); }
		TYPE_LOOKUP(TCH_ASSIGN, dtype)
#undef TCH_ASSIGN
	});
}

int tcr_prefetch (tcr_graph* g, int leaf)
{
	return guarded([&]
	{
		teq::TensptrT tens = g->at(leaf);
		if (nullptr == dynamic_cast<teq::iLeaf*>(tens.get())) { global::fatalf("node %d is not a leaf", leaf); }
		(void) eigen::eigen_ref(*tens).device_data();
	});
}

int tcr_functor (tcr_graph* g, int opcode, int nargs, const int* args, int nattrs,
	const char* const* keys, const int64_t* const* vals, const int* lens, int* node)
{
	return guarded([&]
	{
		teq::TensptrsT children;
		for (int i = 0; i < nargs; ++i) { children.push_back(g->at(args[i])); }
		marsh::Maps attrs;
		for (int i = 0; i < nattrs; ++i)
		{
			std::string key = keys[i];
			std::vector<int64_t> v(vals[i], vals[i] + lens[i]);
			if (key == "rank")
			{
				if (v.size() != 1) { global::fatal("`rank` takes one value"); }
				attrs.add_attr(key, std::make_unique<marsh::Number<int64_t>>(v[0]));
			}
			else if (key == "dtype")
			{
				if (v.size() != 1) { global::fatal("`dtype` takes one value"); }
				attrs.add_attr(key, std::make_unique<marsh::String>(egen::name_type(host_dtype(v[0]))));
			}
			else if (key == "tensor")
			{
				if (v.size() != 1) { global::fatal("`tensor` takes one node"); }
				attrs.add_attr(key, std::make_unique<teq::TensorObj>(g->at((int) v[0])));
			}
			else
			{
				attrs.add_attr(key, std::make_unique<marsh::NumArray<int64_t>>(v));
			}
		}
		auto op = (egen::_GENERATED_OPCODE) opcode;
		if (op <= egen::BAD_OP || op >= egen::_N_GENERATED_OPCODES) { global::fatal("unknown opcode"); }
		*node = g->add(eteq::make_funcattr(op, children, attrs));
	});
}

int tcr_derive (tcr_graph* g, int root, int ntargets, const int* targets, int* grads)
{
	return guarded([&]
	{
		teq::TensptrsT wrt;
		for (int i = 0; i < ntargets; ++i) { wrt.push_back(g->at(targets[i])); }
		auto ders = tcr::derive(g->at(root), wrt);
		for (int i = 0; i < ntargets; ++i) { grads[i] = g->add(ders[i]); }
	});
}

int tcr_local_derivative (tcr_graph* g, int op, int supgrad, int arg_idx, int* grad)
{
	return guarded([&]
	{
		auto func = std::dynamic_pointer_cast<teq::iFunctor>(g->at(op));
		if (nullptr == func) { global::fatal("local derivative of a leaf"); }
		if (arg_idx < 0 || (size_t) arg_idx >= func->get_args().size()) { global::fatalf("no argument %d", arg_idx); }
		eteq::DerivativeFuncs funcs;
		*grad = g->add(funcs.lderive(func, g->at(supgrad), (size_t) arg_idx));
	});
}

int tcr_evaluate (tcr_graph* g, int ntargets, const int* targets)
{
	return guarded([&]
	{
		teq::TensptrsT roots;
		for (int i = 0; i < ntargets; ++i) { roots.push_back(g->at(targets[i])); }
		eteq::run(roots);
	});
}

int tcr_evaluate_ignoring (tcr_graph* g, int ntargets, const int* targets, int nignored, const int* ignored)
{
	return guarded([&]
	{
		teq::TensptrsT roots, skip;
		for (int i = 0; i < ntargets; ++i) { roots.push_back(g->at(targets[i])); }
		for (int i = 0; i < nignored; ++i) { skip.push_back(g->at(ignored[i])); }
		eteq::run(roots, skip);
	});
}

int tcr_sync (tcr_graph*)
{
	return guarded([&] { eigen::hip_check(tcg_sync(eigen::hip_context())); });
}

int tcr_set_evaluator (int kind)
{
	return guarded([&]
	{
		switch (kind)
		{
			case TCR_EVAL_PLAIN: teq::set_eval(new teq::Evaluator()); break;
			case TCR_EVAL_REPLAY: teq::set_eval(new eigen::ReplayEvaluator()); break;
			case TCR_EVAL_REPLAY_UNFUSED: teq::set_eval(new eigen::ReplayEvaluator(1, 16, false)); break;
			case TCR_EVAL_REPLAY_LAUNCHES: teq::set_eval(new eigen::ReplayEvaluator(1, 16, true, false)); break;
			case TCR_EVAL_DEFAULT: teq::set_eval(nullptr); break;
			case TCR_EVAL_TIMING: teq::set_eval(new eigen::TimingEvaluator()); break;
			default: global::fatalf("unknown evaluator kind %d", kind);
		}
	});
}

int tcr_evaluator_stats (uint64_t out[6])
{
	return guarded([&]
	{
		std::fill(out, out + 6, 0);
		if (auto replay = dynamic_cast<eigen::ReplayEvaluator*>(&teq::get_eval()))
		{
			auto& st = replay->stats();
			out[0] = st.plain;
			out[1] = st.recorded;
			out[2] = st.replayed;
			out[3] = st.skipped;
			out[4] = st.launches;
			out[5] = st.reserved_bytes;
		}
	});
}

int tcr_evaluator_timing (char* out, size_t capacity, size_t* needed)
{
	return guarded([&]
	{
		std::string text;
		if (auto timing = dynamic_cast<eigen::TimingEvaluator*>(&teq::get_eval())) { text = timing->report(); }
		if (needed) { *needed = text.size(); }
		if (out && capacity)
		{
			size_t n = std::min(text.size(), capacity - 1);
			memcpy(out, text.data(), n);
			out[n] = '\0';
		}
	});
}

int tcr_evaluator_record_cost (double* record_ms, double* jit_ms, uint64_t* jit_compiled, uint64_t* jit_from_disk)
{
	return guarded([&]
	{
		eigen::ReplayEvaluator::Stats st;
		if (auto replay = dynamic_cast<eigen::ReplayEvaluator*>(&teq::get_eval())) { st = replay->stats(); }
		if (record_ms) { *record_ms = st.record_ms; }
		if (jit_ms) { *jit_ms = st.jit_ms; }
		if (jit_compiled) { *jit_compiled = st.jit_compiled; }
		if (jit_from_disk) { *jit_from_disk = st.jit_from_disk; }
	});
}

int tcr_evaluator_record_error (char* out, size_t capacity, uint64_t* failures)
{
	return guarded([&]
	{
		std::string text;
		uint64_t count = 0;
		if (auto replay = dynamic_cast<eigen::ReplayEvaluator*>(&teq::get_eval()))
		{
			text = replay->stats().record_error;
			count = replay->stats().record_failures;
		}
		if (failures) { *failures = count; }
		if (out && capacity)
		{
			size_t n = std::min(text.size(), capacity - 1);
			memcpy(out, text.data(), n);
			out[n] = '\0';
		}
	});
}

int tcr_shape (tcr_graph* g, int node, uint64_t shape[8])
{
	return guarded([&]
	{
		teq::Shape s = g->at(node)->shape();
		std::copy(s.begin(), s.end(), shape);
	});
}

int tcr_dtype (tcr_graph* g, int node, int* dtype)
{
	return guarded([&] { *dtype = egen::device_type((egen::_GENERATED_DTYPE) g->at(node)->get_meta().type_code()); });
}

int tcr_data (tcr_graph* g, int node, void* out, size_t bytes)
{
	return guarded([&]
	{
		teq::TensptrT tens = g->at(node);
		size_t need = tens->shape().n_elems() * tens->get_meta().type_size();
		if (bytes < need) { global::fatalf("buffer of %d bytes is too small for %d", (int) bytes, (int) need); }
		const void* src = tens->device().data();
		if (nullptr == src) { global::fatalf("node %s has no data", tens->to_string().c_str()); }
		memcpy(out, src, need);
	});
}

int tcr_version (tcr_graph* g, int node, uint64_t* version)
{
	return guarded([&] { *version = g->at(node)->get_meta().state_version(); });
}

int tcr_opcode (tcr_graph* g, int node, int* opcode)
{
	return guarded([&]
	{
		auto f = dynamic_cast<teq::iFunctor*>(g->at(node).get());
		*opcode = f ? (int) f->get_opcode().code_ : 0;
	});
}

int tcr_nargs (tcr_graph* g, int node, int* nargs)
{
	return guarded([&]
	{
		auto f = dynamic_cast<teq::iFunctor*>(g->at(node).get());
		*nargs = f ? (int) f->get_args().size() : 0;
	});
}

int tcr_args (tcr_graph* g, int node, int* args, int capacity)
{
	return guarded([&]
	{
		auto f = dynamic_cast<teq::iFunctor*>(g->at(node).get());
		if (nullptr == f) { return; }
		auto children = f->get_args();
		if ((int) children.size() > capacity) { global::fatal("argument buffer is too small"); }
		for (size_t i = 0; i < children.size(); ++i) { args[i] = g->add(children[i]); }
	});
}

int tcr_attr (tcr_graph* g, int node, const char* key, int64_t* vals, int capacity, int* len)
{
	return guarded([&]
	{
		*len = -1;
		auto f = dynamic_cast<teq::iFunctor*>(g->at(node).get());
		if (nullptr == f) { return; }
		const marsh::iObject* obj = f->get_attr(key);
		if (nullptr == obj) { return; }
		std::vector<int64_t> out;
		if (auto arr = dynamic_cast<const marsh::NumArray<int64_t>*>(obj)) { out = arr->contents_; }
		else if (auto num = dynamic_cast<const marsh::iNumber*>(obj)) { out.push_back(num->to_int64()); }
		else if (auto tens = dynamic_cast<const teq::TensorObj*>(obj)) { out.push_back(g->add(tens->get_tensor())); }
		else if (auto text = dynamic_cast<const marsh::String*>(obj))
		{
			// a type name: its code in the numbering of tcr_variable
			out.push_back((int64_t) egen::device_type(egen::get_type(text->to_string())));
		}
		else { global::fatalf("attribute `%s` holds neither numbers nor a tensor", key); }
		*len = (int) out.size();
		if (nullptr != vals)
		{
			if ((int) out.size() > capacity) { global::fatal("attribute buffer is too small"); }
			std::copy(out.begin(), out.end(), vals);
		}
	});
}

int tcr_to_string (tcr_graph* g, int node, char* out, size_t capacity)
{
	return guarded([&]
	{
		std::ostringstream ss;
		print_tree(ss, g->at(node), "", true, true);
		std::string s = ss.str();
		if (s.size() + 1 > capacity) { global::fatal("string buffer is too small"); }
		memcpy(out, s.c_str(), s.size() + 1);
	});
}

int tcr_count_functors (tcr_graph* g, int nnodes, const int* nodes, int* count)
{
	return guarded([&]
	{
		struct Counter final : public teq::iOnceTraveler
		{
			size_t nfuncs = 0;
			void visit_leaf (teq::iLeaf&) override {}
			void visit_func (teq::iFunctor& f) override
			{
				++nfuncs;
				auto args = f.get_args();
				teq::multi_visit(*this, args);
			}
		} counter;
		for (int i = 0; i < nnodes; ++i) { g->at(nodes[i])->accept(counter); }
		*count = (int) counter.nfuncs;
	});
}

int tcr_launch_plan (tcr_graph* g, int ntargets, const int* targets, char* out, size_t capacity, size_t* needed)
{
	return guarded([&]
	{
		struct Collector final : public teq::iOnceTraveler
		{
			std::vector<eigen::Observable*> funcs;
			void visit_leaf (teq::iLeaf&) override {}
			void visit_func (teq::iFunctor& f) override
			{
				auto args = f.get_args();
				teq::multi_visit(*this, args);
				funcs.push_back(static_cast<eigen::Observable*>(&f));
			}
		} collector;
		teq::TensSetT tset;
		std::vector<teq::iTensor*> key;
		for (int i = 0; i < ntargets; ++i) { key.push_back(g->at(targets[i]).get()); }
		tset.insert(key.begin(), key.end());
		std::sort(key.begin(), key.end());
		teq::multi_visit(collector, eigen::birth_order(key));
		eigen::FusionPlan plan = eigen::plan_fusion(collector.funcs, tset);
		std::stringstream ss;
		// "batch N": the N steps that follow are small and go out as one launch
		for (auto& unit : eigen::launch_units(plan))
		{
			if (unit.second - unit.first > 1) { ss << "batch " << unit.second - unit.first << "\n"; }
			for (size_t i = unit.first; i < unit.second; ++i) { ss << eigen::describe_step(plan, plan.steps[i]) << "\n"; }
		}
		// "padded N": leaves that the pass copies once with a longer leading dim for the
		// products that read them (FusionPlan::padded); only printed when there are any
		if (false == plan.padded.empty()) { ss << "padded " << plan.padded.size() << "\n"; }
		ss << "folded " << plan.absorbed.size() << "\n";
		std::string text = ss.str();
		if (needed) { *needed = text.size(); }
		if (out && capacity)
		{
			size_t n = std::min(text.size(), capacity - 1);
			memcpy(out, text.data(), n);
			out[n] = '\0';
		}
	});
}

int tcr_set_random (int where)
{
	return guarded([&]
	{
		if (TCR_RANDOM_HOST != where && TCR_RANDOM_DEVICE != where) { global::fatalf("unknown generator %d", where); }
		global::device_random() = TCR_RANDOM_DEVICE == where;
	});
}

int tcr_seed (uint64_t seed)
{
	return guarded([&]
	{
		global::seed(seed);
		eigen::hip_check(tcg_rand_seed(eigen::hip_context(), seed));
	});
}

int tcr_optimize (tcr_graph* g, int nroots, const int* roots, const char* rules_json, int fold,
	int* out_roots, uint64_t stats[4])
{
	return guarded([&]
	{
		hone::RulesT rules;
		if (nullptr != rules_json) { rules = hone::parse_rules(rules_json); }
		teq::TensptrsT in;
		for (int i = 0; i < nroots; ++i) { in.push_back(g->at(roots[i])); }
		hone::Stats st;
		teq::TensptrsT out = hone::optimize(in, rules, 0 != fold, &st);
		for (int i = 0; i < nroots; ++i) { out_roots[i] = g->add(out[i]); }
		if (nullptr != stats)
		{
			stats[0] = st.merged;
			stats[1] = st.folded;
			stats[2] = st.converted;
			stats[3] = st.rounds;
		}
	});
}

} // extern "C"
