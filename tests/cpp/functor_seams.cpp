// The node API a tenncor checkout binds to, exercised from C++ the way the
// reference's own unit tests exercise it (tenncor/eteq/test/test_functor.cpp:
// 22-104 Initiation, :107-192 UpdateChild, :195-261 Prop, :264-302 Cache;
// internal/teq/test/test_evaluator.cpp:20-30 SetGet).  The reference runs these
// on gmock doubles; here the operands are real variables and functors of the
// host layer.  Also: the context-keyed registries (internal/teq/src/
// evaluator.cpp:9-30, internal/eigen/src/memory.cpp:8-30) used the way
// tenncor/eteq/etens.hpp:152-162 uses them, and the attribute packers with
// the expectations of internal/eigen/test/test_packer.cpp:23-446 (keys,
// int64 encodings, error strings).  Nothing is launched: no GPU is needed.
// Prints one line per failed expectation and exits with their count.
#include <cstdio>
#include <limits>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

#include "eteq.hpp"
#include "replay_eval.hpp"

static int failures = 0;

#define EXPECT(COND) do { if (!(COND)) { ++failures; std::printf("%s:%d: expected %s\n", __FILE__, __LINE__, #COND); } } while (0)

template <typename F>
static void expect_fatal (F&& call, const std::string& message, int line)
{
	try
	{
		call();
	}
	catch (std::runtime_error& e)
	{
		if (std::string(e.what()).find(message) == std::string::npos)
		{
			++failures;
			std::printf("line %d: expected \"%s\", got \"%s\"\n", line, message.c_str(), e.what());
		}
		return;
	}
	++failures;
	std::printf("line %d: expected failure \"%s\"\n", line, message.c_str());
}

#define EXPECT_FATAL(CALL, MSG) expect_fatal([&] { CALL; }, MSG, __LINE__)

static void initiation (void)
{
	teq::Shape argshape({4, 3});
	std::vector<double> data{1, 2, 3, 4, 5, 6, 1, 2, 3, 4, 5, 6};
	std::vector<float> fdata(12, 1.0f);
	teq::TensptrT leaf = eteq::make_variable<double>(data.data(), argshape, "leaf");
	teq::TensptrT a = eteq::make_functor(egen::NEG, {leaf});
	teq::TensptrT b = eteq::make_functor(egen::ABS, {leaf});
	teq::TensptrT c = eteq::make_variable<float>(fdata.data(), argshape, "c");

	marsh::Maps attrs;
	EXPECT_FATAL(eteq::Functor<double>::get(egen::ADD, teq::TensptrsT{}, std::move(attrs)),
		"cannot perform `ADD` without arguments");
	EXPECT_FATAL(eteq::Functor<double>::get(egen::ADD, teq::TensptrsT{a, c}, std::move(attrs)),
		"children types are not all the same");

	eteq::Functor<double>* f = eteq::Functor<double>::get(egen::ADD, {a, b}, std::move(attrs));
	teq::TensptrT ftens(f);
	auto g = eteq::Functor<double>::get(egen::SIN, {ftens}, std::move(attrs));
	teq::TensptrT gtens(g);

	auto fshape = f->shape();
	EXPECT(std::equal(argshape.begin(), argshape.end(), fshape.begin()));
	EXPECT(egen::ADD == f->get_opcode().code_);
	EXPECT("ADD" == f->get_opcode().name_);
	EXPECT("ADD" == f->to_string());
	EXPECT(false == f->has_data());
	EXPECT_FATAL(static_cast<const eteq::Functor<double>*>(f)->device(), "cannot get device of uninitialized functor");

	// initialising the reader initialises everything under it
	g->must_initialize();
	EXPECT(g->has_data());
	EXPECT(f->has_data());
	// and dropping a node drops its readers
	f->uninitialize();
	EXPECT(false == f->has_data());
	EXPECT(false == g->has_data());
}

static void update_child (void)
{
	teq::Shape argshape({4, 3});
	std::vector<double> data{1, 2, 3, 4, 5, 6, 1, 2, 3, 4, 5, 6};
	std::vector<float> fdata(12, 1.0f);
	teq::TensptrT leaf = eteq::make_variable<double>(data.data(), argshape, "leaf");
	teq::TensptrT a = eteq::make_functor(egen::NEG, {leaf});
	teq::TensptrT b = eteq::make_functor(egen::ABS, {leaf});
	teq::TensptrT c = eteq::make_functor(egen::SIN, {leaf});
	teq::TensptrT leaf2 = eteq::make_variable<double>(data.data(), teq::Shape({3, 4}), "leaf2");
	teq::TensptrT d = eteq::make_functor(egen::COS, {leaf2});
	teq::TensptrT e = eteq::make_variable<float>(fdata.data(), argshape, "e");

	marsh::Maps attrs;
	auto f = eteq::Functor<double>::get(egen::ADD, {a, b}, std::move(attrs));
	teq::TensptrT ftens(f);
	EXPECT(false == f->has_data());
	auto children = f->get_args();
	EXPECT(2 == children.size() && a == children.front() && b == children.back());

	f->must_initialize();
	f->update_child(c, 1);
	EXPECT(false == f->has_data());
	children = f->get_args();
	EXPECT(2 == children.size() && a == children.front() && c == children.back());
	f->update_child(c, 0);
	children = f->get_args();
	EXPECT(c == children.front() && c == children.back());

	EXPECT_FATAL(f->update_child(d, 1), "cannot update child 1 to argument with incompatible shape "
		"[3\\4\\1\\1\\1\\1\\1\\1] (requires shape [4\\3\\1\\1\\1\\1\\1\\1])");
	EXPECT_FATAL(f->update_child(e, 0), "cannot update child 0 to argument with different type FLOAT (requires type DOUBLE)");
	EXPECT_FATAL(f->update_child(a, 2), "cannot replace argument 2 when only there are only 2 available");
}

static void prop (void)
{
	teq::Shape argshape({4, 3});
	std::vector<double> data{1, 2, 3, 4, 5, 6, 1, 2, 3, 4, 5, 6};
	auto leaf = eteq::make_variable<double>(data.data(), argshape, "leaf"); // leaves start at version 1
	teq::TensptrT a = leaf, b = leaf;

	marsh::Maps attrs;
	auto f = eteq::Functor<double>::get(egen::ADD, {a, b}, std::move(attrs));
	teq::TensptrT ftens(f);
	EXPECT(false == f->has_data());
	f->device();
	EXPECT(f->has_data());

	EXPECT(0 == f->get_meta().state_version());
	EXPECT(f->prop_version(3));
	EXPECT(1 == f->get_meta().state_version());
	EXPECT(false == f->prop_version(3));

	// an operator that is not idempotent moves on at every call, up to the cap
	auto g = eteq::Functor<double>::get(egen::RAND_UNIF, {a, b}, std::move(attrs));
	teq::TensptrT gtens(g);
	EXPECT(g->prop_version(3));
	EXPECT(1 == g->get_meta().state_version());
	EXPECT(g->prop_version(3));
	EXPECT(2 == g->get_meta().state_version());
	EXPECT(g->prop_version(3));
	EXPECT(3 == g->get_meta().state_version());
	EXPECT(false == g->prop_version(3));

	// a new value puts the leaf one past the newest version anywhere
	// (tenncor/eteq/variable.hpp:18-27,55-60), which is news for its readers
	leaf->assign(data.data(), argshape);
	size_t leaf_version = leaf->get_meta().state_version();
	EXPECT(4 == leaf_version);
	EXPECT(f->prop_version(99));
	EXPECT(leaf_version == f->get_meta().state_version());
	EXPECT(false == f->prop_version(99));
}

static void cache (void)
{
	teq::Shape argshape({4, 3});
	std::vector<double> data{1, 2, 3, 4, 5, 6, 1, 2, 3, 4, 5, 6};
	teq::TensptrT a = eteq::make_variable<double>(data.data(), argshape, "a");
	marsh::Maps attrs;
	auto f = eteq::Functor<double>::get(egen::SIN, {a}, std::move(attrs));
	teq::TensptrT ftens(f);
	EXPECT(false == f->has_data());
	f->cache_init();
	EXPECT(f->has_data());
	EXPECT(nullptr != dynamic_cast<eigen::CacheEigen*>(&f->device()));
}

namespace
{

struct CountingEvaluator final : public teq::iEvaluator
{
	void evaluate (teq::iDevice&, const teq::TensSetT&, const teq::TensSetT&) override { ++calls_; }
	size_t calls_ = 0;
};

}

static void evaluator_slot (void)
{
	// EVALUATOR.SetGet: the slot owns what it is given and hands it back
	auto counting = new CountingEvaluator();
	teq::set_eval(counting);
	EXPECT(counting == &teq::get_eval());
	eigen::Device device;
	teq::get_eval().evaluate(device, {}, {});
	EXPECT(1 == counting->calls_);
	teq::set_eval(new teq::Evaluator());
	EXPECT(nullptr != dynamic_cast<teq::Evaluator*>(&teq::get_eval()));
}

namespace
{

struct CountingMemory final : public eigen::iRuntimeMemory
{
	void* allocate (size_t size) override { ++allocations_; return ::operator new(size); }
	void deallocate (void* ptr, size_t) override { ::operator delete(ptr); }
	size_t allocations_ = 0;
};

}

static void context_registries (void)
{
	// a context of its own keeps its services apart from the process-wide one
	global::CfgMapptrT ctx = std::make_shared<global::ConfigMap>();
	auto counting = new CountingEvaluator();
	teq::set_eval(counting, ctx);
	EXPECT(counting == &teq::get_eval(ctx));
	EXPECT(counting != &teq::get_eval());
	EXPECT(counting != &teq::get_eval(global::context()));
	EXPECT(&teq::get_eval() == &teq::get_eval(global::context()));

	auto memory = std::make_shared<CountingMemory>();
	eigen::set_runtime(memory, ctx);
	EXPECT(memory == eigen::get_runtime(ctx));
	EXPECT(memory != eigen::get_runtime());
	EXPECT(nullptr != std::dynamic_pointer_cast<eigen::RuntimeMemory>(eigen::get_runtime()));

	// the body of ETensor::calc (tenncor/eteq/etens.hpp:152-162), written out
	teq::Shape shape({3, 2});
	std::vector<double> data{1, 2, 3, 4, 5, 6};
	teq::TensptrT leaf = eteq::make_variable<double>(data.data(), shape, "leaf");
	{
		eigen::Device device(eigen::get_runtime(ctx), std::numeric_limits<size_t>::max());
		teq::get_eval(ctx).evaluate(device, {leaf.get()}, {});
	}
	EXPECT(1 == counting->calls_);
	// ... and through the handle itself
	eteq::ETensor handle(leaf, ctx);
	EXPECT(handle != nullptr);
	EXPECT(ctx == handle.get_context());
	EXPECT(leaf.get() == handle.get());
	EXPECT(leaf == (teq::TensptrT) handle);
	double* got = handle.calc<double>();
	EXPECT(2 == counting->calls_);
	EXPECT(nullptr != got && std::equal(data.begin(), data.end(), got));
	EXPECT_FATAL(handle.data<float>(), "cannot read DOUBLE as FLOAT");
	eteq::run(eteq::ETensorsT{handle, handle});
	EXPECT(3 == counting->calls_);
	EXPECT(1 == eteq::to_tensors({handle}).size());
	// an empty handle and a handle whose context is gone evaluate to nothing
	eteq::ETensor empty;
	EXPECT(empty == nullptr);
	EXPECT(nullptr == empty.calc<double>());
	{
		global::CfgMapptrT brief = std::make_shared<global::ConfigMap>();
		eteq::ETensor orphan(leaf, brief);
		brief = nullptr;
		EXPECT(nullptr == orphan.get_context());
		EXPECT(nullptr == orphan.calc<double>());
	}

	// replacing and removing: the default comes back (src/evaluator.cpp:21-30,
	// src/memory.cpp:19-28)
	// (the default evaluator is the replaying one, which walks like teq::Evaluator
	// whatever it sees for the first time)
	teq::set_eval(nullptr, ctx);
	EXPECT(nullptr != dynamic_cast<eigen::ReplayEvaluator*>(&teq::get_eval(ctx)));
	eigen::set_runtime(nullptr, ctx);
	EXPECT(nullptr != std::dynamic_pointer_cast<eigen::RuntimeMemory>(eigen::get_runtime(ctx)));
	EXPECT(memory != eigen::get_runtime(ctx));

	// the map itself: lazy construction, typed deletion, unknown keys
	static int built = 0, destroyed = 0;
	struct Probe final { Probe (void) { ++built; } ~Probe (void) { ++destroyed; } };
	ctx->add_entry<Probe>("probe", [] { return new Probe(); });
	EXPECT(0 == built);
	void* first = ctx->get_obj("probe");
	EXPECT(nullptr != first && 1 == built && first == ctx->get_obj("probe") && 1 == built);
	EXPECT(nullptr == ctx->get_obj("nothing registered under this"));
	ctx->rm_entry("probe");
	EXPECT(1 == destroyed && nullptr == ctx->get_obj("probe"));
	ctx->add_entry<Probe>("probe", [] { return new Probe(); });
	ctx->get_obj("probe");
	ctx = nullptr; // the map deletes what it still holds
	EXPECT(2 == built && 2 == destroyed);
}

template <typename T, typename EQ>
static void packer_round_trip (const std::string& key, T value, EQ same, int line)
{
	eigen::Packer<T> packer;
	marsh::Maps attrs;
	T out;
	expect_fatal([&] { packer.unpack(out, attrs); }, "cannot find `" + key + "` attribute", line);
	packer.pack(attrs, value);
	if (key != packer.get_key() || nullptr == attrs.get_attr(key))
	{
		++failures;
		std::printf("line %d: expected an attribute under `%s`\n", line, key.c_str());
		return;
	}
	packer.unpack(out, attrs);
	if (false == same(value, out))
	{
		++failures;
		std::printf("line %d: `%s` does not come back as it went in\n", line, key.c_str());
	}
	marsh::Maps attrs2;
	eigen::pack_attr(attrs2, value);
	if (nullptr == attrs2.get_attr(key))
	{
		++failures;
		std::printf("line %d: pack_attr did not file `%s`\n", line, key.c_str());
	}
}

static void packers (void)
{
	auto equal = [](const auto& a, const auto& b) { return a == b; };
	// PACKER.PairEncodeDecode: pairs flatten to int64 (fractions dropped)
	eigen::PairVecT<double> pairs = {{1.2, 2.3}, {3.4, 4.6}, {5.5, 6.7}};
	std::vector<int64_t> flat = eigen::encode_pair(pairs);
	EXPECT((flat == std::vector<int64_t>{1, 2, 3, 4, 5, 6}));
	auto back = eigen::decode_pair<double>(flat);
	EXPECT(3 == back.size() && 1 == back[0].first && 2 == back[0].second && 5 == back[2].first && 6 == back[2].second);
	EXPECT_FATAL(eigen::decode_pair<size_t>(std::vector<int64_t>{1, 2, 3, 4, 5}),
		"cannot decode odd vector [1\\2\\3\\4\\5] into vec of pairs");
	EXPECT("[1:2\\3:4\\5:6]" == eigen::to_string(pairs));

	// PACKER.BadPacker: a type without an attribute
	eigen::Packer<std::string> badpack;
	EXPECT("" == badpack.get_key());
	marsh::Maps none;
	std::string text;
	EXPECT_FATAL(eigen::get_attr(badpack, none), "cannot find `` attribute");
	EXPECT_FATAL(badpack.pack(none, text), "unknown attribute");
	EXPECT_FATAL(badpack.unpack(text, none), "unknown attribute");

	// the keys and what each holds
	packer_round_trip<eigen::PairVecT<teq::DimT>>("dimension_pairs", {{2, 2}, {3, 4}}, equal, __LINE__);
	packer_round_trip<eigen::PairVecT<teq::RankT>>("rank_pairs", {{2, 2}, {3, 4}}, equal, __LINE__);
	packer_round_trip<teq::DimsT>("dimensions", {2, 2, 3, 4}, equal, __LINE__);
	packer_round_trip<teq::RanksT>("ranks", {2, 2, 3, 4}, equal, __LINE__);
	packer_round_trip<std::set<teq::RankT>>("rank_set", {2, 6, 3, 4}, equal, __LINE__);
	packer_round_trip<teq::RankT>("rank", 2, equal, __LINE__);
	packer_round_trip<teq::Shape>("shape", teq::Shape({2, 1, 4}),
		[](const teq::Shape& a, const teq::Shape& b) { return std::equal(a.begin(), a.end(), b.begin()); }, __LINE__);
	std::vector<double> six{1, 2, 3, 4, 5, 6};
	teq::TensptrT tens = eteq::make_variable<double>(six.data(), teq::Shape({3, 2}), "t");
	{
		// PACKER.PackerTensor: no "cannot find" step in the reference's case either
		eigen::Packer<teq::TensptrT> packer;
		marsh::Maps attrs;
		packer.pack(attrs, tens);
		EXPECT("tensor" == packer.get_key() && nullptr != attrs.get_attr("tensor"));
		teq::TensptrT out;
		packer.unpack(out, attrs);
		EXPECT(tens == out);
		marsh::Maps attrs2;
		eigen::pack_attr(attrs2, tens);
		EXPECT(nullptr != attrs2.get_attr("tensor"));
	}
	{
		eigen::Packer<egen::_GENERATED_DTYPE> packer;
		marsh::Maps attrs;
		packer.pack(attrs, egen::INT32);
		EXPECT("dtype" == packer.get_key() && "INT32" == attrs.get_attr("dtype")->to_string());
		egen::_GENERATED_DTYPE out = egen::BAD_TYPE;
		packer.unpack(out, attrs);
		EXPECT(egen::INT32 == out);
	}
	// every numeric list is an array of int64, `rank` a single int64
	{
		marsh::Maps attrs;
		eigen::pack_attr(attrs, eigen::PairVecT<teq::RankT>{{2, 2}, {3, 4}}, teq::DimsT{7, 9}, (teq::RankT) 5);
		auto arr = dynamic_cast<const marsh::NumArray<int64_t>*>(attrs.get_attr("rank_pairs"));
		EXPECT(nullptr != arr && (arr->contents_ == std::vector<int64_t>{2, 2, 3, 4}));
		arr = dynamic_cast<const marsh::NumArray<int64_t>*>(attrs.get_attr("dimensions"));
		EXPECT(nullptr != arr && (arr->contents_ == std::vector<int64_t>{7, 9}));
		auto num = dynamic_cast<const marsh::Number<int64_t>*>(attrs.get_attr("rank"));
		EXPECT(nullptr != num && 5 == num->to_int64());
	}

	// ranks past the cap are refused when packed
	marsh::Maps attrs;
	EXPECT_FATAL(eigen::Packer<eigen::PairVecT<teq::RankT>>().pack(attrs, {{teq::rank_cap, 3}, {4, teq::rank_cap + 2}}),
		"cannot reference ranks beyond rank_cap 8: [8:3\\4:10]");
	EXPECT_FATAL(eigen::Packer<teq::RanksT>().pack(attrs, {teq::rank_cap, 3, 4, teq::rank_cap + 2}),
		"cannot reference ranks beyond rank_cap 8: [8\\3\\4\\10]");
	EXPECT_FATAL(eigen::Packer<std::set<teq::RankT>>().pack(attrs, {teq::rank_cap, 3, 4, teq::rank_cap + 2}),
		"cannot reference ranks beyond rank_cap 8: [3\\4\\8\\10]");
	EXPECT_FATAL(eigen::Packer<std::set<teq::RankT>>().pack(attrs, {1, 2, 3, 4, 5, teq::rank_cap, 6, 7, teq::rank_cap + 2}),
		"cannot specify 9 ranks when 8 (rank_cap) are available");
	EXPECT(0 == attrs.size());

	// PACKER.EmptyPacking
	marsh::Maps empty;
	eigen::pack_attr(empty);
	EXPECT(0 == empty.size());

	// PACKER.ExtendPacking: explicit factors, or the tensor to look like
	teq::Shape inshape({1, 2, 3});
	teq::DimsT extends = {4, 1, 1, 2, 1, 1, 1, 1};
	{
		marsh::Maps byfactor;
		eigen::Packer<teq::DimsT>().pack(byfactor, extends);
		auto ext = eigen::unpack_extend(inshape, byfactor);
		EXPECT(ext && *ext == extends);
	}
	{
		std::vector<double> big(4 * 2 * 3 * 2, 0.0);
		teq::TensptrT like = eteq::make_variable<double>(big.data(), teq::Shape({4, 2, 3, 2}), "like");
		marsh::Maps bytensor;
		eigen::Packer<teq::TensptrT>().pack(bytensor, like);
		auto ext = eigen::unpack_extend(inshape, bytensor);
		EXPECT(ext && *ext == extends);
	}
	EXPECT(false == (bool) eigen::unpack_extend(inshape, empty));
}

int main (void)
{
	initiation();
	update_child();
	prop();
	cache();
	evaluator_slot();
	context_registries();
	packers();
	std::printf("%d failure(s)\n", failures);
	return failures;
}
