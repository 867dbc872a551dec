// The node API a tenncor checkout binds to, exercised from C++ the way the
// reference's own unit tests exercise it (tenncor/eteq/test/test_functor.cpp:
// 22-104 Initiation, :107-192 UpdateChild, :195-261 Prop, :264-302 Cache;
// internal/teq/test/test_evaluator.cpp:20-30 SetGet).  The reference runs these
// on gmock doubles; here the operands are real variables and functors of the
// host layer.  Nothing is launched: no GPU is needed.  Prints one line per
// failed expectation and exits with their count.
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#include "eteq.hpp"

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

int main (void)
{
	initiation();
	update_child();
	prop();
	cache();
	evaluator_slot();
	std::printf("%d failure(s)\n", failures);
	return failures;
}
