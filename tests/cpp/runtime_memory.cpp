// A caller-supplied eigen::iRuntimeMemory on the GPU path, checked the way the
// reference's operator tests check their mock allocator (internal/eigen/test/
// test_operator.cpp:25-67): every operator asks for exactly
// n_elems * sizeof(T) bytes once, writes its result there, and gives the same
// pointer back with the same size exactly once; aliases (ref, last-dim slice)
// ask for nothing (test_operator.cpp:70-91, 423-440).  One operator per family
// is built through its factory (what egen::typed_exec calls) and run with
// assign(ttl, memory); then a two-node graph is evaluated through an
// eigen::Device built on the allocator registered in a context of its own
// (the route of tenncor/eteq/etens.hpp:152-162), where the producer's buffer
// must come back as soon as its only reader has been launched.
// The allocator hands out device memory (tcg_alloc).  Needs a GPU.
// Prints one line per failed expectation and exits with their count.
#include <cmath>
#include <cstdio>
#include <set>
#include <string>
#include <vector>

#include "eteq.hpp"

static int failures = 0;

#define EXPECT(COND) do { if (!(COND)) { ++failures; std::printf("%s:%d: expected %s\n", __FILE__, __LINE__, #COND); } } while (0)

namespace
{

struct RecordingMemory final : public eigen::iRuntimeMemory
{
	struct Event final
	{
		bool alloc;
		void* ptr;
		size_t bytes;
	};

	void* allocate (size_t size) override
	{
		void* ptr = nullptr;
		eigen::hip_check(tcg_alloc(eigen::hip_context(), size, &ptr));
		events_.push_back({true, ptr, size});
		return ptr;
	}

	void deallocate (void* ptr, size_t size) override
	{
		events_.push_back({false, ptr, size});
		eigen::hip_check(tcg_free(eigen::hip_context(), ptr, size));
	}

	std::vector<Event> events_;
};

using MemptrT = std::shared_ptr<RecordingMemory>;

teq::TensptrT leaf (const std::vector<double>& values, teq::Shape shape, const char* label)
{
	if (values.size() != shape.n_elems()) { global::fatalf("%s: %d values", label, (int) values.size()); }
	return eteq::make_variable<double>(values.data(), shape, label);
}

// build -> assign -> read -> destroy, with the allocator's record checked at each point
void run_case (const char* name, MemptrT memory, eigen::EigenptrT op, size_t nout, const std::vector<double>& expect)
{
	size_t bytes = nout * sizeof(double);
	size_t first = memory->events_.size();
	EXPECT(nullptr == op->device_data()); // nothing before the first assign
	eigen::RTMemptrT mem = memory;
	op->assign(1, mem);
	bool asked_once = memory->events_.size() == first + 1 && memory->events_[first].alloc &&
		memory->events_[first].bytes == bytes;
	if (false == asked_once)
	{
		++failures;
		std::printf("%s: expected one allocate(%zu), saw %zu event(s)\n", name, bytes, memory->events_.size() - first);
		return;
	}
	void* handed = memory->events_[first].ptr;
	EXPECT(handed == op->device_data());   // the result is written where the allocator said
	const double* got = (const double*) op->data();
	if (nullptr == got)
	{
		++failures;
		std::printf("%s: no data after assign\n", name);
		return;
	}
	for (size_t i = 0; i < expect.size(); ++i)
	{
		if (std::fabs(got[i] - expect[i]) > 1e-12 * std::max(1.0, std::fabs(expect[i])))
		{
			++failures;
			std::printf("%s: element %zu is %.17g, expected %.17g\n", name, i, got[i], expect[i]);
		}
	}
	EXPECT(memory->events_.size() == first + 1); // reading neither allocates nor frees
	op = nullptr;                                 // the last owner goes away
	bool returned_once = memory->events_.size() == first + 2 && false == memory->events_[first + 1].alloc &&
		memory->events_[first + 1].ptr == handed && memory->events_[first + 1].bytes == bytes;
	if (false == returned_once)
	{
		++failures;
		std::printf("%s: expected one deallocate(%p, %zu)\n", name, handed, bytes);
	}
}

}

int main (void)
{
	try
	{
		auto memory = std::make_shared<RecordingMemory>();
		marsh::Maps attrs;

		// R1 (test_operator.cpp:25-67 values): {3,2} summed over dim 1
		teq::TensptrT edge = leaf({2, 3, 4, 5, 6, 7}, teq::Shape({3, 2}), "edge");
		eigen::pack_attr(attrs, std::set<teq::RankT>{1});
		run_case("reduce_sum", memory, eigen::reduce_sum<double>(teq::Shape({3}), *edge, attrs), 3, {7, 9, 11});
		run_case("reduce_max", memory, eigen::reduce_max<double>(teq::Shape({3}), *edge, attrs), 3, {5, 6, 7});
		// R2: index of the maximum along dim 0
		marsh::Maps rank_attr;
		eigen::pack_attr(rank_attr, (teq::RankT) 0);
		run_case("argmax", memory, eigen::argmax<double>(teq::Shape({1, 2}), *edge, rank_attr), 2, {2, 2});
		// E1, E2, E3, E4
		teq::TensptrT other = leaf({1, -1, 2, -2, 3, -3}, teq::Shape({3, 2}), "other");
		teq::TensptrT third = leaf({10, 20, 30, 40, 50, 60}, teq::Shape({3, 2}), "third");
		run_case("neg", memory, eigen::neg<double>(teq::Shape({3, 2}), *edge), 6, {-2, -3, -4, -5, -6, -7});
		run_case("sub", memory, eigen::sub<double>(teq::Shape({3, 2}), *edge, *other), 6, {1, 4, 2, 7, 3, 10});
		run_case("add3", memory, eigen::add<double>(teq::Shape({3, 2}), teq::TensptrsT{edge, other, third}), 6,
			{13, 22, 36, 43, 59, 64});
		teq::TensptrT cond = leaf({1, 0, 0, 2, 0, -1}, teq::Shape({3, 2}), "cond");
		run_case("select", memory, eigen::select<double>(teq::Shape({3, 2}), *cond, *edge, *other), 6, {2, -1, 2, 5, 3, 7});
		// S1: {3,1,2} tiled 4 times along dim 1
		teq::TensptrT thin = leaf({2, 3, 4, 5, 6, 7}, teq::Shape({3, 1, 2}), "thin");
		marsh::Maps ext_attr;
		eigen::pack_attr(ext_attr, teq::DimsT{1, 4});
		run_case("extend", memory, eigen::extend<double>(teq::Shape({3, 4, 2}), *thin, ext_attr), 24,
			{2, 3, 4, 2, 3, 4, 2, 3, 4, 2, 3, 4, 5, 6, 7, 5, 6, 7, 5, 6, 7, 5, 6, 7});
		// S2: transpose
		marsh::Maps perm_attr;
		eigen::pack_attr(perm_attr, teq::RanksT{1, 0});
		run_case("permute", memory, eigen::permute<double>(teq::Shape({2, 3}), *edge, perm_attr), 6, {2, 5, 3, 6, 4, 7});
		// S3: a slice of the first dim is a copy ...
		marsh::Maps cut_attr;
		eigen::pack_attr(cut_attr, eigen::PairVecT<teq::DimT>{{1, 2}});
		run_case("slice", memory, eigen::slice<double>(teq::Shape({2, 2}), edge, cut_attr), 4, {3, 4, 6, 7});
		// ... a slice of the last dim alone is the operand's memory at an offset: nothing is asked for
		{
			size_t before = memory->events_.size();
			marsh::Maps last_attr;
			eigen::pack_attr(last_attr, eigen::PairVecT<teq::DimT>{{0, 3}, {1, 1}});
			auto alias = eigen::slice<double>(teq::Shape({3, 1}), edge, last_attr);
			eigen::RTMemptrT mem = memory;
			alias->assign(1, mem);
			const double* got = (const double*) alias->data();
			EXPECT(nullptr != got && 5 == got[0] && 6 == got[1] && 7 == got[2]);
			auto same = eigen::ref(edge);
			same->assign(1, mem);
			EXPECT(edge->device().data() == same->data());
			alias = nullptr;
			same = nullptr;
			EXPECT(memory->events_.size() == before);
		}
		// S4
		marsh::Maps pad_attr;
		eigen::pack_attr(pad_attr, eigen::PairVecT<teq::DimT>{{1, 0}});
		run_case("pad", memory, eigen::pad<double>(teq::Shape({4, 2}), *edge, pad_attr), 8, {0, 2, 3, 4, 0, 5, 6, 7});
		marsh::Maps rev_attr;
		eigen::pack_attr(rev_attr, std::set<teq::RankT>{0});
		run_case("reverse", memory, eigen::reverse<double>(teq::Shape({3, 2}), *edge, rev_attr), 6, {4, 3, 2, 7, 6, 5});
		marsh::Maps cat_attr;
		eigen::pack_attr(cat_attr, (teq::RankT) 0);
		run_case("concat", memory, eigen::concat<double>(teq::Shape({6, 2}), teq::TensptrsT{edge, other}, cat_attr), 12,
			{2, 3, 4, 1, -1, 2, 5, 6, 7, -2, 3, -3});
		// M1 / M2 (test_operator.cpp:1969-2000 values): a{4,3} x b{2,4} -> {2,3}
		teq::TensptrT a = leaf({2, 8, 4, 5, 6, 7, 3, 1, 0, 9, 2, 5}, teq::Shape({4, 3}), "a");
		teq::TensptrT b = leaf({1, 3, 2, 6, 7, 5, 4, 2}, teq::Shape({2, 4}), "b");
		std::vector<double> product(6, 0.0);
		{
			const double av[] = {2, 8, 4, 5, 6, 7, 3, 1, 0, 9, 2, 5}, bv[] = {1, 3, 2, 6, 7, 5, 4, 2};
			for (int m = 0; m < 3; ++m) for (int n = 0; n < 2; ++n) for (int k = 0; k < 4; ++k)
			{
				product[n + 2 * m] += av[k + 4 * m] * bv[n + 2 * k];
			}
		}
		run_case("matmul", memory, eigen::matmul<double>(teq::Shape({2, 3}), *a, *b), 6, product);
		marsh::Maps pair_attr;
		eigen::pack_attr(pair_attr, eigen::PairVecT<teq::RankT>{{0, 1}});
		run_case("contract", memory, eigen::contract<double>(teq::Shape({2, 3}), *a, *b, pair_attr), 6, product);
		// C1: a 2-long kernel sliding along dim 0 of {3,2}
		teq::TensptrT kern = leaf({1, -1}, teq::Shape({2}), "kern");
		marsh::Maps conv_attr;
		eigen::pack_attr(conv_attr, teq::RanksT{0});
		run_case("convolution", memory, eigen::convolution<double>(teq::Shape({2, 2}), *edge, *kern, conv_attr), 4,
			{-1, -1, -1, -1});

		// every buffer handed out has come back
		size_t live = 0;
		for (auto& ev : memory->events_) { live += ev.alloc ? 1 : -1; }
		EXPECT(0 == live);

		// through a context of its own: NEG(edge) read only by REDUCE_SUM, the target
		auto graph_memory = std::make_shared<RecordingMemory>();
		global::CfgMapptrT ctx = std::make_shared<global::ConfigMap>();
		eigen::set_runtime(graph_memory, ctx);
		{
			teq::TensptrT negated = eteq::make_functor(egen::NEG, {edge});
			teq::TensptrT summed = eteq::make_functor(egen::REDUCE_SUM, {negated}, std::set<teq::RankT>{1});
			eteq::ETensor handle(summed, ctx);
			double* got = handle.calc<double>();
			EXPECT(nullptr != got && -7 == got[0] && -9 == got[1] && -11 == got[2]);
			auto& ev = graph_memory->events_;
			// NEG's 48 bytes, REDUCE_SUM's 24, and NEG's buffer back after its one read
			EXPECT(3 == ev.size());
			if (3 == ev.size())
			{
				EXPECT(ev[0].alloc && 48 == ev[0].bytes);
				EXPECT(ev[1].alloc && 24 == ev[1].bytes);
				EXPECT(false == ev[2].alloc && ev[2].ptr == ev[0].ptr && 48 == ev[2].bytes);
			}
			// evaluating again without news: the walk finds NEG without a value
			// (its one read is spent) and computes it again, as the reference's
			// does (internal/eigen/device.hpp:555-570); REDUCE_SUM holds its value
			// and is left alone, so NEG's new buffer waits for a reader
			double* again = handle.calc<double>();
			EXPECT(got == again);
			EXPECT(4 == ev.size());
			if (4 == ev.size()) { EXPECT(ev[3].alloc && 48 == ev[3].bytes); }
		}
		// the nodes are gone: both buffers came back, each once, each with its size
		EXPECT(6 == graph_memory->events_.size());
		if (6 == graph_memory->events_.size())
		{
			auto& ev = graph_memory->events_;
			bool target_back = false, operand_back = false;
			for (size_t i = 4; i < 6; ++i)
			{
				target_back = target_back || (false == ev[i].alloc && ev[i].ptr == ev[1].ptr && 24 == ev[i].bytes);
				operand_back = operand_back || (false == ev[i].alloc && ev[i].ptr == ev[3].ptr && 48 == ev[i].bytes);
			}
			EXPECT(target_back && operand_back);
		}
		// the process-wide context was never touched by all this
		EXPECT(nullptr != std::dynamic_pointer_cast<eigen::RuntimeMemory>(eigen::get_runtime()));
	}
	catch (std::exception& e)
	{
		std::printf("error %s\n", e.what());
		return 100;
	}
	std::printf("%d failure(s)\n", failures);
	return failures;
}
