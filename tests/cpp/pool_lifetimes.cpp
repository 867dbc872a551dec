// Lifetime rules of the device block pool and of the arenas of recorded launch
// sequences (tenncor_amd/csrc/tcg_pool.hpp), checked on the host: the pool's
// bookkeeping has no GPU call in it, so here it runs on malloc / free under a
// model that knows who holds what.  A random walk over every operation
// (allocate, free, start / end a recording, claim a result after a launch,
// destroy a sequence, trim, driver out of memory) asserts after each step:
//   - the pool's own audit: every block in exactly one state, counters add up;
//   - no block is handed out while somebody holds it;
//   - a block owned by a live arena is only ever handed out by that arena,
//     and only while that arena is the one being recorded;
//   - destroying a sequence returns exactly its unheld blocks; blocks a caller
//     still holds stay valid and are freed the ordinary way later;
//   - a block cannot be given back twice or with another size.
// The reference's allocator contract (internal/eigen/memory.hpp:14-22:
// deallocate receives the size given to allocate) is what `give` enforces.
// Prints one line per failed expectation and exits with their count.
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <random>

#include "tcg_pool.hpp"

static int failures = 0;

#define EXPECT(COND) do { if (!(COND)) { ++failures; std::printf("%s:%d: expected %s\n", __FILE__, __LINE__, #COND); } } while (0)

namespace
{

struct Driver final
{
	std::set<void*> live;
	size_t live_bytes = 0, limit = (size_t) -1;
	std::map<void*,size_t> sizes;
	size_t drains = 0;
};

struct Held final
{
	void* ptr;
	size_t bytes;       // as asked for
	tcg_arena* arena;   // arena that was recording when it was taken (nullptr: none)
};

void connect (tcg_pool& pool, Driver& drv)
{
	pool.raw_alloc = [&drv](size_t bytes, void** out) -> int
	{
		if (drv.live_bytes + bytes > drv.limit) { return 1; }
		*out = std::malloc(bytes);
		drv.live.insert(*out);
		drv.sizes[*out] = bytes;
		drv.live_bytes += bytes;
		return 0;
	};
	pool.raw_free = [&drv](void* ptr)
	{
		if (0 == drv.live.erase(ptr))
		{
			++failures;
			std::printf("the pool released %p, which the driver does not know (double release?)\n", ptr);
			return;
		}
		drv.live_bytes -= drv.sizes[ptr];
		drv.sizes.erase(ptr);
		std::free(ptr);
	};
	pool.drain = [&drv] { ++drv.drains; };
}

void scripted (void)
{
	Driver drv;
	tcg_pool pool;
	connect(pool, drv);
	std::string why;
	void *a = nullptr, *b = nullptr, *c = nullptr;
	EXPECT(tcg_pool::OK == pool.take(1000, &a, &why));
	EXPECT(1024 == pool.bytes_in_use && 0 == pool.bytes_pooled);
	// the size must be the one asked for (up to the size class), and only once
	EXPECT(tcg_pool::BAD_ARG == pool.give(a, 5000, &why) && why.find("another size") != std::string::npos);
	EXPECT(tcg_pool::OK == pool.give(a, 1000, &why));
	EXPECT(tcg_pool::BAD_ARG == pool.give((char*) a + 8, 1000, &why));
	EXPECT(0 == pool.bytes_in_use && 1024 == pool.bytes_pooled);
	// recycled without going back to the driver
	EXPECT(tcg_pool::OK == pool.take(1024, &b, &why) && a == b && 1 == drv.live.size());

	// a recording adopts what it is handed and reuses what it is given back
	tcg_arena first;
	pool.recording = &first;
	EXPECT(tcg_pool::OK == pool.take(4096, &c, &why));
	EXPECT(1 == first.blocks.count(c) && 1 == first.held.count(c) && 4096 == first.bytes);
	EXPECT(tcg_pool::OK == pool.give(c, 4096, &why));
	EXPECT(tcg_pool::BAD_ARG == pool.give(c, 4096, &why) && why.find("twice") != std::string::npos);
	void* again = nullptr;
	EXPECT(tcg_pool::OK == pool.take(4000, &again, &why) && again == c); // later launches of the pass reuse it
	EXPECT(tcg_pool::OK == pool.give(again, 4000, &why));
	pool.seal(&first);
	EXPECT(nullptr == pool.recording && first.free_blocks.empty());
	EXPECT("" == pool.audit({&first}));
	// sealed: the block stays reserved for the recorded launches
	void* other = nullptr;
	EXPECT(tcg_pool::OK == pool.take(4096, &other, &why) && other != c);
	// a second recording never gets the first one's block either
	tcg_arena second;
	pool.recording = &second;
	void* mine = nullptr;
	EXPECT(tcg_pool::OK == pool.take(4096, &mine, &why) && mine != c && mine != other);
	pool.seal(&second);
	// a result is claimed after a launch, its sequence destroyed, and the block freed the ordinary way
	EXPECT(pool.claim(&first, c) && false == pool.claim(&first, other));
	uint64_t in_use = pool.bytes_in_use;
	pool.dissolve(&first);
	EXPECT(in_use == pool.bytes_in_use);          // still in the caller's hands
	EXPECT(0 == pool.arena_of.count(c));
	EXPECT(tcg_pool::OK == pool.give(c, 4096, &why));
	EXPECT(in_use - 4096 == pool.bytes_in_use);
	EXPECT("" == pool.audit({&second}));
	// a sequence destroyed with nothing held returns everything
	EXPECT(tcg_pool::OK == pool.give(mine, 4096, &why));
	uint64_t pooled = pool.bytes_pooled;
	pool.dissolve(&second);
	EXPECT(pooled + 4096 == pool.bytes_pooled && pool.arena_of.empty());
	EXPECT("" == pool.audit({}));

	// the driver runs out: pooled blocks go back to it (after a drain) and the call succeeds ...
	drv.limit = drv.live_bytes + 100;
	size_t drains = drv.drains;
	void* big = nullptr;
	EXPECT(pool.bytes_pooled >= 8192);
	EXPECT(tcg_pool::OK == pool.take(8192, &big, &why));
	EXPECT(drains + 1 == drv.drains && 0 == pool.bytes_pooled);
	// ... except while recording, when nothing may be drained
	tcg_arena third;
	pool.recording = &third;
	void* none = nullptr;
	EXPECT(tcg_pool::OUT_OF_MEMORY == pool.take(1 << 20, &none, &why) && why.find("while recording") != std::string::npos);
	EXPECT(third.blocks.empty());
	pool.seal(&third);
	pool.dissolve(&third);
	EXPECT(tcg_pool::OUT_OF_MEMORY == pool.take(1 << 20, &none, &why));
	EXPECT("" == pool.audit({}));
	EXPECT(tcg_pool::OK == pool.give(big, 8192, &why) && tcg_pool::OK == pool.give(b, 1024, &why) &&
		tcg_pool::OK == pool.give(other, 4096, &why));
	pool.release_all();
	EXPECT(drv.live.empty());
}

void random_walk (unsigned seed, int steps)
{
	Driver drv;
	tcg_pool pool;
	connect(pool, drv);
	std::mt19937 rng(seed);
	auto pick = [&rng](size_t n) { return (size_t) (rng() % n); };
	std::vector<Held> held;
	std::vector<std::unique_ptr<tcg_arena>> arenas; // live ones; the one being recorded is pool.recording
	const size_t sizes[] = {1, 64, 256, 257, 1000, 4096, 70000, (1u << 20) + 1, 3u << 20};
	std::string why;
	auto all_arenas = [&]
	{
		std::vector<const tcg_arena*> out;
		for (auto& a : arenas) { out.push_back(a.get()); }
		return out;
	};
	for (int step = 0; step < steps; ++step)
	{
		size_t op = pick(100);
		if (op < 40)
		{
			size_t bytes = sizes[pick(sizeof(sizes) / sizeof(sizes[0]))];
			void* p = nullptr;
			int rc = pool.take(bytes, &p, &why);
			if (rc == tcg_pool::OK)
			{
				for (auto& h : held) { EXPECT(h.ptr != p); }           // nobody holds it
				auto owner = pool.arena_of.find(p);
				tcg_arena* arena = owner == pool.arena_of.end() ? nullptr : owner->second;
				EXPECT(arena == pool.recording);                        // a live arena's block only from that arena, while it records
				EXPECT(drv.live.count(p) == 1);
				held.push_back({p, bytes, arena});
			}
			else { EXPECT(rc == tcg_pool::OUT_OF_MEMORY); }
		}
		else if (op < 70 && false == held.empty())
		{
			size_t i = pick(held.size());
			Held h = held[i];
			held.erase(held.begin() + i);
			uint64_t before = pool.bytes_in_use;
			bool owned = pool.arena_of.count(h.ptr) > 0;
			EXPECT(tcg_pool::OK == pool.give(h.ptr, h.bytes, &why));
			// an arena's block stays reserved; an ordinary one returns to the pool
			EXPECT(pool.bytes_in_use == (owned ? before : before - tcg_pool::round_block(h.bytes)));
			EXPECT(tcg_pool::BAD_ARG == pool.give(h.ptr, h.bytes, &why)); // not twice
		}
		else if (op < 76 && nullptr == pool.recording)
		{
			arenas.push_back(std::make_unique<tcg_arena>());
			pool.recording = arenas.back().get();
		}
		else if (op < 84 && nullptr != pool.recording)
		{
			pool.seal(pool.recording);
		}
		else if (op < 90 && false == arenas.empty())
		{
			// after a launch of a sealed sequence: the caller takes one of its blocks for itself
			tcg_arena* arena = arenas[pick(arenas.size())].get();
			if (arena != pool.recording && false == arena->blocks.empty())
			{
				auto it = arena->blocks.begin();
				std::advance(it, pick(arena->blocks.size()));
				bool already = arena->held.count(it->first) > 0;
				EXPECT(pool.claim(arena, it->first));
				if (false == already) { held.push_back({it->first, it->second, arena}); }
			}
		}
		else if (op < 96 && false == arenas.empty())
		{
			size_t i = pick(arenas.size());
			tcg_arena* arena = arenas[i].get();
			if (arena != pool.recording)
			{
				uint64_t unheld = 0;
				for (auto& kv : arena->blocks) { unheld += arena->held.count(kv.first) ? 0 : kv.second; }
				uint64_t pooled = pool.bytes_pooled;
				pool.dissolve(arena);
				EXPECT(pooled + unheld == pool.bytes_pooled);
				for (auto& h : held) { if (h.arena == arena) { h.arena = nullptr; } }
				arenas.erase(arenas.begin() + i);
			}
		}
		else if (op < 98 && nullptr == pool.recording)
		{
			pool.trim();
			EXPECT(0 == pool.bytes_pooled);
		}
		else
		{
			drv.limit = pick(2) ? (size_t) -1 : drv.live_bytes + sizes[pick(6)];
		}
		std::string verdict = pool.audit(all_arenas());
		if (false == verdict.empty())
		{
			++failures;
			std::printf("seed %u step %d: %s\n", seed, step, verdict.c_str());
			break;
		}
		// everything held is memory the driver still knows
		for (auto& h : held) { EXPECT(drv.live.count(h.ptr) == 1); }
	}
	pool.release_all();
	EXPECT(drv.live.empty());
}

}

int main (void)
{
	EXPECT(256 == tcg_pool::round_block(0) && 256 == tcg_pool::round_block(256) && 512 == tcg_pool::round_block(257));
	EXPECT((1u << 20) == tcg_pool::round_block(1u << 20) && (1u << 20) + (1u << 17) == tcg_pool::round_block((1u << 20) + 1));
	scripted();
	for (unsigned seed = 1; seed <= 40; ++seed) { random_walk(seed, 4000); }
	std::printf("%d failure(s)\n", failures);
	return failures > 255 ? 255 : failures;
}
