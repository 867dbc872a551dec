// The stream-ordered block pool of a context and the ownership of blocks by
// recorded launch sequences, without any GPU call in it: where blocks come
// from and go to is a pair of callbacks, so the same bookkeeping runs on the
// device (hipMalloc / hipFree, tcg_ctx.hip) and on the host in tests
// (tests/cpp/pool_lifetimes.cpp checks its invariants with malloc / free).
//
// States of a block, exactly one at a time:
//   pooled        in a free list of the pool, waiting to be handed out
//   in use        handed to a caller by take(), not owned by any arena ("lent")
//   arena, held   owned by an arena and currently handed to a caller
//   arena, free   owned by an arena, given back; only the arena that is being
//                 recorded hands such a block out again
// A block of an arena never returns to the pool before dissolve(): the
// launches recorded with the arena keep its address.
#ifndef TCG_POOL_HPP
#define TCG_POOL_HPP

#include <cstddef>
#include <cstdint>
#include <functional>
#include <map>
#include <set>
#include <string>
#include <vector>

/// Device memory of one recorded launch sequence
struct tcg_arena
{
	std::map<void*,size_t> blocks;                      // block -> rounded size
	std::set<void*> held;                               // blocks a caller currently owns
	std::map<size_t,std::vector<void*>> free_blocks;    // reuse while recording
	uint64_t bytes = 0;
};

struct tcg_pool
{
	enum Status { OK = 0, BAD_ARG = 1, OUT_OF_MEMORY = 4 };

	/// 0 on success; anything else means no memory
	std::function<int(size_t bytes, void** out)> raw_alloc;
	std::function<void(void* ptr)> raw_free;
	/// called before pooled blocks go back to the driver (they may still be
	/// read by work that was enqueued before they were given back)
	std::function<void(void)> drain;

	std::map<size_t,std::vector<void*>> free_blocks;
	std::map<void*,size_t> block_size; // every block the driver has handed over
	std::set<void*> lent;              // blocks in use that no arena owns
	uint64_t bytes_in_use = 0;
	uint64_t bytes_pooled = 0;
	std::map<void*,tcg_arena*> arena_of; // owner of every block that has one
	tcg_arena* recording = nullptr;      // arena of the sequence being recorded

	/// 256-byte granules up to 1 MiB, then 1/8-octave steps: bounded
	/// fragmentation with few distinct size classes
	static size_t round_block (size_t bytes)
	{
		if (bytes == 0) { bytes = 1; }
		if (bytes <= (1u << 20)) { return (bytes + 255) & ~(size_t) 255; }
		size_t p = (size_t) 1 << 20;
		while (p * 2 <= bytes) { p *= 2; }
		size_t step = p / 8;
		return (bytes + step - 1) / step * step;
	}

	int take (size_t bytes, void** out, std::string* why)
	{
		size_t sz = round_block(bytes);
		tcg_arena* rec = recording;
		if (rec)
		{
			// blocks the sequence has already given back are reused first: the
			// recorded launches run in the order they were recorded
			auto mine = rec->free_blocks.find(sz);
			if (mine != rec->free_blocks.end() && !mine->second.empty())
			{
				*out = mine->second.back();
				mine->second.pop_back();
				rec->held.insert(*out);
				return OK;
			}
		}
		auto it = free_blocks.find(sz);
		if (it != free_blocks.end() && !it->second.empty())
		{
			*out = it->second.back();
			it->second.pop_back();
			bytes_pooled -= sz;
			bytes_in_use += sz;
			if (rec) { adopt(rec, *out, sz); }
			else { lent.insert(*out); }
			return OK;
		}
		void* p = nullptr;
		int rc = raw_alloc(sz, &p);
		if (rc != 0 && rec)
		{
			// pooled blocks cannot be drained while a sequence is being recorded
			if (why) { *why = std::to_string(sz) + " bytes while recording"; }
			return OUT_OF_MEMORY;
		}
		if (rc != 0)
		{
			trim(); // give cached blocks back to the driver and retry once
			rc = raw_alloc(sz, &p);
			if (rc != 0)
			{
				if (why) { *why = std::to_string(sz) + " bytes"; }
				return OUT_OF_MEMORY;
			}
		}
		block_size[p] = sz;
		bytes_in_use += sz;
		if (rec) { adopt(rec, p, sz); }
		else { lent.insert(p); }
		*out = p;
		return OK;
	}

	int give (void* ptr, size_t bytes, std::string* why)
	{
		auto it = block_size.find(ptr);
		if (it == block_size.end())
		{
			if (why) { *why = "the block was not allocated by this context"; }
			return BAD_ARG;
		}
		size_t sz = it->second;
		if (round_block(bytes) != sz)
		{
			if (why) { *why = "the block was allocated with another size (" + std::to_string(bytes) + " bytes given)"; }
			return BAD_ARG;
		}
		auto owner = arena_of.find(ptr);
		if (owner != arena_of.end())
		{
			// stays with its arena; reusable only by the sequence being recorded
			tcg_arena* arena = owner->second;
			if (0 == arena->held.erase(ptr))
			{
				if (why) { *why = "the block is not handed out (given back twice?)"; }
				return BAD_ARG;
			}
			if (arena == recording) { arena->free_blocks[sz].push_back(ptr); }
			return OK;
		}
		if (0 == lent.erase(ptr))
		{
			if (why) { *why = "the block is not handed out (given back twice?)"; }
			return BAD_ARG;
		}
		free_blocks[sz].push_back(ptr);
		bytes_in_use -= sz;
		bytes_pooled += sz;
		return OK;
	}

	/// Recording is over: what the sequence gave back stays reserved for its launches
	void seal (tcg_arena* arena)
	{
		arena->free_blocks.clear();
		if (recording == arena) { recording = nullptr; }
	}

	/// A caller takes a block of the arena for itself again (a result it reads
	/// after a launch of the sequence); false when the block is not the arena's
	bool claim (tcg_arena* arena, void* ptr)
	{
		if (0 == arena->blocks.count(ptr)) { return false; }
		arena->held.insert(ptr);
		return true;
	}

	/// The sequence is gone: its blocks return to the pool, except those a
	/// caller still holds, which become ordinary blocks in use
	void dissolve (tcg_arena* arena)
	{
		if (recording == arena) { recording = nullptr; }
		for (auto& kv : arena->blocks)
		{
			arena_of.erase(kv.first);
			if (arena->held.count(kv.first))
			{
				lent.insert(kv.first); // its owner frees it the ordinary way
				continue;
			}
			free_blocks[kv.second].push_back(kv.first);
			bytes_in_use -= kv.second;
			bytes_pooled += kv.second;
		}
		arena->blocks.clear();
		arena->held.clear();
		arena->free_blocks.clear();
		arena->bytes = 0;
	}

	/// Pooled blocks go back to the driver
	void trim (void)
	{
		if (drain) { drain(); }
		for (auto& kv : free_blocks)
		{
			for (void* q : kv.second)
			{
				raw_free(q);
				block_size.erase(q);
			}
			kv.second.clear();
		}
		bytes_pooled = 0;
	}

	/// Everything goes back to the driver (the context is being destroyed)
	void release_all (void)
	{
		for (auto& kv : block_size) { raw_free(kv.first); }
		block_size.clear();
		free_blocks.clear();
		lent.clear();
		arena_of.clear();
		bytes_in_use = bytes_pooled = 0;
		recording = nullptr;
	}

	/// "" when every block is in exactly one state and the byte counters add
	/// up, else what is wrong.  `arenas`: every live arena.
	std::string audit (const std::vector<const tcg_arena*>& arenas) const
	{
		std::map<void*,int> seen;
		uint64_t pooled = 0;
		for (auto& kv : free_blocks)
		{
			for (void* p : kv.second)
			{
				auto it = block_size.find(p);
				if (it == block_size.end()) { return "a pooled block is unknown to the pool"; }
				if (it->second != kv.first) { return "a pooled block sits in the list of another size"; }
				if (arena_of.count(p)) { return "a block of a live arena is in the pool's free list"; }
				if (lent.count(p)) { return "a block in a caller's hands is in the pool's free list"; }
				if (++seen[p] > 1) { return "a block is pooled twice"; }
				pooled += kv.first;
			}
		}
		if (pooled != bytes_pooled) { return "bytes_pooled does not match the free lists"; }
		uint64_t total = 0;
		for (auto& kv : block_size) { total += kv.second; }
		if (total != bytes_pooled + bytes_in_use) { return "bytes_in_use + bytes_pooled does not match the blocks"; }
		size_t owned = 0;
		for (const tcg_arena* arena : arenas)
		{
			uint64_t bytes = 0;
			for (auto& kv : arena->blocks)
			{
				auto owner = arena_of.find(kv.first);
				if (owner == arena_of.end() || owner->second != arena) { return "an arena's block is not registered to it"; }
				auto it = block_size.find(kv.first);
				if (it == block_size.end() || it->second != kv.second) { return "an arena's block has another size in the pool"; }
				bytes += kv.second;
				++owned;
			}
			if (bytes != arena->bytes) { return "an arena's byte count does not match its blocks"; }
			for (void* p : arena->held)
			{
				if (0 == arena->blocks.count(p)) { return "an arena holds a block that is not its own"; }
			}
			for (auto& kv : arena->free_blocks)
			{
				if (arena != recording && !kv.second.empty()) { return "a sealed arena still offers blocks for reuse"; }
				for (void* p : kv.second)
				{
					if (0 == arena->blocks.count(p)) { return "an arena offers a block that is not its own"; }
					if (arena->held.count(p)) { return "an arena offers a block that is handed out"; }
				}
			}
		}
		if (owned != arena_of.size()) { return "a block is registered to an arena that is not alive"; }
		uint64_t in_use = 0;
		for (void* p : lent)
		{
			auto it = block_size.find(p);
			if (it == block_size.end()) { return "a block in a caller's hands is unknown to the pool"; }
			if (arena_of.count(p)) { return "a block is both an arena's and an ordinary one"; }
			in_use += it->second;
		}
		for (const tcg_arena* arena : arenas) { in_use += arena->bytes; }
		if (in_use != bytes_in_use) { return "bytes_in_use does not match the blocks handed out or reserved"; }
		return "";
	}

private:
	void adopt (tcg_arena* arena, void* p, size_t sz)
	{
		arena->blocks[p] = sz;
		arena->held.insert(p);
		arena->bytes += sz;
		arena_of[p] = arena;
	}
};

#endif // TCG_POOL_HPP
