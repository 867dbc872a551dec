// Process-wide helpers of the host layer: error reporting in the style of
// tenncor's global logger (internal/global/logs.hpp:11-81, where the `fatal`
// and `throw_err` levels throw std::runtime_error, internal/global/g3logs.hpp:
// 140-152), the graph-wide version clock and the seeded random generator
// (internal/global/random.hpp:78-146).
#ifndef TCH_GLOBAL_HPP
#define TCH_GLOBAL_HPP

#include <cstdarg>
#include <cstdio>
#include <functional>
#include <memory>
#include <random>
#include <stdexcept>
#include <string>
#include <unordered_map>

namespace global
{

inline std::string vformat (const char* fmt, va_list ap)
{
	char buf[2048];
	vsnprintf(buf, sizeof(buf), fmt, ap);
	return std::string(buf);
}

[[noreturn]] inline void fatal (const std::string& msg)
{
	throw std::runtime_error(msg);
}

[[noreturn]] inline void throw_err (const std::string& msg)
{
	throw std::runtime_error(msg);
}

[[noreturn]] inline void fatalf (const char* fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	std::string msg = vformat(fmt, ap);
	va_end(ap);
	throw std::runtime_error(msg);
}

[[noreturn]] inline void throw_errf (const char* fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	std::string msg = vformat(fmt, ap);
	va_end(ap);
	throw std::runtime_error(msg);
}

// String-keyed registry of the services an evaluation needs (the evaluator,
// the runtime memory): what the reference's global::context() returns
// (internal/global/config.hpp:9-13, src/config.cpp:8-12; its map type is
// estd::ConfigMap<> of the cppkg library).  An entry is registered with a
// factory, created the first time it is asked for and deleted, as the type
// it was registered with, when it is removed or when the map goes away.
struct ConfigMap final
{
	ConfigMap (void) = default;
	ConfigMap (const ConfigMap&) = delete;
	ConfigMap& operator = (const ConfigMap&) = delete;

	~ConfigMap (void)
	{
		for (auto& kv : entries_) { kv.second.drop(); }
	}

	template <typename T>
	void add_entry (const std::string& key, std::function<T*(void)> init)
	{
		if (entries_.count(key) > 0) { return; } // the first registration stays
		Entry entry;
		entry.init_ = [init]() -> void* { return init(); };
		entry.del_ = [](void* obj) { delete static_cast<T*>(obj); };
		entries_.emplace(key, std::move(entry));
	}

	void rm_entry (const std::string& key)
	{
		auto it = entries_.find(key);
		if (it == entries_.end()) { return; }
		it->second.drop();
		entries_.erase(it);
	}

	bool has_entry (const std::string& key) const { return entries_.count(key) > 0; }

	/// The object behind `key`, created on first use; nullptr for an unknown key
	void* get_obj (const std::string& key)
	{
		auto it = entries_.find(key);
		if (it == entries_.end()) { return nullptr; }
		Entry& entry = it->second;
		if (nullptr == entry.obj_ && entry.init_) { entry.obj_ = entry.init_(); }
		return entry.obj_;
	}

private:
	struct Entry final
	{
		void drop (void)
		{
			if (nullptr != obj_ && del_) { del_(obj_); }
			obj_ = nullptr;
		}

		std::function<void*(void)> init_;
		std::function<void(void*)> del_;
		void* obj_ = nullptr;
	};

	std::unordered_map<std::string,Entry> entries_;
};

using CfgMapptrT = std::shared_ptr<ConfigMap>;

using CfgMaprefT = std::weak_ptr<ConfigMap>;

/// The process-wide registry; callers that keep their services apart (a test,
/// a second session) make a map of their own and pass it instead
CfgMapptrT context (void);

// Diagnostics below `error` are routed to an optional sink (none by default)
using LogSinkF = std::function<void(const std::string& level, const std::string& msg)>;
LogSinkF& log_sink (void);

inline void log (const char* level, const std::string& msg)
{
	if (auto& sink = log_sink()) { sink(level, msg); }
}

inline void debug (const std::string& msg) { log("debug", msg); }
inline void warn (const std::string& msg) { log("warn", msg); }

inline void debugf (const char* fmt, ...)
{
	if (!log_sink()) { return; }
	va_list ap;
	va_start(ap, fmt);
	std::string msg = vformat(fmt, ap);
	va_end(ap);
	log("debug", msg);
}

inline void warnf (const char* fmt, ...)
{
	if (!log_sink()) { return; }
	va_list ap;
	va_start(ap, fmt);
	std::string msg = vformat(fmt, ap);
	va_end(ap);
	log("warn", msg);
}

// Highest state version handed out so far; a Variable assignment takes the
// next one so that every dependant recomputes (tenncor/eteq/variable.hpp:55-61)
size_t& last_version (void);

inline void note_version (size_t v)
{
	if (v > last_version()) { last_version() = v; }
}

// Counts events that make remembered node pointers unsafe (a node destroyed,
// an operand replaced, a launch closure rebuilt); whoever caches anything per
// node compares it with the value seen when the cache was filled
size_t& structure_epoch (void);

inline void note_structure_change (void) { ++structure_epoch(); }

// True once the process has begun to exit: device resources are then left to
// the driver rather than released one by one
bool& process_exiting (void);

// Seeded generator behind RAND_UNIF (host side, like the reference)
using RandEngineT = std::default_random_engine;
RandEngineT& get_generator (void);
void seed (size_t s);

// Where RAND_UNIF closures built from now on draw: false = on the host from
// get_generator() (the reference's behaviour and stream family), true = on the
// device (a counter-based generator with its own stream; such nodes can be
// part of a recorded launch sequence)
bool& device_random (void);

}

#endif // TCH_GLOBAL_HPP
