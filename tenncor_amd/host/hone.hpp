// Graph clean-up before evaluation: equal subgraphs are merged, functors that
// depend on constants only are computed once (on the GPU, through the
// registered evaluator) and replaced by constants, and subgraph patterns are
// rewritten by rules read from JSON.  Follows tenncor/hone/optimize.hpp:19-38
// and src/optimize.cpp:13-36 (merge_dups, then up to 50 rounds of constant
// rules + conversions), tenncor/hone/duplicates.hpp:13-95,
// tenncor/hone/cstrules.hpp:48-65 (ConstantTarget), internal/opt/src/parse.cpp
// (conversions: `srcs` patterns and one `dest`) and the pattern language of
// internal/query/query.proto:7-79.
#ifndef TCH_HONE_HPP
#define TCH_HONE_HPP

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "eteq.hpp"

namespace hone
{

/// Parsed JSON value (objects keep their key order)
struct Json final
{
	enum Kind { NUL, BOOL, NUMBER, STRING, ARRAY, OBJECT };

	Kind kind = NUL;
	bool boolean = false;
	double number = 0;
	std::string string;
	std::vector<Json> array;
	std::vector<std::pair<std::string,Json>> object;

	const Json* find (const std::string& key) const
	{
		for (auto& kv : object) { if (kv.first == key) { return &kv.second; } }
		return nullptr;
	}
};

/// Throws std::runtime_error naming the offset of the first malformed byte
Json parse_json (const std::string& text);

/// What a `srcs` entry matches (query.proto Node)
struct Pattern final
{
	enum Kind { SYMBOL, SCALAR, LEAF, OPERATOR };

	Kind kind = SYMBOL;
	std::string symbol;   ///< SYMBOL: binds any node; OPERATOR: optional capture
	double scalar = 0;    ///< SCALAR: constant whose elements all equal this
	// LEAF: every given field must hold
	std::string label, dtype, usage;
	bool has_label = false, has_dtype = false, has_usage = false;
	std::vector<uint64_t> shape;
	// OPERATOR
	std::string opname;
	bool has_args = false;
	std::vector<Pattern> args;
	std::vector<std::pair<std::string,Json>> attrs;
};

/// What a match is replaced by (optimize.proto TargetNode)
struct Target final
{
	enum Kind { SYMBOL, SCALAR, OPERATOR };

	Kind kind = SYMBOL;
	std::string symbol;  ///< SYMBOL: the bound node; SCALAR: node whose shape and dtype the constant takes
	double scalar = 0;
	std::string opname;
	std::vector<Target> args;
	std::vector<std::pair<std::string,Json>> attrs;
};

struct Conversion final
{
	std::vector<Pattern> srcs;
	Target dest;
};

using RulesT = std::vector<Conversion>;

/// {"conversions": [{"srcs": [...], "dest": {...}}, ...]}
RulesT parse_rules (const std::string& json_text);

struct Stats final
{
	size_t merged = 0;    ///< nodes replaced by an equal node
	size_t folded = 0;    ///< functors replaced by the constant they evaluate to
	size_t converted = 0; ///< rule matches rewritten
	size_t rounds = 0;
};

/// Node bindings of one match
using SymbMapT = std::map<std::string,teq::TensptrT>;

/// True when `node` matches; symbols bound so far must agree
bool match (SymbMapT& symbols, const teq::TensptrT& node, const Pattern& pattern);

teq::TensptrT build (const Target& target, const SymbMapT& symbols);

/// Equal immutable leaves and equal functors (same opcode, attributes and
/// operands; operand order ignored for commutative opcodes) become one node
teq::TensptrsT merge_dups (teq::TensptrsT roots, Stats* stats = nullptr);

/// merge_dups, then rounds of constant folding and `rules` until nothing
/// changes (at most 50 rounds).  Parents are rewired in place; the returned
/// roots replace the ones passed in.  `fold` = false skips the evaluation of
/// constant functors (no GPU needed then).
teq::TensptrsT optimize (teq::TensptrsT roots, const RulesT& rules, bool fold = true, Stats* stats = nullptr);

}

#endif // TCH_HONE_HPP
