#include "hone.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <unordered_map>

namespace hone
{

// ---- JSON ------------------------------------------------------------------

namespace
{

struct JsonReader final
{
	const std::string& text;
	size_t pos = 0;

	[[noreturn]] void fail (const char* what) const
	{
		global::fatalf("malformed json at offset %d: %s", (int) pos, what);
	}

	void skip (void)
	{
		while (pos < text.size() && (text[pos] == ' ' || text[pos] == '\t' ||
			text[pos] == '\n' || text[pos] == '\r')) { ++pos; }
	}

	bool take (char c)
	{
		skip();
		if (pos < text.size() && text[pos] == c) { ++pos; return true; }
		return false;
	}

	std::string quoted (void)
	{
		if (!take('"')) { fail("expected a string"); }
		std::string out;
		while (pos < text.size() && text[pos] != '"')
		{
			char c = text[pos++];
			if (c == '\\')
			{
				if (pos >= text.size()) { fail("unfinished escape"); }
				char e = text[pos++];
				switch (e)
				{
					case 'n': out += '\n'; break;
					case 't': out += '\t'; break;
					case 'r': out += '\r'; break;
					case 'b': out += '\b'; break;
					case 'f': out += '\f'; break;
					case 'u':
					{
						if (pos + 4 > text.size()) { fail("unfinished \\u escape"); }
						unsigned code = (unsigned) strtoul(text.substr(pos, 4).c_str(), nullptr, 16);
						pos += 4;
						if (code > 0x7f) { fail("only ascii \\u escapes are read"); }
						out += (char) code;
					}
						break;
					default: out += e; // \" \\ \/
				}
			}
			else { out += c; }
		}
		if (pos >= text.size()) { fail("unterminated string"); }
		++pos;
		return out;
	}

	Json value (void)
	{
		skip();
		if (pos >= text.size()) { fail("unexpected end"); }
		Json out;
		char c = text[pos];
		if (c == '{')
		{
			++pos;
			out.kind = Json::OBJECT;
			if (take('}')) { return out; }
			do
			{
				skip();
				std::string key = quoted();
				if (!take(':')) { fail("expected ':'"); }
				out.object.emplace_back(key, value());
			}
			while (take(','));
			if (!take('}')) { fail("expected '}'"); }
		}
		else if (c == '[')
		{
			++pos;
			out.kind = Json::ARRAY;
			if (take(']')) { return out; }
			do { out.array.push_back(value()); }
			while (take(','));
			if (!take(']')) { fail("expected ']'"); }
		}
		else if (c == '"')
		{
			out.kind = Json::STRING;
			out.string = quoted();
		}
		else if (text.compare(pos, 4, "true") == 0) { out.kind = Json::BOOL; out.boolean = true; pos += 4; }
		else if (text.compare(pos, 5, "false") == 0) { out.kind = Json::BOOL; pos += 5; }
		else if (text.compare(pos, 4, "null") == 0) { pos += 4; }
		else
		{
			const char* begin = text.c_str() + pos;
			char* end = nullptr;
			out.number = strtod(begin, &end);
			if (end == begin) { fail("unexpected character"); }
			out.kind = Json::NUMBER;
			pos += (size_t) (end - begin);
		}
		return out;
	}
};

const Json& member (const Json& obj, const char* key, Json::Kind kind, const char* where)
{
	const Json* found = obj.find(key);
	if (nullptr == found || found->kind != kind)
	{
		global::fatalf("%s: missing or mistyped field `%s`", where, key);
	}
	return *found;
}

std::vector<std::pair<std::string,Json>> attr_fields (const Json& op)
{
	if (const Json* attrs = op.find("attrs"))
	{
		if (attrs->kind != Json::OBJECT) { global::fatal("`attrs` is not an object"); }
		return attrs->object;
	}
	return {};
}

// unknown names fail when the rules are read, not when they first match
void known_op (const std::string& opname)
{
	if (egen::BAD_OP == egen::get_op(opname)) { global::fatalf("unknown opcode `%s` in a conversion", opname.c_str()); }
}

Pattern parse_pattern (const Json& node)
{
	if (node.kind != Json::OBJECT || node.object.size() != 1)
	{
		global::fatal("a pattern node holds exactly one of `cst`, `leaf`, `op`, `symb`");
	}
	const std::string& key = node.object.front().first;
	const Json& val = node.object.front().second;
	Pattern out;
	if (key == "symb")
	{
		if (val.kind != Json::STRING) { global::fatal("`symb` is not a string"); }
		out.kind = Pattern::SYMBOL;
		out.symbol = val.string;
	}
	else if (key == "cst")
	{
		if (val.kind != Json::NUMBER) { global::fatal("`cst` is not a number"); }
		out.kind = Pattern::SCALAR;
		out.scalar = val.number;
	}
	else if (key == "leaf")
	{
		if (val.kind != Json::OBJECT) { global::fatal("`leaf` is not an object"); }
		out.kind = Pattern::LEAF;
		if (const Json* f = val.find("label")) { out.has_label = true; out.label = f->string; }
		if (const Json* f = val.find("dtype")) { out.has_dtype = true; out.dtype = f->string; }
		if (const Json* f = val.find("usage")) { out.has_usage = true; out.usage = f->string; }
		if (const Json* f = val.find("shape"))
		{
			for (auto& d : f->array) { out.shape.push_back((uint64_t) d.number); }
		}
	}
	else if (key == "op")
	{
		if (val.kind != Json::OBJECT) { global::fatal("`op` is not an object"); }
		out.kind = Pattern::OPERATOR;
		out.opname = member(val, "opname", Json::STRING, "pattern op").string;
		known_op(out.opname);
		if (const Json* f = val.find("capture")) { out.symbol = f->string; }
		if (const Json* f = val.find("args"))
		{
			if (f->kind != Json::ARRAY) { global::fatal("`args` is not an array"); }
			out.has_args = true;
			for (auto& arg : f->array) { out.args.push_back(parse_pattern(arg)); }
		}
		out.attrs = attr_fields(val);
	}
	else { global::fatalf("cannot look for unknown node `%s`", key.c_str()); }
	return out;
}

Target parse_target (const Json& node)
{
	if (node.kind != Json::OBJECT || node.object.size() != 1)
	{
		global::fatal("a target node holds exactly one of `cst`, `op`, `symb`");
	}
	const std::string& key = node.object.front().first;
	const Json& val = node.object.front().second;
	Target out;
	if (key == "symb")
	{
		if (val.kind != Json::STRING) { global::fatal("`symb` is not a string"); }
		out.kind = Target::SYMBOL;
		out.symbol = val.string;
	}
	else if (key == "cst")
	{
		if (val.kind != Json::OBJECT) { global::fatal("target `cst` is not an object"); }
		out.kind = Target::SCALAR;
		out.scalar = member(val, "value", Json::NUMBER, "target cst").number;
		out.symbol = member(val, "shape", Json::STRING, "target cst").string;
	}
	else if (key == "op")
	{
		if (val.kind != Json::OBJECT) { global::fatal("`op` is not an object"); }
		out.kind = Target::OPERATOR;
		out.opname = member(val, "opname", Json::STRING, "target op").string;
		known_op(out.opname);
		for (auto& arg : member(val, "args", Json::ARRAY, "target op").array)
		{
			out.args.push_back(parse_target(arg));
		}
		out.attrs = attr_fields(val);
	}
	else { global::fatalf("cannot parse unknown element `%s`", key.c_str()); }
	return out;
}

void pattern_symbols (std::vector<std::string>& out, const Pattern& p)
{
	if (!p.symbol.empty()) { out.push_back(p.symbol); }
	for (auto& arg : p.args) { pattern_symbols(out, arg); }
}

void check_symbols (const Target& t, const std::vector<std::string>& bound)
{
	if (t.kind != Target::OPERATOR &&
		std::find(bound.begin(), bound.end(), t.symbol) == bound.end())
	{
		global::fatalf("dest refers to symbol `%s` that a src does not bind", t.symbol.c_str());
	}
	for (auto& arg : t.args) { check_symbols(arg, bound); }
}

// query.proto Attribute: one of inum, dnum, iarr{values}, darr{values}, str
marsh::ObjptrT attr_object (const std::string& key, const Json& attr)
{
	if (attr.kind != Json::OBJECT || attr.object.size() != 1)
	{
		global::fatalf("attribute `%s` holds exactly one of inum, dnum, iarr, darr, str", key.c_str());
	}
	const std::string& kind = attr.object.front().first;
	const Json& val = attr.object.front().second;
	auto numbers = [&](void) -> const std::vector<Json>&
	{
		return member(val, "values", Json::ARRAY, "array attribute").array;
	};
	if (kind == "inum") { return marsh::ObjptrT(new marsh::Number<int64_t>((int64_t) val.number)); }
	if (kind == "dnum") { return marsh::ObjptrT(new marsh::Number<double>(val.number)); }
	if (kind == "str") { return marsh::ObjptrT(new marsh::String(val.string)); }
	if (kind == "iarr")
	{
		std::vector<int64_t> vals;
		for (auto& v : numbers()) { vals.push_back((int64_t) v.number); }
		return marsh::ObjptrT(new marsh::NumArray<int64_t>(vals));
	}
	if (kind == "darr")
	{
		std::vector<double> vals;
		for (auto& v : numbers()) { vals.push_back(v.number); }
		return marsh::ObjptrT(new marsh::NumArray<double>(vals));
	}
	global::fatalf("cannot parse attribute `%s` of kind `%s`", key.c_str(), kind.c_str());
}

/// First element of an immutable leaf whose elements are all equal
bool scalar_value (double& out, const teq::iLeaf& leaf)
{
	if (teq::IMMUTABLE != leaf.get_usage()) { return false; }
	const void* data = leaf.device().data();
	size_t n = leaf.shape().n_elems();
	bool same = false;
#define TCH_SCALAR(T) {\
	const T* vals = (const T*) data;\
	same = std::all_of(vals + 1, vals + n, [&](const T& e) { return e == vals[0]; });\
	out = (double) vals[0]; }
	TYPE_LOOKUP(TCH_SCALAR, leaf.get_meta().type_code())
#undef TCH_SCALAR
	return same;
}

const char* usage_name (teq::Usage usage)
{
	switch (usage)
	{
		case teq::IMMUTABLE: return "constant";
		case teq::VARUSAGE: return "variable";
		case teq::PLACEHOLDER: return "placeholder";
		default: return "";
	}
}

bool match_args (SymbMapT& symbols, const teq::TensptrsT& args,
	const std::vector<Pattern>& patterns, size_t at, std::vector<bool>& used)
{
	if (at == patterns.size()) { return true; }
	for (size_t i = 0; i < args.size(); ++i)
	{
		if (used[i]) { continue; }
		SymbMapT attempt = symbols;
		if (match(attempt, args[i], patterns[at]))
		{
			used[i] = true;
			if (match_args(attempt, args, patterns, at + 1, used))
			{
				symbols = attempt;
				return true;
			}
			used[i] = false;
		}
	}
	return false;
}

/// Every node under the roots, operands before the functors that read them
struct Index final : public teq::iOnceTraveler
{
	using ParentsT = std::vector<std::pair<teq::iFunctor*,size_t>>;

	explicit Index (const teq::TensptrsT& roots)
	{
		for (auto& root : roots) { enter(root); }
	}

	std::vector<teq::TensptrT> order;
	std::unordered_map<teq::iTensor*,ParentsT> parents;

private:
	void enter (const teq::TensptrT& node)
	{
		if (visited_.find(node.get()) != visited_.end()) { return; }
		owner_ = node;
		node->accept(*this);
	}

	void visit_leaf (teq::iLeaf&) override { order.push_back(owner_); }

	void visit_func (teq::iFunctor& func) override
	{
		teq::TensptrT self = owner_;
		auto args = func.get_args();
		for (size_t i = 0; i < args.size(); ++i)
		{
			parents[args[i].get()].emplace_back(&func, i);
			enter(args[i]);
		}
		order.push_back(self);
	}

	teq::TensptrT owner_;
};

/// Rewire every reader of a replaced node (internal/opt/graph.hpp:40-104)
size_t replace (teq::TensptrsT& roots, const Index& index,
	const std::unordered_map<teq::iTensor*,teq::TensptrT>& converts)
{
	size_t changed = 0;
	for (auto& conv : converts)
	{
		if (conv.first == conv.second.get()) { continue; }
		++changed;
		auto it = index.parents.find(conv.first);
		if (it != index.parents.end())
		{
			for (auto& parent : it->second)
			{
				// a reader that is itself replaced is rewired as well: it may
				// live on inside the replacement of another node
				parent.first->update_child(conv.second, parent.second);
			}
		}
		for (auto& root : roots)
		{
			if (root.get() == conv.first) { root = conv.second; }
		}
	}
	return changed;
}

bool foldable (const teq::iFunctor& func)
{
	switch ((egen::_GENERATED_OPCODE) func.get_opcode().code_)
	{
		// IDENTITY keeps its scheduling dependencies (tenncor/hone/src/
		// cstrules.cpp:31); draws and assignments have effects
		case egen::IDENTITY: case egen::RAND_UNIF: case egen::ASSIGN:
		case egen::ASSIGN_ADD: case egen::ASSIGN_SUB: case egen::ASSIGN_MUL:
		case egen::ASSIGN_DIV:
			return false;
		default:
			break;
	}
	auto args = func.get_args();
	return std::all_of(args.begin(), args.end(), [](const teq::TensptrT& arg)
	{
		auto leaf = dynamic_cast<const teq::iLeaf*>(arg.get());
		return nullptr != leaf && teq::IMMUTABLE == leaf->get_usage();
	});
}

/// tenncor/hone/cstrules.hpp:48-65: evaluate, then wrap the values in a constant
teq::TensptrT evaluated_constant (const teq::TensptrT& root)
{
	eteq::run(teq::TensptrsT{root});
	const void* data = static_cast<const teq::iTensor&>(*root).device().data();
	if (nullptr == data) { global::fatalf("%s holds no value after evaluation", root->to_string().c_str()); }
	teq::TensptrT out;
#define TCH_CST(T) out = eteq::make_constant_tensor<T>((const T*) data, root->shape());
	TYPE_LOOKUP(TCH_CST, root->get_meta().type_code())
#undef TCH_CST
	return out;
}

size_t fold_constants (teq::TensptrsT& roots)
{
	Index index(roots);
	std::unordered_map<teq::iTensor*,teq::TensptrT> converts;
	for (auto& node : index.order)
	{
		auto func = dynamic_cast<teq::iFunctor*>(node.get());
		if (nullptr == func) { continue; }
		// operands folded earlier in this pass
		auto args = func->get_args();
		for (size_t i = 0; i < args.size(); ++i)
		{
			auto it = converts.find(args[i].get());
			if (it != converts.end()) { func->update_child(it->second, i); }
		}
		if (foldable(*func)) { converts.emplace(node.get(), evaluated_constant(node)); }
	}
	for (auto& root : roots)
	{
		auto it = converts.find(root.get());
		if (it != converts.end()) { root = it->second; }
	}
	return converts.size();
}

}

Json parse_json (const std::string& text)
{
	JsonReader reader{text};
	Json out = reader.value();
	reader.skip();
	if (reader.pos != text.size()) { reader.fail("trailing characters"); }
	return out;
}

RulesT parse_rules (const std::string& json_text)
{
	Json root = parse_json(json_text);
	if (root.kind != Json::OBJECT) { global::fatal("failed to parse json optimization"); }
	RulesT rules;
	const Json* convs = root.find("conversions");
	if (nullptr == convs) { return rules; }
	if (convs->kind != Json::ARRAY) { global::fatal("`conversions` is not an array"); }
	for (auto& conv : convs->array)
	{
		if (conv.kind != Json::OBJECT) { global::fatal("a conversion is not an object"); }
		Conversion rule;
		for (auto& src : member(conv, "srcs", Json::ARRAY, "conversion").array)
		{
			rule.srcs.push_back(parse_pattern(src));
		}
		rule.dest = parse_target(member(conv, "dest", Json::OBJECT, "conversion"));
		// a dest symbol must be bound by every src
		for (auto& src : rule.srcs)
		{
			std::vector<std::string> bound;
			pattern_symbols(bound, src);
			check_symbols(rule.dest, bound);
		}
		rules.push_back(std::move(rule));
	}
	return rules;
}

// internal/query/querier.hpp:27-53 (leaves), :186-200 and :289-303 (functors)
bool match (SymbMapT& symbols, const teq::TensptrT& node, const Pattern& pattern)
{
	auto bind = [&](const std::string& symbol)
	{
		auto it = symbols.find(symbol);
		if (it != symbols.end()) { return it->second == node; }
		symbols.emplace(symbol, node);
		return true;
	};
	switch (pattern.kind)
	{
		case Pattern::SYMBOL:
			return bind(pattern.symbol);
		case Pattern::SCALAR:
		{
			auto leaf = dynamic_cast<const teq::iLeaf*>(node.get());
			double value;
			return nullptr != leaf && scalar_value(value, *leaf) && value == pattern.scalar;
		}
		case Pattern::LEAF:
		{
			auto leaf = dynamic_cast<const teq::iLeaf*>(node.get());
			if (nullptr == leaf) { return false; }
			if (pattern.has_label && pattern.label != leaf->to_string()) { return false; }
			if (pattern.has_dtype && pattern.dtype != leaf->get_meta().type_label()) { return false; }
			if (pattern.has_usage && pattern.usage != usage_name(leaf->get_usage())) { return false; }
			if (!pattern.shape.empty())
			{
				teq::DimsT dims(pattern.shape.begin(), pattern.shape.end());
				if (!teq::Shape(dims).compatible_after(leaf->shape(), 0)) { return false; }
			}
			return true;
		}
		case Pattern::OPERATOR:
		{
			auto func = dynamic_cast<const teq::iFunctor*>(node.get());
			if (nullptr == func || func->get_opcode().name_ != pattern.opname) { return false; }
			for (auto& attr : pattern.attrs)
			{
				const marsh::iObject* have = func->get_attr(attr.first);
				if (nullptr == have) { return false; }
				// an empty value matches on the key alone
				if (attr.second.kind == Json::OBJECT && !attr.second.object.empty() &&
					!have->equals(*attr_object(attr.first, attr.second))) { return false; }
			}
			SymbMapT attempt = symbols;
			if (pattern.has_args)
			{
				auto args = func->get_args();
				// the reference accepts functors with more operands than the
				// pattern lists (querier.hpp:195-196), which lets ADD(X, 0) -> X
				// drop operands of a longer sum; here the counts must agree
				if (args.size() != pattern.args.size()) { return false; }
				if (egen::is_commutative((egen::_GENERATED_OPCODE) func->get_opcode().code_))
				{
					std::vector<bool> used(args.size(), false);
					if (!match_args(attempt, args, pattern.args, 0, used)) { return false; }
				}
				else
				{
					for (size_t i = 0; i < args.size(); ++i)
					{
						if (!match(attempt, args[i], pattern.args[i])) { return false; }
					}
				}
			}
			if (!pattern.symbol.empty())
			{
				auto it = attempt.find(pattern.symbol);
				if (it != attempt.end() && it->second != node) { return false; }
				attempt.emplace(pattern.symbol, node);
			}
			symbols = attempt;
			return true;
		}
	}
	return false;
}

// tenncor/hone/target.hpp:13-92
teq::TensptrT build (const Target& target, const SymbMapT& symbols)
{
	switch (target.kind)
	{
		case Target::SYMBOL:
			return symbols.at(target.symbol);
		case Target::SCALAR:
		{
			auto& like = symbols.at(target.symbol);
			return eteq::make_constant_scalar<double>(target.scalar, like->shape(),
				(egen::_GENERATED_DTYPE) like->get_meta().type_code());
		}
		case Target::OPERATOR:
		{
			teq::TensptrsT args;
			for (auto& arg : target.args) { args.push_back(build(arg, symbols)); }
			marsh::Maps attrs;
			for (auto& attr : target.attrs) { attrs.add_attr(attr.first, attr_object(attr.first, attr.second)); }
			return eteq::make_funcattr(egen::get_op(target.opname), args, attrs);
		}
	}
	return nullptr;
}

teq::TensptrsT merge_dups (teq::TensptrsT roots, Stats* stats)
{
	Index index(roots);
	// equal nodes get equal class numbers; a class is described by a string
	// over the class numbers of its operands
	std::unordered_map<std::string,size_t> classes;
	std::unordered_map<teq::iTensor*,size_t> class_of;
	std::vector<teq::TensptrT> first_of;
	std::unordered_map<teq::iTensor*,teq::TensptrT> converts;
	auto classify = [&](const teq::TensptrT& node, const std::string& label, bool unique)
	{
		size_t id = first_of.size();
		if (!unique)
		{
			auto it = classes.find(label);
			if (it != classes.end())
			{
				class_of.emplace(node.get(), it->second);
				converts.emplace(node.get(), first_of[it->second]);
				return;
			}
			classes.emplace(label, id);
		}
		class_of.emplace(node.get(), id);
		first_of.push_back(node);
	};
	for (auto& node : index.order)
	{
		if (auto leaf = dynamic_cast<const teq::iLeaf*>(node.get()))
		{
			if (teq::IMMUTABLE != leaf->get_usage())
			{
				classify(node, "", true);
				continue;
			}
			auto& meta = leaf->get_meta();
			auto bytes = (const char*) leaf->device().data();
			std::string label = "L" + leaf->shape().to_string() + "|" + meta.type_label() + "|" +
				std::string(bytes, bytes + leaf->shape().n_elems() * meta.type_size());
			classify(node, label, false);
			continue;
		}
		auto func = dynamic_cast<const teq::iFunctor*>(node.get());
		auto opcode = (egen::_GENERATED_OPCODE) func->get_opcode().code_;
		std::vector<size_t> operands;
		for (auto& arg : func->get_args()) { operands.push_back(class_of.at(arg.get())); }
		if (egen::is_commutative(opcode)) { std::sort(operands.begin(), operands.end()); }
		std::string label = "F" + func->shape().to_string() + "|" + func->get_opcode().name_ + "|" +
			func->get_meta().type_label() + "\\";
		for (auto& key : func->ls_attrs())
		{
			const marsh::iObject* value = func->get_attr(key);
			if (nullptr == value) { continue; }
			label += key + ":";
			if (auto ref = dynamic_cast<const teq::TensorObj*>(value))
			{
				// a tensor-valued attribute only passes its shape on (EXTEND's `tensor`)
				label += ref->get_tensor()->shape().to_string();
			}
			else { label += value->to_string(); }
			label += ";";
		}
		label += "\\";
		for (size_t operand : operands) { label += std::to_string(operand) + ","; }
		// two draws, two casts of a changing value or two assignments are not one:
		// the reference merges them all the same (tenncor/hone/duplicates.hpp:47-83)
		bool unique = !egen::is_idempotent(opcode) || egen::ASSIGN == opcode;
		classify(node, label, unique && egen::CAST != opcode);
	}
	size_t merged = replace(roots, index, converts);
	if (stats) { stats->merged += merged; }
	return roots;
}

// tenncor/hone/src/optimize.cpp:13-36, internal/opt/src/apply.cpp:9-34
teq::TensptrsT optimize (teq::TensptrsT roots, const RulesT& rules, bool fold, Stats* stats)
{
	Stats local;
	roots = merge_dups(roots, &local);
	const size_t round_limit = 50;
	bool converted = true;
	for (size_t round = 0; converted && round < round_limit; ++round)
	{
		converted = false;
		++local.rounds;
		if (fold)
		{
			size_t folded = fold_constants(roots);
			local.folded += folded;
			converted = folded > 0;
		}
		for (auto& rule : rules)
		{
			Index index(roots);
			std::unordered_map<teq::iTensor*,teq::TensptrT> converts;
			for (auto& node : index.order)
			{
				for (auto& src : rule.srcs)
				{
					SymbMapT symbols;
					if (match(symbols, node, src))
					{
						teq::TensptrT dest = build(rule.dest, symbols);
						if (dest.get() != node.get()) { converts.emplace(node.get(), dest); }
						break;
					}
				}
			}
			size_t changed = replace(roots, index, converts);
			local.converted += changed;
			converted = converted || changed > 0;
		}
	}
	if (stats) { *stats = local; }
	return roots;
}

}
