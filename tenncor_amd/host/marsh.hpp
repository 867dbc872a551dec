// Attribute object model: the subset of tenncor's `marsh` objects
// (internal/marsh/objs.hpp:10-432) that operator attributes use -- String,
// Number<T>, NumArray<T>, Maps -- behind the same iObject / iAttributed
// interfaces, so that attribute keys and encodings stay those of
// internal/eigen/packattr.hpp:60-363.
#ifndef TCH_MARSH_HPP
#define TCH_MARSH_HPP

#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <typeinfo>
#include <vector>

namespace marsh
{

struct iObject
{
	virtual ~iObject (void) = default;
	virtual size_t class_code (void) const = 0;
	virtual std::string to_string (void) const = 0;
	virtual bool equals (const iObject& other) const = 0;
	virtual iObject* clone (void) const = 0;
};

using ObjptrT = std::unique_ptr<iObject>;

struct String final : public iObject
{
	String (const std::string& val) : val_(val) {}
	size_t class_code (void) const override { return typeid(String).hash_code(); }
	std::string to_string (void) const override { return val_; }
	bool equals (const iObject& other) const override
	{
		return other.class_code() == class_code() &&
			static_cast<const String&>(other).val_ == val_;
	}
	iObject* clone (void) const override { return new String(val_); }
	std::string val_;
};

struct iNumber : public iObject
{
	virtual double to_float64 (void) const = 0;
	virtual int64_t to_int64 (void) const = 0;
};

template <typename T>
struct Number final : public iNumber
{
	Number (T val) : val_(val) {}
	size_t class_code (void) const override { return typeid(Number<T>).hash_code(); }
	std::string to_string (void) const override
	{
		std::ostringstream s;
		s << val_;
		return s.str();
	}
	bool equals (const iObject& other) const override
	{
		return other.class_code() == class_code() &&
			static_cast<const Number<T>&>(other).val_ == val_;
	}
	iObject* clone (void) const override { return new Number<T>(val_); }
	double to_float64 (void) const override { return (double) val_; }
	int64_t to_int64 (void) const override { return (int64_t) val_; }
	T val_;
};

template <typename T>
struct NumArray final : public iObject
{
	NumArray (void) = default;
	NumArray (const std::vector<T>& contents) : contents_(contents) {}
	size_t class_code (void) const override { return typeid(NumArray<T>).hash_code(); }
	std::string to_string (void) const override
	{
		std::ostringstream s;
		s << "[";
		for (size_t i = 0; i < contents_.size(); ++i)
		{
			if (i > 0) { s << "\\"; }
			s << contents_[i];
		}
		s << "]";
		return s.str();
	}
	bool equals (const iObject& other) const override
	{
		return other.class_code() == class_code() &&
			static_cast<const NumArray<T>&>(other).contents_ == contents_;
	}
	iObject* clone (void) const override { return new NumArray<T>(contents_); }
	size_t size (void) const { return contents_.size(); }
	std::vector<T> contents_;
};

struct iAttributed
{
	virtual ~iAttributed (void) = default;
	virtual std::vector<std::string> ls_attrs (void) const = 0;
	virtual const iObject* get_attr (const std::string& attr_key) const = 0;
	virtual iObject* get_attr (const std::string& attr_key) = 0;
	virtual void add_attr (const std::string& attr_key, ObjptrT&& attr_val) = 0;
	virtual void rm_attr (const std::string& attr_key) = 0;
	virtual size_t size (void) const = 0;
};

struct Maps final : public iObject, public iAttributed
{
	Maps (void) = default;
	Maps (Maps&&) = default;
	Maps& operator = (Maps&&) = default;
	size_t class_code (void) const override { return typeid(Maps).hash_code(); }
	std::string to_string (void) const override
	{
		std::string out = "{";
		bool first = true;
		for (auto& kv : contents_)
		{
			out += (first ? "" : ",") + kv.first + ":" + kv.second->to_string();
			first = false;
		}
		return out + "}";
	}
	bool equals (const iObject& other) const override
	{
		if (other.class_code() != class_code()) { return false; }
		auto& o = static_cast<const Maps&>(other);
		if (o.contents_.size() != contents_.size()) { return false; }
		for (auto& kv : contents_)
		{
			auto it = o.contents_.find(kv.first);
			if (it == o.contents_.end() || !it->second->equals(*kv.second)) { return false; }
		}
		return true;
	}
	Maps* clone (void) const override
	{
		Maps* out = new Maps();
		for (auto& kv : contents_) { out->contents_.emplace(kv.first, ObjptrT(kv.second->clone())); }
		return out;
	}
	std::vector<std::string> ls_attrs (void) const override
	{
		std::vector<std::string> keys;
		for (auto& kv : contents_) { keys.push_back(kv.first); }
		return keys;
	}
	const iObject* get_attr (const std::string& attr_key) const override
	{
		auto it = contents_.find(attr_key);
		return it == contents_.end() ? nullptr : it->second.get();
	}
	iObject* get_attr (const std::string& attr_key) override
	{
		auto it = contents_.find(attr_key);
		return it == contents_.end() ? nullptr : it->second.get();
	}
	void add_attr (const std::string& attr_key, ObjptrT&& attr_val) override
	{
		contents_[attr_key] = std::move(attr_val);
	}
	void rm_attr (const std::string& attr_key) override { contents_.erase(attr_key); }
	size_t size (void) const override { return contents_.size(); }
	std::map<std::string,ObjptrT> contents_;
};

}

#endif // TCH_MARSH_HPP
