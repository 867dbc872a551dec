// Attribute packers: the nine keys and encodings of tenncor's
// internal/eigen/packattr.hpp:60-363 (every numeric list is a
// NumArray<int64_t>, pairs are flattened, `rank` is a Number<int64_t>, `dtype`
// is the type's name, `tensor` holds the node itself) and unpack_extend of
// internal/eigen/src/packattr.cpp:28-60.
#ifndef TCH_PACKATTR_HPP
#define TCH_PACKATTR_HPP

#include <optional>
#include <set>

#include "egen.hpp"
#include "teq.hpp"

namespace eigen
{

const std::string no_argument_err = "cannot operate without inputs";

using DTypesT = std::vector<egen::_GENERATED_DTYPE>;

template <typename T>
using PairVecT = std::vector<std::pair<T,T>>;

using OptDimsT = std::optional<teq::DimsT>;

template <typename T>
std::string to_string (const PairVecT<T>& pairs)
{
	std::string out = "[";
	for (size_t i = 0; i < pairs.size(); ++i)
	{
		// as integers, first:second
		out += (i ? "\\" : "") + std::to_string((int) pairs[i].first) + ":" + std::to_string((int) pairs[i].second);
	}
	return out + "]";
}

template <typename IT>
std::string range_to_string (IT begin, IT end)
{
	std::string out = "[";
	for (IT it = begin; it != end; ++it)
	{
		out += (it == begin ? "" : "\\") + std::to_string((long long) *it);
	}
	return out + "]";
}

/// A type without an attribute of its own: no key, and packing is an error
template <typename T>
struct Packer final
{
	std::string get_key (void) const { return ""; }
	void pack (marsh::iAttributed&, T) const { global::fatal("unknown attribute"); }
	void unpack (T&, const marsh::iAttributed&) const { global::fatal("unknown attribute"); }
};

template <typename T>
const marsh::iObject* get_attr (const Packer<T>& packer, const marsh::iAttributed& attrib)
{
	auto key = packer.get_key();
	auto attr = attrib.get_attr(key);
	if (nullptr == attr)
	{
		global::fatalf("cannot find `%s` attribute", key.c_str());
	}
	return attr;
}

inline const std::vector<int64_t>& int_contents (const marsh::iObject* attr)
{
	auto arr = dynamic_cast<const marsh::NumArray<int64_t>*>(attr);
	if (nullptr == arr) { global::fatal("attribute is not an integer array"); }
	return arr->contents_;
}

template <typename T>
PairVecT<T> decode_pair (const std::vector<int64_t>& encoding)
{
	if (1 == encoding.size() % 2)
	{
		global::fatalf("cannot decode odd vector %s into vec of pairs",
			range_to_string(encoding.begin(), encoding.end()).c_str());
	}
	PairVecT<T> out;
	for (size_t i = 0; i + 1 < encoding.size(); i += 2)
	{
		out.push_back({(T) encoding[i], (T) encoding[i + 1]});
	}
	return out;
}

template <typename T>
std::vector<int64_t> encode_pair (const PairVecT<T>& pairs)
{
	std::vector<int64_t> out;
	for (auto& p : pairs)
	{
		out.push_back(p.first);
		out.push_back(p.second);
	}
	return out;
}

template <>
struct Packer<egen::_GENERATED_DTYPE>
{
	std::string get_key (void) const { return "dtype"; }
	void pack (marsh::iAttributed& attrib, egen::_GENERATED_DTYPE dtype) const
	{
		attrib.add_attr(get_key(), std::make_unique<marsh::String>(egen::name_type(dtype)));
	}
	void unpack (egen::_GENERATED_DTYPE& out, const marsh::iAttributed& attrib) const
	{
		out = egen::get_type(get_attr(*this, attrib)->to_string());
	}
};

template <>
struct Packer<PairVecT<teq::DimT>>
{
	std::string get_key (void) const { return "dimension_pairs"; }
	void pack (marsh::iAttributed& attrib, PairVecT<teq::DimT> dims) const
	{
		attrib.add_attr(get_key(), std::make_unique<marsh::NumArray<int64_t>>(encode_pair(dims)));
	}
	void unpack (PairVecT<teq::DimT>& out, const marsh::iAttributed& attrib) const
	{
		out = decode_pair<teq::DimT>(int_contents(get_attr(*this, attrib)));
	}
};

template <>
struct Packer<PairVecT<teq::RankT>>
{
	std::string get_key (void) const { return "rank_pairs"; }
	void pack (marsh::iAttributed& attrib, PairVecT<teq::RankT> ranks) const
	{
		for (auto& pr : ranks)
		{
			if (pr.first >= teq::rank_cap || pr.second >= teq::rank_cap)
			{
				global::fatalf("cannot reference ranks beyond rank_cap %d: %s", (int) teq::rank_cap, to_string(ranks).c_str());
			}
		}
		attrib.add_attr(get_key(), std::make_unique<marsh::NumArray<int64_t>>(encode_pair(ranks)));
	}
	void unpack (PairVecT<teq::RankT>& out, const marsh::iAttributed& attrib) const
	{
		out = decode_pair<teq::RankT>(int_contents(get_attr(*this, attrib)));
	}
};

template <>
struct Packer<teq::DimsT>
{
	std::string get_key (void) const { return "dimensions"; }
	void pack (marsh::iAttributed& attrib, teq::DimsT dims) const
	{
		attrib.add_attr(get_key(), std::make_unique<marsh::NumArray<int64_t>>(
			std::vector<int64_t>(dims.begin(), dims.end())));
	}
	void unpack (teq::DimsT& out, const marsh::iAttributed& attrib) const
	{
		auto& enc = int_contents(get_attr(*this, attrib));
		out = teq::DimsT(enc.begin(), enc.end());
	}
};

template <>
struct Packer<teq::RanksT>
{
	std::string get_key (void) const { return "ranks"; }
	void pack (marsh::iAttributed& attrib, teq::RanksT ranks) const
	{
		for (teq::RankT rank : ranks)
		{
			if (rank >= teq::rank_cap)
			{
				global::fatalf("cannot reference ranks beyond rank_cap %d: %s", (int) teq::rank_cap,
					range_to_string(ranks.begin(), ranks.end()).c_str());
			}
		}
		attrib.add_attr(get_key(), std::make_unique<marsh::NumArray<int64_t>>(
			std::vector<int64_t>(ranks.begin(), ranks.end())));
	}
	void unpack (teq::RanksT& out, const marsh::iAttributed& attrib) const
	{
		auto& enc = int_contents(get_attr(*this, attrib));
		out = teq::RanksT(enc.begin(), enc.end());
	}
};

template <>
struct Packer<std::set<teq::RankT>>
{
	std::string get_key (void) const { return "rank_set"; }
	void pack (marsh::iAttributed& attrib, std::set<teq::RankT> ranks) const
	{
		if (ranks.size() > teq::rank_cap)
		{
			global::fatalf("cannot specify %d ranks when %d (rank_cap) are available", (int) ranks.size(), (int) teq::rank_cap);
		}
		// rank_cap itself passes: it stands for "every dim" (internal/eigen/packattr.hpp:262-270)
		if (false == ranks.empty() && *ranks.rbegin() > teq::rank_cap)
		{
			global::fatalf("cannot reference ranks beyond rank_cap %d: %s", (int) teq::rank_cap,
				range_to_string(ranks.begin(), ranks.end()).c_str());
		}
		attrib.add_attr(get_key(), std::make_unique<marsh::NumArray<int64_t>>(
			std::vector<int64_t>(ranks.begin(), ranks.end())));
	}
	void unpack (std::set<teq::RankT>& out, const marsh::iAttributed& attrib) const
	{
		auto& enc = int_contents(get_attr(*this, attrib));
		out = std::set<teq::RankT>(enc.begin(), enc.end());
	}
};

template <>
struct Packer<teq::RankT>
{
	std::string get_key (void) const { return "rank"; }
	void pack (marsh::iAttributed& attrib, teq::RankT rank) const
	{
		attrib.add_attr(get_key(), std::make_unique<marsh::Number<int64_t>>(rank));
	}
	void unpack (teq::RankT& out, const marsh::iAttributed& attrib) const
	{
		auto num = dynamic_cast<const marsh::iNumber*>(get_attr(*this, attrib));
		if (nullptr == num) { global::fatal("`rank` attribute is not a number"); }
		out = (teq::RankT) num->to_int64();
	}
};

template <>
struct Packer<teq::Shape>
{
	std::string get_key (void) const { return "shape"; }
	void pack (marsh::iAttributed& attrib, teq::Shape shape) const
	{
		attrib.add_attr(get_key(), std::make_unique<marsh::NumArray<int64_t>>(
			std::vector<int64_t>(shape.begin(), shape.end())));
	}
	void unpack (teq::Shape& out, const marsh::iAttributed& attrib) const
	{
		auto& enc = int_contents(get_attr(*this, attrib));
		out = teq::Shape(teq::DimsT(enc.begin(), enc.end()));
	}
};

template <>
struct Packer<teq::TensptrT>
{
	std::string get_key (void) const { return "tensor"; }
	void pack (marsh::iAttributed& attrib, teq::TensptrT tens) const
	{
		attrib.add_attr(get_key(), std::make_unique<teq::TensorObj>(tens));
	}
	void unpack (teq::TensptrT& out, const marsh::iAttributed& attrib) const
	{
		auto obj = dynamic_cast<const teq::TensorObj*>(get_attr(*this, attrib));
		if (nullptr == obj) { global::fatal("`tensor` attribute does not hold a tensor"); }
		out = obj->get_tensor();
	}
};

inline void pack_attr (marsh::iAttributed&) {}

template <typename T, typename ...ARGS>
void pack_attr (marsh::iAttributed& attrib, T attr_val, ARGS... args)
{
	Packer<T>().pack(attrib, attr_val);
	pack_attr(attrib, args...);
}

/// Broadcast factors of an EXTEND: the `dimensions` list, or derived from the
/// `tensor` to match (factor = target dim where it differs, else 1)
inline OptDimsT unpack_extend (teq::Shape inshape, const marsh::iAttributed& attrib)
{
	teq::DimsT bcast;
	Packer<teq::DimsT> dimpacker;
	Packer<teq::TensptrT> tenspacker;
	if (nullptr != attrib.get_attr(dimpacker.get_key()))
	{
		dimpacker.unpack(bcast, attrib);
	}
	else if (nullptr != attrib.get_attr(tenspacker.get_key()))
	{
		teq::TensptrT tens;
		tenspacker.unpack(tens, attrib);
		auto target = tens->shape();
		for (teq::RankT i = 0; i < teq::rank_cap; ++i)
		{
			teq::DimT tdim = target.at(i);
			bcast.push_back(inshape.at(i) != tdim ? tdim : 1);
		}
	}
	else
	{
		return OptDimsT();
	}
	return bcast;
}

}

#endif // TCH_PACKATTR_HPP
