// Graph interfaces, shape, evaluator and reverse-mode derivation: the `teq`
// layer the GPU backend plugs into.  Names, signatures and semantics follow
// tenncor's internal/teq (shape.hpp, itensor.hpp, ileaf.hpp, ifunctor.hpp,
// itraveler.hpp, traveler.hpp, once.hpp, ievaluator.hpp, evaluator.hpp,
// derive.hpp, src/derive.cpp) so that code written against those headers
// compiles against this one.
#ifndef TCH_TEQ_HPP
#define TCH_TEQ_HPP

#include <algorithm>
#include <array>
#include <functional>
#include <memory>
#include <numeric>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "global.hpp"
#include "marsh.hpp"

namespace teq
{

// ---- shape (internal/teq/shape.hpp) ----------------------------------------

using RankT = uint8_t;
// the width of a dimension is a build option, as in internal/teq/shape.hpp:27-33
#if !defined(SDIM_BYTES) || SDIM_BYTES <= 2
using DimT = uint16_t;
#elif SDIM_BYTES <= 4
using DimT = uint32_t;
#else
using DimT = uint64_t;
#endif
using RanksT = std::vector<RankT>;
using DimsT = std::vector<DimT>;
using NElemT = uint64_t;
const RankT rank_cap = 8;
using ShapeT = std::array<DimT,rank_cap>;

/// Up to rank_cap dims, dim 0 is the fastest-varying one; missing dims are 1
struct Shape final
{
	Shape (void) { dims_.fill(1); }

	Shape (const std::vector<DimT>& dims) { vector_assign(dims); }

	Shape& operator = (const std::vector<DimT>& dims)
	{
		vector_assign(dims);
		return *this;
	}

	/// "[d0\d1\...\d7]" as printed by the reference's graph dumps
	std::string to_string (void) const
	{
		std::string out = "[";
		for (RankT i = 0; i < rank_cap; ++i)
		{
			out += (i ? "\\" : "") + std::to_string(dims_[i]);
		}
		return out + "]";
	}

	DimT at (RankT idx) const
	{
		if (rank_cap <= idx)
		{
			global::throw_errf("cannot access out of bounds index %d", (int) idx);
		}
		return dims_[idx];
	}

	NElemT n_elems (void) const
	{
		return std::accumulate(dims_.begin(), dims_.end(), (NElemT) 1, std::multiplies<NElemT>());
	}

	/// this[0:idx) equals other[0:idx); a 0 dim matches anything
	bool compatible_before (const Shape& other, RankT idx) const
	{
		return std::equal(dims_.begin(), dims_.begin() + std::min(idx, rank_cap), other.dims_.begin(), wild_equal);
	}

	/// this[idx:rank_cap) equals other[idx:rank_cap)
	bool compatible_after (const Shape& other, RankT idx) const
	{
		return idx < rank_cap && std::equal(dims_.begin() + idx, dims_.end(), other.dims_.begin() + idx, wild_equal);
	}

	ShapeT::iterator begin (void) { return dims_.begin(); }
	ShapeT::iterator end (void) { return dims_.end(); }
	ShapeT::const_iterator begin (void) const { return dims_.begin(); }
	ShapeT::const_iterator end (void) const { return dims_.end(); }

private:
	static bool wild_equal (DimT a, DimT b) { return a == 0 || b == 0 || a == b; }

	void vector_assign (const std::vector<DimT>& dims)
	{
		size_t n = std::min(dims.size(), (size_t) rank_cap);
		std::copy(dims.begin(), dims.begin() + n, dims_.begin());
		std::fill(dims_.begin() + n, dims_.end(), 1);
	}

	ShapeT dims_;
};

using ShapesT = std::vector<Shape>;

/// Dims with the trailing ones removed (internal/teq/src/shape.cpp:8-16)
inline DimsT narrow_shape (const Shape& sign)
{
	auto it = sign.begin(), et = sign.end();
	while (it != et && *(et - 1) <= 1) { --et; }
	return DimsT(it, et);
}

// ---- scope guard (internal/teq/once.hpp) -----------------------------------

/// A value plus a callback fired exactly once, when the last holder lets go
template <typename T>
struct Once final
{
	using GuardOpF = std::function<void(void)>;

	Once (T obj, GuardOpF killsig = GuardOpF()) : term_(killsig), obj_(obj) {}

	template <typename OT>
	Once (T altobj, Once<OT>&& other) : term_(other.release()), obj_(altobj) {}

	Once (const Once<T>&) = delete;
	Once<T>& operator = (const Once<T>&) = delete;

	Once (Once<T>&& other) : term_(std::move(other.term_)), obj_(other.obj_) { other.term_ = nullptr; }

	Once<T>& operator = (Once<T>&& other)
	{
		if (this != &other)
		{
			fire();
			term_ = std::move(other.term_);
			other.term_ = nullptr;
			obj_ = other.obj_;
		}
		return *this;
	}

	~Once (void) { fire(); }

	operator T (void) { return obj_; }

	T get (void) const { return obj_; }

	GuardOpF release (void)
	{
		GuardOpF out = std::move(term_);
		term_ = nullptr;
		return out;
	}

private:
	void fire (void)
	{
		if (term_)
		{
			GuardOpF f = std::move(term_);
			term_ = nullptr;
			f();
		}
	}

	GuardOpF term_;
	T obj_;
};

// ---- tensors (internal/teq/itensor.hpp, ileaf.hpp, ifunctor.hpp) -----------

struct iLeaf;
struct iFunctor;

struct iTraveler
{
	virtual ~iTraveler (void) = default;
	virtual void visit (iLeaf& leaf) = 0;
	virtual void visit (iFunctor& func) = 0;
};

struct iDeviceRef
{
	virtual ~iDeviceRef (void) = default;
	/// Host-dereferenceable pointer, or nullptr when never computed / expired
	virtual void* data (void) = 0;
	virtual const void* data (void) const = 0;
	/// data() plus a guard whose destruction consumes one unit of lifetime
	virtual Once<void*> odata (void) = 0;
	virtual Once<const void*> odata (void) const = 0;
};

struct iMetadata
{
	virtual ~iMetadata (void) = default;
	virtual size_t type_code (void) const = 0;
	virtual std::string type_label (void) const = 0;
	virtual size_t type_size (void) const = 0;
	virtual size_t state_version (void) const = 0;
};

struct iTensor
{
	virtual ~iTensor (void) = default;
	virtual std::string to_string (void) const = 0;
	virtual void accept (iTraveler& visiter) = 0;
	virtual iDeviceRef& device (void) = 0;
	virtual const iDeviceRef& device (void) const = 0;
	virtual const iMetadata& get_meta (void) const = 0;
	virtual Shape shape (void) const = 0;
};

using TensptrT = std::shared_ptr<iTensor>;
using TensT = std::vector<iTensor*>;
using CTensT = std::vector<const iTensor*>;
using TensptrsT = std::vector<TensptrT>;
using TensSetT = std::unordered_set<iTensor*>;
using TensptrSetT = std::unordered_set<TensptrT>;
template <typename V>
using TensMapT = std::unordered_map<iTensor*,V>;

template <typename TS>
void multi_visit (iTraveler& traveler, const TS& tensors)
{
	for (auto tensor : tensors)
	{
		if (nullptr != tensor) { tensor->accept(traveler); }
	}
}

enum Usage { UNKNOWN_USAGE = 0, IMMUTABLE, VARUSAGE, PLACEHOLDER };

struct iLeaf : public iTensor
{
	virtual ~iLeaf (void) = default;
	void accept (iTraveler& visiter) override { visiter.visit(*this); }
	virtual Usage get_usage (void) const = 0;
};

struct Opcode final
{
	std::string name_;
	size_t code_;
};

struct iFunctor : public iTensor, public marsh::iAttributed
{
	virtual ~iFunctor (void) = default;
	void accept (iTraveler& visiter) override { visiter.visit(*this); }
	virtual Opcode get_opcode (void) const = 0;
	virtual TensptrsT get_args (void) const = 0;
	virtual void update_child (TensptrT arg, size_t index) = 0;
};

using FuncptrT = std::shared_ptr<iFunctor>;

/// Attribute value that keeps a tensor alive (the `tensor` key of EXTEND,
/// internal/eigen/packattr.hpp:331-352)
struct TensorObj final : public marsh::iObject
{
	TensorObj (TensptrT tens) : tens_(tens) {}
	size_t class_code (void) const override { return typeid(TensorObj).hash_code(); }
	std::string to_string (void) const override { return tens_->to_string(); }
	bool equals (const marsh::iObject& other) const override
	{
		return other.class_code() == class_code() &&
			static_cast<const TensorObj&>(other).tens_ == tens_;
	}
	marsh::iObject* clone (void) const override { return new TensorObj(tens_); }
	TensptrT get_tensor (void) const { return tens_; }
	TensptrT tens_;
};

// ---- travelers (internal/teq/traveler.hpp) ---------------------------------

/// Visits every node once
struct iOnceTraveler : public iTraveler
{
	virtual ~iOnceTraveler (void) = default;

	void visit (iLeaf& leaf) override
	{
		if (visited_.emplace(&leaf).second) { visit_leaf(leaf); }
	}

	void visit (iFunctor& func) override
	{
		if (visited_.emplace(&func).second) { visit_func(func); }
	}

	virtual void clear (void) { visited_.clear(); }

	TensSetT visited_;

private:
	virtual void visit_leaf (iLeaf& leaf) = 0;
	virtual void visit_func (iFunctor& func) = 0;
};

// ---- evaluation (internal/teq/ievaluator.hpp, evaluator.hpp) ---------------

struct iDevice
{
	virtual ~iDevice (void) = default;
	/// Compute `tens` (an Observable functor); cache_ttl is 1 for targets
	virtual void calc (iTensor& tens, size_t cache_ttl) = 0;
};

struct iEvaluator
{
	virtual ~iEvaluator (void) = default;
	virtual void evaluate (iDevice& device, const TensSetT& targets, const TensSetT& ignored = {}) = 0;
};

/// Post-order walk: children first, every functor once, ignored nodes skipped
struct TravEvaluator final : public iOnceTraveler
{
	TravEvaluator (iDevice& device, const TensSetT& targets, const TensSetT& ignored);

	TensSetT ignored_;

private:
	void visit_leaf (iLeaf&) override {}

	void visit_func (iFunctor& func) override
	{
		if (ignored_.count(&func)) { return; }
		auto dependencies = func.get_args();
		multi_visit(*this, dependencies);
		device_->calc(func, (size_t) (targets_.count(&func) > 0));
	}

	iDevice* device_;
	TensSetT targets_;
};

struct Evaluator final : public iEvaluator
{
	void evaluate (iDevice& device, const TensSetT& targets, const TensSetT& ignored = {}) override
	{
		TravEvaluator eval(device, targets, ignored);
		multi_visit(eval, targets);
	}
};

/// The evaluator registered in `ctx` under "evaluater"
/// (internal/teq/evaluator.hpp:65-67, src/evaluator.cpp:9-30); the context
/// owns the pointer.  A context without one gets what the default factory
/// makes: teq::Evaluator in the reference, and here too until a layer above
/// names another (the GPU layer names its replaying evaluator, which walks a
/// set of targets like teq::Evaluator the first time it sees it and records
/// its launches the second time; TCR_EVAL_PLAIN=1 in the environment keeps
/// the plain walk).
void set_eval (iEvaluator* eval, global::CfgMapptrT ctx = global::context());
iEvaluator& get_eval (const global::CfgMapptrT& ctx = global::context());
using EvalFactoryT = iEvaluator* (*) (void);
void set_default_eval_factory (EvalFactoryT factory);

// ---- derivation (internal/teq/derive.hpp, src/derive.cpp) ------------------

struct iDerivativeFuncs
{
	virtual ~iDerivativeFuncs (void) = default;
	/// d op / d op.args[arg_idx] chained with supgrad
	virtual TensptrT lderive (FuncptrT op, TensptrT supgrad, size_t arg_idx) const = 0;
	virtual TensptrT get_const_one (iTensor& reference) const = 0;
	virtual TensptrT get_const_zero (iTensor& reference) const = 0;
	virtual TensptrT add (TensptrsT elems) const = 0;
};

TensptrsT derive (TensptrT root, const TensptrsT& targets, const iDerivativeFuncs& funcs);

}

#endif // TCH_TEQ_HPP
