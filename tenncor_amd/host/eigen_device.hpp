// Device references, lifetime-counted buffers and the device that runs a
// functor: the GPU counterpart of tenncor's internal/eigen/memory.hpp,
// observable.hpp, emeta.hpp and device.hpp, with the same class names and the
// same TTL / version protocol.  What differs is where the bytes live: every
// buffer handed out by iRuntimeMemory is DEVICE memory of the process-wide
// tcg context, operators are stream-ordered launches through the C ABI
// (include/tcg.h), and iDeviceRef::data() -- which callers dereference on the
// host (tenncor/eteq/etens.hpp:134-139) -- is served from a host mirror that is
// synchronised lazily.
#ifndef TCH_EIGEN_DEVICE_HPP
#define TCH_EIGEN_DEVICE_HPP

#include <atomic>
#include <limits>

#include "tcg.h"

#include "packattr.hpp"

namespace eigen
{

/// Process-wide GPU context, created on first use.  Throws when the HIP
/// library cannot create one: there is no CPU fallback.
tcg_ctx* hip_context (void);

/// Turns a non-zero C-ABI status into the reference's fatal error
inline void hip_check (int status)
{
	if (status != TCG_OK)
	{
		global::fatalf("gpu backend: %s", tcg_last_error(hip_context()));
	}
}

// ---- runtime memory (internal/eigen/memory.hpp) ----------------------------

struct iRuntimeMemory
{
	virtual ~iRuntimeMemory (void) = default;
	/// bytes, not elements
	virtual void* allocate (size_t size) = 0;
	/// receives the size given to allocate
	virtual void deallocate (void* ptr, size_t size) = 0;
};

using RTMemptrT = std::shared_ptr<iRuntimeMemory>;

/// Temporary device memory from the context's stream-ordered pool
struct RuntimeMemory final : public iRuntimeMemory
{
	void* allocate (size_t size) override
	{
		void* ptr = nullptr;
		hip_check(tcg_alloc(hip_context(), size, &ptr));
		return ptr;
	}

	void deallocate (void* ptr, size_t size) override
	{
		hip_check(tcg_free(hip_context(), ptr, size));
	}
};

/// The allocator registered in `ctx` under "runtime_memory"
/// (internal/eigen/memory.hpp:141-143, src/memory.cpp:8-30); defaults to
/// RuntimeMemory.  A custom allocator must hand out device memory.
void set_runtime (RTMemptrT mem, global::CfgMapptrT ctx = global::context());
RTMemptrT get_runtime (const global::CfgMapptrT& ctx = global::context());

/// The buffer a functor's value lives in, on loan from the runtime memory for a
/// number of reads (internal/eigen/memory.hpp:60-115): every consumer that has
/// read the value ticks once, and the tick that uses up the last read hands the
/// buffer back.  Names and error texts are the reference's (its tests name them).
template <typename T>
struct Expirable final
{
	T* get (void) { return loan_.ptr; }

	size_t get_ttl (void) const { return reads_left_; }

	bool is_expired (void) const { return 0 == reads_left_; }

	void borrow (RTMemptrT& memory, size_t nelems, size_t ttl)
	{
		if (nullptr == memory) { global::fatal("cannot borrow from null memory"); }
		if (reads_left_ > 0) { global::throw_err("cannot borrow memory when Expirable is not expired"); }
		const size_t bytes = nelems * sizeof(T);
		loan_ = Loan{static_cast<T*>(memory->allocate(bytes)), bytes, memory};
		extend_life(ttl);
	}

	/// The count only ever grows here: a second reader asking for fewer reads
	/// than are already promised changes nothing
	void extend_life (size_t ttl)
	{
		if (nullptr == loan_.ptr) { global::fatal("cannot extend ttl of expired Expirable"); }
		reads_left_ = std::max(reads_left_, ttl);
	}

	void tick (void)
	{
		if (0 == reads_left_) { return; }
		if (0 == --reads_left_) { give_back(); }
	}

	void expire (void)
	{
		give_back();
		reads_left_ = 0;
	}

	/// Become the owner of `ptr` (a buffer a replayed launch sequence has just
	/// filled) with `ttl` reads left; whatever was held before is returned
	void adopt (RTMemptrT& memory, T* ptr, size_t nelems, size_t ttl)
	{
		if (nullptr == ptr || 0 == ttl)
		{
			expire();
			return;
		}
		if (loan_.ptr != ptr)
		{
			give_back();
			loan_ = Loan{ptr, nelems * sizeof(T), memory};
		}
		reads_left_ = ttl;
	}

private:
	struct Loan final
	{
		T* ptr = nullptr;
		size_t bytes = 0;
		RTMemptrT owner = nullptr;
	};

	void give_back (void)
	{
		if (nullptr != loan_.ptr) { loan_.owner->deallocate(loan_.ptr, loan_.bytes); }
		loan_ = Loan();
	}

	Loan loan_;
	size_t reads_left_ = 0;
};

// ---- metadata (internal/eigen/emeta.hpp) -----------------------------------

template <typename T>
struct EMetadata final : public teq::iMetadata
{
	EMetadata (size_t version = 0) : version_(version) {}
	size_t type_code (void) const override { return egen::get_type<T>(); }
	std::string type_label (void) const override { return egen::name_type(egen::get_type<T>()); }
	size_t type_size (void) const override { return sizeof(T); }
	size_t state_version (void) const override { return version_; }
	size_t version_;
};

// ---- device references (internal/eigen/device.hpp) -------------------------

struct iEigen : public teq::iDeviceRef
{
	virtual ~iEigen (void) = default;
	/// (Re)compute into a buffer that lives for `ttl` reads
	virtual void assign (size_t ttl, RTMemptrT& runtime) = 0;
	virtual bool valid_for (size_t desired_ttl) const = 0;
	virtual void extend_life (size_t ttl) = 0;

	// what the GPU path adds to the reference interface
	/// Device pointer of the current value (nullptr when expired); never
	/// touches the host mirror
	virtual const void* device_data (void) const = 0;
	/// device_data() plus the guard odata() carries
	virtual teq::Once<const void*> odevice (void) const = 0;
	/// True when the last launch filled only the part of the buffer its
	/// consumers read (see convolution); such a value is never reused
	virtual bool is_partial (void) const { return false; }

	// what recording an evaluation and replaying it needs (ReplayEvaluator)
	/// Buffer and reads left, as an evaluation pass leaves them
	struct LifeState final
	{
		void* ptr = nullptr;
		size_t ttl = 0;
	};
	/// False for values produced on the host, which a recording cannot hold
	virtual bool replayable (void) const { return true; }
	/// Forget the current value without counting as a read
	virtual void drop (void) {}
	virtual LifeState save_life (void) const { return LifeState(); }
	/// Put back the state save_life() saw after the recorded launches have
	/// been enqueued again; `graph` owns state.ptr
	virtual void restore_life (const LifeState&, RTMemptrT&, tcg_graph*) {}
	/// Host-side effects of a launch that was replayed rather than issued
	virtual void replayed (void) {}
	/// The buffer a launch issued by someone else (a fused group) fills for
	/// this node, with `ttl` reads to live; nullptr when the node cannot take one
	virtual void* borrow_output (size_t, RTMemptrT&) { return nullptr; }
	/// After borrow_output: the launch fills only part of the buffer
	virtual void mark_partial (void) {}
	/// Leaf storage: where the device copy lives, without bringing it up to
	/// date (nullptr for anything that is not a leaf or has no device copy yet)
	virtual const void* device_address (void) const { return nullptr; }
};

/// Lifetime given to the node whose launch is being enqueued, and a flag the
/// launch closure raises when it fills only part of its output
struct LaunchScope final
{
	size_t ttl = 0;
	bool partial = false;
};

LaunchScope& launch_scope (void);

using EigenptrT = std::shared_ptr<iEigen>;

inline const iEigen& eigen_ref (const teq::iTensor& tens)
{
	return static_cast<const iEigen&>(tens.device());
}

struct iPermEigen : public iEigen
{
	virtual ~iPermEigen (void) = default;
	bool valid_for (size_t) const override { return true; }
	void extend_life (size_t) override {}
};

/// Wraps a ref so that it never expires (Functor::cache_init)
struct CacheEigen final : public iPermEigen
{
	CacheEigen (EigenptrT data) : data_(data)
	{
		if (nullptr == data) { global::fatal("cannot cache null eigen device ref"); }
	}
	void* data (void) override { return data_->data(); }
	const void* data (void) const override { return std::const_pointer_cast<const iEigen>(data_)->data(); }
	teq::Once<void*> odata (void) override { return teq::Once<void*>(data()); }
	teq::Once<const void*> odata (void) const override { return teq::Once<const void*>(data()); }
	void assign (size_t ttl, RTMemptrT& runtime) override { data_->assign(ttl, runtime); }
	const void* device_data (void) const override { return data_->device_data(); }
	teq::Once<const void*> odevice (void) const override { return teq::Once<const void*>(device_data()); }
	bool is_partial (void) const override { return data_->is_partial(); }
	bool replayable (void) const override { return data_->replayable(); }
	void drop (void) override { data_->drop(); }
	LifeState save_life (void) const override { return data_->save_life(); }
	void restore_life (const LifeState& state, RTMemptrT& memory, tcg_graph* graph) override
	{
		data_->restore_life(state, memory, graph);
	}
	void replayed (void) override { data_->replayed(); }
	void* borrow_output (size_t ttl, RTMemptrT& memory) override { return data_->borrow_output(ttl, memory); }
	void mark_partial (void) override { data_->mark_partial(); }
private:
	EigenptrT data_;
};

/// Storage of a leaf: the host copy callers read and write plus a device copy
/// kept coherent by two dirty bits
template <typename T>
struct SrcRef final : public iPermEigen
{
	SrcRef (const T* data, teq::Shape shape) : host_(data, data + shape.n_elems()) {}

	SrcRef (const SrcRef<T>& other) : host_(other.host_snapshot()) {}

	~SrcRef (void)
	{
		global::note_structure_change();
		if (dev_) { tcg_free(hip_context(), dev_, host_.size() * sizeof(T)); }
	}

	void* data (void) override
	{
		pull();
		host_newer_ = true; // the caller may write through the pointer
		return host_.data();
	}

	const void* data (void) const override
	{
		pull();
		return host_.data();
	}

	teq::Once<void*> odata (void) override { return teq::Once<void*>(data()); }

	teq::Once<const void*> odata (void) const override { return teq::Once<const void*>(data()); }

	void assign (size_t, RTMemptrT&) override {}

	/// Replace the value (Variable::assign)
	void assign (const T* input, size_t n)
	{
		if (n != host_.size()) { global::fatal("assigning data of a different size"); }
		std::copy(input, input + n, host_.begin());
		host_newer_ = true;
		dev_newer_ = false;
	}

	const void* device_data (void) const override
	{
		if (nullptr == dev_)
		{
			hip_check(tcg_alloc(hip_context(), host_.size() * sizeof(T), &dev_));
			host_newer_ = true;
		}
		if (host_newer_ && !dev_newer_)
		{
			hip_check(tcg_h2d(hip_context(), dev_, host_.data(), host_.size() * sizeof(T)));
		}
		host_newer_ = false;
		return dev_;
	}

	teq::Once<const void*> odevice (void) const override { return teq::Once<const void*>(device_data()); }

	const void* device_address (void) const override { return dev_; }

	/// A kernel wrote the device copy in place (ASSIGN*)
	void* device_data_mut (void)
	{
		void* out = const_cast<void*>(device_data());
		dev_newer_ = true;
		return out;
	}

private:
	void pull (void) const
	{
		if (dev_newer_ && dev_)
		{
			hip_check(tcg_d2h(hip_context(), host_.data(), dev_, host_.size() * sizeof(T)));
		}
		dev_newer_ = false;
	}

	std::vector<T> host_snapshot (void) const
	{
		pull();
		return host_;
	}

	mutable std::vector<T> host_;
	mutable void* dev_ = nullptr;
	mutable bool host_newer_ = true;
	mutable bool dev_newer_ = false;
};

/// A computed value: device buffer with a reader count, host mirror on demand
template <typename T>
struct iTmpEigen : public iEigen
{
	virtual ~iTmpEigen (void) { data_.expire(); }

	void* data (void) override { return sync_mirror(); }

	const void* data (void) const override { return sync_mirror(); }

	teq::Once<void*> odata (void) override
	{
		return teq::Once<void*>(data(), [this] { data_.tick(); });
	}

	teq::Once<const void*> odata (void) const override
	{
		return teq::Once<const void*>(data(), [this] { data_.tick(); });
	}

	bool valid_for (size_t desired_ttl) const override { return desired_ttl <= data_.get_ttl(); }

	void extend_life (size_t ttl) override { data_.extend_life(ttl); }

	const void* device_data (void) const override { return data_.get(); }

	teq::Once<const void*> odevice (void) const override
	{
		return teq::Once<const void*>(data_.get(), [this] { data_.tick(); });
	}

	void drop (void) override { data_.expire(); }

	iEigen::LifeState save_life (void) const override
	{
		iEigen::LifeState out;
		out.ptr = data_.get();
		out.ttl = data_.get_ttl();
		return out;
	}

	void restore_life (const iEigen::LifeState& state, RTMemptrT& memory, tcg_graph* graph) override
	{
		if (nullptr != state.ptr && state.ttl > 0)
		{
			hip_check(tcg_graph_claim(hip_context(), graph, state.ptr));
		}
		data_.adopt(memory, (T*) state.ptr, nelems_, state.ttl);
		mirror_valid_ = false;
	}

protected:
	T* sync_mirror (void) const
	{
		T* dev = data_.get();
		if (nullptr == dev) { return nullptr; }
		if (!mirror_valid_)
		{
			mirror_.resize(nelems_);
			hip_check(tcg_d2h(hip_context(), mirror_.data(), dev, nelems_ * sizeof(T)));
			mirror_valid_ = true;
		}
		return mirror_.data();
	}

	mutable Expirable<T> data_;
	mutable std::vector<T> mirror_;
	mutable bool mirror_valid_ = false;
	size_t nelems_ = 0;
};

/// One operator node: borrows its output, gathers the operands' device
/// pointers (consuming one read of each) and enqueues the launch
template <typename T>
struct HipOp final : public iTmpEigen<T>
{
	/// out and args are device pointers
	using OpF = std::function<void(tcg_ctx*,T*,const std::vector<const void*>&)>;

	HipOp (const teq::Shape& outshape, const teq::CTensT& args, OpF op) :
		op_(op), args_(args) { this->nelems_ = outshape.n_elems(); }

	void assign (size_t ttl, RTMemptrT& runtime) override
	{
		if (this->data_.is_expired()) { this->data_.borrow(runtime, this->nelems_, ttl); }
		else { this->data_.extend_life(ttl); }
		this->mirror_valid_ = false;
		std::vector<const void*> ptrs;
		std::vector<teq::Once<const void*>> onces;
		ptrs.reserve(args_.size());
		onces.reserve(args_.size());
		for (size_t k = 0, n = args_.size(); k < n; ++k)
		{
			// an operand that appears twice (MUL(x, x)) is one consumer of x, as the
			// producer counts them (a set of observers): one read, one pointer
			size_t same = 0;
			while (same < k && args_[same] != args_[k]) { ++same; }
			if (same < k)
			{
				ptrs.push_back(ptrs[same]);
				continue;
			}
			teq::Once<const void*> argdata = eigen_ref(*args_[k]).odevice();
			if (nullptr == argdata.get())
			{
				global::fatalf("operand %s has no data", args_[k]->to_string().c_str());
			}
			ptrs.push_back(argdata.get());
			onces.push_back(std::move(argdata));
		}
		LaunchScope& scope = launch_scope();
		scope.ttl = ttl;
		scope.partial = false;
		try
		{
			op_(hip_context(), this->data_.get(), ptrs);
		}
		catch (...)
		{
			// nothing was computed: a buffer left in place would read as this
			// node's value at the next evaluation (its version has moved on)
			this->data_.expire();
			throw;
		}
		partial_ = scope.partial;
		// the guards die here: producers whose last reader this was hand their
		// buffer back to the pool, after this launch in stream order
	}

	bool is_partial (void) const override { return partial_; }

	void* borrow_output (size_t ttl, RTMemptrT& runtime) override
	{
		if (this->data_.is_expired()) { this->data_.borrow(runtime, this->nelems_, ttl); }
		else { this->data_.extend_life(ttl); }
		this->mirror_valid_ = false;
		partial_ = false;
		return this->data_.get();
	}

	void mark_partial (void) override { partial_ = true; }

private:
	OpF op_;
	teq::CTensT args_;
	bool partial_ = false;
};

/// An operator evaluated on the host (RAND_UNIF draws from the seeded host
/// generator, like the reference) whose result is then uploaded
template <typename T>
struct HostOp final : public iTmpEigen<T>
{
	using OpF = std::function<void(T*,const std::vector<const void*>&,size_t)>;

	HostOp (const teq::Shape& outshape, const teq::CTensT& args, OpF op) :
		op_(op), args_(args) { this->nelems_ = outshape.n_elems(); }

	void assign (size_t ttl, RTMemptrT& runtime) override
	{
		if (this->data_.is_expired()) { this->data_.borrow(runtime, this->nelems_, ttl); }
		else { this->data_.extend_life(ttl); }
		std::vector<const void*> ptrs;
		std::vector<teq::Once<const void*>> onces;
		for (size_t k = 0, n = args_.size(); k < n; ++k)
		{
			size_t same = 0;
			while (same < k && args_[same] != args_[k]) { ++same; }
			if (same < k)
			{
				ptrs.push_back(ptrs[same]);
				continue;
			}
			teq::Once<const void*> argdata = args_[k]->device().odata();
			ptrs.push_back(argdata.get());
			onces.push_back(std::move(argdata));
		}
		this->mirror_.resize(this->nelems_);
		op_(this->mirror_.data(), ptrs, this->nelems_);
		hip_check(tcg_h2d(hip_context(), this->data_.get(), this->mirror_.data(), this->nelems_ * sizeof(T)));
		this->mirror_valid_ = true;
	}

	bool replayable (void) const override { return false; }

private:
	OpF op_;
	teq::CTensT args_;
};

/// Zero-copy alias of another node's value with a reader count of its own;
/// the aliased producer sees one read when the alias has been read out
struct iRefEigen : public iEigen
{
	iRefEigen (teq::iTensor& ref) : ref_(&ref) {}
	virtual ~iRefEigen (void) = default;

	teq::Once<void*> odata (void) override
	{
		return teq::Once<void*>(data(), [this] { consume(); });
	}

	teq::Once<const void*> odata (void) const override
	{
		return teq::Once<const void*>(data(), [this] { consume(); });
	}

	teq::Once<const void*> odevice (void) const override
	{
		return teq::Once<const void*>(device_data(), [this] { consume(); });
	}

	bool valid_for (size_t desired_ttl) const override { return desired_ttl <= ref_ttl_; }

	void extend_life (size_t ttl) override
	{
		if (ref_ttl_ < ttl) { ref_ttl_ = ttl; }
	}

	void drop (void) override { ref_ttl_ = 0; }

	LifeState save_life (void) const override
	{
		LifeState out;
		out.ttl = ref_ttl_;
		return out;
	}

	void restore_life (const LifeState& state, RTMemptrT&, tcg_graph*) override { ref_ttl_ = state.ttl; }

protected:
	teq::iTensor* ref_;

private:
	void consume (void) const
	{
		if (ref_ttl_ > 0 && 0 == (--ref_ttl_))
		{
			eigen_ref(*ref_).odevice();
		}
	}

	mutable size_t ref_ttl_ = 0;
};

struct TensRef final : public iRefEigen
{
	TensRef (teq::iTensor& ref) : iRefEigen(ref) {}
	void* data (void) override { return ref_->device().data(); }
	const void* data (void) const override { return static_cast<const teq::iTensor*>(ref_)->device().data(); }
	const void* device_data (void) const override { return eigen_ref(*ref_).device_data(); }
	void assign (size_t ttl, RTMemptrT&) override { extend_life(ttl); }
};

/// TensRef displaced by a number of elements (last-dim slices)
template <typename T>
struct UnsafeTensRef final : public iRefEigen
{
	UnsafeTensRef (teq::iTensor& ref, size_t ptr_incrs) : iRefEigen(ref), incrs_(ptr_incrs) {}
	void* data (void) override
	{
		void* base = ref_->device().data();
		return base ? ((T*) base) + incrs_ : nullptr;
	}
	const void* data (void) const override
	{
		const void* base = static_cast<const teq::iTensor*>(ref_)->device().data();
		return base ? ((const T*) base) + incrs_ : nullptr;
	}
	const void* device_data (void) const override
	{
		const void* base = eigen_ref(*ref_).device_data();
		return base ? ((const T*) base) + incrs_ : nullptr;
	}
	void assign (size_t ttl, RTMemptrT&) override { extend_life(ttl); }
private:
	size_t incrs_;
};

struct iMutableLeaf : public teq::iLeaf
{
	virtual ~iMutableLeaf (void) = default;
	virtual void upversion (size_t version) = 0;
};

/// target (op)= source, in place on the target leaf's device copy
template <typename T>
struct TensAssign final : public iRefEigen
{
	TensAssign (teq::iTensor& target, const teq::iTensor& arg, int opcode) :
		iRefEigen(target), arg_(&arg), opcode_(opcode)
	{
		if (nullptr == dynamic_cast<iMutableLeaf*>(&target) ||
			nullptr == dynamic_cast<SrcRef<T>*>(&target.device()))
		{
			global::fatalf("cannot assign to %s: not a mutable leaf", target.to_string().c_str());
		}
	}
	void* data (void) override { return ref_->device().data(); }
	const void* data (void) const override { return static_cast<const teq::iTensor*>(ref_)->device().data(); }
	const void* device_data (void) const override { return eigen_ref(*ref_).device_data(); }
	void assign (size_t ttl, RTMemptrT&) override
	{
		extend_life(ttl);
		auto next_version = arg_->get_meta().state_version() + 1;
		static_cast<iMutableLeaf*>(ref_)->upversion(next_version);
		const void* src = eigen_ref(*arg_).device_data();
		if (nullptr == src) { global::fatalf("operand %s has no data", arg_->to_string().c_str()); }
		void* dst = static_cast<SrcRef<T>&>(ref_->device()).device_data_mut();
		hip_check(tcg_assign(hip_context(), opcode_, egen::device_type<T>(), ref_->shape().n_elems(), dst, src));
	}
	void replayed (void) override
	{
		// the recorded kernel has updated the leaf's device copy again
		static_cast<iMutableLeaf*>(ref_)->upversion(arg_->get_meta().state_version() + 1);
		static_cast<SrcRef<T>&>(ref_->device()).device_data_mut();
	}
private:
	const teq::iTensor* arg_;
	int opcode_;
};

// ---- observable functor base (internal/eigen/observable.hpp) ---------------

struct Observable : public teq::iFunctor
{
	Observable (const teq::TensptrsT& args)
	{
		for (teq::TensptrT arg : args)
		{
			if (auto f = dynamic_cast<Observable*>(arg.get())) { f->subscribe(this); }
		}
	}

	Observable (const teq::TensptrsT& args, marsh::Maps&& attrs) : Observable(args)
	{
		attrs_ = std::move(attrs);
	}

	virtual ~Observable (void) = default;

	/// Position in the order in which the functors of this process were made: a
	/// way to enumerate a set of them that does not depend on where they lie in
	/// memory (launch plans then come out the same from run to run)
	uint64_t born (void) const { return born_; }

	void subscribe (Observable* sub) { subs_.emplace(sub); }
	void unsubscribe (Observable* sub) { subs_.erase(sub); }
	std::unordered_set<Observable*> get_observables (void) const { return subs_; }

	virtual bool has_data (void) const = 0;
	virtual void uninitialize (void) = 0;
	virtual bool initialize (void) = 0;
	virtual void must_initialize (void) = 0;
	virtual void cache_init (void) = 0;
	virtual bool prop_version (size_t max_version) = 0;

	std::vector<std::string> ls_attrs (void) const override { return attrs_.ls_attrs(); }
	const marsh::iObject* get_attr (const std::string& attr_key) const override { return attrs_.get_attr(attr_key); }
	marsh::iObject* get_attr (const std::string& attr_key) override { return attrs_.get_attr(attr_key); }
	void add_attr (const std::string& attr_key, marsh::ObjptrT&& attr_val) override { attrs_.add_attr(attr_key, std::move(attr_val)); }
	void rm_attr (const std::string& attr_key) override { attrs_.rm_attr(attr_key); }
	size_t size (void) const override { return attrs_.size(); }

	/// fan-out: number of functors reading this one
	size_t nsubs (void) const { return subs_.size(); }

	const marsh::Maps& get_attrs (void) const { return attrs_; }

protected:
	std::unordered_set<Observable*> subs_;

private:
	static uint64_t next_born (void)
	{
		static std::atomic<uint64_t> count{0};
		return count.fetch_add(1);
	}

	marsh::Maps attrs_;
	const uint64_t born_ = next_born();
};

// ---- the device (internal/eigen/device.hpp:546-576) ------------------------

struct Device final : public teq::iDevice
{
	Device (size_t max_version = std::numeric_limits<size_t>::max()) :
		max_version_(max_version), memory_(get_runtime()) {}

	Device (RTMemptrT memory, size_t max_version = std::numeric_limits<size_t>::max()) :
		max_version_(max_version), memory_(memory) {}

	void calc (teq::iTensor& tens, size_t cache_ttl) override
	{
		auto& obs = static_cast<Observable&>(tens);
		auto& obsdev = static_cast<iEigen&>(tens.device());
		size_t valid_ttl = obs.nsubs() + cache_ttl;
		// recompute when an operand moved on or when the value is gone
		if (obs.prop_version(max_version_) || nullptr == obsdev.device_data() || obsdev.is_partial())
		{
			obsdev.assign(std::max<size_t>(1, valid_ttl), memory_);
		}
		else if (false == obsdev.valid_for(valid_ttl))
		{
			obsdev.extend_life(valid_ttl);
		}
	}

	/// calc() without the freshness test: always launches
	void calc_forced (teq::iTensor& tens, size_t cache_ttl)
	{
		auto& obs = static_cast<Observable&>(tens);
		auto& obsdev = static_cast<iEigen&>(tens.device());
		obs.prop_version(max_version_);
		obsdev.assign(std::max<size_t>(1, obs.nsubs() + cache_ttl), memory_);
	}

	/// Block until everything enqueued so far has run
	void sync (void) { hip_check(tcg_sync(hip_context())); }

	RTMemptrT& memory (void) { return memory_; }

	size_t max_version_;

private:
	RTMemptrT memory_;
};

}

#endif // TCH_EIGEN_DEVICE_HPP
