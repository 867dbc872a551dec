// Shared declarations of the gfx950 backend: context layout, error helpers,
// dtype dispatch and the small device utilities every kernel file uses.
#ifndef TCG_INTERNAL_HPP
#define TCG_INTERNAL_HPP

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <condition_variable>
#include <cstring>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "tcg.h"
#include "tcg_pool.hpp"

#define TCG_WAVE 64

// One captured launch sequence and the device memory it owns (the arena):
// every block handed out while it was being captured stays with it (never
// returns to the context's pool) until the graph is destroyed, because the
// recorded launches keep addressing it
struct tcg_graph : public tcg_arena
{
	hipGraph_t graph = nullptr;
	hipGraphExec_t exec = nullptr;
	uint64_t kernels = 0;
	// a sequence recorded as the steps of ONE kernel (tcg_capture_begin_small)
	bool small = false;
	struct tcg_small_pass* pass = nullptr;
	// recorded on the context's stream after every launch of the sequence:
	// destroying the graph waits for it, so that neither the executable graph
	// (whose kernel arguments live in memory it owns) nor a compiled pass goes
	// away under a launch that is still running
	hipEvent_t done = nullptr;
	bool launched = false;
};

struct tcg_small_pass;
struct tcg_ctx
{
	int device = 0;
	hipStream_t stream = nullptr;
	hipEvent_t ev_begin = nullptr;
	hipEvent_t ev_end = nullptr;
	int num_cus = 256;
	std::string arch;
	std::string error;

	// stream-ordered pool: freed blocks go back to a per-size free list and are
	// handed out again without a device-wide synchronisation, which is safe
	// because every launch of the context is ordered on `stream`
	tcg_pool pool;

	// pinned staging ring for small host->device copies
	char* staging = nullptr;
	size_t staging_size = 0;
	size_t staging_head = 0;

	// device generator: {key, blocks drawn so far}, read and advanced by
	// kernels only so that recorded launches draw fresh values at every replay
	uint64_t* rng_state = nullptr;

	// row / summed-index tables of convolutions lowered to products, by the bytes
	// of the plan they were computed from: a pass over the same layers finds them
	// again instead of launching the kernel that fills them.  Never evicted
	// (recorded launches keep their addresses); new plans stop being kept at
	// conv_table_limit bytes.
	struct ConvTables
	{
		void* rows = nullptr;
		void* sums = nullptr;
		// what conv_patch.hip needs to know about the plan (worked out on the host, once)
		bool patch_known = false;
		int patch_shape = -1;
		int32_t patch_smin = 0, patch_smax = 0, patch_vlo = 0, patch_vhi = 0;
		uint32_t patch_pad_shift = 0, patch_floats = 0;
	};
	std::map<std::string,ConvTables> conv_tables;
	size_t conv_table_bytes = 0;
	uint64_t conv_patch_launches = 0; // products that read the image out of a patch in LDS (conv_patch.hip)
	uint64_t conv_short_launches = 0; // convolutions with a short summed index done in one launch (conv.hip)
	uint64_t conv_fewrows_launches = 0; // convolutions with few rows under a long summed index, gathered while multiplied (conv.hip)
	// tables first met while launches are being recorded are filled at once on
	// this stream, so that the recording does not fill them again at every replay
	hipStream_t side_stream = nullptr;
	// 256 bytes of zeros in device memory: what a load that goes from memory straight
	// into LDS fetches for an element of a convolution's zero border
	float* zeros = nullptr;
	static constexpr size_t conv_table_limit = (size_t) 256 << 20;

	// launch capture: the graph being recorded (its arena is pool.recording)
	tcg_graph* capturing = nullptr;

	// recorded behind the launches of this context's latest tcg_reduce_noalloc
	hipEvent_t scratch_done = nullptr;

	// tcg_hold: the stream waits in a host function until tcg_release opens this
	struct Hold
	{
		std::mutex mu;
		std::condition_variable cv;
		bool open = false;
	};
	Hold* hold = nullptr;

	// tcg_batch_begin: steps of small work held back, to go out as one launch
	tcg_small_pass* batch = nullptr;

	// tcg_fork: 1 while launches go to fork_stream (`stream` IS fork_stream then and
	// main_stream holds the context's own), 2 while what was enqueued there may
	// still run; memory given back in state 1 is kept until tcg_join
	int fork_state = 0;
	hipStream_t fork_stream = nullptr, main_stream = nullptr;
	hipEvent_t ev_fork = nullptr, ev_join = nullptr;
	std::vector<std::pair<void*,size_t>> fork_frees;
};

int tcg_fail (tcg_ctx* ctx, int status, const char* fmt, ...);

#define TCG_HIP(ctx, call) do {\
	hipError_t err__ = (call);\
	if (err__ != hipSuccess) {\
		return tcg_fail(ctx, TCG_ERR_HIP, "%s failed: %s (%s:%d)", #call,\
			hipGetErrorString(err__), __FILE__, __LINE__);\
	} } while (0)

#define TCG_LAUNCH_CHECK(ctx, what) do {\
	hipError_t err__ = hipGetLastError();\
	if (err__ != hipSuccess) {\
		return tcg_fail(ctx, TCG_ERR_HIP, "launch of %s failed: %s", what,\
			hipGetErrorString(err__));\
	} } while (0)

#define TCG_REQUIRE(ctx, cond, ...) do {\
	if (!(cond)) { return tcg_fail(ctx, TCG_ERR_ARG, __VA_ARGS__); } } while (0)

static inline size_t tcg_type_size (int dtype)
{
	switch (dtype)
	{
		case TCG_DOUBLE: case TCG_INT64: case TCG_UINT64: return 8;
		case TCG_FLOAT: case TCG_INT32: case TCG_UINT32: return 4;
		case TCG_INT16: case TCG_UINT16: return 2;
		case TCG_INT8: case TCG_UINT8: return 1;
		default: return 0;
	}
}

static inline uint64_t tcg_n_elems (const uint64_t shape[8])
{
	uint64_t n = 1;
	for (int i = 0; i < 8; ++i) { n *= shape[i]; }
	return n;
}

static inline bool tcg_aligned16 (const void* p)
{
	return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

// ---- sequences recorded as one kernel (ew_fusedx.hip) ------------------------
// While such a recording is open, entry points hand their work over as a step
// instead of launching; anything that cannot be a step fails the recording.
static inline bool tcg_small_mode (const tcg_ctx* ctx)
{
	return (ctx->capturing && ctx->capturing->small) || nullptr != ctx->batch;
}
// Between tcg_batch_begin and tcg_batch_end the same entry points hand their
// work over when it is small and hold it back; a call that cannot be a step
// sends out the steps held so far, ends the batch and runs as itself.
int tcg_batch_send (tcg_ctx* ctx);     // the steps held so far as one launch; the batch stays open
int tcg_batch_decline (tcg_ctx* ctx);  // tcg_batch_send, and the batch is over
void tcg_batch_discard (tcg_ctx* ctx);  // the batch is over and its steps are dropped
void tcg_batch_note_alloc (tcg_ctx* ctx, const void* ptr, size_t bytes); // tcg_alloc / tcg_free inside a batch
void tcg_batch_note_free (tcg_ctx* ctx, const void* ptr);
#define TCG_SMALL_RETURN(ctx, expr) do {\
	int rc__ = (expr);\
	if (rc__ != TCG_ERR_UNSUPPORTED || nullptr == (ctx)->batch) { return rc__; }\
	rc__ = tcg_batch_decline(ctx);\
	if (rc__ != TCG_OK) { return rc__; } } while (0)
int tcg_small_begin (tcg_ctx* ctx, tcg_graph* g);
int tcg_small_finish (tcg_ctx* ctx, tcg_graph* g);   // compiles; the recording is closed
int tcg_small_launch (tcg_ctx* ctx, tcg_graph* g);
void tcg_small_release (tcg_graph* g);
int tcg_small_contract (tcg_ctx* ctx, int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int npairs, const uint64_t* pairs, const void* a, const void* b, void* out);
int tcg_small_reduce (tcg_ctx* ctx, int opcode, int dtype, const uint64_t shape[8], unsigned rankmask,
	const void* in, void* out);
// out[i] = in[offset + sum_d c_d * stride[d]] over `shape` (zero outside [lo, hi) when given)
int tcg_small_copy (tcg_ctx* ctx, int dtype, int nd, const uint64_t* shape, const int64_t* stride, int64_t offset,
	const uint64_t* lo, const uint64_t* hi, const void* in, void* out);
int tcg_small_unsupported (tcg_ctx* ctx, const char* what);
int tcg_small_declare_feed (tcg_ctx* ctx, const void* devptr, size_t bytes, const void* host);
int tcg_small_feed (tcg_ctx* ctx, tcg_graph* g, const void* devptr, const void* host, size_t bytes);

// A convolution lowered to a matrix product reads A[m][s] = image[rows[m].off +
// sums[s].off], or zero when, for some j < ncheck, rows[m].c[j] + sums[s].c[j]
// falls outside [0, check_ext[j]) (the element lies in the zero border)
struct tcg_conv_tab
{
	int64_t off;
	int32_t c[4];
};

struct tcg_conv_operand
{
	const tcg_conv_tab* rows = nullptr;
	const tcg_conv_tab* sums = nullptr;
	uint32_t check_ext[4] = {0, 0, 0, 0};
	int ncheck = 0;
	// which index runs along memory (consecutive m, or consecutive s), and whether
	// aligned groups of four of them are contiguous and inside or outside together
	// (only then can the product read the image itself)
	bool along_m = false;
	bool vec4 = false;
};

// The same product with the stretch of the image that the rows of a tile can
// touch copied into LDS once per workgroup (conv_patch.hip): which of its tile
// shapes to use (-1: none), the least and greatest offset of the summed index
// over the multiples of four, the image elements [vlo, vhi) that exist, the
// distance between neighbouring rows as a shift, and the floats of LDS the
// padded stretch of the widest tile takes
struct tcg_conv_patch
{
	int shape = -1;
	int32_t smin = 0, smax = 0, vlo = 0, vhi = 0;
	uint32_t pad_shift = 31, patch_floats = 0;
};
constexpr size_t TCG_CONV_PATCH_LDS = 80 * 1024; // per workgroup: two of them fit a CU
int tcg_conv_patch_shapes (void);
void tcg_conv_patch_shape (int which, uint32_t* rows, uint32_t* cols, uint32_t* threads);
size_t tcg_conv_patch_lds (int which, uint32_t patch_floats, uint64_t S, int ncheck);
int tcg_conv_patch_f32 (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t S, const float* image,
	const tcg_conv_operand& op, const tcg_conv_patch& pp, const float* B, uint64_t ldb, float* C, uint64_t ldc, bool* handled);

// C[m][n] = sum_s A[m][s] B[s][n] with A read through `op` (never materialised);
// *handled = false when the shapes do not fit the matrix-core kernel
int tcg_gemm_f32_mfma_conv (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t S,
	const float* image, const tcg_conv_operand& op, const float* B, uint64_t ldb,
	float* C, uint64_t ldc, bool* handled);

// C = sum_t A_t B_t over `terms` products of one shape as one matrix-core
// product over the concatenated summed index (gemm_mfma.hip)
int tcg_gemm_f32_mfma_sum (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint32_t terms,
	const float* const* A, uint64_t lda, int trans_a, const float* const* B, uint64_t ldb, int trans_b,
	float* C, uint64_t ldc, bool* handled);

// the same with a leading dim of its own for every term
int tcg_gemm_f32_mfma_terms (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint32_t terms,
	const float* const* A, const uint64_t* lda, int trans_a, const float* const* B, const uint64_t* ldb, int trans_b,
	float* C, uint64_t ldc, bool* handled);

// blocks of a result whose operands are concatenations along the dims that survive, as one product
int tcg_gemm_f32_mfma_grid (tcg_ctx* ctx, uint32_t mparts, const uint64_t* Mp, uint32_t nparts, const uint64_t* Np,
	uint64_t K, uint32_t terms, const float* const* A, const uint64_t* lda, int trans_a,
	const float* const* B, const uint64_t* ldb, int trans_b, float* C, uint64_t ldc, bool* handled);

// the same with the K ranges left side by side for the reader to add up
int tcg_gemm_f32_mfma_ranges (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint32_t terms,
	const float* const* A, const uint64_t* lda, int trans_a, const float* const* B, const uint64_t* ldb, int trans_b,
	uint32_t nranges, float* ranges, bool* handled);

// reduce.hip: looks up this GPU's copy of the scratch memory of
// tcg_reduce_noalloc; called once per context with the device current
int tcg_reduce_scratch_init (tcg_ctx* ctx);
void tcg_reduce_scratch_release (tcg_ctx* ctx);

// Number of workgroups for a streaming kernel: enough to cover `work` items,
// capped at a multiple of the CU count so that a grid-stride loop takes over
static inline unsigned tcg_grid (const tcg_ctx* ctx, uint64_t work_items,
	unsigned per_block, unsigned blocks_per_cu)
{
	uint64_t need = (work_items + per_block - 1) / per_block;
	uint64_t cap = (uint64_t) ctx->num_cus * blocks_per_cu;
	if (need < 1) { need = 1; }
	return (unsigned) (need < cap ? need : cap);
}

// Runs `stmt` with `T` bound to the C++ type of `dtype`
#define TCG_DISPATCH_TYPE(ctx, dtype, ...) do {\
	switch (dtype) {\
		case TCG_DOUBLE: { using T = double; __VA_ARGS__; } break;\
		case TCG_FLOAT: { using T = float; __VA_ARGS__; } break;\
		case TCG_INT32: { using T = int32_t; __VA_ARGS__; } break;\
		default: return tcg_fail(ctx, TCG_ERR_ARG, "unknown dtype %d", (int) (dtype));\
	} } while (0)

// The same over every dtype, the integer widths of the full type set included
// (cfg/fulltype.yml:11-34): for the entry points whose kernels exist for all of
// them (reductions, casts, products, convolutions).  The streaming elementwise
// kernels are built for the three default types only; the other widths run as
// groups compiled at run time (tcg_ew_fusedx).
#define TCG_DISPATCH_ALL(ctx, dtype, ...) do {\
	switch (dtype) {\
		case TCG_DOUBLE: { using T = double; __VA_ARGS__; } break;\
		case TCG_FLOAT: { using T = float; __VA_ARGS__; } break;\
		case TCG_INT32: { using T = int32_t; __VA_ARGS__; } break;\
		case TCG_INT8: { using T = int8_t; __VA_ARGS__; } break;\
		case TCG_UINT8: { using T = uint8_t; __VA_ARGS__; } break;\
		case TCG_INT16: { using T = int16_t; __VA_ARGS__; } break;\
		case TCG_UINT16: { using T = uint16_t; __VA_ARGS__; } break;\
		case TCG_UINT32: { using T = uint32_t; __VA_ARGS__; } break;\
		case TCG_INT64: { using T = int64_t; __VA_ARGS__; } break;\
		case TCG_UINT64: { using T = uint64_t; __VA_ARGS__; } break;\
		default: return tcg_fail(ctx, TCG_ERR_ARG, "unknown dtype %d", (int) (dtype));\
	} } while (0)

// Data movement only looks at the element size: the integer widths of the
// full type set share the kernels of a type of their size (bytes are copied,
// never computed with; zero fill is all-zero bits for every type)
#define TCG_DISPATCH_MOVE(ctx, dtype, ...) do {\
	switch (dtype) {\
		case TCG_DOUBLE: case TCG_INT64: case TCG_UINT64: { using T = double; __VA_ARGS__; } break;\
		case TCG_FLOAT: { using T = float; __VA_ARGS__; } break;\
		case TCG_INT32: case TCG_UINT32: { using T = int32_t; __VA_ARGS__; } break;\
		case TCG_INT16: case TCG_UINT16: { using T = uint16_t; __VA_ARGS__; } break;\
		case TCG_INT8: case TCG_UINT8: { using T = uint8_t; __VA_ARGS__; } break;\
		default: return tcg_fail(ctx, TCG_ERR_ARG, "unknown dtype %d", (int) (dtype));\
	} } while (0)

static inline bool tcg_default_dtype (int dtype)
{
	return dtype == TCG_DOUBLE || dtype == TCG_FLOAT || dtype == TCG_INT32;
}

// 16-byte vector of T (compiler vector types: the non-temporal load/store
// builtins take these, not the HIP float4 structs)
typedef float tcg_f32x4 __attribute__((ext_vector_type(4)));
typedef int32_t tcg_i32x4 __attribute__((ext_vector_type(4)));
typedef double tcg_f64x2 __attribute__((ext_vector_type(2)));
template <typename T> struct Vec16;
template <> struct Vec16<float> { using type = tcg_f32x4; static constexpr int N = 4; };
template <> struct Vec16<int32_t> { using type = tcg_i32x4; static constexpr int N = 4; };
template <> struct Vec16<double> { using type = tcg_f64x2; static constexpr int N = 2; };
typedef int8_t tcg_i8x16 __attribute__((ext_vector_type(16)));
typedef uint8_t tcg_u8x16 __attribute__((ext_vector_type(16)));
typedef int16_t tcg_i16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t tcg_u16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t tcg_u32x4 __attribute__((ext_vector_type(4)));
typedef int64_t tcg_i64x2 __attribute__((ext_vector_type(2)));
typedef uint64_t tcg_u64x2 __attribute__((ext_vector_type(2)));
template <> struct Vec16<int8_t> { using type = tcg_i8x16; static constexpr int N = 16; };
template <> struct Vec16<uint8_t> { using type = tcg_u8x16; static constexpr int N = 16; };
template <> struct Vec16<int16_t> { using type = tcg_i16x8; static constexpr int N = 8; };
template <> struct Vec16<uint16_t> { using type = tcg_u16x8; static constexpr int N = 8; };
template <> struct Vec16<uint32_t> { using type = tcg_u32x4; static constexpr int N = 4; };
template <> struct Vec16<int64_t> { using type = tcg_i64x2; static constexpr int N = 2; };
template <> struct Vec16<uint64_t> { using type = tcg_u64x2; static constexpr int N = 2; };

template <typename T>
union VecU
{
	typename Vec16<T>::type v;
	T e[Vec16<T>::N];
};

#endif // TCG_INTERNAL_HPP
