// Context, stream-ordered memory pool, host<->device transfers and stream
// timers of the gfx950 backend.
#include "tcg_internal.hpp"

static thread_local std::string g_create_error;

int tcg_fail (tcg_ctx* ctx, int status, const char* fmt, ...)
{
	char buf[1024];
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(buf, sizeof(buf), fmt, ap);
	va_end(ap);
	if (ctx) { ctx->error = buf; }
	else { g_create_error = buf; }
	return status;
}

static __global__ void fill_zero_k (uint32_t* dst, uint64_t nwords)
{
	uint64_t i = (uint64_t) blockIdx.x * blockDim.x + threadIdx.x;
	uint64_t step = (uint64_t) gridDim.x * blockDim.x;
	for (; i < nwords; i += step) { dst[i] = 0u; }
}

static __global__ void fill_zero_bytes_k (uint8_t* dst, uint64_t n)
{
	uint64_t i = (uint64_t) blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) { dst[i] = 0; }
}

extern "C" {

int tcg_ctx_create (int device, tcg_ctx** out)
{
	if (!out) { return tcg_fail(nullptr, TCG_ERR_ARG, "tcg_ctx_create: out is NULL"); }
	*out = nullptr;
	int ndev = 0;
	hipError_t err = hipGetDeviceCount(&ndev);
	if (err != hipSuccess || ndev <= 0)
	{
		return tcg_fail(nullptr, TCG_ERR_HIP,
			"tcg_ctx_create: no HIP device visible (%s); this backend has no CPU fallback",
			err != hipSuccess ? hipGetErrorString(err) : "device count is 0");
	}
	if (device < 0 || device >= ndev)
	{
		return tcg_fail(nullptr, TCG_ERR_ARG, "tcg_ctx_create: device %d of %d", device, ndev);
	}
	tcg_ctx* ctx = new tcg_ctx();
	ctx->device = device;
	hipDeviceProp_t prop;
	if ((err = hipSetDevice(device)) != hipSuccess ||
		(err = hipGetDeviceProperties(&prop, device)) != hipSuccess ||
		(err = hipStreamCreate(&ctx->stream)) != hipSuccess ||
		(err = hipEventCreate(&ctx->ev_begin)) != hipSuccess ||
		(err = hipEventCreate(&ctx->ev_end)) != hipSuccess)
	{
		int rc = tcg_fail(nullptr, TCG_ERR_HIP, "tcg_ctx_create: %s", hipGetErrorString(err));
		delete ctx;
		return rc;
	}
	ctx->pool.raw_alloc = [](size_t bytes, void** out) -> int
	{
		hipError_t rc = hipMalloc(out, bytes);
		if (rc != hipSuccess) { (void) hipGetLastError(); }
		return rc == hipSuccess ? 0 : 1;
	};
	ctx->pool.raw_free = [](void* ptr) { (void) hipFree(ptr); };
	// (a held stream cannot be waited for: see tcg_hold)
	ctx->pool.drain = [ctx]
	{
		if (nullptr != ctx->hold) { return; }
		(void) hipStreamSynchronize(ctx->stream);
		if (ctx->fork_state) { (void) hipStreamSynchronize(ctx->fork_state == 1 ? ctx->main_stream : ctx->fork_stream); }
	};
	ctx->num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
	ctx->arch = prop.gcnArchName;
	size_t colon = ctx->arch.find(':');
	if (colon != std::string::npos) { ctx->arch.resize(colon); }
	ctx->staging_size = 8u << 20;
	if ((err = hipHostMalloc((void**) &ctx->staging, ctx->staging_size, hipHostMallocDefault)) != hipSuccess)
	{
		int rc = tcg_fail(nullptr, TCG_ERR_HIP, "tcg_ctx_create: hipHostMalloc: %s", hipGetErrorString(err));
		delete ctx;
		return rc;
	}
	const uint64_t rng_init[2] = {0, 0};
	if ((err = hipMalloc((void**) &ctx->rng_state, sizeof(rng_init))) != hipSuccess ||
		(err = hipMemcpy(ctx->rng_state, rng_init, sizeof(rng_init), hipMemcpyHostToDevice)) != hipSuccess)
	{
		int rc = tcg_fail(nullptr, TCG_ERR_HIP, "tcg_ctx_create: generator state: %s", hipGetErrorString(err));
		delete ctx;
		return rc;
	}
	if ((err = hipMalloc((void**) &ctx->zeros, 256)) != hipSuccess ||
		(err = hipMemset(ctx->zeros, 0, 256)) != hipSuccess)
	{
		int rc = tcg_fail(nullptr, TCG_ERR_HIP, "tcg_ctx_create: zero buffer: %s", hipGetErrorString(err));
		(void) hipFree(ctx->rng_state);
		(void) hipHostFree(ctx->staging);
		delete ctx;
		return rc;
	}
	// the stream on which convolution tables first met during a recording are filled
	// (made here so that it cannot fail in the middle of a recording)
	if ((err = hipStreamCreate(&ctx->side_stream)) != hipSuccess)
	{
		int rc = tcg_fail(nullptr, TCG_ERR_HIP, "tcg_ctx_create: second stream: %s", hipGetErrorString(err));
		(void) hipFree(ctx->zeros);
		(void) hipFree(ctx->rng_state);
		(void) hipHostFree(ctx->staging);
		delete ctx;
		return rc;
	}
	// the stream and the events of tcg_fork / tcg_join (default priority, like the others)
	if ((err = hipStreamCreate(&ctx->fork_stream)) != hipSuccess ||
		(err = hipEventCreateWithFlags(&ctx->ev_fork, hipEventDisableTiming)) != hipSuccess ||
		(err = hipEventCreateWithFlags(&ctx->ev_join, hipEventDisableTiming)) != hipSuccess)
	{
		int rc = tcg_fail(nullptr, TCG_ERR_HIP, "tcg_ctx_create: third stream: %s", hipGetErrorString(err));
		if (ctx->ev_fork) { (void) hipEventDestroy(ctx->ev_fork); }
		if (ctx->fork_stream) { (void) hipStreamDestroy(ctx->fork_stream); }
		(void) hipStreamDestroy(ctx->side_stream);
		(void) hipFree(ctx->zeros);
		(void) hipFree(ctx->rng_state);
		(void) hipHostFree(ctx->staging);
		delete ctx;
		return rc;
	}
	if (tcg_reduce_scratch_init(ctx) != TCG_OK)
	{
		int rc = tcg_fail(nullptr, TCG_ERR_HIP, "tcg_ctx_create: %s", ctx->error.c_str());
		(void) hipEventDestroy(ctx->ev_join);
		(void) hipEventDestroy(ctx->ev_fork);
		(void) hipStreamDestroy(ctx->fork_stream);
		(void) hipStreamDestroy(ctx->side_stream);
		(void) hipFree(ctx->zeros);
		(void) hipFree(ctx->rng_state);
		(void) hipHostFree(ctx->staging);
		delete ctx;
		return rc;
	}
	*out = ctx;
	return TCG_OK;
}

int tcg_ctx_destroy (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_OK; }
	(void) hipSetDevice(ctx->device);
	tcg_batch_discard(ctx);
	(void) tcg_release(ctx);
	(void) tcg_join(ctx);
	(void) hipStreamSynchronize(ctx->stream);
	tcg_reduce_scratch_release(ctx);
	ctx->pool.release_all();
	if (ctx->staging) { (void) hipHostFree(ctx->staging); }
	if (ctx->rng_state) { (void) hipFree(ctx->rng_state); }
	if (ctx->zeros) { (void) hipFree(ctx->zeros); }
	if (ctx->fork_stream)
	{
		(void) hipStreamSynchronize(ctx->fork_stream);
		(void) hipStreamDestroy(ctx->fork_stream);
		(void) hipEventDestroy(ctx->ev_fork);
		(void) hipEventDestroy(ctx->ev_join);
	}
	if (ctx->side_stream)
	{
		(void) hipStreamSynchronize(ctx->side_stream);
		(void) hipStreamDestroy(ctx->side_stream);
	}
	for (auto& kv : ctx->conv_tables)
	{
		(void) hipFree(kv.second.rows);
		(void) hipFree(kv.second.sums);
	}
	(void) hipEventDestroy(ctx->ev_begin);
	(void) hipEventDestroy(ctx->ev_end);
	(void) hipStreamDestroy(ctx->stream);
	delete ctx;
	return TCG_OK;
}

const char* tcg_last_error (const tcg_ctx* ctx)
{
	return ctx ? ctx->error.c_str() : g_create_error.c_str();
}

const char* tcg_device_arch (const tcg_ctx* ctx)
{
	return ctx ? ctx->arch.c_str() : "";
}

int tcg_alloc (tcg_ctx* ctx, size_t bytes, void** devptr)
{
	if (!ctx || !devptr) { return TCG_ERR_ARG; }
	std::string why;
	int rc = ctx->pool.take(bytes, devptr, &why);
	if (rc != tcg_pool::OK) { return tcg_fail(ctx, TCG_ERR_OOM, "tcg_alloc: %s", why.c_str()); }
	if (ctx->batch) { tcg_batch_note_alloc(ctx, *devptr, bytes); }
	return TCG_OK;
}

int tcg_free (tcg_ctx* ctx, void* devptr, size_t bytes)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (!devptr) { return TCG_OK; }
	if (ctx->fork_state == 1)
	{
		// used by launches of the second stream: back to the pool when the context's
		// own stream has waited for them
		ctx->fork_frees.emplace_back(devptr, bytes);
		return TCG_OK;
	}
	std::string why;
	int rc = ctx->pool.give(devptr, bytes, &why);
	if (rc != tcg_pool::OK) { return tcg_fail(ctx, TCG_ERR_ARG, "tcg_free: %p: %s", devptr, why.c_str()); }
	if (ctx->batch) { tcg_batch_note_free(ctx, devptr); }
	return TCG_OK;
}

int tcg_mem_stats (const tcg_ctx* ctx, uint64_t* in_use, uint64_t* pooled)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (in_use) { *in_use = ctx->pool.bytes_in_use; }
	if (pooled) { *pooled = ctx->pool.bytes_pooled; }
	return TCG_OK;
}

// Launches enqueued between tcg_hold and tcg_release start only at the release,
// back to back: events recorded between them then measure the device, not how
// fast the host enqueues
int tcg_hold (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, nullptr == ctx->capturing, "tcg_hold: not while launches are being recorded");
	TCG_REQUIRE(ctx, nullptr == ctx->hold, "tcg_hold: the stream is held already");
	ctx->hold = new tcg_ctx::Hold();
	hipError_t err = hipLaunchHostFunc(ctx->stream, [](void* arg)
	{
		auto hold = static_cast<tcg_ctx::Hold*>(arg);
		std::unique_lock<std::mutex> lock(hold->mu);
		hold->cv.wait(lock, [hold] { return hold->open; });
	}, ctx->hold);
	if (err != hipSuccess)
	{
		delete ctx->hold;
		ctx->hold = nullptr;
		return tcg_fail(ctx, TCG_ERR_HIP, "tcg_hold: %s", hipGetErrorString(err));
	}
	return TCG_OK;
}

int tcg_release (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (nullptr == ctx->hold) { return TCG_OK; }
	{
		std::lock_guard<std::mutex> lock(ctx->hold->mu);
		ctx->hold->open = true;
	}
	ctx->hold->cv.notify_all();
	// the host function still holds the pointer until it has run
	hipError_t err = hipStreamSynchronize(ctx->stream);
	delete ctx->hold;
	ctx->hold = nullptr;
	if (err != hipSuccess) { return tcg_fail(ctx, TCG_ERR_HIP, "tcg_release: %s", hipGetErrorString(err)); }
	return TCG_OK;
}

// ---- a second stream for work nothing waits for yet -------------------------------
int tcg_fork (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, 0 == ctx->fork_state, "tcg_fork: the launches of an earlier tcg_fork have not been joined");
	// a single-launch recording has no streams to spread its steps over
	if (tcg_small_mode(ctx)) { return TCG_OK; }
	TCG_HIP(ctx, hipEventRecord(ctx->ev_fork, ctx->stream));
	TCG_HIP(ctx, hipStreamWaitEvent(ctx->fork_stream, ctx->ev_fork, 0));
	ctx->main_stream = ctx->stream;
	ctx->stream = ctx->fork_stream;
	ctx->fork_state = 1;
	return TCG_OK;
}

int tcg_fork_end (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (ctx->fork_state != 1) { return TCG_OK; }
	hipError_t err = hipEventRecord(ctx->ev_join, ctx->fork_stream);
	ctx->stream = ctx->main_stream;
	ctx->fork_state = 2;
	if (err != hipSuccess) { return tcg_fail(ctx, TCG_ERR_HIP, "tcg_fork_end: %s", hipGetErrorString(err)); }
	return TCG_OK;
}

int tcg_join (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (0 == ctx->fork_state) { return TCG_OK; }
	int rc = tcg_fork_end(ctx);
	hipError_t err = hipStreamWaitEvent(ctx->stream, ctx->ev_join, 0);
	ctx->fork_state = 0;
	std::vector<std::pair<void*,size_t>> frees;
	frees.swap(ctx->fork_frees);
	for (auto& f : frees)
	{
		int freed = tcg_free(ctx, f.first, f.second);
		if (rc == TCG_OK) { rc = freed; }
	}
	if (rc == TCG_OK && err != hipSuccess) { rc = tcg_fail(ctx, TCG_ERR_HIP, "tcg_join: %s", hipGetErrorString(err)); }
	return rc;
}

int tcg_mem_stats_kept (const tcg_ctx* ctx, uint64_t* conv_tables)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (conv_tables) { *conv_tables = ctx->conv_table_bytes; }
	return TCG_OK;
}

int tcg_h2d (tcg_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (bytes == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, dst_dev && src_host, "tcg_h2d: NULL pointer");
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_h2d: host transfers cannot be part of a captured sequence");
	if (bytes <= ctx->staging_size / 4)
	{
		// small: stage through pinned memory so that the call returns at once
		size_t need = (bytes + 63) & ~(size_t) 63;
		if (ctx->staging_head + need > ctx->staging_size)
		{
			TCG_HIP(ctx, hipStreamSynchronize(ctx->stream));
			ctx->staging_head = 0;
		}
		char* slot = ctx->staging + ctx->staging_head;
		memcpy(slot, src_host, bytes);
		ctx->staging_head += need;
		TCG_HIP(ctx, hipMemcpyAsync(dst_dev, slot, bytes, hipMemcpyHostToDevice, ctx->stream));
		return TCG_OK;
	}
	TCG_HIP(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
	TCG_HIP(ctx, hipStreamSynchronize(ctx->stream));
	return TCG_OK;
}

int tcg_d2h (tcg_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (bytes == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, dst_host && src_dev, "tcg_d2h: NULL pointer");
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_d2h: host transfers cannot be part of a captured sequence");
	if (ctx->batch) { int rc = tcg_batch_end(ctx); if (rc != TCG_OK) { return rc; } }
	if (ctx->fork_state) { int rc = tcg_join(ctx); if (rc != TCG_OK) { return rc; } }
	TCG_HIP(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
	TCG_HIP(ctx, hipStreamSynchronize(ctx->stream));
	return TCG_OK;
}

int tcg_d2d (tcg_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (bytes == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, dst_dev && src_dev, "tcg_d2d: NULL pointer");
	TCG_HIP(ctx, hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream));
	return TCG_OK;
}

int tcg_fill_zero (tcg_ctx* ctx, void* dst_dev, size_t bytes)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (bytes == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, dst_dev, "tcg_fill_zero: NULL pointer");
	// a fill kernel rather than hipMemsetAsync: callers may capture this
	// stream into a graph
	uint8_t* p = (uint8_t*) dst_dev;
	size_t head = (4 - (reinterpret_cast<uintptr_t>(p) & 3)) & 3;
	if (head > bytes) { head = bytes; }
	if (head)
	{
		fill_zero_bytes_k<<<1, 64, 0, ctx->stream>>>(p, head);
	}
	size_t nwords = (bytes - head) / 4;
	if (nwords)
	{
		unsigned grid = tcg_grid(ctx, nwords, 256 * 8, 8);
		fill_zero_k<<<grid, 256, 0, ctx->stream>>>((uint32_t*) (p + head), nwords);
	}
	size_t tail = bytes - head - nwords * 4;
	if (tail)
	{
		fill_zero_bytes_k<<<1, 64, 0, ctx->stream>>>(p + head + nwords * 4, tail);
	}
	TCG_LAUNCH_CHECK(ctx, "fill_zero");
	return TCG_OK;
}

int tcg_sync (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_sync: cannot wait while a sequence is being captured");
	if (ctx->batch) { int rc = tcg_batch_end(ctx); if (rc != TCG_OK) { return rc; } }
	if (ctx->fork_state) { int rc = tcg_join(ctx); if (rc != TCG_OK) { return rc; } }
	TCG_HIP(ctx, hipStreamSynchronize(ctx->stream));
	return TCG_OK;
}

int tcg_timer_begin (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_timer_begin: timers cannot be part of a captured sequence");
	TCG_HIP(ctx, hipEventRecord(ctx->ev_begin, ctx->stream));
	return TCG_OK;
}

int tcg_timer_end (tcg_ctx* ctx, float* ms)
{
	if (!ctx || !ms) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_timer_end: timers cannot be part of a captured sequence");
	TCG_HIP(ctx, hipEventRecord(ctx->ev_end, ctx->stream));
	TCG_HIP(ctx, hipEventSynchronize(ctx->ev_end));
	TCG_HIP(ctx, hipEventElapsedTime(ms, ctx->ev_begin, ctx->ev_end));
	return TCG_OK;
}

int tcg_event_create (tcg_ctx* ctx, void** event)
{
	if (!ctx || !event) { return TCG_ERR_ARG; }
	hipEvent_t ev;
	TCG_HIP(ctx, hipEventCreate(&ev));
	*event = (void*) ev;
	return TCG_OK;
}

int tcg_event_destroy (tcg_ctx* ctx, void* event)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (event) { TCG_HIP(ctx, hipEventDestroy((hipEvent_t) event)); }
	return TCG_OK;
}

int tcg_event_record (tcg_ctx* ctx, void* event)
{
	if (!ctx || !event) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_event_record: timers cannot be part of a captured sequence");
	TCG_HIP(ctx, hipEventRecord((hipEvent_t) event, ctx->stream));
	return TCG_OK;
}

int tcg_event_elapsed (tcg_ctx* ctx, void* start, void* stop, float* ms)
{
	if (!ctx || !start || !stop || !ms) { return TCG_ERR_ARG; }
	TCG_HIP(ctx, hipEventSynchronize((hipEvent_t) stop));
	TCG_HIP(ctx, hipEventElapsedTime(ms, (hipEvent_t) start, (hipEvent_t) stop));
	return TCG_OK;
}

// ---- captured launch sequences -------------------------------------------

int tcg_capture_begin (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_capture_begin: a capture is already in progress");
	if (ctx->fork_state) { int rc = tcg_join(ctx); if (rc != TCG_OK) { return rc; } }
	// relaxed mode: the pool may still call hipMalloc for a size it has not seen
	TCG_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
	ctx->capturing = new tcg_graph();
	ctx->pool.recording = ctx->capturing;
	return TCG_OK;
}

int tcg_capture_begin_small (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_capture_begin_small: a capture is already in progress");
	if (ctx->fork_state) { int rc = tcg_join(ctx); if (rc != TCG_OK) { return rc; } }
	// the stream captures as well: a launch that is not handed over as a step
	// is caught there (and fails tcg_capture_end) instead of running out of turn
	TCG_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
	ctx->capturing = new tcg_graph();
	ctx->pool.recording = ctx->capturing;
	return tcg_small_begin(ctx, ctx->capturing);
}

int tcg_capture_feed (tcg_ctx* ctx, const void* devptr, size_t bytes, const void* host)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, ctx->capturing && ctx->capturing->small, "tcg_capture_feed: no single-launch recording in progress");
	return tcg_small_declare_feed(ctx, devptr, bytes, host);
}

int tcg_graph_feed (tcg_ctx* ctx, tcg_graph* graph, const void* devptr, const void* host, size_t bytes)
{
	if (!ctx || !graph) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, graph->small, "tcg_graph_feed: not a single-launch recording");
	return tcg_small_feed(ctx, graph, devptr, host, bytes);
}

// The launches of `g` that were enqueued have finished when this returns.
// Waits on the graph's own event, which is legal while the stream records
// another sequence (a stream synchronisation would not be).
static void graph_wait (tcg_graph* g)
{
	if (g->launched && g->done) { (void) hipEventSynchronize(g->done); }
	g->launched = false;
}

static void graph_release (tcg_ctx* ctx, tcg_graph* g)
{
	graph_wait(g);
	tcg_small_release(g);
	if (g->exec) { (void) hipGraphExecDestroy(g->exec); }
	if (g->graph) { (void) hipGraphDestroy(g->graph); }
	if (g->done) { (void) hipEventDestroy(g->done); }
	ctx->pool.dissolve(g);
	delete g;
}

int tcg_capture_end (tcg_ctx* ctx, tcg_graph** out)
{
	if (!ctx || !out) { return TCG_ERR_ARG; }
	*out = nullptr;
	TCG_REQUIRE(ctx, ctx->capturing, "tcg_capture_end: no capture in progress");
	// steps still held back belong to the sequence
	int sent = ctx->batch ? tcg_batch_end(ctx) : TCG_OK;
	// the second stream is part of the recording until it has been waited for
	if (sent == TCG_OK && ctx->fork_state) { sent = tcg_join(ctx); }
	if (sent != TCG_OK)
	{
		(void) tcg_capture_abort(ctx);
		return sent;
	}
	tcg_graph* g = ctx->capturing;
	ctx->capturing = nullptr;
	ctx->pool.seal(g);
	hipError_t err = hipStreamEndCapture(ctx->stream, &g->graph);
	if (err == hipSuccess) { err = hipEventCreateWithFlags(&g->done, hipEventDisableTiming); }
	size_t nodes = 0;
	if (err == hipSuccess) { err = hipGraphGetNodes(g->graph, nullptr, &nodes); }
	if (err == hipSuccess && g->small)
	{
		int rc = nodes == 0 ? tcg_small_finish(ctx, g) :
			tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "tcg_capture_end: %zu launches were not steps of the single-launch pass", nodes);
		if (rc != TCG_OK)
		{
			graph_release(ctx, g);
			return rc;
		}
		*out = g;
		return TCG_OK;
	}
	if (err == hipSuccess) { err = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0); }
	if (err != hipSuccess)
	{
		(void) hipGetLastError();
		graph_release(ctx, g);
		return tcg_fail(ctx, TCG_ERR_HIP, "tcg_capture_end: %s", hipGetErrorString(err));
	}
	g->kernels = nodes;
	*out = g;
	return TCG_OK;
}

int tcg_capture_abort (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	tcg_batch_discard(ctx);
	(void) tcg_join(ctx);
	if (!ctx->capturing) { return TCG_OK; }
	tcg_graph* g = ctx->capturing;
	ctx->capturing = nullptr;
	ctx->pool.seal(g);
	(void) hipStreamEndCapture(ctx->stream, &g->graph);
	(void) hipGetLastError();
	graph_release(ctx, g);
	return TCG_OK;
}

int tcg_graph_launch (tcg_ctx* ctx, tcg_graph* graph)
{
	if (!ctx || !graph) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_graph_launch: cannot launch while capturing");
	if (ctx->batch) { int sent = tcg_batch_end(ctx); if (sent != TCG_OK) { return sent; } }
	if (ctx->fork_state) { int joined = tcg_join(ctx); if (joined != TCG_OK) { return joined; } }
	int rc = TCG_OK;
	if (graph->small) { rc = tcg_small_launch(ctx, graph); }
	else
	{
		hipError_t err = hipGraphLaunch(graph->exec, ctx->stream);
		if (err != hipSuccess) { rc = tcg_fail(ctx, TCG_ERR_HIP, "hipGraphLaunch failed: %s", hipGetErrorString(err)); }
	}
	// even a launch that reported a failure may have enqueued part of the sequence
	graph->launched = true;
	hipError_t err = hipEventRecord(graph->done, ctx->stream);
	if (rc == TCG_OK && err != hipSuccess) { rc = tcg_fail(ctx, TCG_ERR_HIP, "hipEventRecord failed: %s", hipGetErrorString(err)); }
	return rc;
}

int tcg_graph_claim (tcg_ctx* ctx, tcg_graph* graph, void* devptr)
{
	if (!ctx || !graph) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, ctx->pool.claim(graph, devptr), "tcg_graph_claim: %p does not belong to this graph", devptr);
	return TCG_OK;
}

int tcg_graph_stats (const tcg_graph* graph, uint64_t* nodes, uint64_t* arena_bytes)
{
	if (!graph) { return TCG_ERR_ARG; }
	if (nodes) { *nodes = graph->kernels; }
	if (arena_bytes) { *arena_bytes = graph->bytes; }
	return TCG_OK;
}

int tcg_graph_destroy (tcg_ctx* ctx, tcg_graph* graph)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (!graph) { return TCG_OK; }
	TCG_REQUIRE(ctx, graph != ctx->capturing, "tcg_graph_destroy: the graph is still being captured");
	// a launch of it may still be in flight: graph_release waits for the
	// graph's last launch (also while another sequence is being recorded, when
	// the stream itself cannot be waited for)
	graph_release(ctx, graph);
	return TCG_OK;
}

} // extern "C"
