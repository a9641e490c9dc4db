// Context lifetime, error reporting, the format table and device-memory entry points of libskainet_hip.
#include "common.h"

static thread_local std::string g_ctxless_error;

int skn_fail(skn_ctx* ctx, int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    if (ctx) ctx->err = buf;
    else g_ctxless_error = buf;
    return code;
}

extern "C" {

int skn_abi_version(void) { return SKN_ABI_VERSION; }

const char* skn_status_string(int code) {
    switch (code) {
        case SKN_OK: return "ok";
        case SKN_ERR_ARG: return "invalid argument";
        case SKN_ERR_TYPE: return "unsupported ggml type";
        case SKN_ERR_SHAPE: return "shape mismatch";
        case SKN_ERR_OOM: return "out of memory";
        case SKN_ERR_HIP: return "HIP runtime error";
        case SKN_ERR_RANGE: return "index out of range";
        case SKN_ERR_POOL: return "KV pool exhausted";
        case SKN_ERR_STATE: return "invalid state";
        default: return "unknown status";
    }
}

const char* skn_last_error(skn_ctx* ctx) { return ctx ? ctx->err.c_str() : g_ctxless_error.c_str(); }

int skn_init(int device, skn_ctx** out) {
    SKN_REQUIRE(nullptr, out != nullptr, SKN_ERR_ARG, "skn_init: out is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return skn_fail(nullptr, SKN_ERR_HIP, "skn_init: no HIP device (%s)", hipGetErrorString(e));
    SKN_REQUIRE(nullptr, device >= 0 && device < count, SKN_ERR_ARG, "skn_init: device %d of %d", device, count);
    SKN_HIP(nullptr, hipSetDevice(device));
    hipDeviceProp_t prop;
    SKN_HIP(nullptr, hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return skn_fail(nullptr, SKN_ERR_STATE, "skn_init: built for gfx950, device is %s", prop.gcnArchName);
    skn_ctx* ctx = new (std::nothrow) skn_ctx();
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_OOM, "skn_init: host allocation failed");
    ctx->device = device;
    ctx->compute_units = prop.multiProcessorCount;
    ctx->lds_per_block = prop.sharedMemPerBlock;
    e = hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev_start);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev_stop);
    if (e != hipSuccess) {
        int rc = skn_fail(nullptr, SKN_ERR_HIP, "skn_init: stream/event creation failed: %s", hipGetErrorString(e));
        skn_shutdown(ctx);
        return rc;
    }
    ctx->stream = ctx->own_stream;
    {
        // rocprofv3 announces its tool library in ROCP_TOOL_LIBRARIES and preloads librocprofiler-sdk-tool; replaying a
        // captured graph under its kernel trace has ended in a fault, so with a profiler attached every decode step
        // is launched kernel by kernel
        const char* tool = getenv("ROCP_TOOL_LIBRARIES");
        const char* pre = getenv("LD_PRELOAD");
        ctx->profiler_attached = (tool && *tool) || (pre && strstr(pre, "rocprofiler"));
        if (ctx->profiler_attached) ctx->opt_llama_graph = 0;
    }
    int rc = skn_matvec_init(ctx);
    if (rc == SKN_OK) rc = skn_gemm_init(ctx);
    if (rc == SKN_OK) rc = skn_attn_init(ctx);
    if (rc != SKN_OK) {
        g_ctxless_error = ctx->err;
        skn_shutdown(ctx);
        return rc;
    }
    *out = ctx;
    return SKN_OK;
}

void skn_shutdown(skn_ctx* ctx) {
    if (!ctx) return;
    if (ctx->own_stream) (void)hipStreamSynchronize(ctx->own_stream);
    if (ctx->attn_scratch) (void)hipFree(ctx->attn_scratch);
    if (ctx->attn_counters) (void)hipFree(ctx->attn_counters);
    if (ctx->gemm_ws) (void)hipFree(ctx->gemm_ws);
    if (ctx->split_scratch) (void)hipFree(ctx->split_scratch);
    if (ctx->prefill_ws) (void)hipFree(ctx->prefill_ws);
    for (hipEvent_t e : ctx->prof_events) (void)hipEventDestroy(e);
    if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
    delete ctx;
}

int skn_device_info(skn_ctx* ctx, char* name, size_t name_len, int* compute_units, size_t* total_bytes) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_device_info: ctx is null");
    hipDeviceProp_t prop;
    SKN_HIP(ctx, hipGetDeviceProperties(&prop, ctx->device));
    if (name && name_len) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_bytes) *total_bytes = prop.totalGlobalMem;
    return SKN_OK;
}

int skn_type_block(int ggml_type, int* block_elems, int* block_bytes) {
    int be, bb;
    // the whole table of gguf/.../Constants.kt:58-90, keyed by the ids of :14-46
    static const struct { int id, elems, bytes; } kTable[] = {
        {0, 1, 4},          // F32
        {1, 1, 2},          // F16
        {2, 32, 2 + 16},    // Q4_0
        {3, 32, 2 + 2 + 16},        // Q4_1
        {6, 32, 2 + 4 + 16},        // Q5_0
        {7, 32, 2 + 2 + 4 + 16},    // Q5_1
        {8, 32, 2 + 32},            // Q8_0
        {9, 32, 4 + 4 + 32},        // Q8_1
        {10, 256, 2 + 2 + 256 / 16 + 256 / 4},            // Q2_K
        {11, 256, 2 + 256 / 4 + 256 / 8 + 12},            // Q3_K
        {12, 256, 2 + 2 + 256 / 2 + 12},                  // Q4_K
        {13, 256, 2 + 2 + 256 / 2 + 256 / 8 + 12},        // Q5_K
        {14, 256, 2 + 256 / 2 + 256 / 4 + 256 / 16},      // Q6_K
        {15, 256, 4 + 256 + 256 / 8},                     // Q8_K
        {16, 256, 2 + 256 / 4},                           // IQ2_XXS
        {17, 256, 2 + 256 / 4 + 256 / 32},                // IQ2_XS
        {18, 256, 2 + 256 / 4 + 256 / 8},                 // IQ3_XXS
        {19, 256, 2 + 256 / 8 + 256 / 16},                // IQ1_S
        {20, 32, 2 + 16},                                 // IQ4_NL
        {21, 256, 2 + 256 / 4 + 256 / 8 + 256 / 32 + 4},  // IQ3_S
        {22, 256, 2 + 256 / 4 + 256 / 16},                // IQ2_S
        {23, 256, 2 + 2 + 256 / 2 + 256 / 64},            // IQ4_XS
        {24, 1, 1}, {25, 1, 2}, {26, 1, 4}, {27, 1, 8},   // I8, I16, I32, I64
        {28, 1, 8},                                       // F64
        {29, 256, 256 / 8 + 256 / 16 + 256 / 32},         // IQ1_M
        {30, 1, 2},                                       // BF16
        {34, 256, 2 + 4 * 13},                            // TQ1_0
        {35, 256, 2 + 64},                                // TQ2_0
    };
    be = bb = 0;
    for (const auto& row : kTable)
        if (row.id == ggml_type) {
            be = row.elems;
            bb = row.bytes;
        }
    if (be == 0) return skn_fail(nullptr, SKN_ERR_TYPE, "ggml type %d is not in the size table", ggml_type);
    if (block_elems) *block_elems = be;
    if (block_bytes) *block_bytes = bb;
    return SKN_OK;
}

int64_t skn_row_bytes(int ggml_type, int64_t k) {
    int be, bb;
    int rc = skn_type_block(ggml_type, &be, &bb);
    if (rc != SKN_OK) return rc;
    if (k < 0 || k % be != 0)
        return skn_fail(nullptr, SKN_ERR_SHAPE, "Quantized tensor row size (%lld) is not a multiple of block size (%d)",
                        (long long)k, be);
    return k / be * bb;
}

int skn_malloc(skn_ctx* ctx, size_t bytes, void** dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_malloc: ctx is null");
    SKN_REQUIRE(ctx, dev != nullptr, SKN_ERR_ARG, "skn_malloc: dev is null");
    *dev = nullptr;
    if (bytes == 0) return SKN_OK;
    hipError_t e = hipMalloc(dev, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return skn_fail(ctx, SKN_ERR_OOM, "skn_malloc: %zu bytes: %s", bytes, hipGetErrorString(e));
    }
    return SKN_OK;
}

int skn_free(skn_ctx* ctx, void* dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_free: ctx is null");
    if (!dev) return SKN_OK;
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    SKN_HIP(ctx, hipFree(dev));
    return SKN_OK;
}

int skn_upload(skn_ctx* ctx, void* dev, const void* host, size_t bytes) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_upload: ctx is null");
    if (bytes == 0) return SKN_OK;
    SKN_REQUIRE(ctx, dev && host, SKN_ERR_ARG, "skn_upload: null pointer");
    SKN_HIP(ctx, hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, ctx->stream));
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SKN_OK;
}

int skn_download(skn_ctx* ctx, void* host, const void* dev, size_t bytes) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_download: ctx is null");
    if (bytes == 0) return SKN_OK;
    SKN_REQUIRE(ctx, dev && host, SKN_ERR_ARG, "skn_download: null pointer");
    SKN_HIP(ctx, hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SKN_OK;
}

__global__ void fill_bytes_kernel(uint8_t* p, uint8_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

int skn_memset(skn_ctx* ctx, void* dev, int byte_value, size_t bytes) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_memset: ctx is null");
    if (bytes == 0) return SKN_OK;
    SKN_REQUIRE(ctx, dev != nullptr, SKN_ERR_ARG, "skn_memset: null pointer");
    // a fill kernel rather than hipMemsetAsync, so that callers may capture this call into a HIP graph
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    skn_launch(ctx, fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, (uint8_t*)dev,
                       (uint8_t)byte_value, bytes);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

__global__ __launch_bounds__(256) void copy16_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

__global__ void copy_bytes_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

int skn_copy(skn_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_copy: ctx is null");
    if (bytes == 0) return SKN_OK;
    SKN_REQUIRE(ctx, dst_dev && src_dev, SKN_ERR_ARG, "skn_copy: null pointer");
    // a plain streaming kernel (128-bit loads and stores when both ends are 16-byte aligned); it doubles as the
    // known-size workload against which hardware traffic counters are calibrated
    if ((((uintptr_t)dst_dev | (uintptr_t)src_dev | bytes) & 15) == 0) {
        const size_t n16 = bytes / 16;
        size_t blocks = (n16 + 255) / 256;
        if (blocks > 2048) blocks = 2048;
        skn_launch(ctx, copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, (const uint4*)src_dev, (uint4*)dst_dev, n16);
    } else {
        size_t blocks = (bytes + 255) / 256;
        if (blocks > 2048) blocks = 2048;
        skn_launch(ctx, copy_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, (const uint8_t*)src_dev,
                   (uint8_t*)dst_dev, bytes);
    }
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_sync(skn_ctx* ctx) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_sync: ctx is null");
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SKN_OK;
}

int skn_set_stream(skn_ctx* ctx, void* hip_stream) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_set_stream: ctx is null");
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
    ctx->opt_generation++;  // graphs captured on the other stream are not replayed on this one
    return SKN_OK;
}

int skn_set_option(skn_ctx* ctx, const char* key, int value) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_set_option: ctx is null");
    SKN_REQUIRE(ctx, key != nullptr, SKN_ERR_ARG, "skn_set_option: key is null");
    if (!strcmp(key, "q4k.waves")) ctx->opt_q4k_waves = value;
    else if (!strcmp(key, "q4k.rows")) ctx->opt_q4k_rows = value;
    else if (!strcmp(key, "q4k.split")) ctx->opt_q4k_split = value;
    else if (!strcmp(key, "attn.splits")) ctx->opt_attn_splits = value;
    else if (!strcmp(key, "llama.graph")) {
        SKN_REQUIRE(ctx, !(value && ctx->profiler_attached), SKN_ERR_STATE,
                    "skn_set_option: llama.graph stays 0 while a rocprofiler tool library is attached to the process");
        ctx->opt_llama_graph = value;
    }
    else if (!strcmp(key, "llama.fused")) ctx->opt_llama_fused = value;
    else if (!strcmp(key, "llama.expand_weights")) ctx->opt_llama_expand = value;
    else if (!strcmp(key, "gemm.tile")) ctx->opt_gemm_tile = value;
    else if (!strcmp(key, "gemm.q6k_fused")) ctx->opt_gemm_q6k_fused = value;
    else if (!strcmp(key, "matvec.stage")) ctx->opt_matvec_stage = value;
    else if (!strcmp(key, "test.rope_table")) ctx->opt_test_rope_table = value;
    else if (!strcmp(key, "llama.attn_wide")) ctx->opt_llama_attn_wide = value;
    else return skn_fail(ctx, SKN_ERR_ARG, "skn_set_option: unknown option '%s'", key);
    ctx->opt_generation++;  // whatever was captured with the old settings is stale
    return SKN_OK;
}

int skn_get_stat(skn_ctx* ctx, const char* key, int64_t* value) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_get_stat: ctx is null");
    SKN_REQUIRE(ctx, key && value, SKN_ERR_ARG, "skn_get_stat: null pointer");
    if (!strcmp(key, "launches")) *value = ctx->stat_launches;
    else if (!strcmp(key, "graph.captures")) *value = ctx->stat_captures;
    else if (!strcmp(key, "llama.expanded_bytes")) *value = ctx->stat_expanded_bytes;
    else if (!strcmp(key, "profiler.attached")) *value = ctx->profiler_attached ? 1 : 0;
    else return skn_fail(ctx, SKN_ERR_ARG, "skn_get_stat: unknown counter '%s'", key);
    return SKN_OK;
}

int skn_timer_start(skn_ctx* ctx) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_timer_start: ctx is null");
    SKN_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
    ctx->timer_running = true;
    return SKN_OK;
}

int skn_timer_stop(skn_ctx* ctx, float* elapsed_ms) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_timer_stop: ctx is null");
    SKN_REQUIRE(ctx, elapsed_ms != nullptr, SKN_ERR_ARG, "skn_timer_stop: elapsed_ms is null");
    SKN_REQUIRE(ctx, ctx->timer_running, SKN_ERR_STATE, "skn_timer_stop: timer was not started");
    SKN_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
    SKN_HIP(ctx, hipEventSynchronize(ctx->ev_stop));
    SKN_HIP(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop));
    ctx->timer_running = false;
    return SKN_OK;
}

}  // extern "C"

extern "C" {

// Per-launch kernel timing: between start and stop every kernel launch of this context carries its own
// start/stop events; stop waits for the stream and returns the summed kernel durations.
int skn_prof_start(skn_ctx* ctx, int max_launches) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_prof_start: ctx is null");
    SKN_REQUIRE(ctx, max_launches > 0 && max_launches <= (1 << 20), SKN_ERR_ARG, "skn_prof_start: bad capacity");
    SKN_REQUIRE(ctx, !ctx->prof_on, SKN_ERR_STATE, "skn_prof_start: already profiling");
    while (ctx->prof_events.size() < 2 * (size_t)max_launches) {
        hipEvent_t e;
        SKN_HIP(ctx, hipEventCreate(&e));
        ctx->prof_events.push_back(e);
    }
    ctx->prof_used = 0;
    ctx->prof_on = true;
    return SKN_OK;
}

int skn_prof_stop(skn_ctx* ctx, double* kernel_ms_total, int* launches) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_prof_stop: ctx is null");
    SKN_REQUIRE(ctx, ctx->prof_on, SKN_ERR_STATE, "skn_prof_stop: not profiling");
    ctx->prof_on = false;
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    double total = 0.0;
    for (size_t i = 0; i < ctx->prof_used; i++) {
        float ms = 0.f;
        SKN_HIP(ctx, hipEventElapsedTime(&ms, ctx->prof_events[2 * i], ctx->prof_events[2 * i + 1]));
        total += ms;
    }
    if (kernel_ms_total) *kernel_ms_total = total;
    if (launches) *launches = (int)ctx->prof_used;
    return SKN_OK;
}

}  // extern "C"
