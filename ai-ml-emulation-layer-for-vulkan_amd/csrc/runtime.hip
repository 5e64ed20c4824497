// Context, device arena, streams, events, HIP-graph capture and the calibration copy kernel of the C ABI
// declared in include/mlel_hip.h.
#include "common.hpp"

#include <cstdlib>
#include <cstring>

namespace mlel {

static thread_local char g_error[1024] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(MLEL_ERR_DEVICE, "%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

int check_tensor(const mlel_tensor *t, const char *what) {
    MLEL_REQUIRE(t != nullptr, MLEL_ERR_INVALID, "%s: null tensor", what);
    MLEL_REQUIRE(t->rank >= 1 && t->rank <= MLEL_MAX_RANK, MLEL_ERR_INVALID, "%s: rank %d outside 1..6", what,
                 t->rank);
    MLEL_REQUIRE(dt_size(t->dtype) != 0, MLEL_ERR_INVALID, "%s: unknown dtype %d", what, t->dtype);
    int64_t n = 1;
    for (int i = 0; i < t->rank; i++) {
        MLEL_REQUIRE(t->dims[i] >= 0, MLEL_ERR_INVALID, "%s: negative dimension", what);
        MLEL_REQUIRE(t->strides[i] >= 0, MLEL_ERR_INVALID, "Strides must be greater than zero.");
        n *= t->dims[i];
    }
    MLEL_REQUIRE(t->ptr != nullptr || n == 0, MLEL_ERR_INVALID, "%s: null data pointer", what);
    return 0;
}

int64_t numel(const mlel_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->rank; i++) n *= t->dims[i];
    return n;
}

bool is_packed(const mlel_tensor *t) {
    int64_t s = dt_size(t->dtype);
    for (int i = t->rank - 1; i >= 0; i--) {
        if (t->dims[i] != 1 && t->strides[i] != s) return false;
        s *= t->dims[i];
    }
    return true;
}

bool same_shape(const mlel_tensor *a, const mlel_tensor *b) {
    if (a->rank != b->rank) return false;
    for (int i = 0; i < a->rank; i++)
        if (a->dims[i] != b->dims[i]) return false;
    return true;
}

int make_rescale_params(const mlel_rescale_attr *attr, int in_dtype, int out_dtype, const mlel_clamp_attr *clamp,
                        RescaleParams *out) {
    MLEL_REQUIRE(dt_is_int(in_dtype) && dt_is_int(out_dtype), MLEL_ERR_INVALID, "rescale: integer types only");
    const int in_dt = dt_unsigned_twin(in_dtype, attr->input_unsigned != 0);
    const int out_dt = dt_unsigned_twin(out_dtype, attr->output_unsigned != 0);
    out->in_zp = (int32_t)narrow_to(in_dt, attr->input_zp);
    out->out_zp = (int32_t)narrow_to(out_dt, attr->output_zp);
    out->double_round = (attr->scale32 && attr->double_round) ? 1 : 0;
    out->per_channel = attr->per_channel ? 1 : 0;
    out->clamp_out = (dt_size(out_dt) < 4) ? 1 : 0;
    int64_t lo = dt_lowest(out_dt), hi = dt_max(out_dt);
    if (dt_size(out_dt) >= 4) {
        lo = INT32_MIN;
        hi = INT32_MAX;
    }
    if (clamp != nullptr) {
        // CLAMP on the narrowed value: clamp(clamp(x, lo, hi), cmin, cmax) == clamp(x, clamp(lo), clamp(hi)).
        // The bounds are converted to the storage type by truncation toward zero (clamp.comp:32-33).
        const int cl_dt = out_dtype;
        int64_t cmin = narrow_to(cl_dt, (int64_t)clamp->min_val);
        int64_t cmax = narrow_to(cl_dt, (int64_t)clamp->max_val);
        MLEL_REQUIRE(cmin <= cmax, MLEL_ERR_INVALID, "clamp: min %lld > max %lld", (long long)cmin, (long long)cmax);
        MLEL_REQUIRE(!attr->output_unsigned, MLEL_ERR_UNSUPPORTED, "fused clamp on an unsigned rescale output");
        auto cl = [&](int64_t v) { return v < cmin ? cmin : (v > cmax ? cmax : v); };
        lo = cl(lo);
        hi = cl(hi);
        out->clamp_out = 1;
    }
    out->out_lo = (int32_t)lo;
    out->out_hi = (int32_t)hi;
    return 0;
}

int check_scale_tensors(const mlel_tensor *mult, const mlel_tensor *shift, const mlel_rescale_attr *attr,
                        int64_t channels) {
    MLEL_TRY(check_tensor(mult, "rescale multiplier"));
    MLEL_TRY(check_tensor(shift, "rescale shift"));
    MLEL_REQUIRE(mult->rank == 1 && shift->rank == 1, MLEL_ERR_INVALID, "rescale: multiplier/shift must be rank 1");
    MLEL_REQUIRE(mult->dtype == (attr->scale32 ? MLEL_I32 : MLEL_I16), MLEL_ERR_INVALID,
                 "rescale: multiplier must be %s", attr->scale32 ? "int32 (scale32)" : "int16");
    MLEL_REQUIRE(shift->dtype == MLEL_I8, MLEL_ERR_INVALID, "rescale: shift must be int8");
    const int64_t need = attr->per_channel ? channels : 1;
    MLEL_REQUIRE(mult->dims[0] >= need && shift->dims[0] >= need, MLEL_ERR_INVALID,
                 "rescale: multiplier/shift shorter than %lld channels", (long long)need);
    return 0;
}

// 128-bit device-to-device copy; tail handled bytewise.
__global__ void __launch_bounds__(256) copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src,
                                                   size_t n_vec, char *__restrict__ dst_tail,
                                                   const char *__restrict__ src_tail, size_t n_tail) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride) dst[i] = src[i];
    if (blockIdx.x == 0 && threadIdx.x < n_tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}

bool stream_is_capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

bool split_workspace(mlel_ctx *ctx, hipStream_t stream, SplitWorkspace *out) {
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    for (int i = 0; i < ctx->n_ws; i++)
        if (ctx->ws[i].stream == stream) {
            *out = ctx->ws[i];
            return true;
        }
    // a new workspace is an allocation: not inside a capture, and not beyond the table
    if (ctx->n_ws >= kMaxSplitWorkspaces || stream_is_capturing(stream)) return false;
    SplitWorkspace w{stream, nullptr, nullptr};
    if (hipMalloc(reinterpret_cast<void **>(&w.partials), kSplitPartialBytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (hipMalloc(reinterpret_cast<void **>(&w.counters), sizeof(uint32_t) * kSplitCounters) != hipSuccess ||
        hipMemset(w.counters, 0, sizeof(uint32_t) * kSplitCounters) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(w.partials);
        if (w.counters) (void)hipFree(w.counters);
        return false;
    }
    ctx->ws[ctx->n_ws++] = w;
    *out = w;
    return true;
}

void free_split_workspaces(mlel_ctx *ctx) {
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    for (int i = 0; i < ctx->n_ws; i++) {
        (void)hipFree(ctx->ws[i].partials);
        (void)hipFree(ctx->ws[i].counters);
    }
    ctx->n_ws = 0;
}

}  // namespace mlel

using namespace mlel;

extern "C" {

const char *mlel_hip_last_error(void) { return g_error; }

int mlel_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int mlel_hip_init(int device, mlel_ctx **out_ctx) {
    MLEL_REQUIRE(out_ctx != nullptr, MLEL_ERR_INVALID, "init: null out_ctx");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        (void)hipGetLastError();
        return set_error(MLEL_ERR_DEVICE, "init: no HIP device visible (%s); this backend has no CPU fallback",
                         e != hipSuccess ? hipGetErrorString(e) : "device count 0");
    }
    MLEL_REQUIRE(device >= 0 && device < n, MLEL_ERR_INVALID, "init: device %d outside 0..%d", device, n - 1);
    MLEL_HIP_CHECK(hipSetDevice(device));
    mlel_ctx *ctx = new mlel_ctx();
    ctx->device = device;
    hipError_t pe = hipGetDeviceProperties(&ctx->props, device);
    if (pe != hipSuccess) {
        delete ctx;
        return set_error(MLEL_ERR_DEVICE, "init: hipGetDeviceProperties: %s", hipGetErrorString(pe));
    }
    if (const char *env = std::getenv("MLEL_SPLIT_K")) ctx->split_k = std::atoi(env);  // 0: off, n: at most n splits
    // this device's address of the static scratch array; a failure only disables the entry point that needs it
    (void)static_scratch_init(ctx);
    *out_ctx = ctx;
    return 0;
}

void mlel_hip_destroy(mlel_ctx *ctx) {
    if (ctx == nullptr) return;
    if (hipSetDevice(ctx->device) == hipSuccess) {
        (void)hipDeviceSynchronize();  // no launch may still be using a workspace that is about to be freed
        free_split_workspaces(ctx);
    }
    delete ctx;
}

int mlel_hip_device_info(mlel_ctx *ctx, int32_t *cu_count, int32_t *clock_khz, int32_t *mem_clock_khz,
                         int32_t *bus_width_bits, char *name, size_t name_len) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "device_info: null ctx");
    if (cu_count) *cu_count = ctx->props.multiProcessorCount;
    if (clock_khz) *clock_khz = ctx->props.clockRate;
    if (mem_clock_khz) *mem_clock_khz = ctx->props.memoryClockRate;
    if (bus_width_bits) *bus_width_bits = ctx->props.memoryBusWidth;
    if (name && name_len) {
        snprintf(name, name_len, "%s (%s)", ctx->props.name, ctx->props.gcnArchName);
    }
    return 0;
}

int mlel_hip_arena_alloc(mlel_ctx *ctx, size_t bytes, void **dptr) {
    MLEL_REQUIRE(ctx != nullptr && dptr != nullptr, MLEL_ERR_INVALID, "arena_alloc: null argument");
    *dptr = nullptr;
    if (bytes == 0) bytes = 16;
    MLEL_HIP_CHECK(hipSetDevice(ctx->device));
    MLEL_HIP_CHECK(hipMalloc(dptr, bytes));
    MLEL_HIP_CHECK(hipMemset(*dptr, 0, bytes));  // tensors start zero-filled, as the reference's test tensors do
    return 0;
}

int mlel_hip_arena_free(mlel_ctx *ctx, void *dptr) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "arena_free: null ctx");
    if (dptr) MLEL_HIP_CHECK(hipFree(dptr));
    return 0;
}

int mlel_hip_arena_import_fd(mlel_ctx *ctx, int fd, size_t bytes, void **dptr, void **out_handle) {
    MLEL_REQUIRE(ctx != nullptr && dptr != nullptr && out_handle != nullptr, MLEL_ERR_INVALID,
                 "arena_import_fd: null argument");
    MLEL_REQUIRE(fd >= 0 && bytes > 0, MLEL_ERR_INVALID, "arena_import_fd: bad fd or size");
    hipExternalMemoryHandleDesc desc;
    memset(&desc, 0, sizeof(desc));
    desc.type = hipExternalMemoryHandleTypeOpaqueFd;
    desc.handle.fd = fd;
    desc.size = bytes;
    hipExternalMemory_t ext = nullptr;
    MLEL_HIP_CHECK(hipImportExternalMemory(&ext, &desc));
    hipExternalMemoryBufferDesc buf;
    memset(&buf, 0, sizeof(buf));
    buf.offset = 0;
    buf.size = bytes;
    hipError_t e = hipExternalMemoryGetMappedBuffer(dptr, ext, &buf);
    if (e != hipSuccess) {
        (void)hipDestroyExternalMemory(ext);
        return set_error(MLEL_ERR_DEVICE, "hipExternalMemoryGetMappedBuffer: %s", hipGetErrorString(e));
    }
    *out_handle = ext;
    return 0;
}

int mlel_hip_arena_release_import(mlel_ctx *ctx, void *handle) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "arena_release_import: null ctx");
    if (handle) MLEL_HIP_CHECK(hipDestroyExternalMemory((hipExternalMemory_t)handle));
    return 0;
}

int mlel_hip_memcpy_h2d(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memcpy_h2d: null ctx");
    if (bytes == 0) return 0;
    MLEL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_memcpy_d2h(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memcpy_d2h: null ctx");
    if (bytes == 0) return 0;
    MLEL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_memcpy_d2d(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memcpy_d2d: null ctx");
    if (bytes == 0) return 0;
    MLEL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return 0;
}

int mlel_hip_memset(mlel_ctx *ctx, void *dst, int value, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memset: null ctx");
    if (bytes == 0) return 0;
    MLEL_HIP_CHECK(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
    return 0;
}

int mlel_hip_stream_create(mlel_ctx *ctx, void **out_stream) {
    MLEL_REQUIRE(ctx != nullptr && out_stream != nullptr, MLEL_ERR_INVALID, "stream_create: null argument");
    hipStream_t s;
    MLEL_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *out_stream = s;
    return 0;
}

int mlel_hip_stream_destroy(mlel_ctx *ctx, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "stream_destroy: null ctx");
    if (stream) MLEL_HIP_CHECK(hipStreamDestroy((hipStream_t)stream));
    return 0;
}

int mlel_hip_sync(mlel_ctx *ctx, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "sync: null ctx");
    if (stream)
        MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    else
        MLEL_HIP_CHECK(hipDeviceSynchronize());
    return 0;
}

int mlel_hip_event_create(mlel_ctx *ctx, void **out_event) {
    MLEL_REQUIRE(ctx != nullptr && out_event != nullptr, MLEL_ERR_INVALID, "event_create: null argument");
    hipEvent_t e;
    MLEL_HIP_CHECK(hipEventCreate(&e));
    *out_event = e;
    return 0;
}

int mlel_hip_event_destroy(mlel_ctx *ctx, void *event) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "event_destroy: null ctx");
    if (event) MLEL_HIP_CHECK(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int mlel_hip_event_record(mlel_ctx *ctx, void *event, void *stream) {
    MLEL_REQUIRE(ctx != nullptr && event != nullptr, MLEL_ERR_INVALID, "event_record: null argument");
    MLEL_HIP_CHECK(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return 0;
}

int mlel_hip_event_elapsed_ms(mlel_ctx *ctx, void *start, void *stop, float *ms) {
    MLEL_REQUIRE(ctx != nullptr && start && stop && ms, MLEL_ERR_INVALID, "event_elapsed_ms: null argument");
    MLEL_HIP_CHECK(hipEventSynchronize((hipEvent_t)stop));
    MLEL_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

int mlel_hip_capture_begin(mlel_ctx *ctx, void *stream) {
    MLEL_REQUIRE(ctx != nullptr && stream != nullptr, MLEL_ERR_INVALID,
                 "capture_begin: a non-null stream is required");
    MLEL_HIP_CHECK(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return 0;
}

int mlel_hip_capture_end(mlel_ctx *ctx, void *stream, void **out_graph_exec) {
    MLEL_REQUIRE(ctx != nullptr && stream != nullptr && out_graph_exec != nullptr, MLEL_ERR_INVALID,
                 "capture_end: null argument");
    hipGraph_t graph = nullptr;
    MLEL_HIP_CHECK(hipStreamEndCapture((hipStream_t)stream, &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return set_error(MLEL_ERR_DEVICE, "hipGraphInstantiate: %s", hipGetErrorString(e));
    *out_graph_exec = exec;
    return 0;
}

int mlel_hip_graph_launch(mlel_ctx *ctx, void *graph_exec, void *stream) {
    MLEL_REQUIRE(ctx != nullptr && graph_exec != nullptr, MLEL_ERR_INVALID, "graph_launch: null argument");
    MLEL_HIP_CHECK(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
    return 0;
}

int mlel_hip_graph_destroy(mlel_ctx *ctx, void *graph_exec) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "graph_destroy: null ctx");
    if (graph_exec) MLEL_HIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return 0;
}

int mlel_hip_copy_kernel(mlel_ctx *ctx, void *stream, void *dst, const void *src, size_t bytes) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "copy_kernel: null ctx");
    if (bytes == 0) return 0;
    MLEL_REQUIRE(dst && src, MLEL_ERR_INVALID, "copy_kernel: null pointer");
    MLEL_REQUIRE(((uintptr_t)dst % 16) == 0 && ((uintptr_t)src % 16) == 0, MLEL_ERR_INVALID,
                 "copy_kernel: pointers must be 16-byte aligned");
    const size_t n_vec = bytes / 16, n_tail = bytes % 16;
    size_t blocks = (n_vec + 255) / 256;
    const size_t max_blocks = (size_t)ctx->props.multiProcessorCount * 16;
    if (blocks > max_blocks) blocks = max_blocks;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint4 *)dst,
                       (const uint4 *)src, n_vec, (char *)dst + n_vec * 16, (const char *)src + n_vec * 16, n_tail);
    return check_launch("copy_kernel");
}

}  // extern "C"
