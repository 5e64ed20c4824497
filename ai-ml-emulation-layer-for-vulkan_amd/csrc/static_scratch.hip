// The statically allocated device scratch behind mlel_hip_conv2d_rescale_clamp_static, the entry point for callers
// that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
//
// `scratch` is a file-scope device array: every GPU the library runs on holds its own copy, at its own address, until
// the process ends.  In host code the array's name is only a stand-in for the symbol, not a device address; the
// address on a device comes from hipGetSymbolAddress with that device current, once per context, and everything on
// the host side (kernel arguments, fills) uses that pointer.  Layout: kStaticScratchPartialBytes of int32 staging
// (split-K partial tiles, or the int32 accumulator of the unfused operator sequence), then kSplitCounters arrival
// counters.  All calls on one GPU share the array, so calls that overlap on one GPU race.
#include "common.hpp"

namespace mlel {
namespace {

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

__global__ void __launch_bounds__(256) clear_words_kernel(uint32_t *p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace

int static_scratch_init(mlel_ctx *ctx) {
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        ctx->static_scratch = nullptr;
        return set_error(MLEL_ERR_DEVICE, "hipGetSymbolAddress(scratch) failed on device %d: %s", ctx->device,
                         hipGetErrorString(e));
    }
    ctx->static_scratch = static_cast<char *>(ptr);
    return 0;
}

// A fill kernel, not hipMemsetAsync: a caller may be capturing the stream into a graph.
int static_scratch_clear_counters(mlel_ctx *ctx, hipStream_t s) {
    MLEL_REQUIRE(ctx->static_scratch != nullptr, MLEL_ERR_DEVICE, "the static scratch has no address on device %d",
                 ctx->device);
    uint32_t *counters = reinterpret_cast<uint32_t *>(ctx->static_scratch + kStaticScratchPartialBytes);
    hipLaunchKernelGGL(clear_words_kernel, dim3((kSplitCounters + 255) / 256), dim3(256), 0, s, counters,
                       kSplitCounters);
    return check_launch("static scratch clear");
}

}  // namespace mlel
