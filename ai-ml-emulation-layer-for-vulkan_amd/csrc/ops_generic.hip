// Generic kernels: one thread per output element, any rank <= 6, any byte strides, every dtype combination the
// backend accepts.  They carry the full operator semantics (out-of-bounds reads give 0, out-of-bounds writes are
// dropped, size-1 broadcast, NaN modes, wraparound integer arithmetic) and serve every case the specialised
// kernels (gemm_i8.hip, ops_fast.hip) do not take.  Each kernel states the reference shader whose results it
// reproduces.
#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {

namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ int64_t global_flat() { return (int64_t)blockIdx.x * blockDim.x + threadIdx.x; }

__device__ __forceinline__ int32_t wadd32(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
__device__ __forceinline__ int32_t wmul32(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }
__device__ __forceinline__ int64_t wadd64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a + (uint64_t)b); }
__device__ __forceinline__ int64_t wmul64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a * (uint64_t)b); }

// ---------------------------------------------------------------------------------------------------------------
// CONV2D, direct form (reference results: conv2d.comp:40-116)
// ---------------------------------------------------------------------------------------------------------------
struct ConvArgs {
    int32_t zi, zw, pad_t, pad_l, sy, sx, dy, dx;
    uint32_t acc;
};

__global__ void __launch_bounds__(kBlock) conv2d_generic(TV out, TV in, TV w, TV bias, ConvArgs a, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t n = o[0], oy = o[1], ox = o[2], oc = o[3];
    const int64_t H = in.dims[1], W = in.dims[2], IC = in.dims[3], KH = w.dims[1], KW = w.dims[2];
    const bool facc = a.acc == MLEL_ACC_F16 || a.acc == MLEL_ACC_F32;
    int64_t iacc = 0;
    float facc_v = 0.f;
    for (int64_t ky = 0; ky < KH; ky++) {
        for (int64_t kx = 0; kx < KW; kx++) {
            const int64_t yy = oy * a.sy - a.pad_t + ky * a.dy;
            const int64_t xx = ox * a.sx - a.pad_l + kx * a.dx;
            if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
            for (int64_t ic = 0; ic < IC; ic++) {
                const int64_t xi[4] = {n, yy, xx, ic};
                const int64_t wi[4] = {oc, ky, kx, ic};
                if (!facc) {
                    const int64_t v = ld_acc_i(in, xi) - a.zi;
                    const int64_t ww = ld_acc_i(w, wi) - a.zw;
                    if (a.acc == MLEL_ACC_I32)
                        iacc = wadd32((int32_t)iacc, wmul32((int32_t)v, (int32_t)ww));
                    else
                        iacc = wadd64(iacc, wmul64(v, ww));
                } else {
                    float v = ld_f(in, xi), ww = ld_f(w, wi);
                    const float p = (v - (float)a.zi) * (ww - (float)a.zw);
                    if (a.acc == MLEL_ACC_F16)
                        facc_v = rnd_f16(facc_v + rnd_f16(p));
                    else
                        facc_v = facc_v + p;
                }
            }
        }
    }
    const int64_t bi[1] = {bias.dims[0] == 1 ? 0 : oc};
    if (!facc) {
        const int64_t b = ld_acc_i(bias, bi);
        st_acc_i(out, o, a.acc == MLEL_ACC_I32 ? (int64_t)wadd32((int32_t)iacc, (int32_t)b) : wadd64(iacc, b));
    } else {
        const float b = ld_f(bias, bi);
        st_f(out, o, a.acc == MLEL_ACC_F16 ? rnd_f16(facc_v + rnd_f16(b)) : facc_v + b, ST_ACC);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// DEPTHWISE_CONV2D, direct form (reference results: depthwise_conv2d.comp:31-78)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) dwconv_generic(TV out, TV in, TV w, TV bias, ConvArgs a, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t n = o[0], oy = o[1], ox = o[2], ocm = o[3];
    const int64_t H = in.dims[1], W = in.dims[2], KH = w.dims[0], KW = w.dims[1], M = w.dims[3];
    const int64_t c = ocm / M, m = ocm % M;
    const bool facc = a.acc == MLEL_ACC_F16 || a.acc == MLEL_ACC_F32;
    int64_t iacc = 0;
    float facc_v = 0.f;
    for (int64_t ky = 0; ky < KH; ky++) {
        for (int64_t kx = 0; kx < KW; kx++) {
            const int64_t yy = oy * a.sy - a.pad_t + ky * a.dy;
            const int64_t xx = ox * a.sx - a.pad_l + kx * a.dx;
            if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
            const int64_t xi[4] = {n, yy, xx, c};
            const int64_t wi[4] = {ky, kx, c, m};
            if (!facc) {
                const int64_t v = ld_acc_i(in, xi) - a.zi;
                const int64_t ww = ld_acc_i(w, wi) - a.zw;
                if (a.acc == MLEL_ACC_I32)
                    iacc = wadd32((int32_t)iacc, wmul32((int32_t)v, (int32_t)ww));
                else
                    iacc = wadd64(iacc, wmul64(v, ww));
            } else {
                const float p = (ld_f(in, xi) - (float)a.zi) * (ld_f(w, wi) - (float)a.zw);
                facc_v = a.acc == MLEL_ACC_F16 ? rnd_f16(facc_v + rnd_f16(p)) : facc_v + p;
            }
        }
    }
    const int64_t bi[1] = {bias.dims[0] == 1 ? 0 : ocm};
    if (!facc) {
        const int64_t b = ld_acc_i(bias, bi);
        st_acc_i(out, o, a.acc == MLEL_ACC_I32 ? (int64_t)wadd32((int32_t)b, (int32_t)iacc) : wadd64(b, iacc));
    } else {
        const float b = ld_f(bias, bi);
        st_f(out, o, a.acc == MLEL_ACC_F16 ? rnd_f16(rnd_f16(b) + facc_v) : b + facc_v, ST_ACC);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// MATMUL, direct form (reference results: matmul.comp:30-73); compute type = output type
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) matmul_generic(TV out, TV A, TV B, int32_t za, int32_t zb, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t C = A.dims[2];
    const int od = out.dtype;
    int64_t iacc = 0;
    float facc = 0.f;
    for (int64_t c = 0; c < C; c++) {
        const int64_t ai[3] = {o[0], o[1], c};
        const int64_t bi[3] = {o[0], c, o[2]};
        if (dt_is_int(od)) {
            const int64_t v1 = ld_i(A, ai) - za, v2 = ld_i(B, bi) - zb;
            if (od == MLEL_I32)
                iacc = wadd32((int32_t)iacc, wmul32((int32_t)v1, (int32_t)v2));
            else
                iacc = wadd64(iacc, wmul64(v1, v2));
        } else {
            const float p = (ld_f(A, ai) - (float)za) * (ld_f(B, bi) - (float)zb);
            facc = dt_comp(od) == MLEL_F16 ? rnd_f16(facc + rnd_f16(p)) : facc + p;
        }
    }
    if (dt_is_int(od))
        st_i(out, o, iacc);
    else
        st_f(out, o, facc);
}

// ---------------------------------------------------------------------------------------------------------------
// RESCALE (reference results: rescale.comp:27-72)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) rescale_generic(TV out, TV in, TV mult, TV shift, RescaleParams p,
                                                          int in_dt, int out_dt, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t c[1] = {p.per_channel ? o[out.rank - 1] : 0};
    TV in_v = in;
    in_v.dtype = in_dt;  // the (un)signed twin of the storage type
    const int64_t value = ld_i(in_v, o) - (int64_t)narrow_to(in_dt, p.in_zp);
    const int32_t m = (int32_t)ld_i(mult, c);
    const int32_t sh = (int32_t)(int8_t)ld_i(shift, c);
    int32_t r = apply_scale(value, m, sh, p.double_round != 0);
    r = wadd32(r, p.out_zp);
    int64_t res = r;
    if (p.clamp_out) res = res < p.out_lo ? p.out_lo : (res > p.out_hi ? p.out_hi : res);
    (void)out_dt;
    st_i(out, o, res);
}

// ---------------------------------------------------------------------------------------------------------------
// CLAMP (reference results: clamp.comp:24-53)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) clamp_generic(TV out, TV in, double mn_d, double mx_d, uint32_t nan_mode,
                                                        int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int dt = out.dtype;
    if (dt_is_int(dt)) {
        const int64_t mn = narrow_to(dt, (int64_t)mn_d), mx = narrow_to(dt, (int64_t)mx_d);
        int64_t v = ld_i(in, o);
        v = v < mn ? mn : v;
        v = v > mx ? mx : v;
        st_i(out, o, v);
    } else {
        const float mn = round_to(dt, (float)mn_d), mx = round_to(dt, (float)mx_d);
        float v = ld_f(in, o);
        if (isnan(v) && nan_mode == MLEL_NAN_IGNORE) v = mn;
        if (!isnan(v)) {
            v = v < mn ? mn : v;
            v = v > mx ? mx : v;
        }
        st_f(out, o, v);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// elementwise binary + MUL (reference results: elementwise_binary.comp:146-173, mul.comp:24-59)
// ---------------------------------------------------------------------------------------------------------------
__device__ inline void broadcast_idx(const TV &t, const int64_t *o, int64_t *idx) {
    for (int i = 0; i < t.rank; i++) idx[i] = t.dims[i] == 1 ? 0 : o[i];
}

__device__ inline float power_f(float base, float e) {
    if (base >= 0.f) return powf(base, e);
    if (e - 2.f * floorf(e / 2.f) == 0.f) return powf(-base, e);
    if (e - floorf(e) == 0.f) return -powf(-base, e);
    return NAN;
}

__global__ void __launch_bounds__(kBlock) binary_generic(int op, TV out, TV in1, TV in2, uint32_t nan_mode,
                                                         int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], i1[MLEL_MAX_RANK], i2[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    broadcast_idx(in1, o, i1);
    broadcast_idx(in2, o, i2);
    const int idt = in1.dtype;
    if (dt_is_float(idt)) {
        const float a = ld_f(in1, i1), b = ld_f(in2, i2);
        float r = 0.f;
        bool is_bool = false, br = false;
        switch (op) {
        case MLEL_BIN_ADD: r = a + b; break;
        case MLEL_BIN_SUB: r = a - b; break;
        case MLEL_BIN_MAXIMUM:
            if (isnan(a)) r = nan_mode == MLEL_NAN_PROPAGATE ? a : b;
            else if (isnan(b)) r = nan_mode == MLEL_NAN_PROPAGATE ? b : a;
            else r = a > b ? a : b;
            break;
        case MLEL_BIN_MINIMUM:
            if (isnan(a)) r = nan_mode == MLEL_NAN_PROPAGATE ? a : b;
            else if (isnan(b)) r = nan_mode == MLEL_NAN_PROPAGATE ? b : a;
            else r = a < b ? a : b;
            break;
        case MLEL_BIN_POW: r = power_f(a, b); break;
        case MLEL_BIN_EQUAL: is_bool = true; br = a == b; break;
        case MLEL_BIN_GREATER: is_bool = true; br = a > b; break;
        case MLEL_BIN_GREATER_EQUAL: is_bool = true; br = a >= b; break;
        default: break;
        }
        if (is_bool)
            st_i(out, o, br);
        else
            st_f(out, o, r, ST_RNE);  // one rounding into the storage type
    } else {
        const int64_t a = ld_i(in1, i1), b = ld_i(in2, i2);
        int64_t r = 0;
        switch (op) {
        case MLEL_BIN_ADD: r = wadd64(a, b); break;
        case MLEL_BIN_SUB: r = wadd64(a, -b); break;
        case MLEL_BIN_BITWISE_AND: r = a & b; break;
        case MLEL_BIN_BITWISE_OR: r = a | b; break;
        case MLEL_BIN_BITWISE_XOR: r = a ^ b; break;
        case MLEL_BIN_INTDIV: r = b == 0 ? 0 : (a == INT64_MIN && b == -1 ? a : a / b); break;
        case MLEL_BIN_LOGICAL_AND: r = (a != 0) && (b != 0); break;
        case MLEL_BIN_LOGICAL_OR: r = (a != 0) || (b != 0); break;
        case MLEL_BIN_LOGICAL_XOR: r = (a != 0) != (b != 0); break;
        case MLEL_BIN_LOGICAL_LEFT_SHIFT: r = (int64_t)((uint32_t)a << ((uint32_t)b & 31u)); break;
        case MLEL_BIN_LOGICAL_RIGHT_SHIFT: {
            const uint32_t z = idt == MLEL_I8 ? (uint8_t)a : idt == MLEL_I16 ? (uint16_t)a : (uint32_t)a;
            r = (int64_t)(z >> ((uint32_t)b & 31u));
            break;
        }
        case MLEL_BIN_MAXIMUM: r = a > b ? a : b; break;
        case MLEL_BIN_MINIMUM: r = a < b ? a : b; break;
        case MLEL_BIN_EQUAL: r = a == b; break;
        case MLEL_BIN_GREATER: r = a > b; break;
        case MLEL_BIN_GREATER_EQUAL: r = a >= b; break;
        default: break;
        }
        st_i(out, o, r);
    }
}

__global__ void __launch_bounds__(kBlock) mul_generic(TV out, TV in1, TV in2, uint32_t shift, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], i1[MLEL_MAX_RANK], i2[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    broadcast_idx(in1, o, i1);
    broadcast_idx(in2, o, i2);
    if (dt_is_float(in1.dtype)) {
        st_f(out, o, round_to(out.dtype, ld_f(in1, i1)) * round_to(out.dtype, ld_f(in2, i2)), ST_RNE);
    } else {
        int64_t r = wmul64(ld_i(in1, i1), ld_i(in2, i2));
        if (shift > 0) r = wadd64(r, int64_t(1) << (shift - 1)) >> (shift > 63 ? 63 : shift);
        st_i(out, o, r);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// elementwise unary (reference results: elementwise_unary.comp:16-205)
// ---------------------------------------------------------------------------------------------------------------
__device__ inline float erf_ref(float x) {
    const float coeffs[12] = {0.08f, 0.08695652173913043f, 0.09523809523809523f, 0.10526315789473684f,
                              0.11764705882352941f, 0.13333333333333333f, 0.15384615384615385f, 0.18181818181818182f,
                              0.22222222222222222f, 0.28571428571428571f, 0.4f, 0.66666666666666666f};
    const float pc[5][2] = {{3.47469513777439592f, 12.07402036406381411f}, {4.00561509202259545f, 9.30596659485887898f},
                            {5.95908795446633271f, 9.19435612886969243f},  {5.16722705817812584f, 9.12661617673673262f},
                            {2.71078540045147805f, 5.80755613130301624f}};
    const float qc[5][2] = {{3.47954057099518960f, 12.06166887286239555f}, {3.72068443960225092f, 8.44319781003968454f},
                            {3.90225704029924078f, 6.36161630953880464f},  {4.03296893109262491f, 5.13578530585681539f},
                            {4.11240942957450885f, 4.48640329523408675f}};
    const float sqrt_pi = 1.7724538509055159f, p0 = 0.56418958354775629f, q0 = 2.06955023132914151f;
    const float s = x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f);
    x = fabsf(x);
    if (x > 4.0f) return s;
    const float x2 = x * x;
    if (x < 0.6f) {
        float tot = 1.0f;
        for (int i = 0; i < 12; i++) tot = 1.0f + tot * coeffs[i] * x2;
        tot *= 2.0f * x * expf(-x2);
        tot /= sqrt_pi;
        return s * tot;
    }
    float prod = p0 / (x + q0);
    for (int i = 0; i < 5; i++) {
        const float p = x2 + x * pc[i][0] + pc[i][1];
        const float q = x2 + x * qc[i][0] + qc[i][1];
        prod *= p / q;
    }
    prod = 1.0f - prod * expf(-x2);
    return s * prod;
}

__device__ inline float sin_hybrid(float x) {
    if (fabsf(x) < 1.0e-3f) {
        const float c3 = -1.0f / 6.0f, c5 = 1.0f / 120.0f, c7 = -1.0f / 5040.0f, c9 = 1.0f / 362880.0f,
                    c11 = -1.0f / 39916800.0f;
        const float x2 = x * x;
        float p = (c11 * x2 + c9) * x2 + c7;
        p = p * x2 + c5;
        p = p * x2 + c3;
        p = p * x2 + 1.0f;
        return x * p;
    }
    return sinf(x);
}

__global__ void __launch_bounds__(kBlock) unary_generic(int op, TV out, TV in, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int dt = in.dtype;
    if (dt_is_float(dt)) {
        const float v = ld_f(in, o);
        float r = v;
        if (!isnan(v)) {
            switch (op) {
            case MLEL_UN_ABS: r = fabsf(v); break;
            case MLEL_UN_CEIL: r = ceilf(v); break;
            case MLEL_UN_FLOOR: r = floorf(v); break;
            case MLEL_UN_COS: r = cosf(v); break;
            case MLEL_UN_EXP: r = expf(v); break;
            case MLEL_UN_LOG: r = v < 0.f ? NAN : logf(v); break;
            case MLEL_UN_RECIPROCAL: r = 1.0f / v; break;
            case MLEL_UN_RSQRT: r = 1.0f / sqrtf(v); break;
            case MLEL_UN_SIGMOID: r = 1.0f / (1.0f + expf(-v)); break;
            case MLEL_UN_SIN: r = sin_hybrid(v); break;
            case MLEL_UN_TANH: r = tanh_clamped(v); break;
            case MLEL_UN_ERF: r = erf_ref(v); break;
            default: break;
            }
        }
        st_f(out, o, r);
    } else {
        const int64_t v = ld_i(in, o);
        int64_t r = v;
        switch (op) {
        case MLEL_UN_ABS: r = v < 0 ? -v : v; break;
        case MLEL_UN_BITWISE_NOT: r = ~v; break;
        case MLEL_UN_LOGICAL_NOT: r = !v; break;
        case MLEL_UN_CLZ: r = (uint32_t)v == 0 ? 32 : __clz((int)(uint32_t)v); break;
        default: break;
        }
        st_i(out, o, r);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// REDUCE_* as a sequential fold per output element (reference results: reduce.comp:24-70)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) reduce_generic(int op, TV out, TV in, uint32_t axis, uint32_t nan_mode,
                                                         int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    for (int i = 0; i < MLEL_MAX_RANK; i++) ii[i] = o[i];
    const int dt = in.dtype;
    if (dt_is_float(dt)) {
        const float lowest = dt_lowest_f(dt);
        float r;
        switch (op) {
        case MLEL_RED_MAX: r = nan_mode == MLEL_NAN_IGNORE ? NAN : lowest; break;
        case MLEL_RED_MIN: r = nan_mode == MLEL_NAN_IGNORE ? NAN : -lowest; break;
        case MLEL_RED_PRODUCT: r = 1.f; break;
        default: r = 0.f; break;
        }
        for (int64_t i = 0; i < in.dims[axis]; i++) {
            ii[axis] = i;
            const float v = ld_f(in, ii);
            if (isnan(v)) {
                if (nan_mode == MLEL_NAN_IGNORE) continue;
                r = v;
                break;
            }
            switch (op) {
            case MLEL_RED_MAX: r = isnan(r) ? v : (r < v ? v : r); break;
            case MLEL_RED_MIN: r = isnan(r) ? v : (v < r ? v : r); break;
            case MLEL_RED_PRODUCT: r = round_to(dt, r * v); break;
            case MLEL_RED_SUM: r = round_to(dt, r + v); break;
            default: break;
            }
        }
        st_f(out, o, r);
    } else {
        int64_t r;
        switch (op) {
        case MLEL_RED_ALL: r = 1; break;
        case MLEL_RED_ANY: r = 0; break;
        case MLEL_RED_MAX: r = dt_lowest(dt); break;
        case MLEL_RED_MIN: r = dt_max(dt); break;
        case MLEL_RED_PRODUCT: r = 1; break;
        default: r = 0; break;
        }
        for (int64_t i = 0; i < in.dims[axis]; i++) {
            ii[axis] = i;
            const int64_t v = ld_i(in, ii);
            switch (op) {
            case MLEL_RED_ALL: r = r && v; break;
            case MLEL_RED_ANY: r = r || v; break;
            case MLEL_RED_MAX: r = r > v ? r : v; break;
            case MLEL_RED_MIN: r = r < v ? r : v; break;
            case MLEL_RED_PRODUCT: r = narrow_to(dt, wmul64(r, v)); break;
            case MLEL_RED_SUM: r = narrow_to(dt, wadd64(r, v)); break;
            default: break;
            }
        }
        st_i(out, o, r);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// pooling (reference results: avgpool2d.comp:27-75, maxpool2d.comp:23-72)
// ---------------------------------------------------------------------------------------------------------------
struct PoolArgs {
    int32_t kh, kw, sy, sx, pad_t, pad_l, zi, zo;
    uint32_t acc, nan_mode;
};

__global__ void __launch_bounds__(kBlock) avgpool_generic(TV out, TV in, PoolArgs a, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t H = in.dims[1], W = in.dims[2];
    const int dt = out.dtype;
    int64_t iacc = 0, count = 0;
    float facc = 0.f;
    for (int64_t ky = 0; ky < a.kh; ky++) {
        for (int64_t kx = 0; kx < a.kw; kx++) {
            const int64_t yy = o[1] * a.sy - a.pad_t + ky;
            const int64_t xx = o[2] * a.sx - a.pad_l + kx;
            if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
            const int64_t xi[4] = {o[0], yy, xx, o[3]};
            if (dt_is_int(dt)) {
                const int64_t v = ld_i(in, xi) - a.zi;
                iacc = a.acc == MLEL_ACC_I64 ? wadd64(iacc, v) : (int64_t)wadd32((int32_t)iacc, (int32_t)v);
            } else {
                const float v = ld_f(in, xi) - (float)a.zi;
                facc = a.acc == MLEL_ACC_F16 ? rnd_f16(facc + rnd_f16(v)) : facc + v;
            }
            count++;
        }
    }
    if (dt_is_int(dt)) {
        int64_t r = 0;
        if (count > 0) {
            const int64_t rnd = iacc < 0 ? -(count >> 1) : (count >> 1);
            r = (iacc + rnd) / count;
        }
        r += a.zo;
        r = r < dt_lowest(dt) ? dt_lowest(dt) : (r > dt_max(dt) ? dt_max(dt) : r);
        st_i(out, o, r);
    } else {
        const float r = facc / (float)count;
        st_f(out, o, a.acc == MLEL_ACC_F16 ? rnd_f16(r) : r);
    }
}

__global__ void __launch_bounds__(kBlock) maxpool_generic(TV out, TV in, PoolArgs a, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t H = in.dims[1], W = in.dims[2];
    const int dt = out.dtype;
    const bool isf = dt_is_float(dt);
    int64_t iacc = dt_lowest(dt);
    float facc = dt_lowest_f(dt);
    if (isf && a.nan_mode == MLEL_NAN_IGNORE) facc = NAN;
    bool done = false;
    for (int64_t ky = 0; ky < a.kh && !done; ky++) {
        for (int64_t kx = 0; kx < a.kw; kx++) {
            const int64_t yy = o[1] * a.sy - a.pad_t + ky;
            const int64_t xx = o[2] * a.sx - a.pad_l + kx;
            if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
            const int64_t xi[4] = {o[0], yy, xx, o[3]};
            if (!isf) {
                const int64_t v = ld_i(in, xi);
                iacc = iacc > v ? iacc : v;
            } else {
                const float v = ld_f(in, xi);
                if (isnan(v)) {
                    if (a.nan_mode == MLEL_NAN_IGNORE) continue;
                    facc = v;
                    done = true;
                    break;
                }
                facc = isnan(facc) ? v : (facc < v ? v : facc);
            }
        }
    }
    if (isf)
        st_f(out, o, facc);
    else
        st_i(out, o, iacc);
}

// ---------------------------------------------------------------------------------------------------------------
// TABLE, CAST, NEGATE (reference results: table.comp:17-52, cast.comp:22-103, negate.comp:29-47)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) table_generic(TV out, TV in, TV table, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t v = ld_i(in, o);
    int64_t r;
    if (in.dtype == MLEL_I8) {
        const int64_t ti[1] = {v + 128};
        r = ld_i(table, ti);
    } else {
        const int32_t index = ((int32_t)v + 32768) >> 7;
        const int32_t fraction = (int32_t)v & 0x7f;
        const int64_t t0[1] = {index}, t1[1] = {index + 1};
        const int32_t base = (int32_t)ld_i(table, t0), next = (int32_t)ld_i(table, t1);
        r = (int32_t)((uint32_t)base << 7) + (next - base) * fraction;
    }
    st_i(out, o, r);
}

__global__ void __launch_bounds__(kBlock) cast_generic(TV out, TV in, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int idt = in.dtype, odt = out.dtype;
    if (odt == MLEL_BOOL) {
        st_i(out, o, dt_is_float(idt) ? (ld_f(in, o) != 0.f) : (ld_i(in, o) != 0));
    } else if (dt_is_float(odt)) {
        // to bf16: round to nearest even; to fp8: the fp32 value is encoded directly (cast.comp:36-56)
        const int mode = odt == MLEL_BF16 ? ST_RNE : ST_ACC;
        if (dt_is_float(idt)) {
            st_f(out, o, ld_f(in, o), mode);
        } else {
            const int64_t v = ld_i(in, o);
            if (odt == MLEL_F16 && idt != MLEL_BOOL && idt != MLEL_I8 && idt != MLEL_U8 && idt != MLEL_I16) {
                if (v > 65504) st_f(out, o, INFINITY);
                else if (v < -65504) st_f(out, o, -INFINITY);
                else st_f(out, o, (float)v);
            } else {
                st_f(out, o, (float)v, mode);
            }
        }
    } else {
        if (dt_is_float(idt)) {
            const float f = ld_f(in, o);
            const float lo = (float)dt_lowest(odt), hi = (float)dt_max(odt);
            int64_t r;
            if (isnan(f)) r = 0;
            else if (f <= lo) r = dt_lowest(odt);
            else if (f >= hi) r = dt_max(odt);
            else r = (int64_t)rintf(f);
            st_i(out, o, r);
        } else {
            st_i(out, o, ld_i(in, o));
        }
    }
}

__global__ void __launch_bounds__(kBlock) negate_generic(TV out, TV in, int32_t zi, int32_t zo, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int dt = out.dtype;
    if (dt_is_float(dt)) {
        const float v = ld_f(in, o);
        st_f(out, o, isnan(v) ? v : -v);
    } else {
        int64_t r = (int64_t)wadd32(wadd32(zi, (int32_t)-ld_i(in, o)), zo);
        r = r < dt_lowest(dt) ? dt_lowest(dt) : (r > dt_max(dt) ? dt_max(dt) : r);
        st_i(out, o, r);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// data movement (reference results: reshape.comp, transpose.comp, concat.comp, slice.comp, pad.comp)
// ---------------------------------------------------------------------------------------------------------------
__device__ inline void copy_elem(const TV &out, const int64_t *oi, const TV &in, const int64_t *ii) {
    int64_t so, si;
    if (!elem_off(out, oi, &so)) return;
    const bool ok = elem_off(in, ii, &si);
    switch (dt_size(out.dtype)) {
    case 1: *(uint8_t *)(out.ptr + so) = ok ? *(const uint8_t *)(in.ptr + si) : (uint8_t)0; break;
    case 2: *(uint16_t *)(out.ptr + so) = ok ? *(const uint16_t *)(in.ptr + si) : (uint16_t)0; break;
    case 4: *(uint32_t *)(out.ptr + so) = ok ? *(const uint32_t *)(in.ptr + si) : 0u; break;
    default: *(uint64_t *)(out.ptr + so) = ok ? *(const uint64_t *)(in.ptr + si) : 0ull; break;
    }
}

struct MoveArgs {
    uint32_t v[MLEL_MAX_RANK];  // perms (transpose) or start (slice)
    uint32_t axis, offset;      // concat
};

__global__ void __launch_bounds__(kBlock) move_generic(int kind, TV out, TV in, MoveArgs a, int64_t total,
                                                       int64_t in_total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK] = {0}, ii[MLEL_MAX_RANK] = {0};
    switch (kind) {
    case kReshape:
        if (flat >= in_total) return;
        unflatten(out, flat, o);
        unflatten(in, flat, ii);
        break;
    case kTranspose:
        unflatten(out, flat, o);
        for (int i = 0; i < out.rank; i++) ii[a.v[i]] = o[i];
        break;
    case kConcat:  // one thread per INPUT element
        unflatten(in, flat, ii);
        for (int i = 0; i < out.rank; i++) o[i] = ii[i];
        o[a.axis] += a.offset;
        break;
    default:
        unflatten(out, flat, o);
        for (int i = 0; i < out.rank; i++) ii[i] = o[i] + a.v[i];
        break;
    }
    copy_elem(out, o, in, ii);
}

__global__ void __launch_bounds__(kBlock) pad_generic(TV out, TV in, TV padding, double pad_const,
                                                      int32_t pad_const_int, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    bool is_pad = false;
    for (int i = 0; i < out.rank; i++) {
        const int64_t pi[1] = {2 * i};
        ii[i] = o[i] - ld_i(padding, pi);
        if (ii[i] < 0 || ii[i] >= in.dims[i]) {
            is_pad = true;
            break;
        }
    }
    const int dt = out.dtype;
    if (!is_pad)
        copy_elem(out, o, in, ii);
    else if (dt == MLEL_I32)
        st_i(out, o, pad_const_int);
    else if (dt_is_float(dt))
        st_f(out, o, (float)pad_const);
    else
        st_i(out, o, (int64_t)pad_const);
}

template <typename... KArgs, typename... Args>
int launch(const char *what, void (*kernel)(KArgs...), int64_t total, hipStream_t stream, Args... args) {
    if (total <= 0) return 0;
    MLEL_REQUIRE(total < (int64_t(1) << 31) * kBlock, MLEL_ERR_LIMIT, "%s: too many elements", what);
    hipLaunchKernelGGL(kernel, grid_1d(total, kBlock), dim3(kBlock), 0, stream, args...);
    return check_launch(what);
}

ConvArgs conv_args(const mlel_conv2d_attr *a) {
    return ConvArgs{a->input_zp, a->weight_zp, a->pad[0], a->pad[2], a->stride[0], a->stride[1], a->dilation[0],
                    a->dilation[1], a->acc_type};
}

}  // namespace

// ---- host entry points of the generic path ----

int conv2d_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                          const mlel_tensor *bias, const mlel_conv2d_attr *a) {
    return launch("conv2d", conv2d_generic, numel(out), s, make_tv(out), make_tv(in), make_tv(w), make_tv(bias),
                  conv_args(a), numel(out));
}

int dwconv_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                          const mlel_tensor *bias, const mlel_conv2d_attr *a) {
    return launch("depthwise_conv2d", dwconv_generic, numel(out), s, make_tv(out), make_tv(in), make_tv(w),
                  make_tv(bias), conv_args(a), numel(out));
}

int matmul_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *a, const mlel_tensor *b,
                          const mlel_matmul_attr *attr) {
    return launch("matmul", matmul_generic, numel(out), s, make_tv(out), make_tv(a), make_tv(b), attr->a_zp,
                  attr->b_zp, numel(out));
}

int rescale_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *mult,
                           const mlel_tensor *shift, const mlel_rescale_attr *attr, const RescaleParams &p) {
    const int in_dt = dt_unsigned_twin(in->dtype, attr->input_unsigned != 0);
    const int out_dt = dt_unsigned_twin(out->dtype, attr->output_unsigned != 0);
    return launch("rescale", rescale_generic, numel(out), s, make_tv(out), make_tv(in), make_tv(mult), make_tv(shift),
                  p, in_dt, out_dt, numel(out));
}

int clamp_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_clamp_attr *a) {
    return launch("clamp", clamp_generic, numel(out), s, make_tv(out), make_tv(in), a->min_val, a->max_val,
                  a->nan_mode, numel(out));
}

int binary_generic_launch(hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in1,
                          const mlel_tensor *in2, uint32_t nan_mode) {
    return launch("elementwise_binary", binary_generic, numel(out), s, op, make_tv(out), make_tv(in1), make_tv(in2),
                  nan_mode, numel(out));
}

int mul_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2,
                       uint32_t shift) {
    return launch("mul", mul_generic, numel(out), s, make_tv(out), make_tv(in1), make_tv(in2), shift, numel(out));
}

int unary_generic_launch(hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in) {
    return launch("elementwise_unary", unary_generic, numel(out), s, op, make_tv(out), make_tv(in), numel(out));
}

int reduce_generic_launch(hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis,
                          uint32_t nan_mode) {
    return launch("reduce", reduce_generic, numel(out), s, op, make_tv(out), make_tv(in), axis, nan_mode, numel(out));
}

int pool_generic_launch(hipStream_t s, bool avg, const mlel_tensor *out, const mlel_tensor *in,
                        const mlel_pool2d_attr *a) {
    PoolArgs p{a->kernel[0], a->kernel[1], a->stride[0], a->stride[1], a->pad[0], a->pad[2],
               a->input_zp,  a->output_zp, a->acc_type,  a->nan_mode};
    if (!avg) {  // reference: maxpool2d.comp:39-42 clamps kernel >= 0 and stride >= 1
        p.kh = p.kh > 0 ? p.kh : 0;
        p.kw = p.kw > 0 ? p.kw : 0;
        p.sy = p.sy > 1 ? p.sy : 1;
        p.sx = p.sx > 1 ? p.sx : 1;
    }
    return launch(avg ? "avg_pool2d" : "max_pool2d", avg ? avgpool_generic : maxpool_generic, numel(out), s,
                  make_tv(out), make_tv(in), p, numel(out));
}

int table_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *table) {
    return launch("table", table_generic, numel(out), s, make_tv(out), make_tv(in), make_tv(table), numel(out));
}

int cast_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in) {
    return launch("cast", cast_generic, numel(out), s, make_tv(out), make_tv(in), numel(out));
}

int negate_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, int32_t zi, int32_t zo) {
    return launch("negate", negate_generic, numel(out), s, make_tv(out), make_tv(in), zi, zo, numel(out));
}

int move_generic_launch(hipStream_t s, int kind, const mlel_tensor *out, const mlel_tensor *in, const uint32_t *v,
                        uint32_t axis, uint32_t offset) {
    MoveArgs a{};
    if (v)
        for (int i = 0; i < out->rank; i++) a.v[i] = v[i];
    a.axis = axis;
    a.offset = offset;
    const int64_t total = kind == kConcat ? numel(in) : numel(out);
    return launch("data movement", move_generic, total, s, kind, make_tv(out), make_tv(in), a, total, numel(in));
}

int pad_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *padding,
                       double pad_const, int32_t pad_const_int) {
    return launch("pad", pad_generic, numel(out), s, make_tv(out), make_tv(in), make_tv(padding), pad_const,
                  pad_const_int, numel(out));
}

}  // namespace mlel
