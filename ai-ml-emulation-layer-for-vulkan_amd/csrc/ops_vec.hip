// Bandwidth-bound integer operators on packed tensors, 128 bits per thread and access where the element size allows:
// stand-alone RESCALE, CLAMP, TABLE, MAX_POOL2D and the same-shape integer elementwise operators (ADD, SUB, MAXIMUM,
// MINIMUM, BITWISE_*).  They are what an unfused graph executes between the contractions (the fused epilogues make
// most of them disappear from the benchmark graphs); each declines (returns 0) whatever it was not written for, and the
// one-thread-per-element kernels of ops_generic.hip take over.  Arithmetic: rescale.comp:27-72, clamp.comp:24-53,
// table.comp:17-52, maxpool2d.comp:23-72, elementwise_binary.comp:146-173 of the reference's shaders.
#include "common.hpp"
#include "dispatch.hpp"

#include <algorithm>

namespace mlel {
namespace {

constexpr int kBlock = 256;

bool aligned16(const void *p) { return ((uintptr_t)p % 16) == 0; }

// ---------------------------------------------------------------------------------------------------------------
// RESCALE.  Work item = 4 consecutive elements (4 consecutive channels: the channel count is a multiple of 4 when the
// scale is per channel).  Thread t takes the items t, t + T, t + 2T, ... with T a multiple of the number of channel
// quads, so its four channels never change: their constants (multiplier, shift, both rounding terms with the input
// zero point folded in) are worked out once and stay in registers.  Consecutive lanes hold consecutive items, so a
// wavefront's loads and stores are contiguous: 16 bytes per lane on a 32-bit side, 4 on an 8-bit side.
// ---------------------------------------------------------------------------------------------------------------
template <int IN_SZ, bool IN_UNSIGNED, int OUT_SZ>
__global__ void __launch_bounds__(kBlock) rescale_vec4_kernel(char *__restrict__ out, const char *__restrict__ in,
                                                              const ScaleRef sc, const int64_t items, const int32_t c4n,
                                                              const int64_t stride) {
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= stride) return;
    const int c0 = (int)(t % c4n) * 4;
    ChanScale q[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int ci = sc.p.per_channel ? c0 + e : 0;
        q[e] = make_chan_scale(load_mult(sc, ci), (int32_t)sc.shift[ci], sc.p);
    }
    for (int64_t g = t; g < items; g += stride) {
        int32_t v[4];
        if (IN_SZ == 4) {
            const int4 x = *reinterpret_cast<const int4 *>(in + g * 16);
            v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
        } else if (IN_SZ == 2) {
            const uint2 x = *reinterpret_cast<const uint2 *>(in + g * 8);
            const uint32_t w[2] = {x.x, x.y};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t h = (w[e >> 1] >> (16 * (e & 1))) & 0xffffu;
                v[e] = IN_UNSIGNED ? (int32_t)h : (int32_t)(int16_t)h;
            }
        } else {
            const uint32_t x = *reinterpret_cast<const uint32_t *>(in + g * 4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t b = (x >> (8 * e)) & 0xffu;
                v[e] = IN_UNSIGNED ? (int32_t)b : (int32_t)(int8_t)b;
            }
        }
        int32_t r[4];
#pragma unroll
        for (int e = 0; e < 4; e++) r[e] = requant_chan(v[e], q[e], sc.p);
        if (OUT_SZ == 4) {
            *reinterpret_cast<int4 *>(out + g * 16) = make_int4(r[0], r[1], r[2], r[3]);
        } else if (OUT_SZ == 2) {
            *reinterpret_cast<uint2 *>(out + g * 8) = make_uint2(((uint32_t)r[0] & 0xffffu) | ((uint32_t)r[1] << 16),
                                                                 ((uint32_t)r[2] & 0xffffu) | ((uint32_t)r[3] << 16));
        } else {
            const uint32_t lo = __builtin_amdgcn_perm((uint32_t)r[1], (uint32_t)r[0], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm((uint32_t)r[3], (uint32_t)r[2], 0x0c0c0400u);
            *reinterpret_cast<uint32_t *>(out + g * 4) = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
    }
}

template <int IN_SZ, bool IN_UNSIGNED>
void launch_rescale(int out_sz, dim3 grid, hipStream_t s, char *out, const char *in, const ScaleRef &sc, int64_t items,
                    int32_t c4n, int64_t stride) {
    if (out_sz == 1)
        rescale_vec4_kernel<IN_SZ, IN_UNSIGNED, 1><<<grid, dim3(kBlock), 0, s>>>(out, in, sc, items, c4n, stride);
    else if (out_sz == 2)
        rescale_vec4_kernel<IN_SZ, IN_UNSIGNED, 2><<<grid, dim3(kBlock), 0, s>>>(out, in, sc, items, c4n, stride);
    else
        rescale_vec4_kernel<IN_SZ, IN_UNSIGNED, 4><<<grid, dim3(kBlock), 0, s>>>(out, in, sc, items, c4n, stride);
}

// ---------------------------------------------------------------------------------------------------------------
// CLAMP on signed 8 / 16 / 32-bit integers: 16 bytes per thread; the elements behind the last whole 16 bytes are
// taken one per thread by the first block.
// ---------------------------------------------------------------------------------------------------------------
template <int SZ>
__device__ __forceinline__ uint32_t clamp_word(uint32_t x, int32_t lo, int32_t hi) {
    if (SZ == 4) {
        int32_t r;
        asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"((int32_t)x), "v"(lo), "v"(hi));
        return (uint32_t)r;
    } else if (SZ == 2) {
        int32_t a, b;
        asm("v_med3_i32 %0, %1, %2, %3" : "=v"(a) : "v"((int32_t)(int16_t)(x & 0xffffu)), "v"(lo), "v"(hi));
        asm("v_med3_i32 %0, %1, %2, %3" : "=v"(b) : "v"((int32_t)x >> 16), "v"(lo), "v"(hi));
        return ((uint32_t)a & 0xffffu) | ((uint32_t)b << 16);
    } else {
        int32_t r[4];
#pragma unroll
        for (int e = 0; e < 4; e++)
            asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r[e]) : "v"((int32_t)(int8_t)(x >> (8 * e))), "v"(lo), "v"(hi));
        const uint32_t l = __builtin_amdgcn_perm((uint32_t)r[1], (uint32_t)r[0], 0x0c0c0400u);
        const uint32_t h = __builtin_amdgcn_perm((uint32_t)r[3], (uint32_t)r[2], 0x0c0c0400u);
        return __builtin_amdgcn_perm(h, l, 0x05040100u);
    }
}

template <int SZ>
__global__ void __launch_bounds__(kBlock) clamp_vec_kernel(char *__restrict__ out, const char *__restrict__ in, int32_t lo,
                                                           int32_t hi, int64_t n_vec, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n_vec) {
        const uint4 x = reinterpret_cast<const uint4 *>(in)[i];
        reinterpret_cast<uint4 *>(out)[i] = make_uint4(clamp_word<SZ>(x.x, lo, hi), clamp_word<SZ>(x.y, lo, hi),
                                                       clamp_word<SZ>(x.z, lo, hi), clamp_word<SZ>(x.w, lo, hi));
    }
    const int64_t e = n_vec * (16 / SZ) + i;  // the tail: fewer than 16 / SZ elements
    if (blockIdx.x == 0 && e < total) {
        if (SZ == 1) {
            const int32_t v = reinterpret_cast<const int8_t *>(in)[e];
            reinterpret_cast<int8_t *>(out)[e] = (int8_t)(v < lo ? lo : (v > hi ? hi : v));
        } else if (SZ == 2) {
            const int32_t v = reinterpret_cast<const int16_t *>(in)[e];
            reinterpret_cast<int16_t *>(out)[e] = (int16_t)(v < lo ? lo : (v > hi ? hi : v));
        } else {
            const int32_t v = reinterpret_cast<const int32_t *>(in)[e];
            reinterpret_cast<int32_t *>(out)[e] = v < lo ? lo : (v > hi ? hi : v);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Same-shape integer elementwise operators on int32: 4 elements per thread.
// ---------------------------------------------------------------------------------------------------------------
template <int OP>
__device__ __forceinline__ int32_t bin_i32(int32_t a, int32_t b) {
    switch (OP) {
    case MLEL_BIN_ADD: return (int32_t)((uint32_t)a + (uint32_t)b);
    case MLEL_BIN_SUB: return (int32_t)((uint32_t)a - (uint32_t)b);
    case MLEL_BIN_MAXIMUM: return a > b ? a : b;
    case MLEL_BIN_MINIMUM: return a < b ? a : b;
    case MLEL_BIN_BITWISE_AND: return a & b;
    case MLEL_BIN_BITWISE_OR: return a | b;
    default: return a ^ b;
    }
}

template <int OP>
__global__ void __launch_bounds__(kBlock) binary_i32x4_kernel(int32_t *__restrict__ out, const int32_t *__restrict__ a,
                                                              const int32_t *__restrict__ b, int64_t n_vec, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n_vec) {
        const int4 x = reinterpret_cast<const int4 *>(a)[i], y = reinterpret_cast<const int4 *>(b)[i];
        reinterpret_cast<int4 *>(out)[i] =
            make_int4(bin_i32<OP>(x.x, y.x), bin_i32<OP>(x.y, y.y), bin_i32<OP>(x.z, y.z), bin_i32<OP>(x.w, y.w));
    }
    const int64_t e = n_vec * 4 + i;
    if (blockIdx.x == 0 && e < total) out[e] = bin_i32<OP>(a[e], b[e]);
}

// ---------------------------------------------------------------------------------------------------------------
// TABLE.  int8: out = table[in + 128], the 256 entries in shared memory, 16 elements per thread.  int16: the 513
// entries in shared memory, out = (table[i] << 7) + (table[i + 1] - table[i]) * (in & 127) with i = (in + 32768) >> 7,
// 8 elements per thread (16 bytes in, 32 bytes out).
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) table_i8x16_kernel(uint8_t *__restrict__ out, const uint8_t *__restrict__ in,
                                                             const uint8_t *__restrict__ table, int64_t n_vec, int64_t total) {
    __shared__ uint8_t tab[256];
    tab[threadIdx.x] = table[threadIdx.x];  // kBlock == 256
    __syncthreads();
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n_vec) {
        const uint4 x = reinterpret_cast<const uint4 *>(in)[i];
        const uint32_t w[4] = {x.x, x.y, x.z, x.w};
        uint32_t r[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t idx = w[k] ^ 0x80808080u;  // value + 128 of every byte
            r[k] = (uint32_t)tab[idx & 0xffu] | ((uint32_t)tab[(idx >> 8) & 0xffu] << 8) |
                   ((uint32_t)tab[(idx >> 16) & 0xffu] << 16) | ((uint32_t)tab[idx >> 24] << 24);
        }
        reinterpret_cast<uint4 *>(out)[i] = make_uint4(r[0], r[1], r[2], r[3]);
    }
    const int64_t e = n_vec * 16 + i;
    if (blockIdx.x == 0 && e < total) out[e] = tab[in[e] ^ 0x80u];
}

__device__ __forceinline__ int32_t table16(const int16_t *tab, int32_t v) {
    const int32_t index = (v + 32768) >> 7, fraction = v & 0x7f;
    const int32_t base = tab[index], next = tab[index + 1];
    return (int32_t)((uint32_t)base << 7) + (next - base) * fraction;
}

__global__ void __launch_bounds__(kBlock) table_i16x8_kernel(int32_t *__restrict__ out, const int16_t *__restrict__ in,
                                                             const int16_t *__restrict__ table, int64_t n_vec, int64_t total) {
    __shared__ int16_t tab[513 + 3];
    for (int k = threadIdx.x; k < 513; k += kBlock) tab[k] = table[k];
    __syncthreads();
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n_vec) {
        const uint4 x = reinterpret_cast<const uint4 *>(in)[i];
        const uint32_t w[4] = {x.x, x.y, x.z, x.w};
        int32_t r[8];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            r[2 * k] = table16(tab, (int32_t)(int16_t)(w[k] & 0xffffu));
            r[2 * k + 1] = table16(tab, (int32_t)w[k] >> 16);
        }
        reinterpret_cast<int4 *>(out)[2 * i] = make_int4(r[0], r[1], r[2], r[3]);
        reinterpret_cast<int4 *>(out)[2 * i + 1] = make_int4(r[4], r[5], r[6], r[7]);
    }
    const int64_t e = n_vec * 8 + i;
    if (blockIdx.x == 0 && e < total) out[e] = table16(tab, in[e]);
}

// ---------------------------------------------------------------------------------------------------------------
// MAX_POOL2D, int8 NHWC.  Work item = 4 consecutive channels of one output position (lanes run over the channel
// quads: a wavefront reads consecutive dwords of each input pixel); taps outside the image are skipped and the
// accumulator starts from the lowest value of the type, as the shader does.
// ---------------------------------------------------------------------------------------------------------------
struct MaxPoolArgs {
    const int8_t *x;
    int8_t *out;
    int32_t H, W, C, OH, OW;
    int64_t x_sn, x_sy, x_sx;
    int32_t kh, kw, sy, sx, pad_t, pad_l;
    int64_t items;  // N * OH * OW * C / 4
};

__global__ void __launch_bounds__(kBlock) maxpool_i8x4_kernel(const MaxPoolArgs a) {
    const int64_t item = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (item >= a.items) return;
    const int c4n = a.C >> 2;
    const int c = (int)(item % c4n) * 4;
    int64_t rest = item / c4n;
    const int ox = (int)(rest % a.OW);
    rest /= a.OW;
    const int oy = (int)(rest % a.OH);
    const int n = (int)(rest / a.OH);
    const int y0 = max(0, oy * a.sy - a.pad_t), y1 = min(a.H, oy * a.sy - a.pad_t + a.kh);
    const int x0 = max(0, ox * a.sx - a.pad_l), x1 = min(a.W, ox * a.sx - a.pad_l + a.kw);
    int32_t m[4] = {-128, -128, -128, -128};
    const int8_t *xb = a.x + (int64_t)n * a.x_sn + c;
    for (int y = y0; y < y1; y++)
        for (int x = x0; x < x1; x++) {
            const uint32_t v = *reinterpret_cast<const uint32_t *>(xb + (int64_t)y * a.x_sy + (int64_t)x * a.x_sx);
#pragma unroll
            for (int e = 0; e < 4; e++) m[e] = max(m[e], (int32_t)(int8_t)(v >> (8 * e)));
        }
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)m[1], (uint32_t)m[0], 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)m[3], (uint32_t)m[2], 0x0c0c0400u);
    reinterpret_cast<uint32_t *>(a.out)[item] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

}  // namespace

int try_rescale_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *mult,
                     const mlel_tensor *shift, const mlel_rescale_attr *attr, const RescaleParams &p) {
    const int in_dt = dt_unsigned_twin(in->dtype, attr->input_unsigned != 0);
    const int in_sz = dt_size(in->dtype), out_sz = dt_size(out->dtype);
    // the kernel's arithmetic takes a 32-bit value: 8 / 16-bit inputs of either signedness and signed 32-bit ones
    if (!(in_dt == MLEL_I8 || in_dt == MLEL_U8 || in_dt == MLEL_I16 || in_dt == MLEL_U16 || in_dt == MLEL_I32)) return 0;
    if (!(out_sz == 1 || out_sz == 2 || out_sz == 4) || !dt_is_int(out->dtype) || out->dtype == MLEL_BOOL) return 0;
    if (!is_packed(in) || !is_packed(out) || !is_packed(mult) || !is_packed(shift)) return 0;
    for (int i = 0; i < out->rank; i++)
        if (in->dims[i] != out->dims[i]) return 0;
    const int64_t total = numel(out);
    if (total == 0) return 1;
    const int64_t C = out->dims[out->rank - 1];
    if (total % 4 != 0 || (attr->per_channel && C % 4 != 0)) return 0;
    if (((uintptr_t)in->ptr % (4 * in_sz)) != 0 || ((uintptr_t)out->ptr % (4 * out_sz)) != 0) return 0;
    if (((uintptr_t)mult->ptr % 4) != 0) return 0;
    const int64_t items = total / 4;
    const int64_t c4n = attr->per_channel ? C / 4 : 1;
    if (c4n >= (int64_t(1) << 30)) return 0;
    // eight items per thread; the thread stride is a whole number of channel-quad rounds
    int64_t stride = (items + 7) / 8;
    stride = (stride + c4n - 1) / c4n * c4n;
    const int64_t blocks = (stride + kBlock - 1) / kBlock;
    if (blocks >= (int64_t(1) << 31)) return 0;
    FusedEpilogue f{mult, shift, p, attr->scale32 != 0, in_dt};
    const ScaleRef sc = make_ref(f);
    const dim3 grid((unsigned)blocks);
    char *o = static_cast<char *>(out->ptr);
    const char *x = static_cast<const char *>(in->ptr);
    (void)ctx;
    switch (in_dt) {
    case MLEL_I8: launch_rescale<1, false>(out_sz, grid, s, o, x, sc, items, (int32_t)c4n, stride); break;
    case MLEL_U8: launch_rescale<1, true>(out_sz, grid, s, o, x, sc, items, (int32_t)c4n, stride); break;
    case MLEL_I16: launch_rescale<2, false>(out_sz, grid, s, o, x, sc, items, (int32_t)c4n, stride); break;
    case MLEL_U16: launch_rescale<2, true>(out_sz, grid, s, o, x, sc, items, (int32_t)c4n, stride); break;
    default: launch_rescale<4, false>(out_sz, grid, s, o, x, sc, items, (int32_t)c4n, stride); break;
    }
    MLEL_TRY(check_launch("rescale (packed)"));
    return 1;
}

int try_clamp_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_clamp_attr *a) {
    (void)ctx;
    const int dt = out->dtype;
    if (!(dt == MLEL_I8 || dt == MLEL_I16 || dt == MLEL_I32) || in->dtype != dt) return 0;
    if (!is_packed(in) || !is_packed(out) || !aligned16(in->ptr) || !aligned16(out->ptr)) return 0;
    for (int i = 0; i < out->rank; i++)
        if (in->dims[i] != out->dims[i]) return 0;
    const int64_t total = numel(out);
    if (total == 0) return 1;
    // the bounds are converted to the storage type by truncation, then narrowed (clamp.comp:32-33)
    const int32_t lo = (int32_t)narrow_to(dt, (int64_t)a->min_val), hi = (int32_t)narrow_to(dt, (int64_t)a->max_val);
    if (lo > hi) return 0;  // the generic kernel applies max then min in that order
    const int sz = dt_size(dt);
    const int64_t n_vec = total * sz / 16;
    const dim3 grid = grid_1d(std::max<int64_t>(n_vec, 16), kBlock);
    char *o = static_cast<char *>(out->ptr);
    const char *x = static_cast<const char *>(in->ptr);
    if (sz == 1)
        clamp_vec_kernel<1><<<grid, dim3(kBlock), 0, s>>>(o, x, lo, hi, n_vec, total);
    else if (sz == 2)
        clamp_vec_kernel<2><<<grid, dim3(kBlock), 0, s>>>(o, x, lo, hi, n_vec, total);
    else
        clamp_vec_kernel<4><<<grid, dim3(kBlock), 0, s>>>(o, x, lo, hi, n_vec, total);
    MLEL_TRY(check_launch("clamp (packed)"));
    return 1;
}

int try_binary_fast(mlel_ctx *ctx, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in1,
                    const mlel_tensor *in2) {
    (void)ctx;
    if (out->dtype != MLEL_I32 || in1->dtype != MLEL_I32 || in2->dtype != MLEL_I32) return 0;
    if (!is_packed(in1) || !is_packed(in2) || !is_packed(out)) return 0;
    if (!aligned16(in1->ptr) || !aligned16(in2->ptr) || !aligned16(out->ptr)) return 0;
    for (int i = 0; i < out->rank; i++)
        if (in1->dims[i] != out->dims[i] || in2->dims[i] != out->dims[i]) return 0;  // no broadcasting here
    const int64_t total = numel(out);
    if (total == 0) return 1;
    const int64_t n_vec = total / 4;
    const dim3 grid = grid_1d(std::max<int64_t>(n_vec, 4), kBlock);
    int32_t *o = static_cast<int32_t *>(out->ptr);
    const int32_t *a = static_cast<const int32_t *>(in1->ptr), *b = static_cast<const int32_t *>(in2->ptr);
#define MLEL_BIN_CASE(OP) \
    case OP: binary_i32x4_kernel<OP><<<grid, dim3(kBlock), 0, s>>>(o, a, b, n_vec, total); break;
    switch (op) {
        MLEL_BIN_CASE(MLEL_BIN_ADD)
        MLEL_BIN_CASE(MLEL_BIN_SUB)
        MLEL_BIN_CASE(MLEL_BIN_MAXIMUM)
        MLEL_BIN_CASE(MLEL_BIN_MINIMUM)
        MLEL_BIN_CASE(MLEL_BIN_BITWISE_AND)
        MLEL_BIN_CASE(MLEL_BIN_BITWISE_OR)
        MLEL_BIN_CASE(MLEL_BIN_BITWISE_XOR)
    default: return 0;
    }
#undef MLEL_BIN_CASE
    MLEL_TRY(check_launch("elementwise_binary (packed int32)"));
    return 1;
}

int try_table_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *table) {
    (void)ctx;
    if (!is_packed(in) || !is_packed(out) || !is_packed(table) || !aligned16(in->ptr) || !aligned16(out->ptr)) return 0;
    for (int i = 0; i < out->rank; i++)
        if (in->dims[i] != out->dims[i]) return 0;
    const int64_t total = numel(out);
    if (total == 0) return 1;
    if (in->dtype == MLEL_I8 && out->dtype == MLEL_I8 && table->dims[0] >= 256) {
        const int64_t n_vec = total / 16;
        table_i8x16_kernel<<<grid_1d(std::max<int64_t>(n_vec, 16), kBlock), dim3(kBlock), 0, s>>>(
            static_cast<uint8_t *>(out->ptr), static_cast<const uint8_t *>(in->ptr),
            static_cast<const uint8_t *>(table->ptr), n_vec, total);
    } else if (in->dtype == MLEL_I16 && out->dtype == MLEL_I32 && table->dims[0] >= 513 && ((uintptr_t)table->ptr % 2) == 0) {
        const int64_t n_vec = total / 8;
        table_i16x8_kernel<<<grid_1d(std::max<int64_t>(n_vec, 8), kBlock), dim3(kBlock), 0, s>>>(
            static_cast<int32_t *>(out->ptr), static_cast<const int16_t *>(in->ptr),
            static_cast<const int16_t *>(table->ptr), n_vec, total);
    } else {
        return 0;
    }
    MLEL_TRY(check_launch("table (packed)"));
    return 1;
}

int try_maxpool_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_pool2d_attr *a) {
    (void)ctx;
    if (in->dtype != MLEL_I8 || out->dtype != MLEL_I8) return 0;
    const int64_t N = out->dims[0], OH = out->dims[1], OW = out->dims[2], C = out->dims[3];
    if (in->dims[3] != C || C % 4 != 0 || in->dims[0] < N || !is_packed(out) || in->strides[3] != 1) return 0;
    if (((uintptr_t)in->ptr % 4) || in->strides[0] % 4 || in->strides[1] % 4 || in->strides[2] % 4) return 0;
    if (((uintptr_t)out->ptr % 4) != 0) return 0;
    if (a->kernel[0] <= 0 || a->kernel[1] <= 0 || a->stride[0] <= 0 || a->stride[1] <= 0) return 0;
    if (a->kernel[0] > (1 << 16) || a->kernel[1] > (1 << 16) || a->stride[0] > (1 << 16) || a->stride[1] > (1 << 16)) return 0;
    if (a->pad[0] < 0 || a->pad[2] < 0 || a->pad[0] > (1 << 16) || a->pad[2] > (1 << 16)) return 0;
    if (in->dims[1] >= (1 << 30) || in->dims[2] >= (1 << 30) || OH >= (1 << 14) || OW >= (1 << 14) || C >= (1 << 24)) return 0;
    const int64_t items = N * OH * OW * (C / 4);
    if (items == 0) return 1;
    if (items >= (int64_t(1) << 40)) return 0;
    MaxPoolArgs g{};
    g.x = static_cast<const int8_t *>(in->ptr);
    g.out = static_cast<int8_t *>(out->ptr);
    g.H = (int)in->dims[1];
    g.W = (int)in->dims[2];
    g.C = (int)C;
    g.OH = (int)OH;
    g.OW = (int)OW;
    g.x_sn = in->strides[0];
    g.x_sy = in->strides[1];
    g.x_sx = in->strides[2];
    g.kh = a->kernel[0];
    g.kw = a->kernel[1];
    g.sy = a->stride[0];
    g.sx = a->stride[1];
    g.pad_t = a->pad[0];
    g.pad_l = a->pad[2];
    g.items = items;
    const int64_t blocks = (items + kBlock - 1) / kBlock;
    if (blocks >= (int64_t(1) << 31)) return 0;
    maxpool_i8x4_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(g);
    MLEL_TRY(check_launch("max_pool2d (int8 quads)"));
    return 1;
}

}  // namespace mlel
