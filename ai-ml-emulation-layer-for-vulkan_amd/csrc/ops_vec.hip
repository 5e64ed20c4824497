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

// `out` may be `in` (CLAMP in place behind an unfused RESCALE): a thread reads its 16 bytes before it writes them, and
// the pointers carry no no-alias promise.  The same holds for the int32 elementwise and the 8-bit TABLE kernels below.
template <int SZ>
__global__ void __launch_bounds__(kBlock) clamp_vec_kernel(char *out, const char *in, int32_t lo,
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
__global__ void __launch_bounds__(kBlock) binary_i32x4_kernel(int32_t *out, const int32_t *a, const int32_t *b, int64_t n_vec,
                                                              int64_t total) {
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
__global__ void __launch_bounds__(kBlock) table_i8x16_kernel(uint8_t *out, const uint8_t *in, const uint8_t *__restrict__ table,
                                                             int64_t n_vec, int64_t total) {
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
// MAX_POOL2D, int8 NHWC (reference: maxpool2d.comp:23-72).  Work item = 4 * V consecutive channels of one output
// position (lanes run over the channel groups: a wavefront reads consecutive pieces of each input pixel, V dwords per
// lane and tap).  A block covers 256 items of one output row (n, oy), so the row is decoded on the scalar unit and a
// thread needs one magic-number division; blocks are dealt to the XCDs in contiguous runs of rows, so the input rows
// that vertically adjacent output rows share are fetched into one L2.  Taps outside the image are replaced by -128,
// the value the shader's accumulator starts from.  The maximum runs on packed 16-bit halves: x ^ 0x80 turns the
// signed order of a byte into the unsigned one, the even and the odd bytes of a dword are two v_pk_max_u16 operands
// (the odd ones in place, as value << 8), and the result is flipped back.
// ---------------------------------------------------------------------------------------------------------------
struct MaxPoolArgs {
    const int8_t *x;
    int8_t *out;
    int32_t H, W, C, OH, OW;
    uint32_t x_sn, x_sy, x_sx, x_bytes, o_bytes;
    int32_t kh, kw, sy, sx, pad_t, pad_l;
    int32_t groups;       // channel groups per pixel: C / (4 V)
    int32_t row_items;    // OW * groups, below 2^16
    int32_t row_blocks;   // ceil(row_items / 256)
    uint32_t groups_magic;  // floor(2^32 / groups) + 1
    int32_t blocks, chunk;  // launch geometry: `chunk` consecutive blocks per XCD
};

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_max_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// K > 0: a K x K window, unrolled, so that all its loads are in flight together; K == 0: any window, tap by tap
template <int V, int K>
__global__ void __launch_bounds__(kBlock) maxpool_i8_kernel(const MaxPoolArgs a) {
    const int bid = (int)(blockIdx.x % 8u) * a.chunk + (int)(blockIdx.x / 8u);
    if (bid >= a.blocks) return;
    const int row = bid / a.row_blocks, part = bid - row * a.row_blocks;  // uniform: scalar unit
    const int n = row / a.OH, oy = row - n * a.OH;
    const uint32_t item = (uint32_t)part * kBlock + threadIdx.x;
    if (item >= (uint32_t)a.row_items) return;
    const uint32_t ox = a.groups == 1 ? item : __umulhi(item, a.groups_magic);
    const uint32_t cg = item - ox * (uint32_t)a.groups;
    const int iy0 = oy * a.sy - a.pad_t, ix0 = (int)ox * a.sx - a.pad_l;
    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(a.out, 0, (int)a.o_bytes, 0x00020000);
    const uint32_t base = (uint32_t)n * a.x_sn + (uint32_t)iy0 * a.x_sy + (uint32_t)ix0 * a.x_sx + cg * (4u * V);
    uint32_t even[V], odd[V];  // running maxima in the flipped (unsigned) order: 0 is the lowest value, -128
#pragma unroll
    for (int v = 0; v < V; v++) even[v] = odd[v] = 0u;
    auto load = [&](uint32_t off, uint32_t (&w)[V]) {
        if constexpr (V == 4) {
            const auto q = __builtin_amdgcn_raw_buffer_load_b128(xres, (int)off, 0, 0);
            w[0] = q[0], w[1] = q[1], w[2] = q[2], w[3] = q[3];
        } else {
            w[0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(xres, (int)off, 0, 0);
        }
    };
    auto fold = [&](bool in, const uint32_t (&w)[V]) {
#pragma unroll
        for (int v = 0; v < V; v++) {
            const uint32_t f = in ? (w[v] ^ 0x80808080u) : 0u;
            even[v] = pk_max_u16(even[v], f & 0x00ff00ffu);
            odd[v] = pk_max_u16(odd[v], f & 0xff00ff00u);
        }
    };
    // The offset of a tap outside the image wraps to another pixel or beyond the extent (such a load returns 0);
    // either way its value is replaced by the lowest one.
    if constexpr (K > 0) {
        uint32_t w[K][K][V];
#pragma unroll
        for (int ky = 0; ky < K; ky++)
#pragma unroll
            for (int kx = 0; kx < K; kx++) load(base + (uint32_t)ky * a.x_sy + (uint32_t)kx * a.x_sx, w[ky][kx]);
#pragma unroll
        for (int ky = 0; ky < K; ky++) {
            const bool yin = (unsigned)(iy0 + ky) < (unsigned)a.H;
#pragma unroll
            for (int kx = 0; kx < K; kx++) fold(yin && (unsigned)(ix0 + kx) < (unsigned)a.W, w[ky][kx]);
        }
    } else {
        for (int ky = 0; ky < a.kh; ky++) {
            if ((unsigned)(iy0 + ky) >= (unsigned)a.H) continue;  // uniform
            const uint32_t rowoff = base + (uint32_t)ky * a.x_sy;
            for (int kx = 0; kx < a.kw; kx++) {
                uint32_t w[V];
                load(rowoff + (uint32_t)kx * a.x_sx, w);
                fold((unsigned)(ix0 + kx) < (unsigned)a.W, w);
            }
        }
    }
    uint32_t r[V];
#pragma unroll
    for (int v = 0; v < V; v++) r[v] = (even[v] | odd[v]) ^ 0x80808080u;
    const uint32_t ooff = (((uint32_t)row * (uint32_t)a.OW + ox) * (uint32_t)a.groups + cg) * (4u * V);
    if constexpr (V == 4) {
        typedef int v4i32 __attribute__((ext_vector_type(4)));
        __builtin_amdgcn_raw_buffer_store_b128(v4i32{(int)r[0], (int)r[1], (int)r[2], (int)r[3]}, ores, (int)ooff, 0, kOutAux);
    } else {
        __builtin_amdgcn_raw_buffer_store_b32(r[0], ores, (int)ooff, 0, 0);
    }
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
    if (N * OH * OW * C == 0) return 1;
    // 32-bit buffer offsets on both sides; taps outside the image are sent to an offset beyond either extent
    if (in->strides[0] < 0 || in->strides[1] < 0 || in->strides[2] < 0) return 0;
    const int64_t x_extent = in->dims[0] * in->strides[0], o_extent = N * OH * OW * C;
    if (x_extent <= 0 || x_extent >= (int64_t(1) << 31) || o_extent >= (int64_t(1) << 31)) return 0;
    // 16 channels per thread when pixels and rows are 16-byte aligned on both sides, else 4
    const bool wide = C % 16 == 0 && ((uintptr_t)in->ptr % 16) == 0 && ((uintptr_t)out->ptr % 16) == 0 &&
                      in->strides[0] % 16 == 0 && in->strides[1] % 16 == 0 && in->strides[2] % 16 == 0;
    const int v = wide ? 4 : 1;
    MaxPoolArgs g{};
    g.x = static_cast<const int8_t *>(in->ptr);
    g.out = static_cast<int8_t *>(out->ptr);
    g.H = (int)in->dims[1];
    g.W = (int)in->dims[2];
    g.C = (int)C;
    g.OH = (int)OH;
    g.OW = (int)OW;
    g.x_sn = (uint32_t)in->strides[0];
    g.x_sy = (uint32_t)in->strides[1];
    g.x_sx = (uint32_t)in->strides[2];
    g.x_bytes = (uint32_t)x_extent;
    g.o_bytes = (uint32_t)o_extent;
    g.kh = a->kernel[0];
    g.kw = a->kernel[1];
    g.sy = a->stride[0];
    g.sx = a->stride[1];
    g.pad_t = a->pad[0];
    g.pad_l = a->pad[2];
    g.groups = (int)(C / (4 * v));
    const int64_t row_items = OW * g.groups;
    if (row_items >= (1 << 16)) return 0;  // the magic-number division holds below 2^16
    g.row_items = (int)row_items;
    g.row_blocks = (int)((row_items + kBlock - 1) / kBlock);
    g.groups_magic = (uint32_t)((uint64_t(1) << 32) / (uint64_t)g.groups + 1);
    const int64_t blocks = N * OH * g.row_blocks;
    if (blocks >= (int64_t(1) << 31) - 8) return 0;
    g.blocks = (int)blocks;
    g.chunk = (int)((blocks + 7) / 8);
    const dim3 grid((unsigned)(g.chunk * 8));
    const int k = (g.kh == g.kw && (g.kh == 2 || g.kh == 3)) ? g.kh : 0;
#define MLEL_MAXPOOL(VV)                                                              \
    if (k == 3)                                                                       \
        maxpool_i8_kernel<VV, 3><<<grid, dim3(kBlock), 0, s>>>(g);                    \
    else if (k == 2)                                                                  \
        maxpool_i8_kernel<VV, 2><<<grid, dim3(kBlock), 0, s>>>(g);                    \
    else                                                                              \
        maxpool_i8_kernel<VV, 0><<<grid, dim3(kBlock), 0, s>>>(g);
    if (wide) {
        MLEL_MAXPOOL(4)
    } else {
        MLEL_MAXPOOL(1)
    }
#undef MLEL_MAXPOOL
    MLEL_TRY(check_launch("max_pool2d (int8)"));
    return 1;
}

}  // namespace mlel
