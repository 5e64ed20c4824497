// Bandwidth-bound specialisations of the floating-point operators (fp16 / fp32 storage): 128-bit accesses, eight
// elements per thread, no per-element index arithmetic.  Arithmetic is the generic kernels' (ops_generic.hip) to the
// bit: operands are widened to fp32, the operator is applied once, and the result is rounded once into the storage
// type (reference: elementwise_binary.comp:146-173, mul.comp:24-59, elementwise_unary.comp:136-205,
// cast.comp:22-103, reduce.comp:24-70).  `try_*` returns 0 to decline a case.
#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {

namespace {

constexpr int kBlock = 256;

enum FOp { F_ADD, F_SUB, F_MUL, F_EXP, F_RECIPROCAL, F_RSQRT, F_TANH, F_COPY };

struct EwArgs {
    char *out;
    const char *a, *b;
    int64_t vecs;     // rows * cols / 8
    int32_t cols8;    // cols / 8
    int32_t cols;
    int32_t a_row, a_col, b_row, b_col;  // 1 when the operand varies along rows / columns, 0 when it is broadcast
};

template <int SIZE>
__device__ __forceinline__ void load8(const char *base, int64_t row, int32_t c8, int32_t cols, int varies_row,
                                      int varies_col, float (&v)[8]) {
    const int64_t r = varies_row ? row : 0;
    if (varies_col) {
        const char *p = base + (r * cols + (int64_t)c8 * 8) * SIZE;
        if (SIZE == 2) {
            const uint4 raw = *reinterpret_cast<const uint4 *>(p);
            const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float2 f = __half22float2(h[i]);
                v[2 * i] = f.x;
                v[2 * i + 1] = f.y;
            }
        } else {
            const float4 lo = *reinterpret_cast<const float4 *>(p), hi = *reinterpret_cast<const float4 *>(p + 16);
            v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
        }
    } else {
        const char *p = base + r * SIZE;
        const float s = SIZE == 2 ? __half2float(*reinterpret_cast<const __half *>(p)) : *reinterpret_cast<const float *>(p);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = s;
    }
}

template <int SIZE>
__device__ __forceinline__ void store8(char *p, const float (&v)[8]) {
    if (SIZE == 2) {
        uint4 raw;
        __half2 *h = reinterpret_cast<__half2 *>(&raw);
#pragma unroll
        for (int i = 0; i < 4; i++) h[i] = __halves2half2(__float2half_rn(v[2 * i]), __float2half_rn(v[2 * i + 1]));
        *reinterpret_cast<uint4 *>(p) = raw;
    } else {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(p + 16) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

template <int OP, int IN_SIZE, int OUT_SIZE>
__global__ void __launch_bounds__(kBlock) ew_float_kernel(const EwArgs g) {
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v >= g.vecs) return;
    const int64_t row = v / g.cols8;
    const int32_t c8 = (int32_t)(v - row * g.cols8);
    float a[8], b[8], r[8];
    load8<IN_SIZE>(g.a, row, c8, g.cols, g.a_row, g.a_col, a);
    if (OP == F_ADD || OP == F_SUB || OP == F_MUL) load8<IN_SIZE>(g.b, row, c8, g.cols, g.b_row, g.b_col, b);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        switch (OP) {
        case F_ADD: r[i] = a[i] + b[i]; break;
        case F_SUB: r[i] = a[i] - b[i]; break;
        case F_MUL: r[i] = a[i] * b[i]; break;  // operands already have the output's storage type
        case F_EXP: r[i] = expf(a[i]); break;
        case F_RECIPROCAL: r[i] = 1.0f / a[i]; break;
        case F_RSQRT: r[i] = 1.0f / sqrtf(a[i]); break;
        case F_TANH: r[i] = tanh_clamped(a[i]); break;
        default: r[i] = a[i]; break;
        }
    }
    store8<OUT_SIZE>(g.out + v * 8 * OUT_SIZE, r);
}

// How `in` relates to the dense output: same extents on every leading dimension (varies along rows) or 1 on all of
// them, and the same last extent (varies along columns) or 1.  Returns false when neither pattern applies.
bool classify(const mlel_tensor *out, const mlel_tensor *in, int *varies_row, int *varies_col) {
    if (in->rank != out->rank || !is_packed(in)) return false;
    const int last = out->rank - 1;
    bool all_same = true, all_one = true;
    for (int i = 0; i < last; i++) {
        all_same = all_same && in->dims[i] == out->dims[i];
        all_one = all_one && in->dims[i] == 1;
    }
    if (!all_same && !all_one) return false;
    if (in->dims[last] != out->dims[last] && in->dims[last] != 1) return false;
    *varies_row = all_same ? 1 : 0;
    *varies_col = in->dims[last] == out->dims[last] ? 1 : 0;
    const int64_t align = *varies_col ? 16 : dt_size(in->dtype);
    return ((uintptr_t)in->ptr % align) == 0;
}

template <int OP>
int launch_ew(hipStream_t s, const EwArgs &g, int in_size, int out_size) {
    const int64_t blocks = (g.vecs + kBlock - 1) / kBlock;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "elementwise: too many work items");
    const dim3 grid((unsigned)blocks), block(kBlock);
    if (in_size == 2 && out_size == 2)
        ew_float_kernel<OP, 2, 2><<<grid, block, 0, s>>>(g);
    else if (in_size == 4 && out_size == 4)
        ew_float_kernel<OP, 4, 4><<<grid, block, 0, s>>>(g);
    else if (in_size == 4 && out_size == 2)
        ew_float_kernel<OP, 4, 2><<<grid, block, 0, s>>>(g);
    else
        ew_float_kernel<OP, 2, 4><<<grid, block, 0, s>>>(g);
    MLEL_TRY(check_launch("elementwise float"));
    return 1;
}

bool float_dt(int dt) { return dt == MLEL_F16 || dt == MLEL_F32; }

// Fills the launch description for a dense output; false when the fast kernel does not apply.
bool describe(const mlel_tensor *out, const mlel_tensor *a, const mlel_tensor *b, EwArgs *g) {
    if (out->rank < 1 || !is_packed(out) || ((uintptr_t)out->ptr % 16) != 0) return false;
    const int64_t cols = out->dims[out->rank - 1];
    const int64_t total = numel(out);
    if (cols <= 0 || cols % 8 != 0 || cols >= (int64_t(1) << 31) || total <= 0) return false;
    g->out = static_cast<char *>(out->ptr);
    g->cols = (int32_t)cols;
    g->cols8 = (int32_t)(cols / 8);
    g->vecs = total / 8;
    if (!classify(out, a, &g->a_row, &g->a_col)) return false;
    g->a = static_cast<const char *>(a->ptr);
    if (b) {
        if (!classify(out, b, &g->b_row, &g->b_col)) return false;
        g->b = static_cast<const char *>(b->ptr);
    }
    return true;
}

}  // namespace

int try_binary_float_fast(mlel_ctx *, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in1,
                          const mlel_tensor *in2) {
    if (!float_dt(out->dtype) || in1->dtype != out->dtype || in2->dtype != out->dtype) return 0;
    EwArgs g{};
    if (!describe(out, in1, in2, &g)) return 0;
    const int sz = dt_size(out->dtype);
    switch (op) {
    case MLEL_BIN_ADD: return launch_ew<F_ADD>(s, g, sz, sz);
    case MLEL_BIN_SUB: return launch_ew<F_SUB>(s, g, sz, sz);
    default: return 0;
    }
}

int try_mul_float_fast(mlel_ctx *, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1,
                       const mlel_tensor *in2) {
    if (!float_dt(out->dtype) || in1->dtype != out->dtype || in2->dtype != out->dtype) return 0;
    EwArgs g{};
    if (!describe(out, in1, in2, &g)) return 0;
    const int sz = dt_size(out->dtype);
    return launch_ew<F_MUL>(s, g, sz, sz);
}

int try_unary_float_fast(mlel_ctx *, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in) {
    if (!float_dt(out->dtype) || in->dtype != out->dtype || !same_shape(out, in)) return 0;
    EwArgs g{};
    if (!describe(out, in, nullptr, &g)) return 0;
    const int sz = dt_size(out->dtype);
    switch (op) {
    case MLEL_UN_EXP: return launch_ew<F_EXP>(s, g, sz, sz);
    case MLEL_UN_RECIPROCAL: return launch_ew<F_RECIPROCAL>(s, g, sz, sz);
    case MLEL_UN_RSQRT: return launch_ew<F_RSQRT>(s, g, sz, sz);
    case MLEL_UN_TANH: return launch_ew<F_TANH>(s, g, sz, sz);
    default: return 0;
    }
}

int try_cast_float_fast(mlel_ctx *, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in) {
    if (!float_dt(out->dtype) || !float_dt(in->dtype) || in->dtype == out->dtype || !same_shape(out, in)) return 0;
    EwArgs g{};
    if (!describe(out, in, nullptr, &g)) return 0;
    return launch_ew<F_COPY>(s, g, dt_size(in->dtype), dt_size(out->dtype));
}

namespace {

// ---------------------------------------------------------------------------------------------------------------
// REDUCE_SUM / REDUCE_MAX along the last axis of a dense fp16 tensor, with the reference's sequential semantics
// (reduce.comp:24-70: a left-to-right fold in the storage type, so every partial sum is rounded to fp16).  Each
// block owns 64 rows: its four wavefronts copy a slab of 64 rows x up to 1024 columns into shared memory with coalesced
// 128-bit loads and then the lanes of the first wavefront fold one row each out of shared memory, element by element.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kSlabMaxCols = 1024;  // halfs per row and slab: 64 rows x 1024 x 2 B = 128 KB of shared memory at most

struct ReduceArgs {
    const char *in;
    char *out;
    int64_t rows;
    int32_t cols;       // multiple of 8
    int32_t slab_cols;  // min(cols, kSlabMaxCols), multiple of 8
    int32_t ignore_nan;
};

template <bool IS_SUM>
__global__ void __launch_bounds__(kBlock) reduce_rows_f16_kernel(const ReduceArgs g) {
    // A block owns 64 rows.  A fold is sequential along its row, so parallelism comes from rows only and small row
    // counts (LayerNorm over a few thousand tokens) must still spread over many compute units; all four wavefronts
    // fetch the slab (many loads in flight), then the first one folds it out of shared memory, one row per lane.
    extern __shared__ __align__(16) char slab[];
    const int pitch = g.slab_cols * 2 + 8;  // bytes; 8-byte aligned, consecutive rows two banks apart
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * 64;
    const int64_t row = row0 + tid;
    float r = IS_SUM ? 0.f : (g.ignore_nan ? NAN : -65504.f);
    bool done = false;
    for (int c0 = 0; c0 < g.cols; c0 += g.slab_cols) {
        const int n = min(g.slab_cols, g.cols - c0);
        const int segs = n >> 3;       // 16-byte pieces per row
        const int pieces = 64 * segs;  // consecutive threads take consecutive pieces of a row
        for (int p0 = 0; p0 < pieces; p0 += kBlock * 8) {
            uint4 v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int p = p0 + i * kBlock + tid;
                const int rr = p / segs, seg = p - rr * segs;
                v[i] = make_uint4(0, 0, 0, 0);
                if (p < pieces && row0 + rr < g.rows)
                    v[i] = *reinterpret_cast<const uint4 *>(g.in + ((row0 + rr) * g.cols + c0 + seg * 8) * 2);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int p = p0 + i * kBlock + tid;
                const int rr = p / segs, seg = p - rr * segs;
                if (p < pieces) {
                    *reinterpret_cast<uint2 *>(slab + rr * pitch + seg * 16) = make_uint2(v[i].x, v[i].y);
                    *reinterpret_cast<uint2 *>(slab + rr * pitch + seg * 16 + 8) = make_uint2(v[i].z, v[i].w);
                }
            }
        }
        __syncthreads();
        if (tid < 64) {
            uint2 next = *reinterpret_cast<const uint2 *>(slab + tid * pitch);
            for (int j = 0; j < n; j += 4) {
                const uint2 raw = next;
                if (j + 4 < n) next = *reinterpret_cast<const uint2 *>(slab + tid * pitch + (j + 4) * 2);
                const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
                // a NaN among the four halfs: exponent all ones and a non-zero mantissa, tested on the packed pairs
                const uint32_t nan_bits = (((raw.x & 0x7fff7fffu) + 0x03ff03ffu) | ((raw.y & 0x7fff7fffu) + 0x03ff03ffu)) &
                                          0x80008000u;
                if (!__any(done || nan_bits != 0)) {
                    // no lane of the wavefront is in a special state: the plain fold.  A native fp16 add rounds the
                    // exact sum once; the generic kernel's fp32 add followed by a conversion gives the same value,
                    // because the fp32 sum of two halfs is inexact only when the smaller one is far below half an ulp
                    // of the larger.
                    if (IS_SUM) {
                        __half acc = __float2half_rn(r);
                        acc = __hadd(acc, __low2half(h[0]));
                        acc = __hadd(acc, __high2half(h[0]));
                        acc = __hadd(acc, __low2half(h[1]));
                        acc = __hadd(acc, __high2half(h[1]));
                        r = __half2float(acc);
                    } else {
                        const float2 f01 = __half22float2(h[0]), f23 = __half22float2(h[1]);
                        const float e[4] = {f01.x, f01.y, f23.x, f23.y};
#pragma unroll
                        for (int t = 0; t < 4; t++) r = isnan(r) ? e[t] : (r < e[t] ? e[t] : r);
                    }
                    continue;
                }
                const float2 f01 = __half22float2(h[0]), f23 = __half22float2(h[1]);
                const float e[4] = {f01.x, f01.y, f23.x, f23.y};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const float v = e[t];
                    if (done) continue;
                    if (isnan(v)) {
                        if (g.ignore_nan) continue;
                        r = v;
                        done = true;
                        continue;
                    }
                    if (IS_SUM)
                        r = rnd_f16(r + v);
                    else
                        r = isnan(r) ? v : (r < v ? v : r);
                }
            }
        }
        __syncthreads();
    }
    if (tid < 64 && row < g.rows) *reinterpret_cast<__half *>(g.out + row * 2) = __float2half_rn(r);
}

}  // namespace

int try_reduce_float_fast(mlel_ctx *, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in,
                          uint32_t axis, uint32_t nan_mode) {
    if (in->dtype != MLEL_F16 || out->dtype != MLEL_F16) return 0;
    if (op != MLEL_RED_SUM && op != MLEL_RED_MAX) return 0;
    const int last = in->rank - 1;
    if (in->rank < 1 || (int)axis != last || out->rank != in->rank || out->dims[last] != 1) return 0;
    for (int i = 0; i < last; i++)
        if (out->dims[i] != in->dims[i]) return 0;
    if (!is_packed(in) || !is_packed(out) || ((uintptr_t)in->ptr % 16) != 0 || ((uintptr_t)out->ptr % 2) != 0) return 0;
    const int64_t cols = in->dims[last];
    if (cols <= 0 || cols % 8 != 0 || cols >= (int64_t(1) << 30)) return 0;
    const int64_t rows = numel(out);
    if (rows <= 0) return 1;
    ReduceArgs g{};
    g.in = static_cast<const char *>(in->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.rows = rows;
    g.cols = (int32_t)cols;
    g.ignore_nan = nan_mode == MLEL_NAN_IGNORE ? 1 : 0;
    const int64_t blocks = (rows + 63) / 64;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "reduce: too many rows");
    g.slab_cols = (int32_t)(cols < kSlabMaxCols ? cols : kSlabMaxCols);
    const size_t smem = (size_t)64 * (g.slab_cols * 2 + 8);
    auto kernel = op == MLEL_RED_SUM ? reduce_rows_f16_kernel<true> : reduce_rows_f16_kernel<false>;
    if (smem > 48 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)smem);
    kernel<<<dim3((unsigned)blocks), dim3(kBlock), smem, s>>>(g);
    MLEL_TRY(check_launch("reduce rows fp16"));
    return 1;
}

}  // namespace mlel
