// Bandwidth-bound specialisations of the floating-point operators (fp16 / fp32 storage): 128-bit accesses, eight
// elements per thread, no per-element index arithmetic.  Arithmetic is the generic kernels' (ops_generic.hip) to the
// bit: operands are widened to fp32, the operator is applied once, and the result is rounded once into the storage
// type (reference: elementwise_binary.comp:146-173, mul.comp:24-59, elementwise_unary.comp:136-205,
// cast.comp:22-103, reduce.comp:24-70).  `try_*` returns 0 to decline a case.
#include <type_traits>
#include <vector>

#include "common.hpp"
#include "dispatch.hpp"
#include "float_programs.hpp"

namespace mlel {

namespace {

constexpr int kBlock = 256;


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
        for (int i = 0; i < 4; i++) h[i] = __halves2half2(f2h(v[2 * i]), f2h(v[2 * i + 1]));
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
        case F_EXP: r[i] = op_exp<OUT_SIZE == 2>(a[i]); break;
        case F_RECIPROCAL: r[i] = op_reciprocal<OUT_SIZE == 2>(a[i]); break;
        case F_RSQRT: r[i] = op_rsqrt<OUT_SIZE == 2>(a[i]); break;
        case F_TANH: r[i] = op_tanh<OUT_SIZE == 2>(a[i]); break;
        default: r[i] = a[i]; break;
        }
    }
    store8<OUT_SIZE>(g.out + v * 8 * OUT_SIZE, r);
}


// ---------------------------------------------------------------------------------------------------------------
// A chain of elementwise operators in one pass.  Eight elements per thread; the values of the chain live in a small
// per-thread register file in shared memory (the program is data, so registers are addressed at run time): slot r of
// thread t holds eight floats at [r][half][t], conflict-free for a wavefront.  Each step applies its operator to the
// fp32 operands and rounds once into the step's storage type, as the stand-alone kernels above do.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kChainRegs = 4;

struct ChainInput {
    const char *ptr;
    int32_t size;        // 2 or 4 bytes per element
    int32_t varies_row;  // as EwArgs
    int32_t varies_col;
    int32_t reg;         // register the value is loaded into; single-element inputs: lane of the scalar file
};

struct alignas(16) ChainStep {  // sixteen bytes at a sixteen-byte boundary: one scalar load fetches a step
    int8_t op;          // FOp
    int8_t f16;         // result rounded to fp16 (else fp32)
    int8_t a, b;        // operand registers (or scalar-file lanes)
    int8_t a_sc, b_sc;  // the operand is a single-element input
    int8_t a_fw, b_fw;  // the operand is the previous step's result, still in vector registers
    int8_t dst;         // result register, or -1 when only the next step reads the result
};

struct ChainArgs {
    char *out;
    int32_t out_size, out_reg;
    int64_t vecs;
    int32_t cols8, cols;
    int32_t n_inputs, n_steps;
    ChainInput in[MLEL_CHAIN_MAX_INPUTS];
    ChainStep step[MLEL_CHAIN_MAX_STEPS];
};

// HALF: every value of the chain (inputs and results) is fp16, so a register is eight halfs (16 bytes) instead of
// eight floats: half the shared memory, twice the resident wavefronts, which is what a latency-bound streaming
// kernel needs.
template <bool HALF>
__global__ void __launch_bounds__(kBlock) ew_chain_kernel(const ChainArgs g) {
    constexpr int kRegs = HALF ? kChainRegs + 2 : kChainRegs;
    __shared__ uint4 regs[kRegs][HALF ? 1 : 2][kBlock];
    // The program is indexed at run time; read straight from the kernel arguments that costs a trip to memory per
    // step and wavefront.  The block copies it into shared memory once and every step is then one broadcast read.
    __shared__ uint4 program[MLEL_CHAIN_MAX_STEPS];
    static_assert(sizeof(ChainStep) == sizeof(uint4), "a step is one 16-byte word");
    const int tid = threadIdx.x;
    const auto step_at = [&](int s) {
        uint4 w = program[s];
        w.x = __builtin_amdgcn_readfirstlane(w.x);
        w.y = __builtin_amdgcn_readfirstlane(w.y);
        w.z = __builtin_amdgcn_readfirstlane(w.z);
        ChainStep st;
        __builtin_memcpy(&st, &w, sizeof st);
        return st;
    };
    // threads past the end repeat the last vector and store nothing: every thread reaches the barrier below
    const int64_t v_raw = (int64_t)blockIdx.x * kBlock + tid;
    const bool active = v_raw < g.vecs;
    const int64_t v = active ? v_raw : g.vecs - 1;
    const int64_t row = v / g.cols8;
    const int32_t c8 = (int32_t)(v - row * g.cols8);
    const auto put = [&](int r, const float (&x)[8]) {
        if (HALF) {  // the values are fp16 numbers already: the conversion is exact
            uint4 raw;
            __half2 *h = reinterpret_cast<__half2 *>(&raw);
#pragma unroll
            for (int i = 0; i < 4; i++) h[i] = __halves2half2(f2h(x[2 * i]), f2h(x[2 * i + 1]));
            regs[r][0][tid] = raw;
        } else {
            regs[r][0][tid] = make_uint4(__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3]));
            regs[r][HALF ? 0 : 1][tid] =
                make_uint4(__float_as_uint(x[4]), __float_as_uint(x[5]), __float_as_uint(x[6]), __float_as_uint(x[7]));
        }
    };
    const auto get = [&](int r, float (&x)[8]) {
        if (HALF) {
            const uint4 raw = regs[r][0][tid];
            const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float2 f = __half22float2(h[i]);
                x[2 * i] = f.x;
                x[2 * i + 1] = f.y;
            }
        } else {
            const uint4 lo = regs[r][0][tid], hi = regs[r][HALF ? 0 : 1][tid];
            x[0] = __uint_as_float(lo.x), x[1] = __uint_as_float(lo.y), x[2] = __uint_as_float(lo.z), x[3] = __uint_as_float(lo.w);
            x[4] = __uint_as_float(hi.x), x[5] = __uint_as_float(hi.y), x[6] = __uint_as_float(hi.z), x[7] = __uint_as_float(hi.w);
        }
    };
    // single-element inputs live in one vector register, lane k holding scalar k (read back with a lane broadcast);
    // the other inputs are all requested before any is stored, so that their loads overlap
    int sc_bits = 0;
    float x[MLEL_CHAIN_MAX_INPUTS][8];
#pragma unroll
    for (int k = 0; k < MLEL_CHAIN_MAX_INPUTS; k++) {
        if (k >= g.n_inputs) continue;  // uniform
        const ChainInput in = g.in[k];
        if (!in.varies_row && !in.varies_col) {
            const float s = in.size == 2 ? __half2float(*reinterpret_cast<const __half *>(in.ptr))
                                         : *reinterpret_cast<const float *>(in.ptr);
            sc_bits = (tid & 63) == in.reg ? __float_as_int(s) : sc_bits;
        } else if (in.size == 2) {
            load8<2>(in.ptr, row, c8, g.cols, in.varies_row, in.varies_col, x[k]);
        } else {
            load8<4>(in.ptr, row, c8, g.cols, in.varies_row, in.varies_col, x[k]);
        }
    }
    // the program is requested after the inputs, so that the two trips to memory overlap
    if (tid < g.n_steps) program[tid] = reinterpret_cast<const uint4 *>(g.step)[tid];
#pragma unroll
    for (int k = 0; k < MLEL_CHAIN_MAX_INPUTS; k++) {
        if (k >= g.n_inputs) continue;
        if (g.in[k].varies_row || g.in[k].varies_col) put(g.in[k].reg, x[k]);
    }
    __syncthreads();  // the program is in place (the registers are private to their thread)
    const auto fetch = [&](int r, int is_scalar, float (&y)[8]) {
        if (is_scalar) {  // uniform
            const float s = __int_as_float(__builtin_amdgcn_readlane(sc_bits, r));
#pragma unroll
            for (int i = 0; i < 8; i++) y[i] = s;
        } else {
            get(r, y);
        }
    };
    if (HALF) {
        // Every value is fp16: ADD, SUB and MUL run on packed halfs.  A native fp16 operation rounds the exact result
        // once; the fp32 operation followed by a conversion (the stand-alone kernels) gives the same value, because
        // the product of two halfs is exact in fp32 and fp32 carries more than twice the fp16 precision plus two bits,
        // so that the second rounding of a sum cannot change the result.
        const auto fetch_h = [&](int r, int is_scalar) {
            if (!is_scalar) return regs[r][0][tid];
            const __half s = f2h(__int_as_float(__builtin_amdgcn_readlane(sc_bits, r)));
            const __half2 s2 = __halves2half2(s, s);
            const uint32_t w = *reinterpret_cast<const uint32_t *>(&s2);
            return make_uint4(w, w, w, w);
        };
        uint4 rp = make_uint4(0, 0, 0, 0);
        for (int s = 0; s < g.n_steps; s++) {
            const ChainStep st = step_at(s);
            const uint4 a = st.a_fw ? rp : fetch_h(st.a, st.a_sc);
            const __half2 *ah = reinterpret_cast<const __half2 *>(&a);
            __half2 *rh = reinterpret_cast<__half2 *>(&rp);
            if (st.op == F_ADD || st.op == F_SUB || st.op == F_MUL) {
                const uint4 b = st.b_fw ? rp : fetch_h(st.b, st.b_sc);
                const __half2 *bh = reinterpret_cast<const __half2 *>(&b);
                uint4 out4;
                __half2 *oh = reinterpret_cast<__half2 *>(&out4);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    oh[i] = st.op == F_ADD ? __hadd2(ah[i], bh[i]) : st.op == F_SUB ? __hsub2(ah[i], bh[i]) : __hmul2(ah[i], bh[i]);
                rp = out4;
            } else {
                float x[8], y[8];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float2 f = __half22float2(ah[i]);
                    x[2 * i] = f.x;
                    x[2 * i + 1] = f.y;
                }
                switch (st.op) {  // uniform
                case F_EXP:
#pragma unroll
                    for (int i = 0; i < 8; i++) y[i] = op_exp<true>(x[i]);
                    break;
                case F_RECIPROCAL:
#pragma unroll
                    for (int i = 0; i < 8; i++) y[i] = op_reciprocal<true>(x[i]);
                    break;
                case F_RSQRT:
#pragma unroll
                    for (int i = 0; i < 8; i++) y[i] = op_rsqrt<true>(x[i]);
                    break;
                case F_TANH:
#pragma unroll
                    for (int i = 0; i < 8; i++) y[i] = op_tanh<true>(x[i]);
                    break;
                default:
#pragma unroll
                    for (int i = 0; i < 8; i++) y[i] = x[i];
                    break;
                }
#pragma unroll
                for (int i = 0; i < 4; i++) rh[i] = __halves2half2(f2h(y[2 * i]), f2h(y[2 * i + 1]));
            }
            if (s + 1 == g.n_steps) {
                if (active) *reinterpret_cast<uint4 *>(g.out + v * 16) = rp;
            } else if (st.dst >= 0) {
                regs[st.dst][0][tid] = rp;
            }
        }
        return;
    }
    float r[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < g.n_steps; s++) {
        const ChainStep st = step_at(s);
        float a[8], b[8];
        if (st.a_fw) {  // uniform
#pragma unroll
            for (int i = 0; i < 8; i++) a[i] = r[i];
        } else {
            fetch(st.a, st.a_sc, a);
        }
        if (st.op == F_ADD || st.op == F_SUB || st.op == F_MUL) {
            if (st.b_fw) {
#pragma unroll
                for (int i = 0; i < 8; i++) b[i] = r[i];
            } else {
                fetch(st.b, st.b_sc, b);
            }
        }
        switch (st.op) {  // uniform
        case F_ADD:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = a[i] + b[i];
            break;
        case F_SUB:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = a[i] - b[i];
            break;
        case F_MUL:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = a[i] * b[i];
            break;
        case F_EXP:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = st.f16 ? op_exp<true>(a[i]) : op_exp<false>(a[i]);
            break;
        case F_RECIPROCAL:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = st.f16 ? op_reciprocal<true>(a[i]) : op_reciprocal<false>(a[i]);
            break;
        case F_RSQRT:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = st.f16 ? op_rsqrt<true>(a[i]) : op_rsqrt<false>(a[i]);
            break;
        case F_TANH:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = st.f16 ? op_tanh<true>(a[i]) : op_tanh<false>(a[i]);
            break;
        default:
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = a[i];
            break;
        }
        if (st.f16) {
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = rnd_f16(r[i]);
        }
        if (s + 1 == g.n_steps) {  // the result goes straight to memory
            if (!active) {
            } else if (g.out_size == 2) {
                store8<2>(g.out + v * 16, r);
            } else {
                store8<4>(g.out + v * 32, r);
            }
        } else if (st.dst >= 0) {
            put(st.dst, r);
        }
    }
}

template <class P>
__global__ void __launch_bounds__(kBlock) ew_static_half_kernel(const StaticArgs g) {
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v >= g.vecs) return;
    uint4 val[P::n_inputs + P::n_steps];
#pragma unroll
    for (int k = 0; k < P::n_inputs; k++) {
        if (P::full[k]) {
            val[k] = *reinterpret_cast<const uint4 *>(g.in[k] + v * 16);
        } else {
            const uint32_t bits = *reinterpret_cast<const uint16_t *>(g.in[k]);
            const uint32_t w = bits | (bits << 16);
            val[k] = make_uint4(w, w, w, w);
        }
    }
    static_run<P, 0>(val);
    store16_result(g.out + v * 16, val[P::n_inputs + P::n_steps - 1]);
}

// the chain is P's program over inputs of P's shapes
template <class P>
bool matches_static(const mlel_tensor *out, const mlel_chain *c, const int *ops) {
    if (c->n_inputs != P::n_inputs || c->n_steps != P::n_steps) return false;
    for (int k = 0; k < P::n_inputs; k++) {
        const mlel_tensor *t = c->inputs[k];
        const bool full = same_shape(t, out) && is_packed(t) && ((uintptr_t)t->ptr % 16) == 0;
        const bool single = numel(t) == 1 && ((uintptr_t)t->ptr % 2) == 0;
        if (t->dtype != MLEL_F16 || !(P::full[k] ? full : single)) return false;
    }
    for (int i = 0; i < P::n_steps; i++) {
        const bool two = ops[i] == F_ADD || ops[i] == F_SUB || ops[i] == F_MUL;
        if (ops[i] != P::steps[i].op || c->steps[i].a != P::steps[i].a || (two && c->steps[i].b != P::steps[i].b) ||
            c->steps[i].dtype != MLEL_F16)
            return false;
    }
    return true;
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

// ---------------------------------------------------------------------------------------------------------------
// The same for the reduced-precision storage types (bf16, fp8 e4m3 / e5m2; reference codecs common.comp:184-611):
// ADD, SUB, MUL and CAST, eight elements per thread with one 64-, 128- or 2 x 128-bit access per operand.  Every
// element goes through the codec functions of the generic kernels (decode to fp32, one operation, raw_st_f's
// rounding rule for the operator), so the results are theirs to the bit.
// ---------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float lowp_decode(int dt, uint32_t bits) {
    switch (dt) {
    case MLEL_F16: return __half2float(__ushort_as_half((unsigned short)bits));
    case MLEL_BF16: return decode_bf16((uint16_t)bits);
    case MLEL_F8E4M3: return decode_f8e4m3((uint8_t)bits);
    case MLEL_F8E5M2: return decode_f8e5m2((uint8_t)bits);
    default: return __uint_as_float(bits);
    }
}
__device__ __forceinline__ uint32_t lowp_encode(int dt, float v, int mode) {
    switch (dt) {
    case MLEL_F16: return (uint32_t)__half_as_ushort(f2h(v));
    case MLEL_BF16: return mode == ST_RNE ? encode_bf16_rne(v) : encode_bf16_trunc(v);
    case MLEL_F8E4M3:
    case MLEL_F8E5M2: return encode_f8(dt, mode == ST_ACC ? v : __half2float(f2h(v)));
    default: return __float_as_uint(v);
    }
}
// eight consecutive elements of `size` bytes each as dwords (size 1: two, 2: four, 4: eight)
template <int SIZE>
__device__ __forceinline__ void lowp_load8(const char *base, int dt, int64_t row, int32_t c8, int32_t cols, int varies_row,
                                           int varies_col, float (&v)[8]) {
    const int64_t r = varies_row ? row : 0;
    if (!varies_col) {
        const char *p = base + r * SIZE;
        const uint32_t bits = SIZE == 1 ? *reinterpret_cast<const uint8_t *>(p)
                                        : (SIZE == 2 ? *reinterpret_cast<const uint16_t *>(p) : *reinterpret_cast<const uint32_t *>(p));
        const float s = lowp_decode(dt, bits);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = s;
        return;
    }
    const char *p = base + (r * cols + (int64_t)c8 * 8) * SIZE;
    uint32_t w[2 * SIZE];
    if (SIZE == 1) {
        const uint2 raw = *reinterpret_cast<const uint2 *>(p);
        w[0] = raw.x, w[1] = raw.y;
    } else {
#pragma unroll
        for (int k = 0; k < SIZE / 2; k++) {
            const uint4 raw = *reinterpret_cast<const uint4 *>(p + 16 * k);
            w[4 * k] = raw.x, w[4 * k + 1] = raw.y, w[4 * k + 2] = raw.z, w[4 * k + 3] = raw.w;
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t bits = SIZE == 1 ? (w[i >> 2] >> (8 * (i & 3))) & 0xffu
                                        : (SIZE == 2 ? (w[i >> 1] >> (16 * (i & 1))) & 0xffffu : w[i]);
        v[i] = lowp_decode(dt, bits);
    }
}
template <int SIZE>
__device__ __forceinline__ void lowp_store8(char *p, int dt, int mode, const float (&v)[8]) {
    uint32_t w[2 * SIZE];
#pragma unroll
    for (int k = 0; k < 2 * SIZE; k++) w[k] = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t bits = lowp_encode(dt, v[i], mode);
        if (SIZE == 1) w[i >> 2] |= (bits & 0xffu) << (8 * (i & 3));
        else if (SIZE == 2) w[i >> 1] |= (bits & 0xffffu) << (16 * (i & 1));
        else w[i] = bits;
    }
    if (SIZE == 1) {
        *reinterpret_cast<uint2 *>(p) = make_uint2(w[0], w[1]);
    } else {
#pragma unroll
        for (int k = 0; k < SIZE / 2; k++) *reinterpret_cast<uint4 *>(p + 16 * k) = make_uint4(w[4 * k], w[4 * k + 1], w[4 * k + 2], w[4 * k + 3]);
    }
}

template <int OP, int IN_SIZE, int OUT_SIZE>
__global__ void __launch_bounds__(kBlock) ew_lowp_kernel(const EwArgs g, int in_dt, int out_dt, int mode) {
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v >= g.vecs) return;
    const int64_t row = v / g.cols8;
    const int32_t c8 = (int32_t)(v - row * g.cols8);
    float a[8], b[8], r[8];
    lowp_load8<IN_SIZE>(g.a, in_dt, row, c8, g.cols, g.a_row, g.a_col, a);
    if (OP != F_COPY) lowp_load8<IN_SIZE>(g.b, in_dt, row, c8, g.cols, g.b_row, g.b_col, b);
#pragma unroll
    for (int i = 0; i < 8; i++) r[i] = OP == F_ADD ? a[i] + b[i] : (OP == F_SUB ? a[i] - b[i] : (OP == F_MUL ? a[i] * b[i] : a[i]));
    lowp_store8<OUT_SIZE>(g.out + v * 8 * OUT_SIZE, out_dt, mode, r);
}

bool lowp_dt(int dt) { return dt == MLEL_BF16 || dt == MLEL_F8E4M3 || dt == MLEL_F8E5M2; }

template <int OP>
int launch_lowp(hipStream_t s, const EwArgs &g, int in_dt, int out_dt, int mode) {
    const int64_t blocks = (g.vecs + kBlock - 1) / kBlock;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "elementwise: too many work items");
    const dim3 grid((unsigned)blocks), block(kBlock);
    const int is = dt_size(in_dt), os = dt_size(out_dt);
#define MLEL_LOWP_CASE(IS, OS) \
    if (is == IS && os == OS) ew_lowp_kernel<OP, IS, OS><<<grid, block, 0, s>>>(g, in_dt, out_dt, mode)
    MLEL_LOWP_CASE(1, 1);
    else MLEL_LOWP_CASE(2, 2);
    else MLEL_LOWP_CASE(1, 2);
    else MLEL_LOWP_CASE(1, 4);
    else MLEL_LOWP_CASE(2, 1);
    else MLEL_LOWP_CASE(2, 4);
    else MLEL_LOWP_CASE(4, 1);
    else MLEL_LOWP_CASE(4, 2);
    else return 0;
#undef MLEL_LOWP_CASE
    MLEL_TRY(check_launch("elementwise reduced precision"));
    return 1;
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
    if (in1->dtype != out->dtype || in2->dtype != out->dtype) return 0;
    if (lowp_dt(out->dtype)) {  // ADD and SUB round to nearest even into the storage type (binary_generic)
        EwArgs l{};
        if ((op != MLEL_BIN_ADD && op != MLEL_BIN_SUB) || !describe(out, in1, in2, &l)) return 0;
        return op == MLEL_BIN_ADD ? launch_lowp<F_ADD>(s, l, out->dtype, out->dtype, ST_RNE)
                                  : launch_lowp<F_SUB>(s, l, out->dtype, out->dtype, ST_RNE);
    }
    if (!float_dt(out->dtype)) return 0;
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
    if (in1->dtype != out->dtype || in2->dtype != out->dtype) return 0;
    if (lowp_dt(out->dtype)) {  // operands of the output's type are their own rounding (mul_generic)
        EwArgs l{};
        if (!describe(out, in1, in2, &l)) return 0;
        return launch_lowp<F_MUL>(s, l, out->dtype, out->dtype, ST_RNE);
    }
    if (!float_dt(out->dtype)) return 0;
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
    if (in->dtype == out->dtype || !same_shape(out, in)) return 0;
    if ((lowp_dt(out->dtype) && (lowp_dt(in->dtype) || float_dt(in->dtype))) || (lowp_dt(in->dtype) && float_dt(out->dtype))) {
        // to bf16: round to nearest even; to fp8: the fp32 value is encoded directly (cast_generic)
        EwArgs l{};
        if (!describe(out, in, nullptr, &l)) return 0;
        return launch_lowp<F_COPY>(s, l, in->dtype, out->dtype, out->dtype == MLEL_BF16 ? ST_RNE : ST_ACC);
    }
    if (!float_dt(out->dtype) || !float_dt(in->dtype)) return 0;
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
constexpr int kSlabCols = 256;  // halfs per row and slab: two buffers of 64 rows x 256 x 2 B (+ padding) = 66 KB

struct ReduceArgs {
    const char *in;
    char *out;
    int64_t rows;
    int32_t cols;       // multiple of 8
    int32_t slab_cols;  // min(cols, kSlabCols), multiple of 8
    int32_t ignore_nan;
};

template <bool IS_SUM>
__global__ void __launch_bounds__(kBlock) reduce_rows_f16_kernel(const ReduceArgs g) {
    // A block owns 64 rows.  A fold is sequential along its row, so parallelism comes from rows only and small row
    // counts (LayerNorm over a few thousand tokens) must still spread over many compute units.  The row is walked in
    // slabs through two buffers: the first wavefront folds slab k out of shared memory, one row per lane, while the
    // other three fetch slab k + 1 (the first slab is fetched by all four).
    extern __shared__ __align__(16) char slab[];
    const int pitch = g.slab_cols * 2 + 16;  // bytes; 16-byte aligned, consecutive rows four banks apart
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * 64;
    const int64_t row = row0 + tid;
    float r = IS_SUM ? 0.f : (g.ignore_nan ? NAN : -65504.f);
    bool done = false;
    // consecutive threads take consecutive 16-byte pieces of a row; eight loads in flight per thread
    const auto stage = [&](int c0, char *buf, int first, int nthreads) {
        const int n = min(g.slab_cols, g.cols - c0);
        const int segs = n >> 3, pieces = 64 * segs;
        for (int p0 = 0; p0 < pieces; p0 += nthreads * 8) {
            uint4 v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int p = p0 + i * nthreads + (tid - first);
                const int rr = p / segs, seg = p - rr * segs;
                v[i] = make_uint4(0, 0, 0, 0);
                if (p < pieces && row0 + rr < g.rows)
                    v[i] = *reinterpret_cast<const uint4 *>(g.in + ((row0 + rr) * g.cols + c0 + seg * 8) * 2);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int p = p0 + i * nthreads + (tid - first);
                const int rr = p / segs, seg = p - rr * segs;
                if (p < pieces) *reinterpret_cast<uint4 *>(buf + rr * pitch + seg * 16) = v[i];
            }
        }
    };
    const int buf_bytes = 64 * pitch;
    stage(0, slab, 0, kBlock);
    __syncthreads();
    int which = 0;
    for (int c0 = 0; c0 < g.cols; c0 += g.slab_cols, which ^= 1) {
        const int n = min(g.slab_cols, g.cols - c0);
        if (tid >= 64) {
            if (c0 + g.slab_cols < g.cols) stage(c0 + g.slab_cols, slab + (which ^ 1) * buf_bytes, 64, kBlock - 64);
        } else {
            const char *mine = slab + which * buf_bytes + tid * pitch;
            // a NaN among eight halfs: exponent all ones and a non-zero mantissa, tested on the packed pairs
            const auto nan_bits = [](const uint4 &raw) {
                return (((raw.x & 0x7fff7fffu) + 0x03ff03ffu) | ((raw.y & 0x7fff7fffu) + 0x03ff03ffu) |
                        ((raw.z & 0x7fff7fffu) + 0x03ff03ffu) | ((raw.w & 0x7fff7fffu) + 0x03ff03ffu)) & 0x80008000u;
            };
            // No lane of the wavefront in a special state: the plain fold.  A native fp16 add rounds the exact sum
            // once; the generic kernel's fp32 add followed by a conversion gives the same value (fp32 carries more
            // than twice the fp16 precision plus two bits, so the second rounding cannot change the result).
            const auto fold_plain = [&](const uint4 &raw, __half &acc, float &mx) {
                const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
                if (IS_SUM) {
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        acc = __hadd(acc, __low2half(h[t]));
                        acc = __hadd(acc, __high2half(h[t]));
                    }
                } else {
                    // the order of a maximum is free: pairwise on the packed halfs, then against the state
                    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
                    const h2_t *p = reinterpret_cast<const h2_t *>(&raw);
                    const h2_t m = __builtin_elementwise_max(__builtin_elementwise_max(p[0], p[1]),
                                                             __builtin_elementwise_max(p[2], p[3]));
                    const float e = (float)(m.x > m.y ? m.x : m.y);
                    mx = isnan(mx) ? e : (mx < e ? e : mx);
                }
            };
            const auto fold_careful = [&](const uint4 &raw) {  // NaN-aware, element by element
                const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
                float e[8];
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const float2 f = __half22float2(h[t]);
                    e[2 * t] = f.x;
                    e[2 * t + 1] = f.y;
                }
#pragma unroll
                for (int t = 0; t < 8; t++) {
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
            };
            // groups of 32 elements: one test for special values per group keeps the dependent chain of the fold short
            int j = 0;
            uint4 nxt[4];
            if (n >= 32) {
#pragma unroll
                for (int t = 0; t < 4; t++) nxt[t] = *reinterpret_cast<const uint4 *>(mine + t * 16);
            }
            for (; j + 32 <= n; j += 32) {
                uint4 raw[4];
#pragma unroll
                for (int t = 0; t < 4; t++) raw[t] = nxt[t];
                if (j + 64 <= n) {
#pragma unroll
                    for (int t = 0; t < 4; t++) nxt[t] = *reinterpret_cast<const uint4 *>(mine + (j + 32) * 2 + t * 16);
                }
                const uint32_t special = nan_bits(raw[0]) | nan_bits(raw[1]) | nan_bits(raw[2]) | nan_bits(raw[3]);
                if (!__any(done || special != 0)) {
                    __half acc = f2h(r);
                    float mx = r;
#pragma unroll
                    for (int t = 0; t < 4; t++) fold_plain(raw[t], acc, mx);
                    r = IS_SUM ? __half2float(acc) : mx;
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++) fold_careful(raw[t]);
                }
            }
            for (; j < n; j += 8) fold_careful(*reinterpret_cast<const uint4 *>(mine + j * 2));
        }
        __syncthreads();
    }
    if (tid < 64 && row < g.rows) *reinterpret_cast<__half *>(g.out + row * 2) = f2h(r);
}


// ---------------------------------------------------------------------------------------------------------------
// A chain of fp16 operators with reductions over the last axis in it (LayerNorm's moments, softmax with its scale,
// ...), in one pass.  Values come in four shapes: full [rows, cols], one per row [rows, 1], one per column
// [1, cols] and single elements.  A block owns R = 4 .. 64 rows; the full values that are alive at the same time
// sit in shared memory ("row registers", R rows of cols halfs each), the per-row values in a small file of their own.
// 256 / R threads share a row: elementwise steps walk the row's 16-byte pieces with them (a piece is always handled
// by the same thread, so consecutive elementwise steps need no barrier), REDUCE_SUM is folded left to right in fp16
// by the row's first thread (reduce.comp:24-70), REDUCE_MAX is taken pairwise by all of them.  Every step rounds to
// fp16 where the stand-alone operator rounds, with the same device functions.  A reduction over a row that holds a
// NaN yields a NaN (the stand-alone kernels return the first one met; payload and sign are not kept here).
// ---------------------------------------------------------------------------------------------------------------
enum { F_RED_SUM = 16, F_RED_MAX = 17 };
enum RowClass : int8_t { RC_ONE = 0, RC_COL = 1, RC_ROW_IN = 2, RC_ROW = 3, RC_FULL = 4 };
constexpr int kRowRegs = 4;       // full values alive at once
constexpr int kRowScalars = 8;    // per-row values alive at once
constexpr int kRowLdsBudget = 64 * 1024;

struct RowOperand {
    int8_t cls;  // RowClass
    int8_t idx;  // RC_FULL: row register; RC_ROW: slot of the per-row file; RC_COL: slot of the column file;
                 // otherwise the input's index
};
struct alignas(8) RowStep {  // eight bytes: one scalar load fetches a step
    int8_t op;      // FOp or F_RED_*
    int8_t cls;     // RC_FULL or RC_ROW: shape of the result
    RowOperand a, b;
    int8_t dst;     // row register / per-row slot of the result; -1: the result is the output
    int8_t pad;
};
struct RowArgs {
    char *out;
    int64_t rows;
    const char *in[MLEL_CHAIN_MAX_INPUTS];
    RowStep step[MLEL_CHAIN_MAX_STEPS];
    int32_t cols;
    int32_t log2_r;
    int32_t n_inputs, n_steps, n_regs;
    int32_t n_cols;                        // per-column inputs
    int8_t in_reg[MLEL_CHAIN_MAX_INPUTS];  // row register a full input is fetched into, -1 for the other shapes
    int8_t in_cls[MLEL_CHAIN_MAX_INPUTS];  // RowClass of the input
    int8_t in_col[MLEL_CHAIN_MAX_INPUTS];  // per-column inputs: slot of the column file
};

__device__ __forceinline__ float row_apply(int op, float a, float b) {
    switch (op) {
    case F_ADD: return a + b;
    case F_SUB: return a - b;
    case F_MUL: return a * b;
    case F_EXP: return op_exp<true>(a);
    case F_RECIPROCAL: return op_reciprocal<true>(a);
    case F_RSQRT: return op_rsqrt<true>(a);
    case F_TANH: return op_tanh<true>(a);
    default: return a;
    }
}

__global__ void __launch_bounds__(kBlock) row_chain_f16_kernel(const RowArgs g) {
    extern __shared__ __align__(16) char lds[];
    const int R = 1 << g.log2_r, tpr_log = 8 - g.log2_r, TPR = 1 << tpr_log;
    const int pitch = g.cols * 2 + 16, reg_bytes = R * pitch;
    __half *row_file = reinterpret_cast<__half *>(lds + g.n_regs * reg_bytes);  // [kRowScalars][64]
    __half *one_file = row_file + kRowScalars * 64;                              // [MLEL_CHAIN_MAX_INPUTS]
    char *col_file = reinterpret_cast<char *>(one_file + MLEL_CHAIN_MAX_INPUTS); // [n_cols][cols] halfs
    const int tid = threadIdx.x, rr = tid >> tpr_log, part = tid & (TPR - 1);
    const int64_t row = (int64_t)blockIdx.x * R + rr;
    const bool live = row < g.rows;
    const int segs = g.cols >> 3;
    char *mine = lds + rr * pitch;  // this thread's row inside row register 0

    // ---- single elements and per-column inputs into their files (read by every thread later: one barrier below),
    // the full inputs into their row registers, four loads in flight per thread
    for (int k = 0; k < g.n_inputs; k++) {
        if (g.in_cls[k] == RC_ONE) {
            if (tid == k) one_file[k] = *reinterpret_cast<const __half *>(g.in[k]);
        } else if (g.in_cls[k] == RC_COL) {
            for (int sg = tid; sg < segs; sg += kBlock)
                *reinterpret_cast<uint4 *>(col_file + g.in_col[k] * g.cols * 2 + sg * 16) =
                    *reinterpret_cast<const uint4 *>(g.in[k] + sg * 16);
        }
    }
    for (int k = 0; k < g.n_inputs; k++) {
        if (g.in_reg[k] < 0) continue;  // uniform
        const char *src = g.in[k] + row * g.cols * 2;
        char *dst = mine + g.in_reg[k] * reg_bytes;
        for (int sg0 = part; sg0 < segs; sg0 += 4 * TPR) {
            uint4 v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int sg = sg0 + i * TPR;
                v[i] = make_uint4(0, 0, 0, 0);
                if (live && sg < segs) v[i] = *reinterpret_cast<const uint4 *>(src + sg * 16);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int sg = sg0 + i * TPR;
                if (sg < segs) *reinterpret_cast<uint4 *>(dst + sg * 16) = v[i];
            }
        }
    }

    const auto unpack = [](const uint4 &raw, float (&x)[8]) {
        const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float2 f = __half22float2(h[i]);
            x[2 * i] = f.x;
            x[2 * i + 1] = f.y;
        }
    };
    // one element of an operand that does not vary along the row
    const auto row_value = [&](const RowOperand o) {
        switch (o.cls) {
        case RC_ROW: return __half2float(row_file[o.idx * 64 + rr]);
        case RC_ROW_IN: return live ? __half2float(*reinterpret_cast<const __half *>(g.in[o.idx] + row * 2)) : 0.f;
        default: return __half2float(one_file[o.idx]);
        }
    };
    // An operand of a full-shaped step is either a row of halfs in shared memory (a row register or a per-column
    // input) or one value for the whole row.  `OP` is a template argument so that the loop over the pieces holds no
    // dispatch on the operator.
    struct Source {
        const char *base;  // null: `value` for every element
        float value;
    };
    const auto source = [&](const RowOperand o) {
        if (o.cls == RC_FULL) return Source{mine + o.idx * reg_bytes, 0.f};
        if (o.cls == RC_COL) return Source{col_file + o.idx * g.cols * 2, 0.f};
        return Source{nullptr, row_value(o)};
    };
    const auto full_step = [&](auto op_tag, const RowStep &st) {
        constexpr int OP = decltype(op_tag)::value;
        constexpr bool two = OP == F_ADD || OP == F_SUB || OP == F_MUL;
        const Source sa = source(st.a), sb = two ? source(st.b) : Source{nullptr, 0.f};
        char *dst = st.dst >= 0 ? mine + st.dst * reg_bytes : nullptr;
        char *out_row = g.out + row * g.cols * 2;
        // an operand that is one value for the whole row, as four packed pairs
        const auto splat = [](float v) {
            const __half h = f2h(v);
            const __half2 h2 = __halves2half2(h, h);
            const uint32_t w = *reinterpret_cast<const uint32_t *>(&h2);
            return make_uint4(w, w, w, w);
        };
        const uint4 a_row = splat(sa.value), b_row = splat(sb.value);
        for (int sg = part; sg < segs; sg += TPR) {
            const uint4 pa = sa.base ? *reinterpret_cast<const uint4 *>(sa.base + sg * 16) : a_row;
            uint4 raw;
            __half2 *h = reinterpret_cast<__half2 *>(&raw);
            if (two) {
                // packed fp16 arithmetic: one rounding of the exact result, which is what the fp32 operation followed
                // by a conversion yields for sums, differences and products of halfs
                const uint4 pb = sb.base ? *reinterpret_cast<const uint4 *>(sb.base + sg * 16) : b_row;
                const __half2 *ah = reinterpret_cast<const __half2 *>(&pa), *bh = reinterpret_cast<const __half2 *>(&pb);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    h[i] = OP == F_ADD ? __hadd2(ah[i], bh[i]) : OP == F_SUB ? __hsub2(ah[i], bh[i]) : __hmul2(ah[i], bh[i]);
            } else {
                float a[8];
                unpack(pa, a);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    h[i] = __halves2half2(f2h(row_apply(OP, a[2 * i], 0.f)), f2h(row_apply(OP, a[2 * i + 1], 0.f)));
            }
            if (dst)
                *reinterpret_cast<uint4 *>(dst + sg * 16) = raw;
            else if (live)
                *reinterpret_cast<uint4 *>(out_row + sg * 16) = raw;
        }
    };

    // the program as well: indexed at run time, a read from the kernel arguments would be a trip to memory per step
    __shared__ uint2 program[MLEL_CHAIN_MAX_STEPS];
    static_assert(sizeof(RowStep) == sizeof(uint2), "a step is one 8-byte word");
    if (tid < g.n_steps) program[tid] = reinterpret_cast<const uint2 *>(g.step)[tid];
    __syncthreads();  // the files are filled
    for (int s = 0; s < g.n_steps; s++) {
        uint2 w = program[s];
        w.x = __builtin_amdgcn_readfirstlane(w.x);
        w.y = __builtin_amdgcn_readfirstlane(w.y);
        RowStep st;  // uniform
        __builtin_memcpy(&st, &w, sizeof st);
        if (st.op == F_RED_SUM || st.op == F_RED_MAX) {
            __syncthreads();  // the row register is complete
            const char *src = mine + st.a.idx * reg_bytes;
            float result = 0.f;
            if (st.op == F_RED_SUM) {
                if (part == 0) {
                    __half acc = f2h(0.f);
                    const auto add8 = [&](const uint4 &raw) {
                        const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
                        for (int t = 0; t < 4; t++) {
                            acc = __hadd(acc, __low2half(h[t]));
                            acc = __hadd(acc, __high2half(h[t]));
                        }
                    };
                    // the adds form one dependent chain: four pieces are requested while the four before them are
                    // folded, alternating between two sets of registers
                    const auto load4 = [&](uint4 (&v)[4], int first) {
#pragma unroll
                        for (int t = 0; t < 4; t++) v[t] = *reinterpret_cast<const uint4 *>(src + (first + t) * 16);
                    };
                    int sg = 0;
                    uint4 even[4], odd[4];
                    if (segs >= 4) load4(even, 0);
                    for (; sg + 8 <= segs; sg += 8) {
                        load4(odd, sg + 4);
#pragma unroll
                        for (int t = 0; t < 4; t++) add8(even[t]);
                        if (sg + 12 <= segs) load4(even, sg + 8);
#pragma unroll
                        for (int t = 0; t < 4; t++) add8(odd[t]);
                    }
                    if (sg + 4 <= segs) {  // `even` holds the pieces sg .. sg + 3
#pragma unroll
                        for (int t = 0; t < 4; t++) add8(even[t]);
                        sg += 4;
                    }
                    for (; sg < segs; sg++) add8(*reinterpret_cast<const uint4 *>(src + sg * 16));
                    result = __half2float(acc);
                }
            } else {
                typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
                h2_t m2 = {(_Float16)-65504.f, (_Float16)-65504.f};
                uint32_t special = 0;
                for (int sg = part; sg < segs; sg += TPR) {
                    const uint4 raw = *reinterpret_cast<const uint4 *>(src + sg * 16);
                    special |= (((raw.x & 0x7fff7fffu) + 0x03ff03ffu) | ((raw.y & 0x7fff7fffu) + 0x03ff03ffu) |
                                ((raw.z & 0x7fff7fffu) + 0x03ff03ffu) | ((raw.w & 0x7fff7fffu) + 0x03ff03ffu)) & 0x80008000u;
                    const h2_t *p = reinterpret_cast<const h2_t *>(&raw);
                    m2 = __builtin_elementwise_max(m2, __builtin_elementwise_max(__builtin_elementwise_max(p[0], p[1]),
                                                                                   __builtin_elementwise_max(p[2], p[3])));
                }
                float mx = (float)(m2.x > m2.y ? m2.x : m2.y);
                for (int d = 1; d < TPR; d <<= 1) {  // the row's threads are neighbouring lanes of one wavefront
                    mx = fmaxf(mx, __shfl_xor(mx, d));
                    special |= (uint32_t)__shfl_xor((int)special, d);
                }
                result = special != 0 ? __builtin_nanf("") : mx;
            }
            if (part == 0) {
                if (st.dst >= 0)
                    row_file[st.dst * 64 + rr] = f2h(result);
                else if (live)
                    *reinterpret_cast<__half *>(g.out + row * 2) = f2h(result);
            }
            __syncthreads();
            continue;
        }
        const bool two = st.op == F_ADD || st.op == F_SUB || st.op == F_MUL;
        if (st.cls == RC_ROW) {  // one value per row: the row's first thread
            if (part == 0) {
                const float a = row_value(st.a), b = two ? row_value(st.b) : 0.f;
                const __half r = f2h(row_apply(st.op, a, b));
                if (st.dst >= 0)
                    row_file[st.dst * 64 + rr] = r;
                else if (live)
                    *reinterpret_cast<__half *>(g.out + row * 2) = r;
            }
            __syncthreads();
            continue;
        }
        switch (st.op) {  // uniform
        case F_ADD: full_step(std::integral_constant<int, F_ADD>{}, st); break;
        case F_SUB: full_step(std::integral_constant<int, F_SUB>{}, st); break;
        case F_MUL: full_step(std::integral_constant<int, F_MUL>{}, st); break;
        case F_EXP: full_step(std::integral_constant<int, F_EXP>{}, st); break;
        case F_RECIPROCAL: full_step(std::integral_constant<int, F_RECIPROCAL>{}, st); break;
        case F_RSQRT: full_step(std::integral_constant<int, F_RSQRT>{}, st); break;
        case F_TANH: full_step(std::integral_constant<int, F_TANH>{}, st); break;
        default: break;
        }
    }
}


// ---------------------------------------------------------------------------------------------------------------
// Chains with reductions that are known at compile time (LayerNorm and the scaled softmax as TOSA graphs spell them,
// in the order in which the region builder emits them).  Same shapes of values and same arithmetic as
// row_chain_f16_kernel, but the program is a template argument: 2^k threads of one wavefront share a row and keep
// their pieces of every full value in vector registers (at most four 16-byte pieces per thread and value), per-row
// values live in a register of every thread of the row, REDUCE_MAX is a few shuffles, and only REDUCE_SUM goes
// through shared memory: the row's threads lay the operand down, the row's first thread folds it left to right in
// fp16 and hands the sum back with a shuffle.  A row never leaves its wavefront, so there is no block-wide barrier.
// ---------------------------------------------------------------------------------------------------------------
enum { SC_FULL, SC_ROW, SC_COL, SC_ONE };
struct LayerNormProgram {
    static constexpr int n_inputs = 5, n_steps = 11, n_full = 2, n_row = 2;
    // values: 0 x, 1 1/N, 2 eps, 3 gamma, 4 beta, then one per step
    static constexpr int cls[16] = {SC_FULL, SC_ONE, SC_ONE, SC_COL, SC_COL, SC_ROW, SC_ROW, SC_FULL,
                                    SC_FULL, SC_ROW, SC_ROW, SC_ROW, SC_ROW, SC_FULL, SC_FULL, SC_FULL};
    // register slot of full and per-row values (a slot is reused once its value is dead); the input index otherwise
    static constexpr int slot[16] = {0, 1, 2, 3, 4, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 1};
    static constexpr StaticStep steps[n_steps] = {{F_RED_SUM, 0, 0}, {F_MUL, 5, 1},  {F_SUB, 0, 6},    {F_MUL, 7, 7},
                                                  {F_RED_SUM, 8, 0}, {F_MUL, 9, 1},  {F_ADD, 10, 2},   {F_RSQRT, 11, 0},
                                                  {F_MUL, 7, 12},    {F_MUL, 13, 3}, {F_ADD, 14, 4}};
};
struct ScaledSoftmaxProgram {
    static constexpr int n_inputs = 2, n_steps = 7, n_full = 1, n_row = 1;
    // values: 0 x, 1 scale, then one per step
    static constexpr int cls[9] = {SC_FULL, SC_ONE, SC_FULL, SC_ROW, SC_FULL, SC_FULL, SC_ROW, SC_ROW, SC_FULL};
    static constexpr int slot[9] = {0, 1, 0, 0, 0, 0, 0, 0, 0};
    static constexpr StaticStep steps[n_steps] = {{F_MUL, 0, 1},     {F_RED_MAX, 2, 0},    {F_SUB, 2, 3}, {F_EXP, 4, 0},
                                                  {F_RED_SUM, 5, 0}, {F_RECIPROCAL, 6, 0}, {F_MUL, 5, 7}};
};
struct SoftmaxProgram {  // the six operators without a scale in front (mlel_hip_softmax_rows)
    static constexpr int n_inputs = 1, n_steps = 6, n_full = 1, n_row = 1;
    static constexpr int cls[7] = {SC_FULL, SC_ROW, SC_FULL, SC_FULL, SC_ROW, SC_ROW, SC_FULL};
    static constexpr int slot[7] = {0, 0, 0, 0, 0, 0, 0};
    static constexpr StaticStep steps[n_steps] = {{F_RED_MAX, 0, 0}, {F_SUB, 0, 1},        {F_EXP, 2, 0},
                                                  {F_RED_SUM, 3, 0}, {F_RECIPROCAL, 4, 0}, {F_MUL, 3, 5}};
};
struct RowStaticArgs {
    char *out;
    int64_t rows;
    int32_t cols, tpr_log;
    const char *in[MLEL_CHAIN_MAX_INPUTS];
};
constexpr int kRowStaticPieces = 4;      // pieces per thread and value when a row is spread as widely as it goes
constexpr int kRowStaticMaxPieces = 12;  // the most a thread holds when rows are packed more densely into wavefronts

template <class P, int NP>
struct RowStaticState {
    uint4 f[P::n_full][NP];
    uint32_t r[P::n_row];              // a per-row value, the half in both halves of the word
    uint32_t one[P::n_inputs];         // single-element inputs, likewise
    const RowStaticArgs *g;
    char *stage;                       // this row's staging area in shared memory
    int part, tpr, segs;
    int64_t row;
    bool live;
};

__device__ __forceinline__ uint4 splat_word(uint32_t w) { return make_uint4(w, w, w, w); }

template <class P, int NP, int V>
__device__ __forceinline__ uint4 row_static_piece(const RowStaticState<P, NP> &c, int u) {
    if constexpr (P::cls[V] == SC_FULL) {
        return c.f[P::slot[V]][u];
    } else if constexpr (P::cls[V] == SC_ROW) {
        return splat_word(c.r[P::slot[V]]);
    } else if constexpr (P::cls[V] == SC_ONE) {
        return splat_word(c.one[V]);
    } else {
        const int sg = c.part + u * c.tpr;
        return sg < c.segs ? *reinterpret_cast<const uint4 *>(c.g->in[V] + sg * 16) : make_uint4(0, 0, 0, 0);
    }
}

template <class P, int NP, int S>
__device__ __forceinline__ void row_static_run(RowStaticState<P, NP> &c) {
    if constexpr (S < P::n_steps) {
        constexpr int OP = P::steps[S].op, A = P::steps[S].a, B = P::steps[S].b, V = P::n_inputs + S;
        constexpr bool last = S + 1 == P::n_steps;
        if constexpr (OP == F_RED_SUM) {
            // the operand into the row's staging area, then the row's first thread folds it; the row's threads are
            // lanes of one wavefront, whose shared-memory operations complete in program order
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
            for (int u = 0; u < NP; u++) {
                const int sg = c.part + u * c.tpr;
                if (sg < c.segs) *reinterpret_cast<uint4 *>(c.stage + sg * 16) = c.f[P::slot[A]][u];
            }
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __half acc = f2h(0.f);
            // lgkmcnt(0): no scalar load of a kernel argument is left in flight.  With one pending the compiler cannot
            // count shared-memory reads (scalar loads return out of order) and waits for all of them at every use.
            __builtin_amdgcn_s_waitcnt(0xc07f);
            if (c.part == 0) {
                const auto add8 = [&](const uint4 &raw) {
                    const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        acc = __hadd(acc, __low2half(h[t]));
                        acc = __hadd(acc, __high2half(h[t]));
                    }
                };
                const auto load4 = [&](uint4 (&v)[4], int first) {
#pragma unroll
                    for (int t = 0; t < 4; t++) v[t] = *reinterpret_cast<const uint4 *>(c.stage + (first + t) * 16);
                };
                // batches of four pieces, two register sets: while one is added the other is on its way.  Every load is
                // issued unconditionally (the last one of an even count reads the last batch again and is not used),
                // so the sets keep their registers and the waits count exactly the loads of the other set.
                const int n4 = c.segs >> 2;
                int done = 0;
                if (n4 >= 2) {
                    uint4 even[4], odd[4];
                    int i = 0;
                    load4(even, 0);
                    for (; i + 2 <= n4; i += 2) {
                        load4(odd, (i + 1) * 4);
                        __builtin_amdgcn_sched_barrier(0);  // the loads first: they travel while the other set is added
#pragma unroll
                        for (int t = 0; t < 4; t++) add8(even[t]);
                        __builtin_amdgcn_sched_barrier(0);
                        load4(even, min(i + 2, n4 - 1) * 4);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int t = 0; t < 4; t++) add8(odd[t]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if (i < n4) {
#pragma unroll
                        for (int t = 0; t < 4; t++) add8(even[t]);
                    }
                    done = n4 * 4;
                }
                for (int sg = done; sg < c.segs; sg++) add8(*reinterpret_cast<const uint4 *>(c.stage + sg * 16));
            }
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const uint32_t bits = (uint32_t)__half_as_ushort(acc);
            const int first_lane = (int)(threadIdx.x & 63u) & ~(c.tpr - 1);
            const uint32_t sum = (uint32_t)__shfl((int)bits, first_lane);
            c.r[P::slot[V]] = sum | (sum << 16);
        } else if constexpr (OP == F_RED_MAX) {
            typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
            h2_t m2 = {(_Float16)-65504.f, (_Float16)-65504.f};
            uint32_t special = 0;
#pragma unroll
            for (int u = 0; u < NP; u++) {
                const int sg = c.part + u * c.tpr;
                if (sg >= c.segs) continue;
                const uint4 raw = c.f[P::slot[A]][u];
                special |= (((raw.x & 0x7fff7fffu) + 0x03ff03ffu) | ((raw.y & 0x7fff7fffu) + 0x03ff03ffu) |
                            ((raw.z & 0x7fff7fffu) + 0x03ff03ffu) | ((raw.w & 0x7fff7fffu) + 0x03ff03ffu)) & 0x80008000u;
                const h2_t *p = reinterpret_cast<const h2_t *>(&raw);
                m2 = __builtin_elementwise_max(m2, __builtin_elementwise_max(__builtin_elementwise_max(p[0], p[1]),
                                                                               __builtin_elementwise_max(p[2], p[3])));
            }
            float mx = (float)(m2.x > m2.y ? m2.x : m2.y);
            for (int d = 1; d < c.tpr; d <<= 1) {
                mx = fmaxf(mx, __shfl_xor(mx, d));
                special |= (uint32_t)__shfl_xor((int)special, d);
            }
            const uint32_t bits = (uint32_t)__half_as_ushort(f2h(special != 0 ? __builtin_nanf("") : mx));
            c.r[P::slot[V]] = bits | (bits << 16);
        } else if constexpr (P::cls[V] == SC_ROW) {
            uint4 r = static_apply<OP>(row_static_piece<P, NP, A>(c, 0), row_static_piece<P, NP, B>(c, 0));
            asm volatile("" : "+v"(r.x));  // rounded here, as the stand-alone operator rounds: no contraction across steps
            c.r[P::slot[V]] = r.x;
        } else {
#pragma unroll
            for (int u = 0; u < NP; u++) {
                uint4 r = static_apply<OP>(row_static_piece<P, NP, A>(c, u), row_static_piece<P, NP, B>(c, u));
                asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
                if constexpr (last) {
                    const int sg = c.part + u * c.tpr;
                    if (c.live && sg < c.segs)
                        store16_result(c.g->out + (c.row * c.g->cols + sg * 8) * 2, r);
                } else {
                    c.f[P::slot[V]][u] = r;
                }
            }
        }
        row_static_run<P, NP, S + 1>(c);
    }
}

// the full inputs into registers (four pieces requested at once), the single elements into both halves of a word
template <class P, int NP, int K>
__device__ __forceinline__ void row_static_load(RowStaticState<P, NP> &c) {
    if constexpr (K < P::n_inputs) {
        if constexpr (P::cls[K] == SC_FULL) {
#pragma unroll
            for (int u = 0; u < NP; u++) {
                const int sg = c.part + u * c.tpr;
                c.f[P::slot[K]][u] = (c.live && sg < c.segs)
                                         ? *reinterpret_cast<const uint4 *>(c.g->in[K] + (c.row * c.g->cols + sg * 8) * 2)
                                         : make_uint4(0, 0, 0, 0);
            }
        } else if constexpr (P::cls[K] == SC_ONE) {
            const uint32_t bits = *reinterpret_cast<const uint16_t *>(c.g->in[K]);
            c.one[K] = bits | (bits << 16);
        }
        row_static_load<P, NP, K + 1>(c);
    }
}

template <class P, int NP>
__global__ void __launch_bounds__(kBlock) row_static_f16_kernel(const RowStaticArgs g) {
    extern __shared__ __align__(16) char lds[];
    RowStaticState<P, NP> c;
    c.g = &g;
    c.tpr = 1 << g.tpr_log;
    c.part = (int)threadIdx.x & (c.tpr - 1);
    const int rr = (int)threadIdx.x >> g.tpr_log;
    c.row = (int64_t)blockIdx.x * (kBlock >> g.tpr_log) + rr;
    c.live = c.row < g.rows;
    c.segs = g.cols >> 3;
    c.stage = lds + rr * (g.cols * 2 + 16);
    row_static_load<P, NP, 0>(c);
    row_static_run<P, NP, 0>(c);
}

// the chain is P's program over inputs of P's shapes (`classes`: the RowClass of every input, `ops`: FOp / F_RED_*)
template <class P>
bool matches_row_static(const mlel_chain *c, const int8_t *classes, const int *ops) {
    if (c->n_inputs != P::n_inputs || c->n_steps != P::n_steps) return false;
    for (int k = 0; k < P::n_inputs; k++) {
        const int want = P::cls[k] == SC_FULL ? RC_FULL : P::cls[k] == SC_COL ? RC_COL : RC_ONE;
        if (classes[k] != want) return false;
    }
    for (int i = 0; i < P::n_steps; i++) {
        const bool two = ops[i] == F_ADD || ops[i] == F_SUB || ops[i] == F_MUL;
        if (ops[i] != P::steps[i].op || c->steps[i].a != P::steps[i].a || (two && c->steps[i].b != P::steps[i].b)) return false;
    }
    return true;
}

template <class P, int NP>
int launch_row_static_pieces(hipStream_t s, const RowStaticArgs &g, int64_t rows, int64_t cols) {
    const int64_t rows_per_block = kBlock >> g.tpr_log;
    const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "row chain: too many rows");
    const size_t smem = (size_t)rows_per_block * (size_t)(cols * 2 + 16);
    row_static_f16_kernel<P, NP><<<dim3((unsigned)blocks), dim3(kBlock), smem, s>>>(g);
    return check_launch("row chain (compiled program)");
}

template <class P>
int launch_row_static(hipStream_t s, const mlel_tensor *out, const mlel_chain *c, int64_t rows, int64_t cols) {
    RowStaticArgs g{};
    g.out = static_cast<char *>(out->ptr);
    g.rows = rows;
    g.cols = (int32_t)cols;
    const int64_t segs = cols / 8;
    int tpr_log = 0;
    while ((int64_t(kRowStaticPieces) << tpr_log) < segs) tpr_log++;  // as wide as a row goes: four pieces per thread
    // The left-to-right fold of a REDUCE_SUM is issued once per wavefront whatever the number of rows in it.  One
    // wavefront alone issues a vector instruction every 6.5 clocks (measured: dependent or not), a SIMD takes one
    // every 4: two wavefronts fold side by side on a SIMD at full speed each, a third slows all three.  Rows are
    // therefore packed more densely (fewer threads per row, more pieces per thread) until there are at most two
    // wavefronts per SIMD of the device (256 compute units of four) or a thread is full.
    const auto pieces = [&](int log) { return (segs + (int64_t(1) << log) - 1) >> log; };
    const auto wavefronts = [&](int log) { return (rows + (64 >> log) - 1) / (64 >> log); };
    while (tpr_log > 0 && wavefronts(tpr_log) > 2048 && pieces(tpr_log - 1) <= kRowStaticMaxPieces) tpr_log--;
    g.tpr_log = tpr_log;
    for (int k = 0; k < c->n_inputs; k++) g.in[k] = static_cast<const char *>(c->inputs[k]->ptr);
    const int64_t np = pieces(tpr_log);
    if (np <= 4) return launch_row_static_pieces<P, 4>(s, g, rows, cols);
    if (np <= 8) return launch_row_static_pieces<P, 8>(s, g, rows, cols);
    return launch_row_static_pieces<P, kRowStaticMaxPieces>(s, g, rows, cols);
}

}  // namespace

// MLEL_ERR_UNSUPPORTED when the chain does not fit the kernel (types, shapes, alignment, live values): the caller
// then runs the operators one by one.
int elementwise_chain_launch(hipStream_t s, const mlel_tensor *out, const mlel_chain *c) {
    const auto decline = [](const char *why) { return set_error(MLEL_ERR_UNSUPPORTED, "elementwise chain: %s", why); };
    if (c->n_inputs < 1 || c->n_inputs > MLEL_CHAIN_MAX_INPUTS || c->n_steps < 1 || c->n_steps > MLEL_CHAIN_MAX_STEPS)
        return set_error(MLEL_ERR_INVALID, "elementwise chain: %d inputs, %d steps", c->n_inputs, c->n_steps);
    if ((out->dtype != MLEL_F16 && out->dtype != MLEL_F32) || !is_packed(out)) return decline("output type or strides");
    const int last = out->rank - 1;
    int64_t cols = out->dims[last];
    const int64_t total = numel(out);
    // rows shorter than a vector: the tensors are walked as one long row, which needs every input to have the
    // output's shape or a single element
    const bool flat = cols % 8 != 0;
    if (flat) cols = total;
    if (cols % 8 != 0 || cols >= (int64_t(1) << 31) || ((uintptr_t)out->ptr % 16) != 0) return decline("row length or alignment");
    if (total == 0) return 0;
    ChainArgs g{};
    g.out = static_cast<char *>(out->ptr);
    g.out_size = dt_size(out->dtype);
    g.vecs = total / 8;
    g.cols = (int32_t)cols;
    g.cols8 = (int32_t)(cols / 8);
    g.n_inputs = c->n_inputs;
    g.n_steps = c->n_steps;
    const int n_values = c->n_inputs + c->n_steps;
    // last use of every value, then registers by linear scan
    std::vector<int> last_use(n_values, -1), reg(n_values, -1);
    for (int i = 0; i < c->n_steps; i++) {
        const mlel_chain_step &st = c->steps[i];
        const bool two = st.kind == MLEL_CHAIN_BINARY || st.kind == MLEL_CHAIN_MUL;
        if (st.a < 0 || st.a >= c->n_inputs + i || (two && (st.b < 0 || st.b >= c->n_inputs + i)))
            return set_error(MLEL_ERR_INVALID, "elementwise chain: step %d reads a value that does not exist yet", i);
        last_use[st.a] = i;
        if (two) last_use[st.b] = i;
    }
    last_use[n_values - 1] = c->n_steps;  // the result
    bool all_half = out->dtype == MLEL_F16;
    for (int k = 0; k < c->n_inputs; k++) all_half = all_half && c->inputs[k] != nullptr && c->inputs[k]->dtype == MLEL_F16;
    for (int i = 0; i < c->n_steps; i++) all_half = all_half && c->steps[i].dtype == MLEL_F16;
    if (all_half && total % 8 == 0) {  // a program compiled ahead of time?
        int ops[MLEL_CHAIN_MAX_STEPS];
        for (int i = 0; i < c->n_steps; i++) {
            const mlel_chain_step &st = c->steps[i];
            ops[i] = st.kind == MLEL_CHAIN_MUL ? F_MUL
                     : st.kind == MLEL_CHAIN_BINARY ? (st.selector == MLEL_BIN_ADD ? F_ADD : st.selector == MLEL_BIN_SUB ? F_SUB : -1)
                     : st.kind == MLEL_CHAIN_UNARY
                         ? (st.selector == MLEL_UN_EXP ? F_EXP : st.selector == MLEL_UN_RECIPROCAL ? F_RECIPROCAL
                            : st.selector == MLEL_UN_RSQRT ? F_RSQRT : st.selector == MLEL_UN_TANH ? F_TANH : -1)
                         : -1;
        }
        if (matches_static<GeluTanhProgram>(out, c, ops)) {
            StaticArgs sa{};
            sa.out = static_cast<char *>(out->ptr);
            sa.vecs = total / 8;
            for (int k = 0; k < c->n_inputs; k++) sa.in[k] = static_cast<const char *>(c->inputs[k]->ptr);
            const int64_t static_blocks = (sa.vecs + kBlock - 1) / kBlock;
            MLEL_REQUIRE(static_blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "elementwise chain: too many work items");
            ew_static_half_kernel<GeluTanhProgram><<<dim3((unsigned)static_blocks), dim3(kBlock), 0, s>>>(sa);
            return check_launch("elementwise chain (compiled program)");
        }
    }
    const int n_regs = all_half ? kChainRegs + 2 : kChainRegs;
    std::vector<int> free_regs;
    for (int r = n_regs - 1; r >= 0; r--) free_regs.push_back(r);
    const auto take = [&](int value) {
        if (free_regs.empty()) return false;
        reg[value] = free_regs.back();
        free_regs.pop_back();
        return true;
    };
    std::vector<bool> is_scalar(n_values, false);
    int scalars = 0;
    for (int k = 0; k < c->n_inputs; k++) {
        const mlel_tensor *t = c->inputs[k];
        if (t == nullptr || (t->dtype != MLEL_F16 && t->dtype != MLEL_F32)) return decline("input type");
        int vr = 0, vc = 0;
        if (!classify(out, t, &vr, &vc)) return decline("input shape, strides or alignment");
        if (flat) {
            const bool single = numel(t) == 1, same = numel(t) == total && vr == 1;
            if (!single && !same) return decline("input shape for short rows");
            vr = 0;
            vc = single ? 0 : 1;
            if (!single && ((uintptr_t)t->ptr % 16) != 0) return decline("input alignment");
        }
        if (!vr && !vc) {  // one element: a lane of the scalar file
            is_scalar[k] = true;
            reg[k] = scalars++;
        } else if (last_use[k] >= 0) {
            if (!take(k)) return decline("too many live values");
        } else {
            reg[k] = 0;  // never read: loaded into a register nothing else holds yet
        }
        g.in[k] = ChainInput{static_cast<const char *>(t->ptr), dt_size(t->dtype), vr, vc, reg[k]};
    }
    for (int i = 0; i < c->n_steps; i++) {
        const mlel_chain_step &st = c->steps[i];
        int op;
        if (st.kind == MLEL_CHAIN_BINARY && st.selector == MLEL_BIN_ADD) op = F_ADD;
        else if (st.kind == MLEL_CHAIN_BINARY && st.selector == MLEL_BIN_SUB) op = F_SUB;
        else if (st.kind == MLEL_CHAIN_MUL) op = F_MUL;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_EXP) op = F_EXP;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_RECIPROCAL) op = F_RECIPROCAL;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_RSQRT) op = F_RSQRT;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_TANH) op = F_TANH;
        else if (st.kind == MLEL_CHAIN_CAST) op = F_COPY;
        else return decline("operator");
        if (st.dtype != MLEL_F16 && st.dtype != MLEL_F32) return decline("step type");
        const bool two = op == F_ADD || op == F_SUB || op == F_MUL;
        const int value = c->n_inputs + i, prev = value - 1;
        const bool a_fw = i > 0 && st.a == prev, b_fw = two && i > 0 && st.b == prev;
        // operands die here: their registers may take the result
        if (!is_scalar[st.a] && last_use[st.a] == i && reg[st.a] >= 0) free_regs.push_back(reg[st.a]);
        if (two && st.b != st.a && !is_scalar[st.b] && last_use[st.b] == i && reg[st.b] >= 0) free_regs.push_back(reg[st.b]);
        // a result that only the next step reads stays in vector registers and needs no slot
        bool needs_slot = i + 1 < c->n_steps && last_use[value] > i + 1;
        if (i + 1 < c->n_steps && last_use[value] == i + 1) {
            const mlel_chain_step &nx = c->steps[i + 1];
            const bool nx_two = nx.kind == MLEL_CHAIN_BINARY || nx.kind == MLEL_CHAIN_MUL;
            needs_slot = !(nx.a == value || (nx_two && nx.b == value));
        }
        if (needs_slot && !take(value)) return decline("too many live values");
        g.step[i] = ChainStep{(int8_t)op, (int8_t)(st.dtype == MLEL_F16), (int8_t)(a_fw ? 0 : reg[st.a]),
                              (int8_t)(two && !b_fw ? reg[st.b] : 0), (int8_t)is_scalar[st.a],
                              (int8_t)(two && is_scalar[st.b]), (int8_t)a_fw, (int8_t)b_fw,
                              (int8_t)(needs_slot ? reg[value] : -1)};
    }
    if (c->steps[c->n_steps - 1].dtype != out->dtype) return decline("the last step must have the output's type");
    const int64_t blocks = (g.vecs + kBlock - 1) / kBlock;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "elementwise chain: too many work items");
    if (all_half)
        ew_chain_kernel<true><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(g);
    else
        ew_chain_kernel<false><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(g);
    return check_launch("elementwise chain");
}

// The chain with reductions.  MLEL_ERR_UNSUPPORTED when it does not fit the kernel (types other than fp16, shapes,
// alignment, too many values alive at once, rows too long for shared memory).
bool chain_is_gelu_tanh(const mlel_chain *c) {
    typedef GeluTanhProgram P;
    if (c->n_inputs != P::n_inputs || c->n_steps != P::n_steps) return false;
    for (int k = 1; k < P::n_inputs; k++)
        if (c->inputs[k] == nullptr || c->inputs[k]->dtype != MLEL_F16 || numel(c->inputs[k]) != 1) return false;
    for (int i = 0; i < P::n_steps; i++) {
        const mlel_chain_step &st = c->steps[i];
        const int op = st.kind == MLEL_CHAIN_MUL ? F_MUL
                       : st.kind == MLEL_CHAIN_BINARY && st.selector == MLEL_BIN_ADD ? F_ADD
                       : st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_TANH ? F_TANH : -1;
        const bool two = op == F_ADD || op == F_MUL;
        if (op != P::steps[i].op || st.a != P::steps[i].a || (two && st.b != P::steps[i].b) || st.dtype != MLEL_F16) return false;
    }
    return true;
}

int row_chain_launch(hipStream_t s, const mlel_tensor *out, const mlel_chain *c) {
    const auto decline = [](const char *why) { return set_error(MLEL_ERR_UNSUPPORTED, "row chain: %s", why); };
    if (c->n_inputs < 1 || c->n_inputs > MLEL_CHAIN_MAX_INPUTS || c->n_steps < 1 || c->n_steps > MLEL_CHAIN_MAX_STEPS)
        return set_error(MLEL_ERR_INVALID, "row chain: %d inputs, %d steps", c->n_inputs, c->n_steps);
    if (out->dtype != MLEL_F16 || !is_packed(out) || out->rank < 1) return decline("output type or strides");
    // the full shape: that of the input with the most elements
    const mlel_tensor *full = nullptr;
    for (int k = 0; k < c->n_inputs; k++) {
        const mlel_tensor *t = c->inputs[k];
        if (t == nullptr || t->dtype != MLEL_F16 || !is_packed(t) || t->rank != out->rank) return decline("input type, rank or strides");
        if (full == nullptr || numel(t) > numel(full)) full = t;
    }
    const int last = full->rank - 1;
    const int64_t cols = full->dims[last], total = numel(full);
    if (total == 0) return 0;
    if (cols < 8 || cols % 8 != 0) return decline("row length");
    const int64_t rows = total / cols;
    const int n_values = c->n_inputs + c->n_steps;
    std::vector<int8_t> cls(n_values, RC_ONE);
    const auto class_of = [&](const mlel_tensor *t, int8_t *out_cls) {
        bool same = true, ones = true;
        for (int i = 0; i < last; i++) {
            same = same && t->dims[i] == full->dims[i];
            ones = ones && t->dims[i] == 1;
        }
        const bool wide = t->dims[last] == cols;
        if (!wide && t->dims[last] != 1) return false;
        if (same && wide) *out_cls = RC_FULL;
        else if (ones && wide) *out_cls = RC_COL;
        else if (ones) *out_cls = RC_ONE;
        else if (same) *out_cls = RC_ROW_IN;
        else return false;
        return true;
    };
    RowArgs g{};
    for (int k = 0; k < c->n_inputs; k++) {
        const mlel_tensor *t = c->inputs[k];
        if (!class_of(t, &cls[k])) return decline("input shape");
        const bool wide = cls[k] == RC_FULL || cls[k] == RC_COL;
        if (((uintptr_t)t->ptr % (wide ? 16 : 2)) != 0) return decline("input alignment");
        g.in[k] = static_cast<const char *>(t->ptr);
        g.in_reg[k] = -1;
        g.in_cls[k] = cls[k];
        g.in_col[k] = cls[k] == RC_COL ? (int8_t)g.n_cols++ : (int8_t)-1;
    }
    // shapes of the results, last uses
    std::vector<int> last_use(n_values, -1), op_of(c->n_steps, 0);
    for (int i = 0; i < c->n_steps; i++) {
        const mlel_chain_step &st = c->steps[i];
        if (st.dtype != MLEL_F16) return decline("step type");
        int op;
        if (st.kind == MLEL_CHAIN_BINARY && st.selector == MLEL_BIN_ADD) op = F_ADD;
        else if (st.kind == MLEL_CHAIN_BINARY && st.selector == MLEL_BIN_SUB) op = F_SUB;
        else if (st.kind == MLEL_CHAIN_MUL) op = F_MUL;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_EXP) op = F_EXP;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_RECIPROCAL) op = F_RECIPROCAL;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_RSQRT) op = F_RSQRT;
        else if (st.kind == MLEL_CHAIN_UNARY && st.selector == MLEL_UN_TANH) op = F_TANH;
        else if (st.kind == MLEL_CHAIN_REDUCE && st.selector == MLEL_RED_SUM) op = F_RED_SUM;
        else if (st.kind == MLEL_CHAIN_REDUCE && st.selector == MLEL_RED_MAX) op = F_RED_MAX;
        else return decline("operator");
        op_of[i] = op;
        const bool two = op == F_ADD || op == F_SUB || op == F_MUL;
        const int value = c->n_inputs + i;
        if (st.a < 0 || st.a >= value || (two && (st.b < 0 || st.b >= value)))
            return set_error(MLEL_ERR_INVALID, "row chain: step %d reads a value that does not exist yet", i);
        last_use[st.a] = i;
        if (two) last_use[st.b] = i;
        const auto along_rows = [](int8_t k) { return k == RC_FULL || k == RC_ROW || k == RC_ROW_IN; };
        const auto along_cols = [](int8_t k) { return k == RC_FULL || k == RC_COL; };
        if (op == F_RED_SUM || op == F_RED_MAX) {
            if (cls[st.a] != RC_FULL) return decline("reduction of a value that is not a full row");
            cls[value] = RC_ROW;
        } else {
            const bool r = along_rows(cls[st.a]) || (two && along_rows(cls[st.b]));
            const bool w = along_cols(cls[st.a]) || (two && along_cols(cls[st.b]));
            if (!r) return decline("a step whose result does not vary from row to row");
            cls[value] = w ? RC_FULL : RC_ROW;
        }
    }
    const int result = n_values - 1;
    last_use[result] = c->n_steps;
    {   // the output has the result's shape
        int8_t out_cls = RC_ONE;
        if (!class_of(out, &out_cls)) return decline("output shape");
        const bool want_full = cls[result] == RC_FULL;
        const bool ok = want_full ? (out_cls == RC_FULL)
                                  : (out_cls == RC_ROW_IN || (rows == 1 && out_cls == RC_ONE));
        if (!ok || ((uintptr_t)out->ptr % (want_full ? 16 : 2)) != 0) return decline("output shape or alignment");
    }
    // a program compiled ahead of time?  (rows of at most 4 x 64 pieces: a row stays inside one wavefront)
    if (cols <= 8 * kRowStaticPieces * 64 && cls[result] == RC_FULL) {
        if (matches_row_static<LayerNormProgram>(c, cls.data(), op_of.data()))
            return launch_row_static<LayerNormProgram>(s, out, c, rows, cols);
        if (matches_row_static<ScaledSoftmaxProgram>(c, cls.data(), op_of.data()))
            return launch_row_static<ScaledSoftmaxProgram>(s, out, c, rows, cols);
        if (matches_row_static<SoftmaxProgram>(c, cls.data(), op_of.data()))
            return launch_row_static<SoftmaxProgram>(s, out, c, rows, cols);
    }
    // row registers for full values, slots of the per-row file for the others, both by linear scan
    std::vector<int> slot(n_values, -1), free_regs, free_slots;
    for (int r = kRowRegs - 1; r >= 0; r--) free_regs.push_back(r);
    for (int r = kRowScalars - 1; r >= 0; r--) free_slots.push_back(r);
    int regs_used = 0;
    const auto take = [&](int value) {
        std::vector<int> &pool = cls[value] == RC_FULL ? free_regs : free_slots;
        if (pool.empty()) return false;
        slot[value] = pool.back();
        pool.pop_back();
        if (cls[value] == RC_FULL) regs_used = std::max(regs_used, slot[value] + 1);
        return true;
    };
    const auto release = [&](int value) {
        if (slot[value] < 0) return;
        (cls[value] == RC_FULL ? free_regs : free_slots).push_back(slot[value]);
        slot[value] = -1;
    };
    for (int k = 0; k < c->n_inputs; k++) {
        if (cls[k] != RC_FULL || last_use[k] < 0) continue;
        if (!take(k)) return decline("too many full values alive at once");
        g.in_reg[k] = (int8_t)slot[k];
    }
    for (int i = 0; i < c->n_steps; i++) {
        const mlel_chain_step &st = c->steps[i];
        const int op = op_of[i], value = c->n_inputs + i;
        const bool two = op == F_ADD || op == F_SUB || op == F_MUL;
        const auto operand = [&](int v) {
            const bool held = cls[v] == RC_FULL || cls[v] == RC_ROW;
            return RowOperand{cls[v], (int8_t)(held ? slot[v] : cls[v] == RC_COL ? g.in_col[v] : v)};
        };
        RowStep rs{};
        rs.op = (int8_t)op;
        rs.cls = cls[value];
        rs.a = operand(st.a);
        rs.b = two ? operand(st.b) : RowOperand{RC_ONE, 0};
        // operands that die here give their place to the result (a piece is read and written by the same thread)
        if (last_use[st.a] == i) release(st.a);
        if (two && st.b != st.a && last_use[st.b] == i) release(st.b);
        rs.dst = -1;
        if (value != result) {
            if (last_use[value] < 0) return decline("a step whose result is never read");
            if (!take(value)) return decline(cls[value] == RC_FULL ? "too many full values alive at once" : "too many per-row values alive at once");
            rs.dst = (int8_t)slot[value];
        }
        g.step[i] = rs;
    }
    if (regs_used == 0) return decline("no full value");
    const int64_t pitch = cols * 2 + 16;
    int log2_r = 6;
    const auto lds_bytes = [&](int lr) {
        return (int64_t)regs_used * (int64_t(1) << lr) * pitch + kRowScalars * 64 * 2 + MLEL_CHAIN_MAX_INPUTS * 2 +
               (int64_t)g.n_cols * cols * 2;
    };
    while (log2_r > 2 && lds_bytes(log2_r) > kRowLdsBudget) log2_r--;
    if (lds_bytes(log2_r) > kRowLdsBudget) return decline("rows too long for shared memory");
    // few rows: smaller blocks, so that the sequential folds spread over the compute units
    while (log2_r > 2 && (rows + (int64_t(1) << log2_r) - 1) / (int64_t(1) << log2_r) < 512) log2_r--;
    const int64_t blocks = (rows + (int64_t(1) << log2_r) - 1) >> log2_r;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "row chain: too many rows");
    g.out = static_cast<char *>(out->ptr);
    g.rows = rows;
    g.cols = (int32_t)cols;
    g.log2_r = log2_r;
    g.n_inputs = c->n_inputs;
    g.n_steps = c->n_steps;
    g.n_regs = regs_used;
    static const bool raised = hipFuncSetAttribute(reinterpret_cast<const void *>(row_chain_f16_kernel),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, kRowLdsBudget) == hipSuccess;
    (void)raised;
    row_chain_f16_kernel<<<dim3((unsigned)blocks), dim3(kBlock), (size_t)lds_bytes(log2_r), s>>>(g);
    return check_launch("row chain");
}

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
    g.slab_cols = (int32_t)(cols < kSlabCols ? cols : kSlabCols);
    const size_t smem = (size_t)2 * 64 * (g.slab_cols * 2 + 16);
    auto kernel = op == MLEL_RED_SUM ? reduce_rows_f16_kernel<true> : reduce_rows_f16_kernel<false>;
    if (smem > 48 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)smem);
    kernel<<<dim3((unsigned)blocks), dim3(kBlock), smem, s>>>(g);
    MLEL_TRY(check_launch("reduce rows fp16"));
    return 1;
}

}  // namespace mlel
