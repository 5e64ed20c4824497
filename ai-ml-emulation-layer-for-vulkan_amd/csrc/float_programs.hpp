// Device functions shared by the floating-point kernels: the transcendental operators, and operator chains that are
// known at compile time (used by the elementwise kernels of ops_float.hip and by the epilogue of gemm_f16.hip).
#pragma once

#include <hip/hip_fp16.h>

#include "common.hpp"

namespace mlel {

enum FOp { F_ADD, F_SUB, F_MUL, F_EXP, F_RECIPROCAL, F_RSQRT, F_TANH, F_COPY };

// Transcendentals.  Results that are stored as fp32 use the accurate library functions; results that are rounded to
// fp16 use the hardware approximations (v_exp_f32, v_rcp_f32, v_rsq_f32: about one ulp of fp32, three decimal
// orders below half an ulp of fp16), which matter because these operators are otherwise bound by the vector ALU, not
// by memory.  The stand-alone kernels and the one-pass chain kernel share these functions, so they agree bit for
// bit.  (In the reference these functions are the Vulkan driver's and differ from driver to driver.)
template <bool F16>
__device__ __forceinline__ float op_exp(float x) {
    // v_exp_f32 of x * log2(e); written as a fused multiply-add with zero so that an argument that has just been
    // widened from fp16 takes one v_fma_mix_f32 instead of a conversion and a multiplication (same bits: the
    // product is rounded once either way)
    return F16 ? __builtin_amdgcn_exp2f(__builtin_fmaf(x, 1.44269504088896340736f, 0.0f)) : expf(x);
}
template <bool F16>
__device__ __forceinline__ float op_reciprocal(float x) {
    return F16 ? __builtin_amdgcn_rcpf(x) : 1.0f / x;
}
template <bool F16>
__device__ __forceinline__ float op_rsqrt(float x) {
    return F16 ? __builtin_amdgcn_rsqf(x) : 1.0f / sqrtf(x);
}
template <bool F16>
__device__ __forceinline__ float op_tanh(float x) {
    if (!F16) return tanh_clamped(x);
    // the reference's three ranges (elementwise_unary.comp:136-155) with tanh(x) = 1 - 2 / (exp(2x) + 1) in between
    // exp(2x) as one v_exp_f32 of x * 2 log2(e) (doubling commutes with the rounding of the product).  Beyond
    // |x| = 10 the middle formula already gives exactly +-1 (and NaN for NaN), so the third range needs no test.
    const float x2 = x * x;
    const float small = x * (1.0f - x2 * (1.0f / 3.0f - x2 * (2.0f / 15.0f - 17.0f / 315.0f * x2)));
    const float e2x = __builtin_amdgcn_exp2f(__builtin_fmaf(x, 2.0f * 1.44269504088896340736f, 0.0f));
    const float mid = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e2x + 1.0f);
    return fabsf(x) < 0.2f ? small : mid;
}

// ---------------------------------------------------------------------------------------------------------------
// Chains that are known at compile time.  The interpreter above pays for every step with shared-memory round trips
// and a decode; a chain whose program is a template argument unrolls into straight-line code with every value in
// vector registers and runs like a stand-alone operator.  A program lists, per step, the operator and the values it
// reads (value v < n_inputs is input v, value n_inputs + i the result of step i); `full` marks the inputs that have
// the output's shape, the others are single elements.  The arithmetic is the interpreter's (packed fp16 ADD / SUB /
// MUL, the shared device functions for the rest, one rounding per step).
// ---------------------------------------------------------------------------------------------------------------
struct StaticStep {
    int op, a, b;
};
// x * c1 * (TANH((x + x * x * x * c2) * c3) + c4): the tanh form of GELU as TOSA graphs spell it, in the order in
// which the region builder emits it
struct GeluTanhProgram {
    static constexpr int n_inputs = 5, n_steps = 9;
    static constexpr bool full[n_inputs] = {true, false, false, false, false};
    static constexpr StaticStep steps[n_steps] = {{F_MUL, 0, 1}, {F_MUL, 0, 0},  {F_MUL, 6, 0},  {F_MUL, 7, 2}, {F_ADD, 0, 8},
                                                  {F_MUL, 9, 3}, {F_TANH, 10, 0}, {F_ADD, 11, 4}, {F_MUL, 5, 12}};
};
struct StaticArgs {
    char *out;
    int64_t vecs;
    const char *in[MLEL_CHAIN_MAX_INPUTS];
};

// two fp32 results rounded to fp16 (nearest even) with one v_cvt_pk_f16_f32
__device__ __forceinline__ __half2 pack_f16(float a, float b) {
    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
    typedef float f2_t __attribute__((ext_vector_type(2)));
    asm("" : "+v"(a), "+v"(b));  // the values as computed: nothing is folded into the rounding
    const f2_t v = {a, b};
    const h2_t h = __builtin_convertvector(v, h2_t);
    return __builtin_bit_cast(__half2, h);
}

template <int OP>
__device__ __forceinline__ uint4 static_apply(const uint4 &a, const uint4 &b) {
    uint4 r;
    __half2 *rh = reinterpret_cast<__half2 *>(&r);
    const __half2 *ah = reinterpret_cast<const __half2 *>(&a), *bh = reinterpret_cast<const __half2 *>(&b);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (OP == F_ADD) {
            rh[i] = __hadd2(ah[i], bh[i]);
        } else if (OP == F_SUB) {
            rh[i] = __hsub2(ah[i], bh[i]);
        } else if (OP == F_MUL) {
            rh[i] = __hmul2(ah[i], bh[i]);
        } else {
            const float2 f = __half22float2(ah[i]);
            const float y0 = OP == F_EXP ? op_exp<true>(f.x) : OP == F_RECIPROCAL ? op_reciprocal<true>(f.x)
                           : OP == F_RSQRT ? op_rsqrt<true>(f.x) : OP == F_TANH ? op_tanh<true>(f.x) : f.x;
            const float y1 = OP == F_EXP ? op_exp<true>(f.y) : OP == F_RECIPROCAL ? op_reciprocal<true>(f.y)
                           : OP == F_RSQRT ? op_rsqrt<true>(f.y) : OP == F_TANH ? op_tanh<true>(f.y) : f.y;
            rh[i] = pack_f16(y0, y1);
        }
    }
    return r;
}

template <class P, int S>
__device__ __forceinline__ void static_run(uint4 (&val)[P::n_inputs + P::n_steps]) {
    if constexpr (S < P::n_steps) {
        uint4 r = static_apply<P::steps[S].op>(val[P::steps[S].a], val[P::steps[S].b]);
        // every step's result is rounded where the stand-alone operator rounds it: the compiler must not see through
        // it, or it contracts a multiplication and the addition of the next step into one fused operation
        asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
        val[P::n_inputs + S] = r;
        static_run<P, S + 1>(val);
    }
}


// One 16-byte piece (eight halfs) through the GELU program: `c` holds the program's four single-element inputs, each
// in both halves of a word.
__device__ __forceinline__ uint4 gelu_tanh_piece(const uint4 &h, const uint32_t (&c)[4]) {
    uint4 val[GeluTanhProgram::n_inputs + GeluTanhProgram::n_steps];
    val[0] = h;
#pragma unroll
    for (int k = 0; k < 4; k++) val[1 + k] = make_uint4(c[k], c[k], c[k], c[k]);
    static_run<GeluTanhProgram, 0>(val);
    return val[GeluTanhProgram::n_inputs + GeluTanhProgram::n_steps - 1];
}

}  // namespace mlel
