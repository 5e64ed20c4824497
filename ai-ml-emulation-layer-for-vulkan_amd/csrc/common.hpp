// Shared host/device helpers of the gfx950 TOSA backend: error reporting, tensor views passed by value to
// kernels, the dtype table and generic element accessors with the reference's out-of-bounds semantics.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>

#include "../../include/mlel_hip.h"

namespace mlel {

// Cache policy of the stores that write an operator's result: sc0 | sc1 (write-through).  A result is read next by
// another launch, usually under another XCD's L2, so keeping it dirty in this one only moves its write-back to the
// end of the kernel, where nothing overlaps it.
#ifndef MLEL_OUT_AUX
#define MLEL_OUT_AUX 17
#endif
constexpr int kOutAux = MLEL_OUT_AUX;
// The same policy for a 16-byte result store through a plain pointer.
__device__ __forceinline__ void store16_result(void *p, uint4 v) {
    typedef unsigned int u32x4_st __attribute__((ext_vector_type(4)));
    const u32x4_st d = {v.x, v.y, v.z, v.w};
    // The two wait states behind the store belong to it: a store of more than eight bytes reads its data registers
    // after it has issued, and a vector instruction that overwrites them within two wait states changes what is
    // stored.  The compiler keeps that distance for the stores it emits itself; it cannot see into this one.
    if (kOutAux == 17)
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(d) : "memory");
    else
        *reinterpret_cast<uint4 *>(p) = v;
}


// floor(n / d) for 0 <= n < 2^31 as (n * m) >> (31 + s) with s = ceil(log2 d), m = ceil(2^(31 + s) / d)
// (2^(31+s) <= m d <= 2^(31+s) + 2^s, the condition of Granlund and Montgomery's theorem 4.2 for 31-bit n)
struct DivMagic {
    uint32_t m, s;
};
inline DivMagic make_div_magic(uint32_t d) {
    DivMagic r{1u << 31, 0};
    if (d <= 1) return r;
    uint32_t s = 0;
    while ((uint64_t(1) << s) < d) s++;
    const uint64_t p = uint64_t(1) << (31 + s);
    r.m = (uint32_t)((p + d - 1) / d);
    r.s = s;
    return r;
}
__device__ __forceinline__ int div_magic(int n, const DivMagic &d) {
    return (int)(((uint64_t)(uint32_t)n * d.m) >> (31 + d.s));
}

// ---------------------------------------------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------------------------------------------
int set_error(int code, const char *fmt, ...);

#define MLEL_HIP_CHECK(expr)                                                                                           \
    do {                                                                                                               \
        hipError_t e_ = (expr);                                                                                        \
        if (e_ != hipSuccess)                                                                                          \
            return ::mlel::set_error(MLEL_ERR_DEVICE, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, \
                                     __LINE__);                                                                        \
    } while (0)

#define MLEL_REQUIRE(cond, code, ...)                                                                                  \
    do {                                                                                                               \
        if (!(cond)) return ::mlel::set_error((code), __VA_ARGS__);                                                    \
    } while (0)

#define MLEL_TRY(expr)                                                                                                 \
    do {                                                                                                               \
        int rc_ = (expr);                                                                                              \
        if (rc_ != 0) return rc_;                                                                                      \
    } while (0)

int check_launch(const char *what);

// ---------------------------------------------------------------------------------------------------------------
// dtype table (mirrors the format table of the reference: common/utils.cpp:119-228)
// ---------------------------------------------------------------------------------------------------------------
__host__ __device__ inline int dt_size(int dt) {
    switch (dt) {
    case MLEL_BOOL: case MLEL_I8: case MLEL_U8: case MLEL_F8E4M3: case MLEL_F8E5M2: return 1;
    case MLEL_I16: case MLEL_U16: case MLEL_F16: case MLEL_BF16: return 2;
    case MLEL_I32: case MLEL_U32: case MLEL_F32: return 4;
    case MLEL_I64: case MLEL_U64: case MLEL_F64: return 8;
    default: return 0;
    }
}
__host__ __device__ inline bool dt_is_int(int dt) { return dt >= MLEL_BOOL && dt <= MLEL_U64; }
__host__ __device__ inline bool dt_is_float(int dt) {
    return dt == MLEL_F16 || dt == MLEL_F32 || dt == MLEL_F64 || dt == MLEL_BF16 || dt == MLEL_F8E4M3 || dt == MLEL_F8E5M2;
}
__host__ __device__ inline bool dt_is_fp8(int dt) { return dt == MLEL_F8E4M3 || dt == MLEL_F8E5M2; }
// The type arithmetic runs in (getFormatInfo's compType, common/utils.cpp:119-228): fp8 computes in fp16, bf16 in fp32.
__host__ __device__ inline int dt_comp(int dt) { return dt_is_fp8(dt) ? MLEL_F16 : (dt == MLEL_BF16 ? MLEL_F32 : dt); }
__host__ __device__ inline int64_t dt_lowest(int dt) {
    switch (dt) {
    case MLEL_I8: return -128;
    case MLEL_I16: return -32768;
    case MLEL_I32: return INT32_MIN;
    case MLEL_I64: return INT64_MIN;
    default: return 0;
    }
}
__host__ __device__ inline int64_t dt_max(int dt) {
    switch (dt) {
    case MLEL_BOOL: return 1;
    case MLEL_I8: return 127;
    case MLEL_U8: return 255;
    case MLEL_I16: return 32767;
    case MLEL_U16: return 65535;
    case MLEL_I32: return INT32_MAX;
    case MLEL_U32: return UINT32_MAX;
    default: return INT64_MAX;
    }
}
inline int dt_unsigned_twin(int dt, bool is_unsigned) {
    if (is_unsigned) {
        switch (dt) {
        case MLEL_I8: return MLEL_U8;
        case MLEL_I16: return MLEL_U16;
        case MLEL_I32: return MLEL_U32;
        case MLEL_I64: return MLEL_U64;
        default: return dt;
        }
    }
    switch (dt) {
    case MLEL_U8: return MLEL_I8;
    case MLEL_U16: return MLEL_I16;
    case MLEL_U32: return MLEL_I32;
    case MLEL_U64: return MLEL_I64;
    default: return dt;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// tensor view handed to kernels by value
// ---------------------------------------------------------------------------------------------------------------
struct TV {
    char *ptr;
    int32_t dtype;
    int32_t rank;
    int64_t dims[MLEL_MAX_RANK];
    int64_t strides[MLEL_MAX_RANK];
};

inline TV make_tv(const mlel_tensor *t) {
    TV v{};
    v.ptr = static_cast<char *>(t->ptr);
    v.dtype = t->dtype;
    v.rank = t->rank;
    for (int i = 0; i < MLEL_MAX_RANK; i++) {
        v.dims[i] = i < t->rank ? t->dims[i] : 1;
        v.strides[i] = i < t->rank ? t->strides[i] : 0;
    }
    return v;
}

int check_tensor(const mlel_tensor *t, const char *what);
int64_t numel(const mlel_tensor *t);
bool is_packed(const mlel_tensor *t);
bool same_shape(const mlel_tensor *a, const mlel_tensor *b);

// flat invocation index -> multi-index over `t`'s dims, row-major
__device__ inline void unflatten(const TV &t, int64_t flat, int64_t *idx) {
    for (int i = t.rank - 1; i >= 0; i--) {
        const int64_t d = t.dims[i];
        if (flat < (int64_t(1) << 31) && d < (int64_t(1) << 31)) {
            const uint32_t f = (uint32_t)flat, dd = (uint32_t)d;
            idx[i] = f % dd;
            flat = f / dd;
        } else {
            idx[i] = flat % d;
            flat /= d;
        }
    }
}

__device__ inline bool elem_off(const TV &t, const int64_t *idx, int64_t *off) {
    int64_t o = 0;
    for (int i = 0; i < t.rank; i++) {
        if (idx[i] < 0 || idx[i] >= t.dims[i]) return false;
        o += idx[i] * t.strides[i];
    }
    *off = o;
    return true;
}

__device__ inline int64_t raw_ld_i(const char *p, int dt) {
    switch (dt) {
    case MLEL_BOOL: return *(const uint8_t *)p != 0;
    case MLEL_I8: return *(const int8_t *)p;
    case MLEL_U8: case MLEL_F8E4M3: case MLEL_F8E5M2: return *(const uint8_t *)p;
    case MLEL_I16: return *(const int16_t *)p;
    case MLEL_U16: case MLEL_F16: case MLEL_BF16: return *(const uint16_t *)p;
    case MLEL_I32: return *(const int32_t *)p;
    case MLEL_U32: return *(const uint32_t *)p;
    case MLEL_I64: case MLEL_U64: return *(const int64_t *)p;
    default: return 0;
    }
}
__device__ inline void raw_st_i(char *p, int dt, int64_t v) {
    switch (dt) {
    case MLEL_BOOL: *(uint8_t *)p = (uint8_t)(v != 0); break;
    case MLEL_I8: case MLEL_U8: case MLEL_F8E4M3: case MLEL_F8E5M2: *(uint8_t *)p = (uint8_t)v; break;
    case MLEL_I16: case MLEL_U16: case MLEL_F16: case MLEL_BF16: *(uint16_t *)p = (uint16_t)v; break;
    case MLEL_I32: case MLEL_U32: *(uint32_t *)p = (uint32_t)v; break;
    case MLEL_I64: case MLEL_U64: *(int64_t *)p = v; break;
    default: break;
    }
}
// fp32 -> fp16, nearest even.  The value is made opaque first: the compiler otherwise folds a multiplication that
// feeds the conversion into v_fma_mix*_f16 with a +0 addend, and (-0) * x + (+0) is +0 where the product is -0.
__device__ __forceinline__ __half f2h(float v) {
    asm("" : "+v"(v));
    return __float2half_rn(v);
}

// ---- reduced-precision storage formats (graph/shaders/graph_op/common.comp:184-232, 300-418) ----
// bf16 is the upper half of an fp32; fp8 e5m2 the upper byte of an fp16; fp8 e4m3 has bias 7, no infinities and
// one NaN code per sign (0x7f).  Every fp8 value is an fp16 value, every bf16 value an fp32 value.
__device__ inline float decode_bf16(uint16_t x) { return __uint_as_float((uint32_t)x << 16); }
__device__ inline float decode_f8e5m2(uint8_t x) { return __half2float(__ushort_as_half((unsigned short)((uint32_t)x << 8))); }
__device__ inline float decode_f8e4m3(uint8_t x) {
    const uint32_t sign = (x >> 7) & 1u, e = (x >> 3) & 0xfu, m = x & 7u;
    if (e == 0xfu && m == 7u) return NAN;
    const float v = e == 0 ? (float)m / 512.0f : ldexpf(1.0f + (float)m / 8.0f, (int)e - 7);
    return sign ? -v : v;
}
// bf16 by truncation (the default store of most operators) and by round-to-nearest-even (ADD-like operators, MUL, CAST)
__device__ inline uint16_t encode_bf16_trunc(float v) { return (uint16_t)(__float_as_uint(v) >> 16); }
__device__ inline uint16_t encode_bf16_rne(float v) {
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7f800000u) == 0x7f800000u) return (uint16_t)((u >> 16) | ((u & 0x007fffffu) ? 0x0040u : 0u));
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
// fp8 from fp32: e5m2 rounds to fp16 (nearest even) and drops the low byte; beyond +-57344 it saturates to infinity
__device__ inline uint8_t encode_f8e5m2(float v) {
    const uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
    if (isnan(v)) return (uint8_t)(sign | 0x7du);
    if (isinf(v) || v > 57344.0f || v < -57344.0f) return (uint8_t)(sign | 0x7cu);
    return (uint8_t)(__half_as_ushort(f2h(v)) >> 8);
}
// e4m3 rounds the mantissa to nearest even; NaN, infinities and magnitudes above 448 give the NaN code
__device__ inline uint8_t encode_f8e4m3(float v) {
    const uint32_t bits = __float_as_uint(v), sign = (bits >> 24) & 0x80u;
    const float ax = fabsf(v);
    if (isnan(v) || isinf(v) || ax > 448.0f) return (uint8_t)(sign | 0x7fu);
    if (ax == 0.0f) return (uint8_t)sign;
    if (ax < 0.015625f) {  // below 2^-6: multiples of 2^-9
        float r = rintf(ax * 512.0f);
        r = r < 0.f ? 0.f : (r > 8.f ? 8.f : r);
        const uint32_t m = (uint32_t)r;
        if (m == 0) return (uint8_t)sign;
        if (m >= 8) return (uint8_t)(sign | 0x08u);
        return (uint8_t)(sign | m);
    }
    int exponent = (int)((bits >> 23) & 0xffu) - 127;   // floor(log2(ax)) of a normal fp32
    const uint32_t frac = bits & 0x007fffffu;           // (scaled - 1) * 2^23
    uint32_t m = (frac + 0x7ffffu + ((frac >> 20) & 1u)) >> 20;  // roundEven((scaled - 1) * 8)
    if (m == 8u) {
        m = 0;
        exponent += 1;
    }
    if (exponent > 8) return (uint8_t)(sign | 0x7fu);
    const uint32_t field = (uint32_t)(exponent + 7);
    if (field == 0xfu && m == 7u) m = 6u;
    return (uint8_t)(sign | (field << 3) | m);
}
__device__ inline uint8_t encode_f8(int dt, float v) { return dt == MLEL_F8E4M3 ? encode_f8e4m3(v) : encode_f8e5m2(v); }

__device__ inline float raw_ld_f(const char *p, int dt) {
    switch (dt) {
    case MLEL_F16: return __half2float(*(const __half *)p);
    case MLEL_F32: return *(const float *)p;
    case MLEL_F64: return (float)*(const double *)p;
    case MLEL_BF16: return decode_bf16(*(const uint16_t *)p);
    case MLEL_F8E4M3: return decode_f8e4m3(*(const uint8_t *)p);
    case MLEL_F8E5M2: return decode_f8e5m2(*(const uint8_t *)p);
    default: return (float)raw_ld_i(p, dt);
    }
}
// How a computed value becomes storage.  ST_TRUNC is the reference's ENCODE_COMP_TO_STORAGE (bf16 truncates), ST_RNE
// its ENCODE_COMP_TO_STORAGE_RNE (bf16 rounds to nearest even); both take fp8 through fp16 first (common.comp:618-633).
// ST_ACC is the convolution family's acc_to_out (common.comp:651-652): bf16 truncates, fp8 encodes the fp32 value.
enum { ST_TRUNC = 0, ST_RNE = 1, ST_ACC = 2 };
__device__ inline void raw_st_f(char *p, int dt, float v, int mode = ST_TRUNC) {
    switch (dt) {
    case MLEL_F16: *(__half *)p = f2h(v); break;
    case MLEL_F32: *(float *)p = v; break;
    case MLEL_F64: *(double *)p = (double)v; break;
    case MLEL_BF16: *(uint16_t *)p = mode == ST_RNE ? encode_bf16_rne(v) : encode_bf16_trunc(v); break;
    case MLEL_F8E4M3:
    case MLEL_F8E5M2: *(uint8_t *)p = encode_f8(dt, mode == ST_ACC ? v : __half2float(f2h(v))); break;
    default: break;
    }
}
__device__ inline int64_t ld_i(const TV &t, const int64_t *idx) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return 0;
    return raw_ld_i(t.ptr + off, t.dtype);
}
__device__ inline float ld_f(const TV &t, const int64_t *idx) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return 0.f;
    return raw_ld_f(t.ptr + off, t.dtype);
}
__device__ inline void st_i(const TV &t, const int64_t *idx, int64_t v) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return;
    raw_st_i(t.ptr + off, t.dtype, v);
}
__device__ inline void st_f(const TV &t, const int64_t *idx, float v, int mode = ST_TRUNC) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return;
    raw_st_f(t.ptr + off, t.dtype, v, mode);
}
// Integer accumulators over floating-point storage (the convolution shaders' to_acc / acc_to_out for an integer
// ACC_TYPE, common.comp:636-660): operands are truncated toward zero, the result is converted back and encoded.
__device__ inline int64_t ld_acc_i(const TV &t, const int64_t *idx) {
    return dt_is_float(t.dtype) ? (int64_t)ld_f(t, idx) : ld_i(t, idx);
}
__device__ inline void st_acc_i(const TV &t, const int64_t *idx, int64_t v) {
    if (dt_is_float(t.dtype))
        st_f(t, idx, (float)v, ST_ACC);
    else
        st_i(t, idx, v);
}
__device__ inline float rnd_f16(float v) { return __half2float(f2h(v)); }
// lowest finite value of a floating-point storage type (getFormatInfo's `lowest`, common/utils.cpp:125-131)
__device__ inline float dt_lowest_f(int dt) {
    switch (dt) {
    case MLEL_F16: return -65504.f;
    case MLEL_BF16: return -3.3895313892515355e+38f;
    case MLEL_F8E5M2: return -57344.f;
    case MLEL_F8E4M3: return -448.f;
    default: return -3.402823466e+38f;
    }
}
// rounding of an intermediate result to the type the arithmetic runs in
__device__ inline float round_to(int dt, float v) { return dt_comp(dt) == MLEL_F16 ? rnd_f16(v) : v; }

// TANH as the reference computes it (elementwise_unary.comp:136-205): saturated beyond |x| > 10, an odd polynomial
// below 0.2, the library function in between.
__device__ inline float tanh_clamped(float x) {
    const float ax = fabsf(x);
    if (x > 10.0f) return 1.0f;
    if (x < -10.0f) return -1.0f;
    if (ax < 0.2f) {
        const float x2 = x * x;
        return x * (1.0f - x2 * (1.0f / 3.0f - x2 * (2.0f / 15.0f - 17.0f / 315.0f * x2)));
    }
    return tanhf(x);
}


__host__ __device__ inline int64_t narrow_to(int dt, int64_t v) {
    switch (dt) {
    case MLEL_BOOL: return v != 0;
    case MLEL_I8: return (int8_t)v;
    case MLEL_U8: return (uint8_t)v;
    case MLEL_I16: return (int16_t)v;
    case MLEL_U16: return (uint16_t)v;
    case MLEL_I32: return (int32_t)v;
    case MLEL_U32: return (uint32_t)v;
    default: return v;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// RESCALE arithmetic shared by the stand-alone kernel and the fused epilogues
// (follows the reference shader graph/shaders/graph_op/tosa/rescale.comp:27-46)
// ---------------------------------------------------------------------------------------------------------------
struct RescaleParams {
    int32_t in_zp;   // already narrowed to the (un)signed input type
    int32_t out_zp;  // already narrowed to the (un)signed output type
    int32_t out_lo;  // clamp range: output type range intersected with a fused CLAMP
    int32_t out_hi;
    int32_t double_round;  // scale32 && double_round
    int32_t per_channel;
    int32_t clamp_out;  // 0 for 32-bit outputs (the clamp is the identity there)
};

__device__ __forceinline__ int32_t apply_scale(int64_t value, int32_t mult, int32_t shift, bool double_round) {
    int64_t round = shift > 0 ? (int64_t(1) << (shift - 1)) : 0;
    if (double_round && shift > 31) round += value >= 0 ? (int64_t(1) << 30) : -(int64_t(1) << 30);
    const uint64_t prod = (uint64_t)value * (uint64_t)(int64_t)mult + (uint64_t)round;
    const int s = shift < 0 ? 0 : (shift > 63 ? 63 : shift);
    return (int32_t)((int64_t)prod >> s);
}

// int32 accumulator -> requantised value (any shift, general form)
__device__ __forceinline__ int32_t requant_i32(int32_t acc, int32_t mult, int32_t shift, const RescaleParams &p) {
    const int64_t value = (int64_t)acc - (int64_t)p.in_zp;
    int32_t r = apply_scale(value, mult, shift, p.double_round != 0);
    r = (int32_t)((uint32_t)r + (uint32_t)p.out_zp);
    if (p.clamp_out) r = r < p.out_lo ? p.out_lo : (r > p.out_hi ? p.out_hi : r);
    return r;
}

// Per-channel RESCALE constants with everything that does not depend on the accumulator folded in:
//   result = clamp(int32((int64(acc) * mult + R) >> shift) + out_zp),
//   R = 2^(shift-1) - in_zp * mult  (+ 2^30 when acc >= in_zp, - 2^30 otherwise, if double rounding applies).
// Both signed variants of R are stored so that the choice is one compare and two selects.
struct ChanScale {
    int64_t round_pos;
    int64_t round_neg;
    int32_t mult;
    int32_t shift;
};

__host__ __device__ inline ChanScale make_chan_scale(int32_t mult, int32_t shift, const RescaleParams &p) {
    ChanScale c;
    c.mult = mult;
    c.shift = shift < 0 ? 0 : (shift > 63 ? 63 : shift);
    const uint64_t nudge = (p.double_round && shift > 31) ? (uint64_t(1) << 30) : 0;
    const uint64_t base = shift > 0 ? (uint64_t(1) << (c.shift - 1)) : 0;
    const uint64_t round = base - (uint64_t)(int64_t)p.in_zp * (uint64_t)(int64_t)mult;
    c.round_pos = (int64_t)(round + nudge);
    c.round_neg = (int64_t)(round - nudge);
#if defined(__HIP_DEVICE_COMPILE__)
    {
        // In a kernel the compiler sees how the two constants were made and would multiply their exact 64-bit
        // difference by the sign bit with two unsigned 64-bit multiply-adds per value (requant_acc); as an opaque
        // pair of registers the difference is truncated to 32 bits there and the product is one v_mad_i64_i32.
        int32_t lo = (int32_t)(uint32_t)(uint64_t)c.round_neg, hi = (int32_t)((uint64_t)c.round_neg >> 32);
        asm volatile("" : "+v"(lo), "+v"(hi));
        c.round_neg = (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo);
    }
#endif
    return c;
}

// out_lo / out_hi span the whole int32 range for 32-bit outputs, so the clamp is always applied.
__device__ __forceinline__ int32_t requant_chan(int32_t acc, const ChanScale &c, const RescaleParams &p) {
    const int64_t r = acc < p.in_zp ? c.round_neg : c.round_pos;
    const uint64_t t = (uint64_t)((int64_t)acc * (int64_t)c.mult) + (uint64_t)r;
    int32_t v = (int32_t)((int64_t)t >> c.shift);
    v = (int32_t)((uint32_t)v + (uint32_t)p.out_zp);
    // clamp(v, lo, hi) as the median of the three (out_lo <= out_hi always): one instruction instead of max + min
    int32_t clamped;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(clamped) : "v"(v), "v"(p.out_lo), "v"(p.out_hi));
    return clamped;
}

// The same for an int32 accumulator whose RESCALE has input_zp == 0 (TOSA allows no other for int32 inputs; the
// host sends operators that name one to the general kernels): the signed rounding constant is
// round_pos + sign bit * (round_neg - round_pos), the difference being 0 or -2^31, i.e. one shift and one
// multiply-add in place of the compare and the two selects (measured: 10.9 against 12.7 ns per wavefront of 64 values).
__device__ __forceinline__ int32_t requant_acc(int32_t acc, const ChanScale &c, const RescaleParams &p) {
    const int32_t fix = (int32_t)((uint64_t)c.round_neg - (uint64_t)c.round_pos);
    const int64_t r = (int64_t)(int32_t)((uint32_t)acc >> 31) * (int64_t)fix + c.round_pos;
    const uint64_t t = (uint64_t)((int64_t)acc * (int64_t)c.mult) + (uint64_t)r;
    int32_t v = (int32_t)((int64_t)t >> c.shift);
    v = (int32_t)((uint32_t)v + (uint32_t)p.out_zp);
    int32_t clamped;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(clamped) : "v"(v), "v"(p.out_lo), "v"(p.out_hi));
    return clamped;
}

// 4 rows x 4 channels (bytes) -> 4 channels x 4 vertical taps: output row 0 multiplies the column by the weights
// (w0, w1, w2, 0), output row 1 by (0, w0, w1, w2), so one transpose serves both rows of a work item
__device__ __forceinline__ void transpose_4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t (&col)[4]) {
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // [r0.b0 r1.b0 r0.b1 r1.b1]
    const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // [r0.b2 r1.b2 r0.b3 r1.b3]
    const uint32_t u0 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);  // [r2.b0 r3.b0 r2.b1 r3.b1]
    const uint32_t u1 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    col[0] = __builtin_amdgcn_perm(u0, t0, 0x05040100u);             // [t0.b0 t0.b1 u0.b0 u0.b1]
    col[1] = __builtin_amdgcn_perm(u0, t0, 0x07060302u);
    col[2] = __builtin_amdgcn_perm(u1, t1, 0x05040100u);
    col[3] = __builtin_amdgcn_perm(u1, t1, 0x07060302u);
}

// d = dot4(a, b) + c with c in a register of its own: the first tap of an output starts from the bias term without
// a copy of it into the accumulator (the two-operand form the compiler prefers accumulates in place)
__device__ __forceinline__ int32_t dot4_from(uint32_t a, uint32_t b, int32_t c) {
    int32_t d;
    asm("v_dot4_i32_i8 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

// The clamp's upper bound in a vector register that the compiler may not re-create from the scalar one: v_med3 takes
// one scalar operand only, and left alone the compiler moves both bounds into registers again for every few values
// (3 - 4 % of the vector instructions of the requantisation-bound kernels).  The staged matrix kernel keeps the
// three-argument form: its 128 x 128 direct-to-LDS variant measured 1 % slower with this one.
__device__ __forceinline__ int32_t pin_vgpr(int32_t s) {
    int32_t v;
    asm volatile("v_mov_b32 %0, %1" : "=v"(v) : "s"(s));
    return v;
}
__device__ __forceinline__ int32_t requant_acc(int32_t acc, const ChanScale &c, const RescaleParams &p, int32_t hi_v) {
    const int32_t fix = (int32_t)((uint64_t)c.round_neg - (uint64_t)c.round_pos);
    const int64_t r = (int64_t)(int32_t)((uint32_t)acc >> 31) * (int64_t)fix + c.round_pos;
    const uint64_t t = (uint64_t)((int64_t)acc * (int64_t)c.mult) + (uint64_t)r;
    int32_t v = (int32_t)((int64_t)t >> c.shift);
    v = (int32_t)((uint32_t)v + (uint32_t)p.out_zp);
    int32_t clamped;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(clamped) : "v"(v), "s"(p.out_lo), "v"(hi_v));
    return clamped;
}

int make_rescale_params(const mlel_rescale_attr *attr, int in_dtype, int out_dtype, const mlel_clamp_attr *clamp,
                        RescaleParams *out);
int check_scale_tensors(const mlel_tensor *mult, const mlel_tensor *shift, const mlel_rescale_attr *attr,
                        int64_t channels);

inline dim3 grid_1d(int64_t work_items, int block) { return dim3((unsigned)((work_items + block - 1) / block)); }

}  // namespace mlel

// Device scratch for the contraction kernels' split-K mode: int32 partial tiles and one arrival counter per tile.
// One workspace per stream that has used the mode (the calls of one stream are ordered, those of different streams
// are not), created the first time a stream asks for it outside a graph capture and freed with the context.
struct SplitWorkspace {
    hipStream_t stream;
    char *partials;      // kSplitPartialBytes
    uint32_t *counters;  // kSplitCounters, zero between launches (the last block to arrive resets its counter)
};
constexpr size_t kSplitPartialBytes = size_t(16) << 20;
constexpr int kSplitCounters = 4096;
constexpr int kMaxSplitWorkspaces = 16;

// Device staging memory of the operators that rearrange an operand before the kernel proper (CONV3D as CONV2D): one
// grow-only buffer per stream that has used such an operator (the calls of one stream are ordered, so the next call may
// overwrite it), freed with the stream or the context.
struct StageWorkspace {
    hipStream_t stream;
    char *ptr;
    size_t bytes;
};
constexpr size_t kMaxStageBytes = size_t(2) << 30;

struct mlel_ctx {
    int device;
    hipDeviceProp_t props;
    std::mutex ws_lock;
    SplitWorkspace ws[kMaxSplitWorkspaces];
    int n_ws = 0;
    StageWorkspace stage[kMaxSplitWorkspaces];
    int n_stage = 0;
    int split_k = 8;  // most blocks per tile in split-K mode; 0 or 1: never split (MLEL_SPLIT_K in the environment)
    // the statically allocated scratch of the entry point that must not allocate: this device's address of the
    // array (hipGetSymbolAddress at context creation), nullptr if that failed
    char *static_scratch = nullptr;
    int static_last_use = 0;  // what the last call of that entry point kept there: 0 nothing, 1 split-K tiles, 2 accumulator
};

namespace mlel {
// The split-K workspace of `stream`, or false when there is none and none can be made now (stream is being
// captured, table full, allocation failed): the caller then runs without splitting.
bool split_workspace(mlel_ctx *ctx, hipStream_t stream, SplitWorkspace *out);
void free_split_workspaces(mlel_ctx *ctx);
// `bytes` of staging memory for `stream`, or nullptr when it cannot be had now: growing it allocates (and waits for the
// stream, whose earlier calls may still read the old buffer), which a capturing stream cannot do.
char *stage_workspace(mlel_ctx *ctx, hipStream_t stream, size_t bytes);
// static_scratch.hip: the file-scope device array behind mlel_hip_conv2d_rescale_clamp_static
constexpr size_t kStaticScratchPartialBytes = size_t(8) << 20;
constexpr size_t kStaticScratchBytes = kStaticScratchPartialBytes + size_t(kSplitCounters) * 4;
int static_scratch_init(mlel_ctx *ctx);
int static_scratch_clear_counters(mlel_ctx *ctx, hipStream_t s);
bool stream_is_capturing(hipStream_t s);
}  // namespace mlel
