/*
 * mlel_oracle.c -- CPU restatement of the reference's TOSA operator shaders.  TEST INFRASTRUCTURE ONLY:
 * see mlel_oracle.h for the rules on who may call it and for the per-function reference citations.
 *
 * Style: one scalar code path per operator that follows the shader's arithmetic literally (types, truncation
 * points, rounding, accumulation order for floats), written over generic element accessors.  The int8
 * contractions additionally have a packed-layout fast path whose result is identical because int32
 * wraparound addition is order independent; tests compare the two paths.
 */
#include "mlel_oracle.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static __thread char g_err[512];

const char *mlel_cpu_last_error(void) { return g_err; }

int mlel_cpu_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

/* ------------------------------------------------------------------------------------------------------------
 * dtype table (reference: common/utils.cpp:119-228)
 * ---------------------------------------------------------------------------------------------------------- */
static int dt_size(int dt) {
    switch (dt) {
    case MLEL_BOOL: case MLEL_I8: case MLEL_U8: case MLEL_F8E4M3: case MLEL_F8E5M2: return 1;
    case MLEL_I16: case MLEL_U16: case MLEL_F16: case MLEL_BF16: return 2;
    case MLEL_I32: case MLEL_U32: case MLEL_F32: return 4;
    case MLEL_I64: case MLEL_U64: case MLEL_F64: return 8;
    default: return 0;
    }
}
static int dt_is_int(int dt) { return dt >= MLEL_BOOL && dt <= MLEL_U64; }
static int dt_is_float(int dt) {
    return dt == MLEL_F16 || dt == MLEL_F32 || dt == MLEL_F64 || dt == MLEL_BF16 || dt == MLEL_F8E4M3 || dt == MLEL_F8E5M2;
}
static int dt_is_fp8(int dt) { return dt == MLEL_F8E4M3 || dt == MLEL_F8E5M2; }
/* the type arithmetic runs in: fp8 -> fp16, bf16 -> fp32 (getFormatInfo compType, common/utils.cpp:125-131) */
static int dt_comp(int dt) { return dt_is_fp8(dt) ? MLEL_F16 : (dt == MLEL_BF16 ? MLEL_F32 : dt); }
static double dt_lowest_f(int dt) { /* getFormatInfo `lowest`, common/utils.cpp:119-131 */
    switch (dt) {
    case MLEL_F16: return -65504.0;
    case MLEL_BF16: return -3.3895313892515355e+38;
    case MLEL_F8E5M2: return -57344.0;
    case MLEL_F8E4M3: return -448.0;
    case MLEL_F32: return -(double)3.402823466e+38F;
    default: return -1.7976931348623157e308;
    }
}
static int64_t dt_lowest(int dt) {
    switch (dt) {
    case MLEL_I8: return -128;
    case MLEL_I16: return -32768;
    case MLEL_I32: return INT32_MIN;
    case MLEL_I64: return INT64_MIN;
    default: return 0;
    }
}
static int64_t dt_max(int dt) {
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
static int dt_unsigned_twin(int dt, int is_unsigned) {
    /* reference: common/utils.cpp:189-228 */
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

/* ------------------------------------------------------------------------------------------------------------
 * binary16 / bfloat16 codecs
 * ---------------------------------------------------------------------------------------------------------- */
float mlel_cpu_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* double -> binary16, round to nearest even, one rounding. */
static uint16_t f64_to_f16(double d) {
    uint64_t b;
    memcpy(&b, &d, 8);
    uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
    int64_t exp = (int64_t)((b >> 52) & 0x7ff);
    uint64_t man = b & 0xfffffffffffffull;
    if (exp == 0x7ff) {
        if (man) return (uint16_t)(sign | 0x7e00u | (uint16_t)(man >> 42));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (exp == 0) return sign; /* double denormals are far below half's range */
    int64_t e = exp - 1023;    /* unbiased */
    man |= 1ull << 52;         /* 53-bit significand, value = man * 2^(e-52) */
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    int shift;   /* number of low bits to drop from the 53-bit significand */
    int64_t he;  /* biased half exponent */
    if (e >= -14) {
        shift = 42;
        he = e + 15;
    } else {
        /* subnormal half: value = m * 2^-24 */
        shift = (int)(42 + (-14 - e));
        he = 0;
        if (shift > 63) return sign;
    }
    uint64_t kept = man >> shift;
    uint64_t rem = man & ((1ull << shift) - 1);
    uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (kept & 1))) kept++;
    uint32_t out;
    if (he == 0) {
        out = (uint32_t)kept; /* may carry into exponent 1: correct encoding */
    } else {
        out = (uint32_t)(((uint64_t)(he - 1) << 10) + kept); /* kept has the implicit bit at position 10 */
    }
    if (out >= 0x7c00u) out = 0x7c00u;
    return (uint16_t)(sign | out);
}
uint16_t mlel_cpu_f32_to_f16(float f) { return f64_to_f16((double)f); }
static double rnd_f16(double d) { return (double)mlel_cpu_f16_to_f32(f64_to_f16(d)); }
static double rnd_f32(double d) { return (double)(float)d; }

static float bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* ------------------------------------------------------------------------------------------------------------
 * element access: out-of-bounds reads give 0, out-of-bounds writes are dropped
 * (reference: tensor/shaders/tensor.glsl:26-81)
 * ---------------------------------------------------------------------------------------------------------- */
static int64_t numel(const mlel_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->rank; i++) n *= t->dims[i];
    return n;
}

static inline int elem_off(const mlel_tensor *t, const int64_t *idx, int64_t *off) {
    int64_t o = 0;
    for (int i = 0; i < t->rank; i++) {
        if (idx[i] < 0 || idx[i] >= t->dims[i]) return 0;
        o += idx[i] * t->strides[i];
    }
    *off = o;
    return 1;
}

static inline int64_t raw_ld_i(const void *p, int dt) {
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
static inline void raw_st_i(void *p, int dt, int64_t v) {
    switch (dt) {
    case MLEL_BOOL: *(uint8_t *)p = (uint8_t)(v != 0); break;
    case MLEL_I8: case MLEL_U8: case MLEL_F8E4M3: case MLEL_F8E5M2: *(uint8_t *)p = (uint8_t)v; break;
    case MLEL_I16: case MLEL_U16: case MLEL_F16: case MLEL_BF16: *(uint16_t *)p = (uint16_t)v; break;
    case MLEL_I32: case MLEL_U32: *(uint32_t *)p = (uint32_t)v; break;
    case MLEL_I64: case MLEL_U64: *(int64_t *)p = v; break;
    default: break;
    }
}
/* ---- reduced-precision storage formats, written after graph/shaders/graph_op/common.comp ----
 * decode: bf16 :185-189, e5m2 :191-195, e4m3 :197-215; encode: bf16 truncation :300-305, bf16 nearest-even :403-418,
 * e5m2 :312-327, e4m3 :329-371.  The e4m3 encoder keeps the shader's floating-point formulation (floor(log2), exp2,
 * roundEven) in double precision, where every step is exact for fp32 inputs. */
static double f8e5m2_to_f64(uint8_t x) { return (double)mlel_cpu_f16_to_f32((uint16_t)((uint32_t)x << 8)); }
static double f8e4m3_to_f64(uint8_t x) {
    const unsigned sign = (x >> 7) & 1u, exponent = (x >> 3) & 0xFu, mantissa = x & 7u;
    if (exponent == 0xFu && mantissa == 7u) return NAN;
    double value;
    if (exponent == 0u)
        value = mantissa == 0u ? 0.0 : (double)mantissa / 512.0;
    else
        value = exp2((double)((int)exponent - 7)) * (1.0 + (double)mantissa / 8.0);
    return sign ? -value : value;
}
static uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static uint16_t f32_to_bf16_trunc(float x) { return (uint16_t)(f32_bits(x) >> 16); }
static uint16_t f32_to_bf16_rne(float x) {
    uint32_t u = f32_bits(x);
    const uint32_t exp = u & 0x7F800000u, mantissa = u & 0x007FFFFFu;
    if (exp == 0x7F800000u) return mantissa != 0u ? (uint16_t)((u >> 16) | 0x0040u) : (uint16_t)(u >> 16);
    const uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}
static uint8_t f32_to_f8e5m2(float x) {
    const uint32_t sign = (f32_bits(x) >> 24) & 0x80u;
    if (isnan(x)) return (uint8_t)(sign | 0x7Du);
    if (isinf(x) || x > 57344.0f || x < -57344.0f) return (uint8_t)(sign | 0x7Cu);
    return (uint8_t)(mlel_cpu_f32_to_f16(x) >> 8); /* packHalf2x16 (nearest even), upper byte */
}
static double round_even(double v) { return nearbyint(v); } /* default rounding mode: ties to even */
static double clampd(double v, double lo, double hi) { return v < lo ? lo : (v > hi ? hi : v); }
static uint8_t f32_to_f8e4m3(float x) {
    const uint32_t sign = (f32_bits(x) >> 24) & 0x80u;
    const double ax = fabs((double)x);
    if (isnan(x) || isinf(x) || ax > 448.0) return (uint8_t)(sign | 0x7Fu);
    if (ax == 0.0) return (uint8_t)sign;
    if (ax < exp2(-6.0)) {
        const unsigned mantissa = (unsigned)clampd(round_even(ax * 512.0), 0.0, 8.0);
        if (mantissa == 0u) return (uint8_t)sign;
        if (mantissa >= 8u) return (uint8_t)(sign | 0x08u);
        return (uint8_t)(sign | mantissa);
    }
    int exponent = (int)floor(log2(ax));
    if (exp2((double)exponent) > ax) exponent--; /* guard the library's log2 at exact powers of two */
    if (exp2((double)(exponent + 1)) <= ax) exponent++;
    const double scaled = ax * exp2((double)-exponent);
    unsigned mantissa = (unsigned)clampd(round_even((scaled - 1.0) * 8.0), 0.0, 8.0);
    if (mantissa == 8u) {
        mantissa = 0u;
        exponent += 1;
    }
    if (exponent > 8) return (uint8_t)(sign | 0x7Fu);
    const unsigned field = (unsigned)(exponent + 7);
    if (field == 0xFu && mantissa == 0x7u) mantissa = 0x6u;
    return (uint8_t)(sign | (field << 3) | mantissa);
}
uint16_t mlel_cpu_f32_to_bf16(float x, int nearest_even) { return nearest_even ? f32_to_bf16_rne(x) : f32_to_bf16_trunc(x); }
uint8_t mlel_cpu_f32_to_f8(float x, int dtype) { return dtype == MLEL_F8E4M3 ? f32_to_f8e4m3(x) : f32_to_f8e5m2(x); }
float mlel_cpu_f8_to_f32(uint8_t x, int dtype) { return (float)(dtype == MLEL_F8E4M3 ? f8e4m3_to_f64(x) : f8e5m2_to_f64(x)); }

static inline double raw_ld_f(const void *p, int dt) {
    switch (dt) {
    case MLEL_F16: return (double)mlel_cpu_f16_to_f32(*(const uint16_t *)p);
    case MLEL_BF16: return (double)bf16_to_f32(*(const uint16_t *)p);
    case MLEL_F8E4M3: return f8e4m3_to_f64(*(const uint8_t *)p);
    case MLEL_F8E5M2: return f8e5m2_to_f64(*(const uint8_t *)p);
    case MLEL_F32: return (double)*(const float *)p;
    case MLEL_F64: return *(const double *)p;
    default: return (double)raw_ld_i(p, dt);
    }
}
/* How a computed value becomes storage (common.comp:611-633, 651-652).  ST_TRUNC = ENCODE_COMP_TO_STORAGE: bf16
 * truncates; ST_RNE = ENCODE_COMP_TO_STORAGE_RNE: bf16 rounds to nearest even; both send fp8 through fp16 first.
 * ST_ACC = the convolution family's acc_to_out and CAST to fp8: bf16 truncates, fp8 encodes the fp32 value itself. */
enum { ST_TRUNC = 0, ST_RNE = 1, ST_ACC = 2 };
static inline void raw_st_f_mode(void *p, int dt, double v, int mode) {
    switch (dt) {
    case MLEL_F16: *(uint16_t *)p = f64_to_f16(v); break;
    case MLEL_F32: *(float *)p = (float)v; break;
    case MLEL_F64: *(double *)p = v; break;
    case MLEL_BF16: *(uint16_t *)p = mode == ST_RNE ? f32_to_bf16_rne((float)v) : f32_to_bf16_trunc((float)v); break;
    case MLEL_F8E4M3:
    case MLEL_F8E5M2: {
        const float f = mode == ST_ACC ? (float)v : mlel_cpu_f16_to_f32(f64_to_f16(v));
        *(uint8_t *)p = dt == MLEL_F8E4M3 ? f32_to_f8e4m3(f) : f32_to_f8e5m2(f);
        break;
    }
    default: break;
    }
}

static inline int64_t ld_i(const mlel_tensor *t, const int64_t *idx) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return 0;
    return raw_ld_i((const char *)t->ptr + off, t->dtype);
}
static inline double ld_f(const mlel_tensor *t, const int64_t *idx) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return 0.0;
    return raw_ld_f((const char *)t->ptr + off, t->dtype);
}
static inline void st_i(const mlel_tensor *t, const int64_t *idx, int64_t v) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return;
    raw_st_i((char *)t->ptr + off, t->dtype, v);
}
static inline void st_f_mode(const mlel_tensor *t, const int64_t *idx, double v, int mode) {
    int64_t off;
    if (!elem_off(t, idx, &off)) return;
    raw_st_f_mode((char *)t->ptr + off, t->dtype, v, mode);
}
static inline void st_f(const mlel_tensor *t, const int64_t *idx, double v) { st_f_mode(t, idx, v, ST_TRUNC); }

/* Integer accumulators over floating-point storage (the convolution shaders' to_acc / acc_to_out with an integer
 * ACC_TYPE, common.comp:636-660): operands are truncated toward zero, the result is converted back and encoded. */
static inline int64_t ld_acc_i(const mlel_tensor *t, const int64_t *idx) {
    return dt_is_float(t->dtype) ? (int64_t)(float)ld_f(t, idx) : ld_i(t, idx);
}
static inline void st_acc_i(const mlel_tensor *t, const int64_t *idx, int64_t v) {
    if (dt_is_float(t->dtype))
        st_f_mode(t, idx, (double)(float)v, ST_ACC);
    else
        st_i(t, idx, v);
}

/* flat invocation index -> row-major multi-index over `t`'s dims (reference: common.comp:74-128) */
static inline void unflatten(const mlel_tensor *t, int64_t flat, int64_t *idx) {
    for (int i = t->rank - 1; i >= 0; i--) {
        idx[i] = flat % t->dims[i];
        flat /= t->dims[i];
    }
}

static int check_tensor(const mlel_tensor *t, const char *what) {
    if (!t || !t->ptr) return fail(MLEL_ERR_INVALID, "%s: null tensor", what);
    if (t->rank < 1 || t->rank > MLEL_MAX_RANK) return fail(MLEL_ERR_INVALID, "%s: rank %d", what, t->rank);
    if (dt_size(t->dtype) == 0) return fail(MLEL_ERR_INVALID, "%s: dtype %d", what, t->dtype);
    for (int i = 0; i < t->rank; i++)
        if (t->dims[i] < 0) return fail(MLEL_ERR_INVALID, "%s: negative dim", what);
    return 0;
}
#define CHECK(t, what)                                                                                                 \
    do {                                                                                                               \
        int rc_ = check_tensor((t), (what));                                                                           \
        if (rc_) return rc_;                                                                                           \
    } while (0)

static int is_packed(const mlel_tensor *t) {
    int64_t s = dt_size(t->dtype);
    for (int i = t->rank - 1; i >= 0; i--) {
        if (t->strides[i] != s) return 0;
        s *= t->dims[i];
    }
    return 1;
}

/* wraparound helpers (signed overflow is undefined in C; do the arithmetic unsigned) */
static inline int32_t wadd32(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
static inline int32_t wmul32(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }
static inline int64_t wadd64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a + (uint64_t)b); }
static inline int64_t wmul64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a * (uint64_t)b); }
static inline int64_t asr64(int64_t v, int s) {
    /* arithmetic shift right on int64 (floor), defined for 0 <= s <= 63 */
    if (s <= 0) return v;
    if (s > 63) s = 63;
    return v < 0 ? ~((~v) >> s) : v >> s;
}

/* ------------------------------------------------------------------------------------------------------------
 * CONV2D (reference: conv2d.comp:40-116)
 * ---------------------------------------------------------------------------------------------------------- */
static int acc_is_float(uint32_t acc) { return acc == MLEL_ACC_F16 || acc == MLEL_ACC_F32; }

int mlel_cpu_conv2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w, const mlel_tensor *bias,
                    const mlel_conv2d_attr *a) {
    CHECK(out, "conv2d out");
    CHECK(in, "conv2d in");
    CHECK(w, "conv2d weights");
    CHECK(bias, "conv2d bias");
    if (out->rank != 4 || in->rank != 4 || w->rank != 4 || bias->rank != 1)
        return fail(MLEL_ERR_INVALID, "conv2d: ranks must be 4,4,4,1");
    if (a->acc_type < 1 || a->acc_type > 4) return fail(MLEL_ERR_INVALID, "Unsupported acc type %u", a->acc_type);
    const int64_t N = out->dims[0], OH = out->dims[1], OW = out->dims[2], OC = out->dims[3];
    const int64_t H = in->dims[1], W = in->dims[2], IC = in->dims[3];
    const int64_t KH = w->dims[1], KW = w->dims[2];
    const int facc = acc_is_float(a->acc_type);
    const int64_t total = N * OH * OW * OC;

    /* packed int8 x int8 -> int32 fast path: same sums, contiguous inner loop */
    if (!facc && a->acc_type == MLEL_ACC_I32 && in->dtype == MLEL_I8 && w->dtype == MLEL_I8 &&
        out->dtype == MLEL_I32 && bias->dtype == MLEL_I32 && is_packed(in) && is_packed(w) && is_packed(out) &&
        is_packed(bias) && w->dims[3] == IC && w->dims[0] >= OC && in->dims[0] >= N &&
        (bias->dims[0] == 1 || bias->dims[0] >= OC)) {
        const int8_t *x = (const int8_t *)in->ptr;
        const int8_t *wt = (const int8_t *)w->ptr;
        const int32_t *bs = (const int32_t *)bias->ptr;
        int32_t *y = (int32_t *)out->ptr;
        const int32_t zi = a->input_zp, zw = a->weight_zp;
#pragma omp parallel for schedule(static)
        for (int64_t pix = 0; pix < N * OH * OW; pix++) {
            const int64_t n = pix / (OH * OW), oy = (pix / OW) % OH, ox = pix % OW;
            for (int64_t oc = 0; oc < OC; oc++) {
                int32_t acc = 0;
                for (int64_t ky = 0; ky < KH; ky++) {
                    const int64_t yy = oy * a->stride[0] - a->pad[0] + ky * a->dilation[0];
                    if (yy < 0 || yy >= H) continue;
                    for (int64_t kx = 0; kx < KW; kx++) {
                        const int64_t xx = ox * a->stride[1] - a->pad[2] + kx * a->dilation[1];
                        if (xx < 0 || xx >= W) continue;
                        const int8_t *xp = x + ((n * H + yy) * W + xx) * IC;
                        const int8_t *wp = wt + ((oc * KH + ky) * KW + kx) * IC;
                        int32_t s = 0;
                        for (int64_t ic = 0; ic < IC; ic++) s += ((int32_t)xp[ic] - zi) * ((int32_t)wp[ic] - zw);
                        acc = wadd32(acc, s);
                    }
                }
                acc = wadd32(acc, bs[bias->dims[0] == 1 ? 0 : oc]);
                y[pix * OC + oc] = acc;
            }
        }
        return 0;
    }

#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[4];
        unflatten(out, flat, o);
        const int64_t n = o[0], oy = o[1], ox = o[2], oc = o[3];
        int64_t iacc = 0;
        double dacc = 0.0;
        for (int64_t ky = 0; ky < KH; ky++) {
            for (int64_t kx = 0; kx < KW; kx++) {
                const int64_t yy = oy * a->stride[0] - a->pad[0] + ky * a->dilation[0];
                const int64_t xx = ox * a->stride[1] - a->pad[2] + kx * a->dilation[1];
                if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue; /* padded taps contribute nothing */
                for (int64_t ic = 0; ic < IC; ic++) {
                    const int64_t xi[4] = {n, yy, xx, ic};
                    const int64_t wi[4] = {oc, ky, kx, ic};
                    if (!facc) {
                        const int64_t v = ld_acc_i(in, xi) - a->input_zp;
                        const int64_t ww = ld_acc_i(w, wi) - a->weight_zp;
                        if (a->acc_type == MLEL_ACC_I32)
                            iacc = wadd32((int32_t)iacc, wmul32((int32_t)v, (int32_t)ww));
                        else
                            iacc = wadd64(iacc, wmul64(v, ww));
                    } else {
                        /* values are converted to the accumulator type, the products are formed in fp32 and
                         * converted back to the accumulator type before being added one by one */
                        double v = ld_f(in, xi), ww = ld_f(w, wi);
                        if (a->acc_type == MLEL_ACC_F16) {
                            v = rnd_f16(v);
                            ww = rnd_f16(ww);
                        }
                        double p = rnd_f32(rnd_f32(v - (double)a->input_zp) * rnd_f32(ww - (double)a->weight_zp));
                        if (a->acc_type == MLEL_ACC_F16)
                            dacc = rnd_f16(dacc + rnd_f16(p));
                        else
                            dacc = rnd_f32(dacc + p);
                    }
                }
            }
        }
        const int64_t bi[1] = {bias->dims[0] == 1 ? 0 : oc};
        if (!facc) {
            const int64_t b = ld_acc_i(bias, bi);
            if (a->acc_type == MLEL_ACC_I32)
                iacc = wadd32((int32_t)iacc, (int32_t)b);
            else
                iacc = wadd64(iacc, b);
            st_acc_i(out, o, iacc);
        } else {
            double b = ld_f(bias, bi);
            if (a->acc_type == MLEL_ACC_F16)
                dacc = rnd_f16(dacc + rnd_f16(b));
            else
                dacc = rnd_f32(dacc + b);
            st_f_mode(out, o, dacc, ST_ACC);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * DEPTHWISE_CONV2D (reference: depthwise_conv2d.comp:31-78)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_depthwise_conv2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                              const mlel_tensor *bias, const mlel_conv2d_attr *a) {
    CHECK(out, "dwconv out");
    CHECK(in, "dwconv in");
    CHECK(w, "dwconv weights");
    CHECK(bias, "dwconv bias");
    if (out->rank != 4 || in->rank != 4 || w->rank != 4 || bias->rank != 1)
        return fail(MLEL_ERR_INVALID, "depthwise_conv2d: ranks must be 4,4,4,1");
    if (a->acc_type < 1 || a->acc_type > 4) return fail(MLEL_ERR_INVALID, "Unsupported acc type %u", a->acc_type);
    const int64_t H = in->dims[1], W = in->dims[2];
    const int64_t KH = w->dims[0], KW = w->dims[1], M = w->dims[3];
    const int facc = acc_is_float(a->acc_type);
    const int64_t total = numel(out);
    if (M <= 0) return fail(MLEL_ERR_INVALID, "depthwise_conv2d: multiplier dim must be > 0");
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[4];
        unflatten(out, flat, o);
        const int64_t n = o[0], oy = o[1], ox = o[2], ocm = o[3];
        const int64_t c = ocm / M, m = ocm % M;
        int64_t iacc = 0;
        double dacc = 0.0;
        for (int64_t ky = 0; ky < KH; ky++) {
            for (int64_t kx = 0; kx < KW; kx++) {
                const int64_t yy = oy * a->stride[0] - a->pad[0] + ky * a->dilation[0];
                const int64_t xx = ox * a->stride[1] - a->pad[2] + kx * a->dilation[1];
                if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
                const int64_t xi[4] = {n, yy, xx, c};
                const int64_t wi[4] = {ky, kx, c, m};
                if (!facc) {
                    const int64_t v = ld_acc_i(in, xi) - a->input_zp;
                    const int64_t ww = ld_acc_i(w, wi) - a->weight_zp;
                    if (a->acc_type == MLEL_ACC_I32)
                        iacc = wadd32((int32_t)iacc, wmul32((int32_t)v, (int32_t)ww));
                    else
                        iacc = wadd64(iacc, wmul64(v, ww));
                } else if (a->acc_type == MLEL_ACC_F16) {
                    double v = rnd_f16(rnd_f16(ld_f(in, xi)) - rnd_f16((double)a->input_zp));
                    double ww = rnd_f16(rnd_f16(ld_f(w, wi)) - rnd_f16((double)a->weight_zp));
                    dacc = rnd_f16(dacc + rnd_f16(v * ww));
                } else {
                    double v = rnd_f32(ld_f(in, xi) - (double)a->input_zp);
                    double ww = rnd_f32(ld_f(w, wi) - (double)a->weight_zp);
                    dacc = rnd_f32(dacc + rnd_f32(v * ww));
                }
            }
        }
        const int64_t bi[1] = {bias->dims[0] == 1 ? 0 : ocm};
        if (!facc) {
            const int64_t b = ld_acc_i(bias, bi);
            st_acc_i(out, o, a->acc_type == MLEL_ACC_I32 ? (int64_t)wadd32((int32_t)b, (int32_t)iacc) : wadd64(b, iacc));
        } else if (a->acc_type == MLEL_ACC_F16) {
            st_f_mode(out, o, rnd_f16(rnd_f16(ld_f(bias, bi)) + dacc), ST_ACC);
        } else {
            st_f_mode(out, o, rnd_f32(ld_f(bias, bi) + dacc), ST_ACC);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * MATMUL (reference: matmul.comp:30-73).  Compute type = output type.
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_matmul(const mlel_tensor *out, const mlel_tensor *A, const mlel_tensor *B, const mlel_matmul_attr *at) {
    CHECK(out, "matmul out");
    CHECK(A, "matmul a");
    CHECK(B, "matmul b");
    if (out->rank != 3 || A->rank != 3 || B->rank != 3) return fail(MLEL_ERR_INVALID, "matmul: rank must be 3");
    const int64_t N = out->dims[0], H = out->dims[1], W = out->dims[2], C = A->dims[2];

    if (A->dtype == MLEL_I8 && B->dtype == MLEL_I8 && out->dtype == MLEL_I32 && is_packed(A) && is_packed(B) &&
        is_packed(out) && A->dims[0] >= N && B->dims[0] >= N && A->dims[1] >= H && B->dims[1] >= C &&
        B->dims[2] >= W && B->dims[2] == W && A->dims[1] == H) {
        const int8_t *a = (const int8_t *)A->ptr;
        const int8_t *b = (const int8_t *)B->ptr;
        int32_t *y = (int32_t *)out->ptr;
        const int32_t za = at->a_zp, zb = at->b_zp;
#pragma omp parallel for schedule(static)
        for (int64_t row = 0; row < N * H; row++) {
            const int64_t n = row / H;
            int32_t *yr = y + row * W;
            for (int64_t x = 0; x < W; x++) yr[x] = 0;
            for (int64_t c = 0; c < C; c++) {
                const int32_t av = (int32_t)a[row * C + c] - za;
                const int8_t *br = b + (n * C + c) * W;
                for (int64_t x = 0; x < W; x++) yr[x] = wadd32(yr[x], wmul32(av, (int32_t)br[x] - zb));
            }
        }
        return 0;
    }

    const int64_t total = N * H * W;
    const int od = out->dtype;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[3];
        unflatten(out, flat, o);
        int64_t iacc = 0;
        double dacc = 0.0;
        for (int64_t c = 0; c < C; c++) {
            const int64_t ai[3] = {o[0], o[1], c};
            const int64_t bi[3] = {o[0], c, o[2]};
            if (dt_is_int(od)) {
                const int64_t v1 = ld_i(A, ai) - at->a_zp, v2 = ld_i(B, bi) - at->b_zp;
                if (od == MLEL_I32)
                    iacc = wadd32((int32_t)iacc, wmul32((int32_t)v1, (int32_t)v2));
                else
                    iacc = wadd64(iacc, wmul64(v1, v2));
            } else if (dt_comp(od) == MLEL_F16) {
                double v1 = rnd_f16(ld_f(A, ai) - rnd_f16((double)at->a_zp));
                double v2 = rnd_f16(ld_f(B, bi) - rnd_f16((double)at->b_zp));
                dacc = rnd_f16(dacc + rnd_f16(v1 * v2));
            } else {
                double v1 = rnd_f32(ld_f(A, ai) - (double)at->a_zp);
                double v2 = rnd_f32(ld_f(B, bi) - (double)at->b_zp);
                dacc = rnd_f32(dacc + rnd_f32(v1 * v2));
            }
        }
        if (dt_is_int(od))
            st_i(out, o, iacc);
        else
            st_f(out, o, dacc);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * RESCALE (reference: rescale.comp:27-72)
 * ---------------------------------------------------------------------------------------------------------- */
static inline int64_t narrow_to(int dt, int64_t v) {
    /* C-style conversion of an integer to the storage type `dt`, returned sign/zero extended */
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

static inline int32_t apply_scale(int64_t value, int32_t multiplier, int shift, int double_round) {
    /* reference: rescale.comp:27-46.  shift == 0 shifts by -1 in the shader, which is undefined there; the
     * rounding term is taken as 0 in that case. */
    int64_t round = shift > 0 ? (int64_t)1 << (shift - 1) : 0;
    if (double_round && shift > 31) round += value >= 0 ? ((int64_t)1 << 30) : -((int64_t)1 << 30);
    int64_t result = wmul64(value, (int64_t)multiplier);
    result = wadd64(result, round);
    result = asr64(result, shift);
    return (int32_t)result;
}

int mlel_cpu_rescale(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *mult, const mlel_tensor *shift,
                     const mlel_rescale_attr *a) {
    CHECK(out, "rescale out");
    CHECK(in, "rescale in");
    CHECK(mult, "rescale multiplier");
    CHECK(shift, "rescale shift");
    if (!dt_is_int(in->dtype) || !dt_is_int(out->dtype)) return fail(MLEL_ERR_INVALID, "rescale: integer types only");
    const int in_dt = dt_unsigned_twin(in->dtype, (int)a->input_unsigned);
    const int out_dt = dt_unsigned_twin(out->dtype, (int)a->output_unsigned);
    const int64_t total = numel(out);
    const int64_t zi = narrow_to(in_dt, a->input_zp);
    const int64_t zo = narrow_to(out_dt, a->output_zp);
    const int64_t lo = dt_lowest(out_dt), hi = dt_max(out_dt);
    mlel_tensor in_v = *in; /* view the bytes as the (un)signed twin */
    in_v.dtype = in_dt;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        const int64_t c[1] = {a->per_channel ? o[out->rank - 1] : 0};
        const int64_t value = ld_i(&in_v, o) - zi;
        const int32_t m = (int32_t)ld_i(mult, c);
        const int sh = (int)(int8_t)ld_i(shift, c);
        int32_t r = apply_scale(value, m, sh, a->scale32 && a->double_round);
        r = wadd32(r, (int32_t)zo);
        int64_t res = r;
        if (out_dt != MLEL_I32 && out_dt != MLEL_U32) {
            if (res < lo) res = lo;
            if (res > hi) res = hi;
        }
        st_i(out, o, res);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * CLAMP (reference: clamp.comp:24-53)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_clamp(const mlel_tensor *out, const mlel_tensor *in, const mlel_clamp_attr *a) {
    CHECK(out, "clamp out");
    CHECK(in, "clamp in");
    const int64_t total = numel(out);
    const int dt = out->dtype;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        if (dt_is_int(dt)) {
            /* COMP_T(double): conversion truncates toward zero; out-of-range conversions are undefined */
            const int64_t mn = narrow_to(dt, (int64_t)a->min_val), mx = narrow_to(dt, (int64_t)a->max_val);
            int64_t v = ld_i(in, o);
            v = v < mn ? mn : v;
            v = v > mx ? mx : v;
            st_i(out, o, v);
        } else {
            double mn = a->min_val, mx = a->max_val, v = ld_f(in, o);
            if (dt_comp(dt) == MLEL_F16) {
                mn = rnd_f16(mn);
                mx = rnd_f16(mx);
            } else if (dt_comp(dt) == MLEL_F32) {
                mn = rnd_f32(mn);
                mx = rnd_f32(mx);
            }
            if (isnan(v) && a->nan_mode == MLEL_NAN_IGNORE) v = mn;
            if (!isnan(v)) {
                v = v < mn ? mn : v;
                v = v > mx ? mx : v;
            }
            st_f(out, o, v);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * elementwise binary (reference: elementwise_binary.comp:146-173; broadcast common.comp:64-72)
 * ---------------------------------------------------------------------------------------------------------- */
static inline void broadcast_idx(const mlel_tensor *t, const int64_t *o, int64_t *idx) {
    for (int i = 0; i < t->rank; i++) idx[i] = t->dims[i] == 1 ? 0 : o[i];
}

static double round_to(int dt, double v) {
    dt = dt_comp(dt);
    if (dt == MLEL_F16) return rnd_f16(v);
    if (dt == MLEL_F32) return rnd_f32(v);
    return v;
}

static double glsl_mod(double x, double y) { return x - y * floor(x / y); }

static double power_f(double base, double e) {
    /* reference: elementwise_binary.comp:69-89 */
    if (base >= 0.0) return pow(base, e);
    if (glsl_mod(e, 2.0) == 0.0) return pow(-base, e);
    if (glsl_mod(e, 1.0) == 0.0) return -pow(-base, e);
    return NAN;
}

int mlel_cpu_elementwise_binary(int32_t op, const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2,
                                uint32_t nan_mode) {
    CHECK(out, "binary out");
    CHECK(in1, "binary in1");
    CHECK(in2, "binary in2");
    if (op < 0 || op >= MLEL_BIN_COUNT) return fail(MLEL_ERR_INVALID, "binary: unknown op %d", op);
    if (in1->dtype != in2->dtype) return fail(MLEL_ERR_INVALID, "binary: input types differ");
    if (in1->rank != out->rank || in2->rank != out->rank) return fail(MLEL_ERR_INVALID, "binary: ranks differ");
    const int64_t total = numel(out);
    const int idt = in1->dtype;
    const int isf = dt_is_float(idt);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], i1[MLEL_MAX_RANK], i2[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        broadcast_idx(in1, o, i1);
        broadcast_idx(in2, o, i2);
        if (isf) {
            const double a = ld_f(in1, i1), b = ld_f(in2, i2);
            double r = 0.0;
            int is_bool = 0, br = 0;
            switch (op) {
            case MLEL_BIN_ADD: r = round_to(idt, a + b); break;
            case MLEL_BIN_SUB: r = round_to(idt, a - b); break;
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
            case MLEL_BIN_POW: r = round_to(idt, power_f(a, b)); break;
            case MLEL_BIN_EQUAL: is_bool = 1; br = a == b; break;
            case MLEL_BIN_GREATER: is_bool = 1; br = a > b; break;
            case MLEL_BIN_GREATER_EQUAL: is_bool = 1; br = a >= b; break;
            default: break;
            }
            if (is_bool)
                st_i(out, o, br);
            else
                st_f_mode(out, o, r, ST_RNE);
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
                /* zeroExtend(value1) >> uint(value2) (reference: elementwise_binary.comp:33-37) */
                uint32_t z = idt == MLEL_I8 ? (uint8_t)a : idt == MLEL_I16 ? (uint16_t)a : (uint32_t)a;
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
            st_i(out, o, r); /* truncating store into the output type */
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * MUL (reference: mul.comp:24-59)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_mul(const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2, uint32_t shift) {
    CHECK(out, "mul out");
    CHECK(in1, "mul in1");
    CHECK(in2, "mul in2");
    if (in1->dtype != in2->dtype) return fail(MLEL_ERR_INVALID, "mul: input types differ");
    if (in1->rank != out->rank || in2->rank != out->rank) return fail(MLEL_ERR_INVALID, "mul: ranks differ");
    const int64_t total = numel(out);
    const int isf = dt_is_float(in1->dtype);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], i1[MLEL_MAX_RANK], i2[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        broadcast_idx(in1, o, i1);
        broadcast_idx(in2, o, i2);
        if (isf) {
            st_f_mode(out, o, round_to(out->dtype, round_to(out->dtype, ld_f(in1, i1)) * round_to(out->dtype, ld_f(in2, i2))), ST_RNE);
        } else {
            int64_t r = wmul64(ld_i(in1, i1), ld_i(in2, i2));
            if (shift > 0) r = asr64(wadd64(r, (int64_t)1 << (shift - 1)), (int)shift);
            st_i(out, o, r);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * elementwise unary (reference: elementwise_unary.comp:16-205)
 * ---------------------------------------------------------------------------------------------------------- */
static float erf_ref(float x) {
    /* reference: elementwise_unary.comp:54-134, evaluated in fp32 */
    static const float coeffs[12] = {0.08f, 0.08695652173913043f, 0.09523809523809523f, 0.10526315789473684f,
                                     0.11764705882352941f, 0.13333333333333333f, 0.15384615384615385f,
                                     0.18181818181818182f, 0.22222222222222222f, 0.28571428571428571f, 0.4f,
                                     0.66666666666666666f};
    static const float pc[5][2] = {{3.47469513777439592f, 12.07402036406381411f},
                                   {4.00561509202259545f, 9.30596659485887898f},
                                   {5.95908795446633271f, 9.19435612886969243f},
                                   {5.16722705817812584f, 9.12661617673673262f},
                                   {2.71078540045147805f, 5.80755613130301624f}};
    static const float qc[5][2] = {{3.47954057099518960f, 12.06166887286239555f},
                                   {3.72068443960225092f, 8.44319781003968454f},
                                   {3.90225704029924078f, 6.36161630953880464f},
                                   {4.03296893109262491f, 5.13578530585681539f},
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
        float p = x2 + x * pc[i][0] + pc[i][1];
        float q = x2 + x * qc[i][0] + qc[i][1];
        prod *= p / q;
    }
    prod = 1.0f - prod * expf(-x2);
    return s * prod;
}

static float tanh_clamped(float x) {
    /* reference: elementwise_unary.comp:136-155 */
    const float ax = fabsf(x);
    if (x > 10.0f) return 1.0f;
    if (x < -10.0f) return -1.0f;
    if (ax < 0.2f) {
        const float x2 = x * x;
        return x * (1.0f - x2 * (1.0f / 3.0f - x2 * (2.0f / 15.0f - 17.0f / 315.0f * x2)));
    }
    return tanhf(x);
}

static float sin_hybrid(float x) {
    /* reference: elementwise_unary.comp:161-186 */
    if (fabsf(x) < 1.0e-3f) {
        const float c3 = -1.0f / 6.0f, c5 = 1.0f / 120.0f, c7 = -1.0f / 5040.0f, c9 = 1.0f / 362880.0f,
                    c11 = -1.0f / 39916800.0f;
        float x2 = x * x;
        float p = (c11 * x2 + c9) * x2 + c7;
        p = p * x2 + c5;
        p = p * x2 + c3;
        p = p * x2 + 1.0f;
        return x * p;
    }
    return sinf(x);
}

int mlel_cpu_elementwise_unary(int32_t op, const mlel_tensor *out, const mlel_tensor *in) {
    CHECK(out, "unary out");
    CHECK(in, "unary in");
    if (op < 0 || op >= MLEL_UN_COUNT) return fail(MLEL_ERR_INVALID, "unary: unknown op %d", op);
    const int64_t total = numel(out);
    const int dt = in->dtype;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        if (dt_is_float(dt)) {
            const double v = ld_f(in, o);
            double r = v;
            if (!isnan(v)) {
                const float vf = (float)v;
                switch (op) {
                case MLEL_UN_ABS: r = fabs(v); break;
                case MLEL_UN_CEIL: r = ceil(v); break;
                case MLEL_UN_FLOOR: r = floor(v); break;
                case MLEL_UN_COS: r = cos(v); break;
                case MLEL_UN_EXP: r = exp(v); break;
                case MLEL_UN_LOG: r = v < 0.0 ? NAN : log(v); break;
                case MLEL_UN_RECIPROCAL: r = 1.0 / v; break;
                case MLEL_UN_RSQRT: r = 1.0 / sqrt(v); break;
                case MLEL_UN_SIGMOID: r = 1.0 / (1.0 + exp(-v)); break;
                case MLEL_UN_SIN: r = (double)sin_hybrid(vf); break;
                case MLEL_UN_TANH: r = (double)tanh_clamped(vf); break;
                case MLEL_UN_ERF: r = (double)erf_ref(vf); break;
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
            case MLEL_UN_CLZ: {
                int i;
                for (i = 0; i < 32; i++)
                    if (((uint32_t)v >> (31 - i)) & 1u) break;
                r = i;
                break;
            }
            default: break;
            }
            st_i(out, o, r);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * REDUCE_* (reference: reduce.comp:24-70): sequential fold in the compute type
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_reduce(int32_t op, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t nan_mode) {
    CHECK(out, "reduce out");
    CHECK(in, "reduce in");
    if (op < 0 || op >= MLEL_RED_COUNT) return fail(MLEL_ERR_INVALID, "reduce: unknown op %d", op);
    if ((int)axis >= in->rank || in->rank != out->rank) return fail(MLEL_ERR_INVALID, "reduce: bad axis/rank");
    const int64_t total = numel(out);
    const int dt = in->dtype;
    const int isf = dt_is_float(dt);
    if (!isf) nan_mode = MLEL_NAN_PROPAGATE; /* reference: compute_graph_op.cpp:1674-1680 */
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        memcpy(ii, o, sizeof(ii));
        if (isf) {
            double lowest = dt_lowest_f(dt);
            double r;
            switch (op) {
            case MLEL_RED_MAX: r = nan_mode == MLEL_NAN_IGNORE ? NAN : lowest; break;
            case MLEL_RED_MIN: r = nan_mode == MLEL_NAN_IGNORE ? NAN : -lowest; break;
            case MLEL_RED_PRODUCT: r = 1.0; break;
            default: r = 0.0; break;
            }
            for (int64_t i = 0; i < in->dims[axis]; i++) {
                ii[axis] = i;
                const double v = ld_f(in, ii);
                if (isnan(v)) {
                    if (nan_mode == MLEL_NAN_IGNORE) continue;
                    if (nan_mode == MLEL_NAN_PROPAGATE) {
                        r = v;
                        break;
                    }
                }
                switch (op) {
                /* GLSL max(x,y) = (x < y) ? y : x; min(x,y) = (y < x) ? y : x.  A NaN accumulator (ignore-mode
                 * start value) therefore is replaced by the first real value only if the comparison is
                 * written the other way round; drivers differ here, so the first real value is taken. */
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
            for (int64_t i = 0; i < in->dims[axis]; i++) {
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
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * AVG_POOL2D (reference: avgpool2d.comp:27-75), MAX_POOL2D (reference: maxpool2d.comp:23-72)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_avg_pool2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_pool2d_attr *a) {
    CHECK(out, "avg_pool2d out");
    CHECK(in, "avg_pool2d in");
    if (out->rank != 4 || in->rank != 4) return fail(MLEL_ERR_INVALID, "avg_pool2d: rank must be 4");
    if (a->acc_type < 1 || a->acc_type > 4)
        return fail(MLEL_ERR_INVALID, "Unsupported AVG_POOL2D acc type %u", a->acc_type);
    const int64_t H = in->dims[1], W = in->dims[2];
    const int64_t total = numel(out);
    const int dt = out->dtype;
    const int isf = dt_is_float(dt);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[4];
        unflatten(out, flat, o);
        int64_t iacc = 0, count = 0;
        double dacc = 0.0;
        for (int64_t ky = 0; ky < a->kernel[0]; ky++) {
            for (int64_t kx = 0; kx < a->kernel[1]; kx++) {
                const int64_t yy = o[1] * a->stride[0] - a->pad[0] + ky;
                const int64_t xx = o[2] * a->stride[1] - a->pad[2] + kx;
                if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
                const int64_t xi[4] = {o[0], yy, xx, o[3]};
                if (!isf) {
                    iacc = a->acc_type == MLEL_ACC_I64 ? wadd64(iacc, ld_i(in, xi) - a->input_zp)
                                                       : (int64_t)wadd32((int32_t)iacc, (int32_t)(ld_i(in, xi) - a->input_zp));
                } else if (a->acc_type == MLEL_ACC_F16) {
                    dacc = rnd_f16(dacc + rnd_f16(rnd_f16(ld_f(in, xi)) - rnd_f16((double)a->input_zp)));
                } else {
                    dacc = rnd_f32(dacc + rnd_f32(ld_f(in, xi) - (double)a->input_zp));
                }
                count++;
            }
        }
        if (!isf) {
            /* divide with rounding half away from zero, truncating signed division; an empty window divides by
             * zero in the shader (undefined): written as 0 here */
            int64_t r = 0;
            if (count > 0) {
                const int64_t rnd = iacc < 0 ? -(count >> 1) : (count >> 1);
                r = (iacc + rnd) / count;
            }
            r += a->output_zp;
            if (r < dt_lowest(dt)) r = dt_lowest(dt);
            if (r > dt_max(dt)) r = dt_max(dt);
            st_i(out, o, r);
        } else {
            double r = a->acc_type == MLEL_ACC_F16 ? rnd_f16(dacc / (double)count) : rnd_f32(dacc / (double)count);
            st_f(out, o, r);
        }
    }
    return 0;
}

int mlel_cpu_max_pool2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_pool2d_attr *a) {
    CHECK(out, "max_pool2d out");
    CHECK(in, "max_pool2d in");
    if (out->rank != 4 || in->rank != 4) return fail(MLEL_ERR_INVALID, "max_pool2d: rank must be 4");
    const int64_t H = in->dims[1], W = in->dims[2];
    const int64_t total = numel(out);
    const int dt = out->dtype;
    const int isf = dt_is_float(dt);
    const int64_t kh = a->kernel[0] > 0 ? a->kernel[0] : 0, kw = a->kernel[1] > 0 ? a->kernel[1] : 0;
    const int64_t sy = a->stride[0] > 1 ? a->stride[0] : 1, sx = a->stride[1] > 1 ? a->stride[1] : 1;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[4];
        unflatten(out, flat, o);
        int64_t iacc = dt_lowest(dt);
        double dacc = dt_lowest_f(dt);
        if (isf && a->nan_mode == MLEL_NAN_IGNORE) dacc = NAN; /* reference: compute_graph_op.cpp:1490 */
        int done = 0;
        for (int64_t ky = 0; ky < kh && !done; ky++) {
            for (int64_t kx = 0; kx < kw; kx++) {
                const int64_t yy = o[1] * sy - a->pad[0] + ky;
                const int64_t xx = o[2] * sx - a->pad[2] + kx;
                if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;
                const int64_t xi[4] = {o[0], yy, xx, o[3]};
                if (!isf) {
                    const int64_t v = ld_i(in, xi);
                    iacc = iacc > v ? iacc : v;
                } else {
                    const double v = ld_f(in, xi);
                    if (isnan(v)) {
                        if (a->nan_mode == MLEL_NAN_IGNORE) continue;
                        dacc = v;
                        done = 1;
                        break;
                    }
                    dacc = isnan(dacc) ? v : (dacc < v ? v : dacc);
                }
            }
        }
        if (isf)
            st_f(out, o, dacc);
        else
            st_i(out, o, iacc);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * TABLE (reference: table.comp:17-52)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_table(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *table) {
    CHECK(out, "table out");
    CHECK(in, "table in");
    CHECK(table, "table table");
    if (in->dtype != MLEL_I8 && in->dtype != MLEL_I16) return fail(MLEL_ERR_UNSUPPORTED, "table: i8 or i16 input");
    if (table->dtype != in->dtype || table->rank != 1) return fail(MLEL_ERR_INVALID, "table: table type/rank");
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        const int64_t v = ld_i(in, o);
        int64_t r;
        if (in->dtype == MLEL_I8) {
            const int64_t ti[1] = {v + 128};
            r = ld_i(table, ti);
        } else {
            const int32_t index = ((int32_t)v + 32768) >> 7;
            const int32_t fraction = (int32_t)v & 0x7f;
            const int64_t t0[1] = {index}, t1[1] = {index + 1};
            const int32_t base = (int32_t)ld_i(table, t0), next = (int32_t)ld_i(table, t1);
            const int32_t slope = next - base;
            r = (int32_t)((uint32_t)base << 7) + slope * fraction;
        }
        st_i(out, o, r);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * CAST (reference: cast.comp:22-103)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_cast(const mlel_tensor *out, const mlel_tensor *in) {
    CHECK(out, "cast out");
    CHECK(in, "cast in");
    const int64_t total = numel(out);
    const int idt = in->dtype, odt = out->dtype;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        if (odt == MLEL_BOOL) {
            st_i(out, o, dt_is_float(idt) ? (ld_f(in, o) != 0.0) : (ld_i(in, o) != 0));
        } else if (dt_is_float(odt)) {
            /* to bf16: nearest even (cast.comp:36-46); to fp8: the fp32 value is encoded directly (:47-56) */
            const int mode = odt == MLEL_BF16 ? ST_RNE : ST_ACC;
            if (dt_is_float(idt)) {
                st_f_mode(out, o, ld_f(in, o), mode);
            } else {
                const int64_t v = ld_i(in, o);
                /* a wide integer going to a narrower float range saturates to +/-Inf */
                if (odt == MLEL_F16 && idt != MLEL_BOOL && idt != MLEL_I8 && idt != MLEL_U8 && idt != MLEL_I16) {
                    if (v > 65504) st_f(out, o, INFINITY);
                    else if (v < -65504) st_f(out, o, -INFINITY);
                    else st_f(out, o, (double)v);
                } else {
                    st_f_mode(out, o, (double)v, mode);
                }
            }
        } else {
            if (dt_is_float(idt)) {
                const float f = (float)ld_f(in, o);
                const float lo = (float)dt_lowest(odt), hi = (float)dt_max(odt);
                int64_t r;
                if (f <= lo) r = dt_lowest(odt);
                else if (f >= hi) r = dt_max(odt);
                else r = (int64_t)nearbyintf(f); /* roundEven: the default rounding mode */
                if (isnan(f)) r = 0;
                st_i(out, o, r);
            } else {
                st_i(out, o, ld_i(in, o)); /* truncating store */
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * NEGATE (reference: negate.comp:29-47)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_negate(const mlel_tensor *out, const mlel_tensor *in, int32_t input_zp, int32_t output_zp) {
    CHECK(out, "negate out");
    CHECK(in, "negate in");
    const int64_t total = numel(out);
    const int dt = out->dtype;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        if (dt_is_float(dt)) {
            const double v = ld_f(in, o);
            st_f(out, o, isnan(v) ? v : -v);
        } else {
            /* accumulate in int32 (int64 for 32-bit storage would need acc_t; the reference uses int32_t) */
            int64_t r = (int64_t)wadd32(wadd32(input_zp, (int32_t)-ld_i(in, o)), output_zp);
            if (r < dt_lowest(dt)) r = dt_lowest(dt);
            if (r > dt_max(dt)) r = dt_max(dt);
            st_i(out, o, r);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * data movement (reference: reshape.comp, transpose.comp, concat.comp, slice.comp, pad.comp)
 * ---------------------------------------------------------------------------------------------------------- */
static inline void copy_elem(const mlel_tensor *out, const int64_t *oi, const mlel_tensor *in, const int64_t *ii) {
    int64_t so, si;
    if (!elem_off(out, oi, &so)) return;
    uint64_t v = 0;
    if (elem_off(in, ii, &si)) memcpy(&v, (const char *)in->ptr + si, (size_t)dt_size(in->dtype));
    memcpy((char *)out->ptr + so, &v, (size_t)dt_size(out->dtype));
}

int mlel_cpu_reshape(const mlel_tensor *out, const mlel_tensor *in) {
    CHECK(out, "reshape out");
    CHECK(in, "reshape in");
    if (dt_size(out->dtype) != dt_size(in->dtype)) return fail(MLEL_ERR_INVALID, "reshape: element size differs");
    const int64_t total = numel(out), in_total = numel(in);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        if (flat >= in_total) continue; /* the invocation returns when the input index overflows */
        unflatten(out, flat, o);
        unflatten(in, flat, ii);
        copy_elem(out, o, in, ii);
    }
    return 0;
}

int mlel_cpu_transpose(const mlel_tensor *out, const mlel_tensor *in, const uint32_t *perms) {
    CHECK(out, "transpose out");
    CHECK(in, "transpose in");
    if (out->rank != in->rank) return fail(MLEL_ERR_INVALID, "transpose: ranks differ");
    for (int i = 0; i < out->rank; i++)
        if ((int)perms[i] >= out->rank) return fail(MLEL_ERR_INVALID, "transpose: bad perms");
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK] = {0};
        unflatten(out, flat, o);
        for (int i = 0; i < out->rank; i++) ii[perms[i]] = o[i];
        copy_elem(out, o, in, ii);
    }
    return 0;
}

int mlel_cpu_concat(const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t offset) {
    CHECK(out, "concat out");
    CHECK(in, "concat in");
    if (out->rank != in->rank || (int)axis >= in->rank) return fail(MLEL_ERR_INVALID, "concat: bad rank/axis");
    const int64_t total = numel(in);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t ii[MLEL_MAX_RANK], o[MLEL_MAX_RANK];
        unflatten(in, flat, ii);
        memcpy(o, ii, sizeof(o));
        o[axis] += offset;
        copy_elem(out, o, in, ii);
    }
    return 0;
}

int mlel_cpu_slice(const mlel_tensor *out, const mlel_tensor *in, const uint32_t *start) {
    CHECK(out, "slice out");
    CHECK(in, "slice in");
    if (out->rank != in->rank) return fail(MLEL_ERR_INVALID, "slice: ranks differ");
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        for (int i = 0; i < out->rank; i++) ii[i] = o[i] + start[i];
        copy_elem(out, o, in, ii);
    }
    return 0;
}

int mlel_cpu_pad(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *padding, double pad_const,
                 int32_t pad_const_int) {
    CHECK(out, "pad out");
    CHECK(in, "pad in");
    CHECK(padding, "pad padding");
    if (out->rank != in->rank) return fail(MLEL_ERR_INVALID, "pad: ranks differ");
    const int64_t total = numel(out);
    const int dt = out->dtype;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        int is_pad = 0;
        for (int i = 0; i < out->rank; i++) {
            const int64_t pi[1] = {2 * i};
            ii[i] = o[i] - ld_i(padding, pi);
            if (ii[i] < 0 || ii[i] >= in->dims[i]) {
                is_pad = 1;
                break;
            }
        }
        if (!is_pad) {
            copy_elem(out, o, in, ii);
        } else if (dt == MLEL_I32) {
            st_i(out, o, pad_const_int);
        } else if (dt_is_float(dt)) {
            st_f(out, o, pad_const);
        } else {
            st_i(out, o, (int64_t)pad_const);
        }
    }
    return 0;
}

/* ============================================================================================================
 * The remaining TOSA operators
 * ========================================================================================================== */

/* one multiply-accumulate of a convolution in the accumulator type (as in mlel_cpu_conv2d above) */
static inline void conv_mac(uint32_t acc_type, int64_t *iacc, double *dacc, const mlel_tensor *in, const int64_t *xi,
                            const mlel_tensor *w, const int64_t *wi, int32_t zi, int32_t zw) {
    if (!acc_is_float(acc_type)) {
        const int64_t v = ld_acc_i(in, xi) - zi;
        const int64_t ww = ld_acc_i(w, wi) - zw;
        if (acc_type == MLEL_ACC_I32)
            *iacc = wadd32((int32_t)*iacc, wmul32((int32_t)v, (int32_t)ww));
        else
            *iacc = wadd64(*iacc, wmul64(v, ww));
    } else {
        double v = ld_f(in, xi), ww = ld_f(w, wi);
        if (acc_type == MLEL_ACC_F16) {
            v = rnd_f16(v);
            ww = rnd_f16(ww);
        }
        const double p = rnd_f32(rnd_f32(v - (double)zi) * rnd_f32(ww - (double)zw));
        *dacc = acc_type == MLEL_ACC_F16 ? rnd_f16(*dacc + rnd_f16(p)) : rnd_f32(*dacc + p);
    }
}

static inline void conv_finish(uint32_t acc_type, int64_t iacc, double dacc, const mlel_tensor *bias, int64_t oc,
                               const mlel_tensor *out, const int64_t *o) {
    const int64_t bi[1] = {bias->dims[0] == 1 ? 0 : oc};
    if (!acc_is_float(acc_type)) {
        const int64_t b = ld_acc_i(bias, bi);
        st_acc_i(out, o, acc_type == MLEL_ACC_I32 ? (int64_t)wadd32((int32_t)iacc, (int32_t)b) : wadd64(iacc, b));
    } else {
        const double b = ld_f(bias, bi);
        st_f_mode(out, o, acc_type == MLEL_ACC_F16 ? rnd_f16(dacc + rnd_f16(b)) : rnd_f32(dacc + b), ST_ACC);
    }
}

/* ------------------------------------------------------------------------------------------------------------
 * CONV3D (reference: conv3d.comp:37-104): NDHWC input, ODHWI weights; taps outside the input contribute nothing
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_conv3d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w, const mlel_tensor *bias,
                    const mlel_conv3d_attr *a) {
    CHECK(out, "conv3d out");
    CHECK(in, "conv3d in");
    CHECK(w, "conv3d weights");
    CHECK(bias, "conv3d bias");
    if (out->rank != 5 || in->rank != 5 || w->rank != 5 || bias->rank != 1)
        return fail(MLEL_ERR_INVALID, "conv3d: ranks must be 5,5,5,1");
    if (a->acc_type < 1 || a->acc_type > 4) return fail(MLEL_ERR_INVALID, "Unsupported acc type %u", a->acc_type);
    const int64_t D = in->dims[1], H = in->dims[2], W = in->dims[3], IC = w->dims[4];
    const int64_t KD = w->dims[1], KH = w->dims[2], KW = w->dims[3];
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        int64_t iacc = 0;
        double dacc = 0.0;
        for (int64_t kd = 0; kd < KD; kd++) {
            const int64_t d = o[1] * a->stride[0] - a->pad[0] + kd * a->dilation[0];
            if (d < 0 || d >= D) continue;
            for (int64_t ky = 0; ky < KH; ky++) {
                const int64_t y = o[2] * a->stride[1] - a->pad[2] + ky * a->dilation[1];
                if (y < 0 || y >= H) continue;
                for (int64_t kx = 0; kx < KW; kx++) {
                    const int64_t x = o[3] * a->stride[2] - a->pad[4] + kx * a->dilation[2];
                    if (x < 0 || x >= W) continue;
                    for (int64_t ic = 0; ic < IC; ic++) {
                        const int64_t xi[5] = {o[0], d, y, x, ic};
                        const int64_t wi[5] = {o[4], kd, ky, kx, ic};
                        conv_mac(a->acc_type, &iacc, &dacc, in, xi, w, wi, a->input_zp, a->weight_zp);
                    }
                }
            }
        }
        conv_finish(a->acc_type, iacc, dacc, bias, o[4], out, o);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * TRANSPOSE_CONV2D (reference: transpose_conv2d.comp:31-70): output position oy receives input row iy through
 * kernel row ky when oy - out_pad_top - ky == iy * stride_y; the accumulator starts from the bias
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_transpose_conv2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                              const mlel_tensor *bias, const mlel_tconv2d_attr *a) {
    CHECK(out, "transpose_conv2d out");
    CHECK(in, "transpose_conv2d in");
    CHECK(w, "transpose_conv2d weights");
    CHECK(bias, "transpose_conv2d bias");
    if (out->rank != 4 || in->rank != 4 || w->rank != 4 || bias->rank != 1)
        return fail(MLEL_ERR_INVALID, "transpose_conv2d: ranks must be 4,4,4,1");
    if (a->acc_type < 1 || a->acc_type > 4) return fail(MLEL_ERR_INVALID, "Unsupported acc type %u", a->acc_type);
    if (a->stride[0] <= 0 || a->stride[1] <= 0) return fail(MLEL_ERR_INVALID, "transpose_conv2d: stride must be positive");
    const int64_t H = in->dims[1], W = in->dims[2], IC = in->dims[3], KH = w->dims[1], KW = w->dims[2];
    const int64_t total = numel(out);
    const int facc = acc_is_float(a->acc_type);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        const int64_t bi[1] = {bias->dims[0] == 1 ? 0 : o[3]};
        int64_t iacc = facc ? 0 : ld_acc_i(bias, bi);
        if (!facc && a->acc_type == MLEL_ACC_I32) iacc = (int32_t)iacc;
        double dacc = facc ? ld_f(bias, bi) : 0.0;
        if (a->acc_type == MLEL_ACC_F16) dacc = rnd_f16(dacc);
        for (int64_t ky = 0; ky < KH; ky++) {
            for (int64_t kx = 0; kx < KW; kx++) {
                int64_t iy = o[1] - a->out_pad[0] - ky, ix = o[2] - a->out_pad[2] - kx;
                if (iy % a->stride[0] != 0 || ix % a->stride[1] != 0) continue; /* C remainder, as in GLSL */
                iy /= a->stride[0];
                ix /= a->stride[1];
                if (iy < 0 || ix < 0 || iy >= H || ix >= W) continue;
                for (int64_t ic = 0; ic < IC; ic++) {
                    const int64_t xi[4] = {o[0], iy, ix, ic};
                    const int64_t wi[4] = {o[3], ky, kx, ic};
                    conv_mac(a->acc_type, &iacc, &dacc, in, xi, w, wi, a->input_zp, a->weight_zp);
                }
            }
        }
        if (!facc)
            st_acc_i(out, o, iacc);
        else
            st_f_mode(out, o, dacc, ST_ACC);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * ARGMAX (reference: argmax.comp:26-66): int32 output without the axis; the running maximum starts at the lowest
 * value of the type and only a strictly greater value replaces it, so the first maximum wins
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_argmax(const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t nan_mode) {
    CHECK(out, "argmax out");
    CHECK(in, "argmax in");
    if ((int)axis >= in->rank || out->rank != in->rank - 1) return fail(MLEL_ERR_INVALID, "argmax: bad axis or ranks");
    const int64_t total = numel(out), len = in->dims[axis];
    const int isf = dt_is_float(in->dtype);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        for (uint32_t i = 0; i < axis; i++) ii[i] = o[i];
        for (int i = (int)axis; i < out->rank; i++) ii[i + 1] = o[i];
        int64_t best = 0;
        if (isf) {
            /* the shader starts from the lowest FINITE value of the type, so a -inf input never wins */
            double mx = dt_lowest_f(in->dtype);
            for (int64_t i = 0; i < len; i++) {
                ii[axis] = i;
                const double v = ld_f(in, ii);
                if (isnan(v)) {
                    if (nan_mode == MLEL_NAN_IGNORE) continue;
                    best = i;
                    break;
                }
                if (v > mx) {
                    mx = v;
                    best = i;
                }
            }
        } else {
            int64_t mx = dt_lowest(in->dtype);
            for (int64_t i = 0; i < len; i++) {
                ii[axis] = i;
                const int64_t v = ld_i(in, ii);
                if (v > mx) {
                    mx = v;
                    best = i;
                }
            }
        }
        st_i(out, o, best);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * ARITHMETIC_RIGHT_SHIFT (reference: arithmetic_right_shift.comp:22-48)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_arithmetic_right_shift(const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2,
                                    uint32_t round) {
    CHECK(out, "arithmetic_right_shift out");
    CHECK(in1, "arithmetic_right_shift in1");
    CHECK(in2, "arithmetic_right_shift in2");
    if (!dt_is_int(out->dtype)) return fail(MLEL_ERR_INVALID, "arithmetic_right_shift: integer types only");
    const int64_t total = numel(out);
    const int bits = 8 * dt_size(out->dtype);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], a[MLEL_MAX_RANK], b[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        broadcast_idx(in1, o, a);
        broadcast_idx(in2, o, b);
        const int64_t v = ld_i(in1, a), s = ld_i(in2, b);
        const int sh = (int)(s & (bits - 1)); /* shift counts are taken modulo the width on every target tested */
        int64_t r = asr64(v, sh);
        if (round && s > 0 && ((asr64(v, (int)((s - 1) & (bits - 1))) & 1) != 0)) r++;
        st_i(out, o, narrow_to(out->dtype, r));
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * GATHER / SCATTER (reference: gather.comp:13-25, scatter.comp:14-34)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_gather(const mlel_tensor *out, const mlel_tensor *values, const mlel_tensor *indices) {
    CHECK(out, "gather out");
    CHECK(values, "gather values");
    CHECK(indices, "gather indices");
    if (out->rank != 3 || values->rank != 3 || indices->rank != 2) return fail(MLEL_ERR_INVALID, "gather: ranks must be 3,3,2");
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        const int64_t xi[2] = {o[0], o[1]};
        const int64_t k = (int64_t)(uint32_t)ld_i(indices, xi);
        const int64_t vi[3] = {o[0], k, o[2]};
        copy_elem(out, o, values, vi);
    }
    return 0;
}

int mlel_cpu_scatter(const mlel_tensor *out, const mlel_tensor *values_in, const mlel_tensor *indices,
                     const mlel_tensor *input) {
    CHECK(out, "scatter out");
    CHECK(values_in, "scatter values_in");
    CHECK(indices, "scatter indices");
    CHECK(input, "scatter input");
    if (out->rank != 3 || values_in->rank != 3 || indices->rank != 2 || input->rank != 3)
        return fail(MLEL_ERR_INVALID, "scatter: ranks must be 3,3,2,3");
    const int64_t total = numel(out), W = indices->dims[1];
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        int64_t w_hit = -1;
        for (int64_t wv = 0; wv < W && w_hit < 0; wv++) {
            const int64_t xi[2] = {o[0], wv};
            if ((int64_t)(uint32_t)ld_i(indices, xi) == o[1]) w_hit = wv; /* the first matching row wins */
        }
        if (w_hit < 0) {
            copy_elem(out, o, values_in, o);
        } else {
            const int64_t ii[3] = {o[0], w_hit, o[2]};
            copy_elem(out, o, input, ii);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * REVERSE / TILE / SELECT (reference: reverse.comp:14-30, tile.comp:12-30, select.comp:15-41)
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_reverse(const mlel_tensor *out, const mlel_tensor *in, uint32_t axis) {
    CHECK(out, "reverse out");
    CHECK(in, "reverse in");
    if (out->rank != in->rank || (int)axis >= out->rank) return fail(MLEL_ERR_INVALID, "reverse: bad rank or axis");
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        unflatten(out, flat, ii); /* the shader walks the output grid, reads the input there and writes mirrored */
        for (int i = 0; i < out->rank; i++) o[i] = ii[i];
        o[axis] = out->dims[axis] - 1 - ii[axis];
        copy_elem(out, o, in, ii);
    }
    return 0;
}

int mlel_cpu_tile(const mlel_tensor *out, const mlel_tensor *in) {
    CHECK(out, "tile out");
    CHECK(in, "tile in");
    if (out->rank != in->rank) return fail(MLEL_ERR_INVALID, "tile: ranks differ");
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        for (int i = 0; i < out->rank; i++) ii[i] = o[i] % in->dims[i];
        copy_elem(out, o, in, ii);
    }
    return 0;
}

int mlel_cpu_select(const mlel_tensor *out, const mlel_tensor *condition, const mlel_tensor *in_true,
                    const mlel_tensor *in_false) {
    CHECK(out, "select out");
    CHECK(condition, "select condition");
    CHECK(in_true, "select in_true");
    CHECK(in_false, "select in_false");
    const int64_t total = numel(out);
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK], c[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        broadcast_idx(condition, o, c);
        const mlel_tensor *src = ld_i(condition, c) != 0 ? in_true : in_false;
        broadcast_idx(src, o, ii);
        copy_elem(out, o, src, ii);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * RESIZE (reference: resize.comp:57-134).  Coordinates are computed in int32 and narrowed to int16 exactly where
 * the shader narrows them; integer types interpolate with integer weights (unit = scale numerator), floats with
 * weights in [0, 1].
 * ---------------------------------------------------------------------------------------------------------- */
static inline int32_t idiv_floor(int32_t n, int32_t d) {
    int32_t r = n / d;
    if ((int64_t)r * d > n) r--;
    return r;
}

int mlel_cpu_resize(const mlel_tensor *out, const mlel_tensor *in, const mlel_resize_attr *a) {
    CHECK(out, "resize out");
    CHECK(in, "resize in");
    if (out->rank != 4 || in->rank != 4) return fail(MLEL_ERR_INVALID, "resize: ranks must be 4");
    if (a->scale[0] <= 0 || a->scale[2] <= 0) return fail(MLEL_ERR_INVALID, "resize: scale numerators must be positive");
    if (a->mode != MLEL_RESIZE_NEAREST && a->mode != MLEL_RESIZE_BILINEAR) return fail(MLEL_ERR_INVALID, "resize: bad mode");
    const int64_t total = numel(out);
    const int isf = dt_is_float(out->dtype);
    const int32_t yn = a->scale[0], yd = a->scale[1], xn = a->scale[2], xd = a->scale[3];
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out, flat, o);
        const int32_t y = (int32_t)((uint32_t)o[1] * (uint32_t)yd + (uint32_t)a->offset[0]);
        const int16_t iy = (int16_t)idiv_floor(y, yn);
        const int16_t ry = (int16_t)(y - iy * yn);
        const int32_t x = (int32_t)((uint32_t)o[2] * (uint32_t)xd + (uint32_t)a->offset[1]);
        const int16_t ix = (int16_t)idiv_floor(x, xn);
        const int16_t rx = (int16_t)(x - ix * xn);
        const int16_t iy0 = (int16_t)(iy > 0 ? iy : 0);
        const int16_t ix0 = (int16_t)(ix > 0 ? ix : 0);
        /* min(iy + 1, H - 1) is evaluated in unsigned arithmetic in the shader (the shape is unsigned) */
        const uint32_t uy1 = (uint32_t)(int32_t)(iy + 1), ux1 = (uint32_t)(int32_t)(ix + 1);
        const uint32_t hy = (uint32_t)in->dims[1] - 1u, hx = (uint32_t)in->dims[2] - 1u;
        const int16_t iy1 = (int16_t)(uy1 < hy ? uy1 : hy), ix1 = (int16_t)(ux1 < hx ? ux1 : hx);
        const int64_t p00[4] = {o[0], iy0, ix0, o[3]}, p01[4] = {o[0], iy0, ix1, o[3]};
        const int64_t p10[4] = {o[0], iy1, ix0, o[3]}, p11[4] = {o[0], iy1, ix1, o[3]};
        if (isf) {
            const int dt = out->dtype;
            const double dy = round_to(dt, round_to(dt, (double)ry) / round_to(dt, (double)yn));
            const double dx = round_to(dt, round_to(dt, (double)rx) / round_to(dt, (double)xn));
            double acc;
            if (a->mode == MLEL_RESIZE_BILINEAR) {
                const double wy0 = round_to(dt, 1.0 - dy), wx0 = round_to(dt, 1.0 - dx);
                acc = round_to(dt, round_to(dt, round_to(dt, ld_f(in, p00)) * wy0) * wx0);
                acc = round_to(dt, acc + round_to(dt, round_to(dt, round_to(dt, ld_f(in, p01)) * wy0) * dx));
                acc = round_to(dt, acc + round_to(dt, round_to(dt, round_to(dt, ld_f(in, p10)) * dy) * wx0));
                acc = round_to(dt, acc + round_to(dt, round_to(dt, round_to(dt, ld_f(in, p11)) * dy) * dx));
            } else {
                const int64_t p[4] = {o[0], dy >= 0.5 ? iy1 : iy0, dx >= 0.5 ? ix1 : ix0, o[3]};
                acc = ld_f(in, p);
            }
            st_f(out, o, acc);
        } else {
            /* the computation type is that of the output (int32 for int8 data, int64 for int16 data) */
            const int wide = dt_size(out->dtype) == 8;
            int64_t acc;
            if (a->mode == MLEL_RESIZE_BILINEAR) {
                const int64_t wy1 = ry, wx1 = rx, wy0 = (int16_t)(yn) - ry, wx0 = (int16_t)(xn) - rx;
                const int64_t v[4] = {ld_i(in, p00), ld_i(in, p01), ld_i(in, p10), ld_i(in, p11)};
                const int64_t wy[4] = {wy0, wy0, wy1, wy1}, wx[4] = {wx0, wx1, wx0, wx1};
                acc = 0;
                for (int t = 0; t < 4; t++) {
                    if (wide)
                        acc = wadd64(acc, wmul64(wmul64(v[t], wy[t]), wx[t]));
                    else
                        acc = wadd32((int32_t)acc, wmul32(wmul32((int32_t)v[t], (int32_t)wy[t]), (int32_t)wx[t]));
                }
            } else {
                const int64_t p[4] = {o[0], 2 * (int32_t)ry >= yn ? iy1 : iy0, 2 * (int32_t)rx >= xn ? ix1 : ix0, o[3]};
                acc = ld_i(in, p);
            }
            st_i(out, o, narrow_to(out->dtype, acc));
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * FFT2D / RFFT2D (reference: fft2d.comp:17-52, rfft2d.comp:13-71): the transform sums evaluated directly.  The
 * reference's sine and cosine come from the Vulkan driver; here they are the C library's, so results agree with
 * the reference to rounding, not bit for bit (parity unpinned beyond the transform's mathematics).
 * ---------------------------------------------------------------------------------------------------------- */
int mlel_cpu_fft2d(const mlel_tensor *out_real, const mlel_tensor *out_imag, const mlel_tensor *in_real,
                   const mlel_tensor *in_imag, int32_t inverse) {
    CHECK(out_real, "fft2d out_real");
    CHECK(out_imag, "fft2d out_imag");
    CHECK(in_real, "fft2d in_real");
    CHECK(in_imag, "fft2d in_imag");
    if (out_real->rank != 3 || out_imag->rank != 3 || in_real->rank != 3 || in_imag->rank != 3)
        return fail(MLEL_ERR_INVALID, "fft2d: ranks must be 3");
    const int64_t total = numel(out_real), H = out_real->dims[1], W = out_real->dims[2];
    const float sign = inverse ? -1.0f : 1.0f;
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out_real, flat, o);
        double sr = 0.0, si = 0.0;
        for (int64_t iy = 0; iy < H; iy++) {
            for (int64_t ix = 0; ix < W; ix++) {
                const int64_t ii[3] = {o[0], iy, ix};
                const float re = (float)ld_f(in_real, ii), im = (float)ld_f(in_imag, ii);
                /* angle in fp32 as in the shader: sign * 2 pi * (float(iy * oy) / H + float(ix) * ox / W) */
                const float frac = (float)(uint32_t)(iy * o[1]) / (float)H + ((float)ix * (float)o[2]) / (float)W;
                const float angle = sign * 2.0f * 3.14159265358979323846f * frac;
                const float c = cosf(angle), s = sinf(angle);
                sr += (double)(re * c) + (double)(im * s);
                si += (double)(-(re * s)) + (double)(im * c);
            }
        }
        st_f(out_real, o, (double)(float)sr);
        st_f(out_imag, o, (double)(float)si);
    }
    return 0;
}

int mlel_cpu_rfft2d(const mlel_tensor *out_real, const mlel_tensor *out_imag, const mlel_tensor *in) {
    CHECK(out_real, "rfft2d out_real");
    CHECK(out_imag, "rfft2d out_imag");
    CHECK(in, "rfft2d in");
    if (out_real->rank != 3 || out_imag->rank != 3 || in->rank != 3) return fail(MLEL_ERR_INVALID, "rfft2d: ranks must be 3");
    const int64_t total = numel(out_real), H = in->dims[1], W = in->dims[2];
#pragma omp parallel for schedule(static)
    for (int64_t flat = 0; flat < total; flat++) {
        int64_t o[MLEL_MAX_RANK];
        unflatten(out_real, flat, o);
        const int64_t oy = o[1], ox = o[2];
        /* purely real bins: the imaginary part is left at exactly zero */
        const int skip_imag = (oy == 0 || oy == H / 2) && (ox == 0 || ox == W / 2);
        double sr = 0.0, si = 0.0;
        for (int64_t iy = 0; iy < H; iy++) {
            for (int64_t ix = 0; ix < W; ix++) {
                const int64_t ii[3] = {o[0], iy, ix};
                const double v = ld_f(in, ii);
                /* the angle numerator is reduced modulo W * H before the division, as in the shader */
                const double num = fmod((double)(iy * oy * W + ix * ox * H), (double)(W * H));
                const double angle = 2.0 * 3.14159265358979323846 * num / (double)(W * H);
                sr += v * cos(angle);
                if (!skip_imag) si -= v * sin(angle);
            }
        }
        st_f(out_real, o, (double)(float)sr);
        st_f(out_imag, o, (double)(float)si);
    }
    return 0;
}
