// Context, device arena, streams, events, HIP-graph capture and the calibration copy kernel of the C ABI
// declared in include/mlel_hip.h.
#include "common.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace mlel {

static thread_local char g_error[1024] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(MLEL_ERR_DEVICE, "%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

int check_tensor(const mlel_tensor *t, const char *what) {
    MLEL_REQUIRE(t != nullptr, MLEL_ERR_INVALID, "%s: null tensor", what);
    MLEL_REQUIRE(t->rank >= 1 && t->rank <= MLEL_MAX_RANK, MLEL_ERR_INVALID, "%s: rank %d outside 1..6", what,
                 t->rank);
    MLEL_REQUIRE(dt_size(t->dtype) != 0, MLEL_ERR_INVALID, "%s: unknown dtype %d", what, t->dtype);
    int64_t n = 1;
    for (int i = 0; i < t->rank; i++) {
        MLEL_REQUIRE(t->dims[i] >= 0, MLEL_ERR_INVALID, "%s: negative dimension", what);
        MLEL_REQUIRE(t->strides[i] >= 0, MLEL_ERR_INVALID, "Strides must be greater than zero.");
        n *= t->dims[i];
    }
    MLEL_REQUIRE(t->ptr != nullptr || n == 0, MLEL_ERR_INVALID, "%s: null data pointer", what);
    return 0;
}

int64_t numel(const mlel_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->rank; i++) n *= t->dims[i];
    return n;
}

bool is_packed(const mlel_tensor *t) {
    int64_t s = dt_size(t->dtype);
    for (int i = t->rank - 1; i >= 0; i--) {
        if (t->dims[i] != 1 && t->strides[i] != s) return false;
        s *= t->dims[i];
    }
    return true;
}

bool same_shape(const mlel_tensor *a, const mlel_tensor *b) {
    if (a->rank != b->rank) return false;
    for (int i = 0; i < a->rank; i++)
        if (a->dims[i] != b->dims[i]) return false;
    return true;
}

int make_rescale_params(const mlel_rescale_attr *attr, int in_dtype, int out_dtype, const mlel_clamp_attr *clamp,
                        RescaleParams *out) {
    MLEL_REQUIRE(dt_is_int(in_dtype) && dt_is_int(out_dtype), MLEL_ERR_INVALID, "rescale: integer types only");
    const int in_dt = dt_unsigned_twin(in_dtype, attr->input_unsigned != 0);
    const int out_dt = dt_unsigned_twin(out_dtype, attr->output_unsigned != 0);
    out->in_zp = (int32_t)narrow_to(in_dt, attr->input_zp);
    out->out_zp = (int32_t)narrow_to(out_dt, attr->output_zp);
    out->double_round = (attr->scale32 && attr->double_round) ? 1 : 0;
    out->per_channel = attr->per_channel ? 1 : 0;
    out->clamp_out = (dt_size(out_dt) < 4) ? 1 : 0;
    int64_t lo = dt_lowest(out_dt), hi = dt_max(out_dt);
    if (dt_size(out_dt) >= 4) {
        lo = INT32_MIN;
        hi = INT32_MAX;
    }
    if (clamp != nullptr) {
        // CLAMP on the narrowed value: clamp(clamp(x, lo, hi), cmin, cmax) == clamp(x, clamp(lo), clamp(hi)).
        // The bounds are converted to the storage type by truncation toward zero (clamp.comp:32-33).
        const int cl_dt = out_dtype;
        int64_t cmin = narrow_to(cl_dt, (int64_t)clamp->min_val);
        int64_t cmax = narrow_to(cl_dt, (int64_t)clamp->max_val);
        MLEL_REQUIRE(cmin <= cmax, MLEL_ERR_INVALID, "clamp: min %lld > max %lld", (long long)cmin, (long long)cmax);
        MLEL_REQUIRE(!attr->output_unsigned, MLEL_ERR_UNSUPPORTED, "fused clamp on an unsigned rescale output");
        auto cl = [&](int64_t v) { return v < cmin ? cmin : (v > cmax ? cmax : v); };
        lo = cl(lo);
        hi = cl(hi);
        out->clamp_out = 1;
    }
    out->out_lo = (int32_t)lo;
    out->out_hi = (int32_t)hi;
    return 0;
}

int check_scale_tensors(const mlel_tensor *mult, const mlel_tensor *shift, const mlel_rescale_attr *attr,
                        int64_t channels) {
    MLEL_TRY(check_tensor(mult, "rescale multiplier"));
    MLEL_TRY(check_tensor(shift, "rescale shift"));
    MLEL_REQUIRE(mult->rank == 1 && shift->rank == 1, MLEL_ERR_INVALID, "rescale: multiplier/shift must be rank 1");
    MLEL_REQUIRE(mult->dtype == (attr->scale32 ? MLEL_I32 : MLEL_I16), MLEL_ERR_INVALID,
                 "rescale: multiplier must be %s", attr->scale32 ? "int32 (scale32)" : "int16");
    MLEL_REQUIRE(shift->dtype == MLEL_I8, MLEL_ERR_INVALID, "rescale: shift must be int8");
    const int64_t need = attr->per_channel ? channels : 1;
    MLEL_REQUIRE(mult->dims[0] >= need && shift->dims[0] >= need, MLEL_ERR_INVALID,
                 "rescale: multiplier/shift shorter than %lld channels", (long long)need);
    return 0;
}

// 128-bit device-to-device copy; tail handled bytewise.
__global__ void __launch_bounds__(256) copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src,
                                                   size_t n_vec, char *__restrict__ dst_tail,
                                                   const char *__restrict__ src_tail, size_t n_tail) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride) dst[i] = src[i];
    if (blockIdx.x == 0 && threadIdx.x < n_tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}

// The copy kernel's launch geometry as parameters, for the measurement of the HBM ceiling: U 16-byte pieces in flight
// per thread (all loads issued before the first store), temporal or non-temporal accesses, any grid; MODE 1 only
// reads (the sum keeps the loads alive, one conditional store that never happens), MODE 2 only writes.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int U, bool NT, int MODE>
__global__ void __launch_bounds__(256) copy_variant_kernel(uint4 *__restrict__ dst_, const uint4 *__restrict__ src_,
                                                           size_t n_vec) {
    u32x4 *__restrict__ dst = reinterpret_cast<u32x4 *>(dst_);
    const u32x4 *__restrict__ src = reinterpret_cast<const u32x4 *>(src_);
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const u32x4 fill = {1u, 2u, 3u, 4u};
    uint32_t acc = 0;
    for (; i + (U - 1) * stride < n_vec; i += U * stride) {
        u32x4 v[U];
        if (MODE != 2) {
#pragma unroll
            for (int u = 0; u < U; u++)
                v[u] = NT ? __builtin_nontemporal_load(&src[i + u * stride]) : src[i + u * stride];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (MODE == 1) {
                acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
            } else {
                const u32x4 w = MODE == 2 ? fill : v[u];
                if (NT)
                    __builtin_nontemporal_store(w, &dst[i + u * stride]);
                else
                    dst[i + u * stride] = w;
            }
        }
    }
    for (; i < n_vec; i += stride) {
        if (MODE == 1) {
            acc += src[i].x;
        } else {
            dst[i] = MODE == 2 ? fill : src[i];
        }
    }
    if (MODE == 1 && acc == 0x9e3779b9u && n_vec == 1) dst[0].x = acc;
}

template <int U, bool NT>
void launch_copy_variant(int mode, unsigned blocks, hipStream_t s, uint4 *dst, const uint4 *src, size_t n_vec) {
    if (mode == 1)
        hipLaunchKernelGGL((copy_variant_kernel<U, NT, 1>), dim3(blocks), dim3(256), 0, s, dst, src, n_vec);
    else if (mode == 2)
        hipLaunchKernelGGL((copy_variant_kernel<U, NT, 2>), dim3(blocks), dim3(256), 0, s, dst, src, n_vec);
    else
        hipLaunchKernelGGL((copy_variant_kernel<U, NT, 0>), dim3(blocks), dim3(256), 0, s, dst, src, n_vec);
}

// The matrix cores on their own: every wavefront keeps eight independent 32 x 32 int8 accumulator tiles going from
// operands that sit in registers (loaded once from `operands`: zeros, or random bytes -- the rate this part sustains
// depends on how many bits toggle), `iters` rounds of eight v_mfma_i32_32x32x32_i8, then one store per lane so that
// nothing is optimised away.  What a contraction kernel could reach if operand delivery cost nothing.
typedef int v4i_probe __attribute__((ext_vector_type(4)));
typedef int v16i_probe __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(256) mfma_rate_kernel(const v4i_probe *__restrict__ operands, int32_t *__restrict__ out,
                                                        int iters) {
    const int tid = threadIdx.x + blockIdx.x * 256;
    v4i_probe a[2], b[4];
#pragma unroll
    for (int i = 0; i < 2; i++) a[i] = operands[(tid * 6 + i) & 4095];
#pragma unroll
    for (int j = 0; j < 4; j++) b[j] = operands[(tid * 6 + 2 + j) & 4095];
    v16i_probe acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    int32_t sum = 0;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) sum += acc[i][j][r];
    out[tid] = sum;
}

// What a wavefront that is alone on its SIMD can issue while its matrix instructions run: one round of `MODE` per
// iteration, written as inline assembly so that the order is the order below; the first wavefront of block 0 reports
// the clocks it took (s_memtime) per iteration.  The modes are the pieces of a contraction loop: four
// v_mfma_i32_32x32x32_i8; sixteen v_dot4 / v_add_u32 / v_sad_u8 (zero-point sums); six 128-bit reads of shared memory;
// four 16-byte-per-lane loads into shared memory; four v_mfma_i32_16x16x64_i8 -- each alone, behind the four matrix
// instructions, and dealt out between them.
#define MLEL_PROBE_MF(a, x, w) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(a) : "v"(x), "v"(w))
#define MLEL_PROBE_MS(a, x, w) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(a) : "v"(x), "v"(w))
#define MLEL_PROBE_DOT(s, x) asm volatile("v_dot4c_i32_i8 %0, %1, %2" : "+v"(s) : "v"(ones), "v"(x))
#define MLEL_PROBE_ADD(s, x) asm volatile("v_add_u32 %0, %0, %1" : "+v"(s) : "v"(x))
#define MLEL_PROBE_SAD(s, x) asm volatile("v_sad_u8 %0, %1, 0, %0" : "+v"(s) : "v"(x))
#define MLEL_PROBE_READ(d, p, off) asm volatile("ds_read_b128 %0, %1 offset:" #off : "=v"(d) : "v"(p))
#define MLEL_PROBE_LOAD(off)                                                                                      \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_wave + off), "v"(goff), \
                 "s"(rs)                                                                                          \
                 : "memory")
template <int MODE>
__global__ void __launch_bounds__(256) issue_probe_kernel(const int32_t *__restrict__ operands, uint32_t *__restrict__ out,
                                                          int iters) {
    __shared__ __align__(16) char lds[32768];
    v16i_probe a0, a1, a2, a3;
#pragma unroll
    for (int r = 0; r < 16; r++) a0[r] = a1[r] = a2[r] = a3[r] = 0;
    const int t = threadIdx.x;
    v4i_probe x0, x1, w0, w1, m0 = {0, 0, 0, 0}, m1 = {0, 0, 0, 0}, m2 = {0, 0, 0, 0}, m3 = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 4; e++) {
        x0[e] = operands[(t * 16 + e) & 16383];
        x1[e] = operands[(t * 16 + 4 + e) & 16383];
        w0[e] = operands[(t * 16 + 8 + e) & 16383];
        w1[e] = operands[(t * 16 + 12 + e) & 16383];
    }
    int s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    const int ones = 0x01010101;
    const uint32_t p = (uint32_t)(t * 16);
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
        (uint32_t) reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char *)lds) + (uint32_t)(t >> 6) * 4096u);
    const uint32_t goff = (uint32_t)(t & 63) * 16u + (uint32_t)(blockIdx.x & 15) * 4096u;
    const uint64_t ga = reinterpret_cast<uint64_t>(operands);
    const v4i_probe rs = {(int)(uint32_t)ga, (int)(uint32_t)(ga >> 32), 65536, 0x00020000};
    v4i_probe d0 = x0, d1 = x0, d2 = x0, d3 = x0, d4 = x0, d5 = x0;
    for (int i = t; i < 8192; i += 256) reinterpret_cast<int *>(lds)[i] = i;
    __syncthreads();
    const uint64_t t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; it++) {
        if (MODE == 0) { MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_MF(a3, x1, w1); }
        if (MODE == 1 || MODE == 2) {
            if (MODE == 2) { MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_MF(a3, x1, w1); }
#pragma unroll
            for (int e = 0; e < 4; e++) { MLEL_PROBE_DOT(s0, x0[e]); MLEL_PROBE_DOT(s1, x1[e]); MLEL_PROBE_DOT(s2, w0[e]); MLEL_PROBE_DOT(s3, w1[e]); }
        }
        if (MODE == 3) {
            MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_DOT(s0, x0[0]); MLEL_PROBE_DOT(s1, x1[0]); MLEL_PROBE_DOT(s2, w0[0]); MLEL_PROBE_DOT(s3, w1[0]);
            MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_DOT(s0, x0[1]); MLEL_PROBE_DOT(s1, x1[1]); MLEL_PROBE_DOT(s2, w0[1]); MLEL_PROBE_DOT(s3, w1[1]);
            MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_DOT(s0, x0[2]); MLEL_PROBE_DOT(s1, x1[2]); MLEL_PROBE_DOT(s2, w0[2]); MLEL_PROBE_DOT(s3, w1[2]);
            MLEL_PROBE_MF(a3, x1, w1); MLEL_PROBE_DOT(s0, x0[3]); MLEL_PROBE_DOT(s1, x1[3]); MLEL_PROBE_DOT(s2, w0[3]); MLEL_PROBE_DOT(s3, w1[3]);
        }
        if (MODE == 4 || MODE == 5) {
            if (MODE == 5) { MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_MF(a3, x1, w1); }
#pragma unroll
            for (int e = 0; e < 4; e++) { MLEL_PROBE_ADD(s0, x0[e]); MLEL_PROBE_ADD(s1, x1[e]); MLEL_PROBE_ADD(s2, w0[e]); MLEL_PROBE_ADD(s3, w1[e]); }
        }
        if (MODE == 6) {
            MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_ADD(s0, x0[0]); MLEL_PROBE_ADD(s1, x1[0]); MLEL_PROBE_ADD(s2, w0[0]); MLEL_PROBE_ADD(s3, w1[0]);
            MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_ADD(s0, x0[1]); MLEL_PROBE_ADD(s1, x1[1]); MLEL_PROBE_ADD(s2, w0[1]); MLEL_PROBE_ADD(s3, w1[1]);
            MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_ADD(s0, x0[2]); MLEL_PROBE_ADD(s1, x1[2]); MLEL_PROBE_ADD(s2, w0[2]); MLEL_PROBE_ADD(s3, w1[2]);
            MLEL_PROBE_MF(a3, x1, w1); MLEL_PROBE_ADD(s0, x0[3]); MLEL_PROBE_ADD(s1, x1[3]); MLEL_PROBE_ADD(s2, w0[3]); MLEL_PROBE_ADD(s3, w1[3]);
        }
        if (MODE == 7) {
            MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_SAD(s0, x0[0]); MLEL_PROBE_SAD(s1, x1[0]); MLEL_PROBE_SAD(s2, w0[0]); MLEL_PROBE_SAD(s3, w1[0]);
            MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_SAD(s0, x0[1]); MLEL_PROBE_SAD(s1, x1[1]); MLEL_PROBE_SAD(s2, w0[1]); MLEL_PROBE_SAD(s3, w1[1]);
            MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_SAD(s0, x0[2]); MLEL_PROBE_SAD(s1, x1[2]); MLEL_PROBE_SAD(s2, w0[2]); MLEL_PROBE_SAD(s3, w1[2]);
            MLEL_PROBE_MF(a3, x1, w1); MLEL_PROBE_SAD(s0, x0[3]); MLEL_PROBE_SAD(s1, x1[3]); MLEL_PROBE_SAD(s2, w0[3]); MLEL_PROBE_SAD(s3, w1[3]);
        }
        if (MODE == 8 || MODE == 9) {
            if (MODE == 9) { MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_MF(a3, x1, w1); }
            MLEL_PROBE_READ(d0, p, 0); MLEL_PROBE_READ(d1, p, 4096); MLEL_PROBE_READ(d2, p, 8192);
            MLEL_PROBE_READ(d3, p, 12288); MLEL_PROBE_READ(d4, p, 16384); MLEL_PROBE_READ(d5, p, 20480);
            asm volatile("s_waitcnt lgkmcnt(0)");
        }
        if (MODE == 10) {
            MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_READ(d0, p, 0); MLEL_PROBE_READ(d1, p, 4096);
            MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_READ(d2, p, 8192); MLEL_PROBE_READ(d3, p, 12288);
            MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_READ(d4, p, 16384); MLEL_PROBE_READ(d5, p, 20480);
            MLEL_PROBE_MF(a3, x1, w1);
            asm volatile("s_waitcnt lgkmcnt(0)");
        }
        if (MODE == 11 || MODE == 12) {
            if (MODE == 12) { MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_MF(a3, x1, w1); }
            MLEL_PROBE_LOAD(0); MLEL_PROBE_LOAD(1024); MLEL_PROBE_LOAD(2048); MLEL_PROBE_LOAD(3072);
            asm volatile("s_waitcnt vmcnt(4)");
        }
        if (MODE == 13) {
            MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_LOAD(0); MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_LOAD(1024);
            MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_LOAD(2048); MLEL_PROBE_MF(a3, x1, w1); MLEL_PROBE_LOAD(3072);
            asm volatile("s_waitcnt vmcnt(4)");
        }
        if (MODE == 14) {
            MLEL_PROBE_MF(a0, x0, w0); MLEL_PROBE_MS(m0, x0, w0); MLEL_PROBE_MF(a1, x0, w1); MLEL_PROBE_MS(m1, x1, w0);
            MLEL_PROBE_MF(a2, x1, w0); MLEL_PROBE_MS(m2, w0, x0); MLEL_PROBE_MF(a3, x1, w1); MLEL_PROBE_MS(m3, w1, x0);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)");
    const uint64_t t1 = __builtin_readcyclecounter();
    int sum = s0 + s1 + s2 + s3 + d0[0] + d1[1] + d2[2] + d3[3] + d4[0] + d5[1] + m0[0] + m1[1] + m2[2] + m3[3];
#pragma unroll
    for (int r = 0; r < 16; r++) sum += a0[r] + a1[r] + a2[r] + a3[r];
    out[2 + blockIdx.x * 256 + t] = (uint32_t)sum;
    if (t == 0 && blockIdx.x == 0) {
        out[0] = (uint32_t)(t1 - t0);
        out[1] = (uint32_t)((t1 - t0) >> 32);
    }
}

// Byte fill for streams under capture, where a memset node must not be recorded: 16-byte stores over the aligned
// middle, single bytes at the two ragged ends.
__global__ void __launch_bounds__(256) fill_kernel(unsigned char *__restrict__ dst, size_t head, size_t n_vec,
                                                   size_t tail, uint32_t word) {
    uint4 *mid = reinterpret_cast<uint4 *>(dst + head);
    const uint4 v = make_uint4(word, word, word, word);
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride) mid[i] = v;
    if (blockIdx.x == 0) {
        if (threadIdx.x < head) dst[threadIdx.x] = (unsigned char)word;
        if (threadIdx.x < tail) dst[head + n_vec * 16 + threadIdx.x] = (unsigned char)word;
    }
}

bool stream_is_capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

bool split_workspace(mlel_ctx *ctx, hipStream_t stream, SplitWorkspace *out) {
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    for (int i = 0; i < ctx->n_ws; i++)
        if (ctx->ws[i].stream == stream) {
            *out = ctx->ws[i];
            return true;
        }
    // a new workspace is an allocation: not inside a capture, and not beyond the table
    if (ctx->n_ws >= kMaxSplitWorkspaces || stream_is_capturing(stream)) return false;
    SplitWorkspace w{stream, nullptr, nullptr};
    if (hipMalloc(reinterpret_cast<void **>(&w.partials), kSplitPartialBytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (hipMalloc(reinterpret_cast<void **>(&w.counters), sizeof(uint32_t) * kSplitCounters) != hipSuccess ||
        hipMemset(w.counters, 0, sizeof(uint32_t) * kSplitCounters) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(w.partials);
        if (w.counters) (void)hipFree(w.counters);
        return false;
    }
    ctx->ws[ctx->n_ws++] = w;
    *out = w;
    return true;
}

// The stream is going away: its workspace goes with it, and the table is compacted so that the slot serves the next
// stream that splits K.  The caller has synchronised the stream.
void release_split_workspace(mlel_ctx *ctx, hipStream_t stream) {
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    for (int i = 0; i < ctx->n_ws; i++)
        if (ctx->ws[i].stream == stream) {
            (void)hipFree(ctx->ws[i].partials);
            (void)hipFree(ctx->ws[i].counters);
            ctx->ws[i] = ctx->ws[--ctx->n_ws];
            return;
        }
}

void free_split_workspaces(mlel_ctx *ctx) {
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    for (int i = 0; i < ctx->n_ws; i++) {
        (void)hipFree(ctx->ws[i].partials);
        (void)hipFree(ctx->ws[i].counters);
    }
    ctx->n_ws = 0;
    for (int i = 0; i < ctx->n_stage; i++) (void)hipFree(ctx->stage[i].ptr);
    ctx->n_stage = 0;
}

char *stage_workspace(mlel_ctx *ctx, hipStream_t stream, size_t bytes) {
    if (bytes == 0 || bytes > kMaxStageBytes) return nullptr;
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    int slot = -1;
    for (int i = 0; i < ctx->n_stage; i++)
        if (ctx->stage[i].stream == stream) slot = i;
    if (slot >= 0 && ctx->stage[slot].bytes >= bytes) return ctx->stage[slot].ptr;
    if (stream_is_capturing(stream) || (slot < 0 && ctx->n_stage >= kMaxSplitWorkspaces)) return nullptr;
    if (slot >= 0) {  // grow: earlier calls of the stream may still be reading the old buffer
        if (hipStreamSynchronize(stream) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        (void)hipFree(ctx->stage[slot].ptr);
        ctx->stage[slot] = ctx->stage[--ctx->n_stage];
    }
    char *p = nullptr;
    const size_t rounded = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    if (hipMalloc(reinterpret_cast<void **>(&p), rounded) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    ctx->stage[ctx->n_stage++] = StageWorkspace{stream, p, rounded};
    return p;
}

void release_stage_workspace(mlel_ctx *ctx, hipStream_t stream) {
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    for (int i = 0; i < ctx->n_stage; i++)
        if (ctx->stage[i].stream == stream) {
            (void)hipFree(ctx->stage[i].ptr);
            ctx->stage[i] = ctx->stage[--ctx->n_stage];
            return;
        }
}

}  // namespace mlel

using namespace mlel;

extern "C" {

const char *mlel_hip_last_error(void) { return g_error; }

int mlel_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int mlel_hip_init(int device, mlel_ctx **out_ctx) {
    MLEL_REQUIRE(out_ctx != nullptr, MLEL_ERR_INVALID, "init: null out_ctx");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        (void)hipGetLastError();
        return set_error(MLEL_ERR_DEVICE, "init: no HIP device visible (%s); this backend has no CPU fallback",
                         e != hipSuccess ? hipGetErrorString(e) : "device count 0");
    }
    MLEL_REQUIRE(device >= 0 && device < n, MLEL_ERR_INVALID, "init: device %d outside 0..%d", device, n - 1);
    MLEL_HIP_CHECK(hipSetDevice(device));
    mlel_ctx *ctx = new mlel_ctx();
    ctx->device = device;
    hipError_t pe = hipGetDeviceProperties(&ctx->props, device);
    if (pe != hipSuccess) {
        delete ctx;
        return set_error(MLEL_ERR_DEVICE, "init: hipGetDeviceProperties: %s", hipGetErrorString(pe));
    }
    if (const char *env = std::getenv("MLEL_SPLIT_K")) ctx->split_k = std::atoi(env);  // 0: off, n: at most n splits
    // this device's address of the static scratch array; a failure only disables the entry point that needs it
    (void)static_scratch_init(ctx);
    *out_ctx = ctx;
    return 0;
}

void mlel_hip_destroy(mlel_ctx *ctx) {
    if (ctx == nullptr) return;
    if (hipSetDevice(ctx->device) == hipSuccess) {
        (void)hipDeviceSynchronize();  // no launch may still be using a workspace that is about to be freed
        free_split_workspaces(ctx);
    }
    delete ctx;
}

int mlel_hip_device_info(mlel_ctx *ctx, int32_t *cu_count, int32_t *clock_khz, int32_t *mem_clock_khz,
                         int32_t *bus_width_bits, char *name, size_t name_len) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "device_info: null ctx");
    if (cu_count) *cu_count = ctx->props.multiProcessorCount;
    if (clock_khz) *clock_khz = ctx->props.clockRate;
    if (mem_clock_khz) *mem_clock_khz = ctx->props.memoryClockRate;
    if (bus_width_bits) *bus_width_bits = ctx->props.memoryBusWidth;
    if (name && name_len) {
        snprintf(name, name_len, "%s (%s)", ctx->props.name, ctx->props.gcnArchName);
    }
    return 0;
}

int mlel_hip_arena_alloc(mlel_ctx *ctx, size_t bytes, void **dptr) {
    MLEL_REQUIRE(ctx != nullptr && dptr != nullptr, MLEL_ERR_INVALID, "arena_alloc: null argument");
    *dptr = nullptr;
    if (bytes == 0) bytes = 16;
    MLEL_HIP_CHECK(hipSetDevice(ctx->device));
    MLEL_HIP_CHECK(hipMalloc(dptr, bytes));
    MLEL_HIP_CHECK(hipMemset(*dptr, 0, bytes));  // tensors start zero-filled, as the reference's test tensors do
    return 0;
}

int mlel_hip_arena_free(mlel_ctx *ctx, void *dptr) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "arena_free: null ctx");
    if (dptr) MLEL_HIP_CHECK(hipFree(dptr));
    return 0;
}

int mlel_hip_arena_import_fd(mlel_ctx *ctx, int fd, size_t bytes, void **dptr, void **out_handle) {
    MLEL_REQUIRE(ctx != nullptr && dptr != nullptr && out_handle != nullptr, MLEL_ERR_INVALID,
                 "arena_import_fd: null argument");
    MLEL_REQUIRE(fd >= 0 && bytes > 0, MLEL_ERR_INVALID, "arena_import_fd: bad fd or size");
    hipExternalMemoryHandleDesc desc;
    memset(&desc, 0, sizeof(desc));
    desc.type = hipExternalMemoryHandleTypeOpaqueFd;
    desc.handle.fd = fd;
    desc.size = bytes;
    hipExternalMemory_t ext = nullptr;
    MLEL_HIP_CHECK(hipImportExternalMemory(&ext, &desc));
    hipExternalMemoryBufferDesc buf;
    memset(&buf, 0, sizeof(buf));
    buf.offset = 0;
    buf.size = bytes;
    hipError_t e = hipExternalMemoryGetMappedBuffer(dptr, ext, &buf);
    if (e != hipSuccess) {
        (void)hipDestroyExternalMemory(ext);
        return set_error(MLEL_ERR_DEVICE, "hipExternalMemoryGetMappedBuffer: %s", hipGetErrorString(e));
    }
    *out_handle = ext;
    return 0;
}

int mlel_hip_arena_release_import(mlel_ctx *ctx, void *handle) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "arena_release_import: null ctx");
    if (handle) MLEL_HIP_CHECK(hipDestroyExternalMemory((hipExternalMemory_t)handle));
    return 0;
}

int mlel_hip_memcpy_h2d(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memcpy_h2d: null ctx");
    if (bytes == 0) return 0;
    MLEL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_memcpy_d2h(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memcpy_d2h: null ctx");
    if (bytes == 0) return 0;
    MLEL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_memcpy_d2d(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memcpy_d2d: null ctx");
    if (bytes == 0) return 0;
    MLEL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return 0;
}

int mlel_hip_memset(mlel_ctx *ctx, void *dst, int value, size_t bytes, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "memset: null ctx");
    if (bytes == 0) return 0;
    MLEL_REQUIRE(dst != nullptr, MLEL_ERR_INVALID, "memset: null pointer");
    if (!stream_is_capturing((hipStream_t)stream)) {
        MLEL_HIP_CHECK(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
        return 0;
    }
    // a memset node recorded into a graph has replayed wrongly on this part: a captured fill is a kernel
    const size_t head = std::min<size_t>((16 - ((uintptr_t)dst & 15)) & 15, bytes);
    const size_t n_vec = (bytes - head) / 16, tail = (bytes - head) % 16;
    size_t blocks = std::min<size_t>(std::max<size_t>((n_vec + 255) / 256, 1), (size_t)ctx->props.multiProcessorCount * 16);
    const uint32_t word = 0x01010101u * (uint32_t)(value & 0xff);
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (unsigned char *)dst,
                       head, n_vec, tail, word);
    return check_launch("memset (fill kernel)");
}

int mlel_hip_stream_create(mlel_ctx *ctx, void **out_stream) {
    MLEL_REQUIRE(ctx != nullptr && out_stream != nullptr, MLEL_ERR_INVALID, "stream_create: null argument");
    hipStream_t s;
    MLEL_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *out_stream = s;
    return 0;
}

int mlel_hip_stream_destroy(mlel_ctx *ctx, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "stream_destroy: null ctx");
    if (stream) {
        // the stream's split-K workspace (if it ever split) is freed with it; nothing may still be using it
        MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
        release_split_workspace(ctx, (hipStream_t)stream);
        release_stage_workspace(ctx, (hipStream_t)stream);
        MLEL_HIP_CHECK(hipStreamDestroy((hipStream_t)stream));
    }
    return 0;
}

int mlel_hip_split_workspaces(mlel_ctx *ctx) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "split_workspaces: null ctx");
    std::lock_guard<std::mutex> guard(ctx->ws_lock);
    return ctx->n_ws;
}

int mlel_hip_sync(mlel_ctx *ctx, void *stream) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "sync: null ctx");
    if (stream)
        MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    else
        MLEL_HIP_CHECK(hipDeviceSynchronize());
    return 0;
}

int mlel_hip_event_create(mlel_ctx *ctx, void **out_event) {
    MLEL_REQUIRE(ctx != nullptr && out_event != nullptr, MLEL_ERR_INVALID, "event_create: null argument");
    hipEvent_t e;
    MLEL_HIP_CHECK(hipEventCreate(&e));
    *out_event = e;
    return 0;
}

int mlel_hip_event_destroy(mlel_ctx *ctx, void *event) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "event_destroy: null ctx");
    if (event) MLEL_HIP_CHECK(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int mlel_hip_event_record(mlel_ctx *ctx, void *event, void *stream) {
    MLEL_REQUIRE(ctx != nullptr && event != nullptr, MLEL_ERR_INVALID, "event_record: null argument");
    MLEL_HIP_CHECK(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return 0;
}

int mlel_hip_stream_wait_event(mlel_ctx *ctx, void *stream, void *event) {
    MLEL_REQUIRE(ctx != nullptr && event != nullptr, MLEL_ERR_INVALID, "stream_wait_event: null argument");
    MLEL_HIP_CHECK(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0));
    return 0;
}

int mlel_hip_event_elapsed_ms(mlel_ctx *ctx, void *start, void *stop, float *ms) {
    MLEL_REQUIRE(ctx != nullptr && start && stop && ms, MLEL_ERR_INVALID, "event_elapsed_ms: null argument");
    MLEL_HIP_CHECK(hipEventSynchronize((hipEvent_t)stop));
    MLEL_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

int mlel_hip_capture_begin(mlel_ctx *ctx, void *stream) {
    MLEL_REQUIRE(ctx != nullptr && stream != nullptr, MLEL_ERR_INVALID,
                 "capture_begin: a non-null stream is required");
    MLEL_HIP_CHECK(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return 0;
}

int mlel_hip_capture_end(mlel_ctx *ctx, void *stream, void **out_graph_exec) {
    MLEL_REQUIRE(ctx != nullptr && stream != nullptr && out_graph_exec != nullptr, MLEL_ERR_INVALID,
                 "capture_end: null argument");
    hipGraph_t graph = nullptr;
    MLEL_HIP_CHECK(hipStreamEndCapture((hipStream_t)stream, &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return set_error(MLEL_ERR_DEVICE, "hipGraphInstantiate: %s", hipGetErrorString(e));
    *out_graph_exec = exec;
    return 0;
}

int mlel_hip_graph_launch(mlel_ctx *ctx, void *graph_exec, void *stream) {
    MLEL_REQUIRE(ctx != nullptr && graph_exec != nullptr, MLEL_ERR_INVALID, "graph_launch: null argument");
    MLEL_HIP_CHECK(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
    return 0;
}

int mlel_hip_graph_destroy(mlel_ctx *ctx, void *graph_exec) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "graph_destroy: null ctx");
    if (graph_exec) MLEL_HIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return 0;
}

int mlel_hip_copy_kernel(mlel_ctx *ctx, void *stream, void *dst, const void *src, size_t bytes) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "copy_kernel: null ctx");
    if (bytes == 0) return 0;
    MLEL_REQUIRE(dst && src, MLEL_ERR_INVALID, "copy_kernel: null pointer");
    MLEL_REQUIRE(((uintptr_t)dst % 16) == 0 && ((uintptr_t)src % 16) == 0, MLEL_ERR_INVALID,
                 "copy_kernel: pointers must be 16-byte aligned");
    // One pass: a 16-byte piece per thread, non-temporal accesses, as many blocks as that takes.  Measured on this
    // part over 1 GiB: 6.7 TB/s (read + write) against 5.0 TB/s for a grid-stride loop of 16 blocks per compute unit
    // and 5.0 - 5.6 TB/s with more pieces in flight per thread; a read-only pass reaches 7.1, a write-only pass 6.9.
    const size_t n_vec = bytes / 16, n_tail = bytes % 16;
    if (n_vec > 0) {
        const size_t blocks = std::min<size_t>((n_vec + 255) / 256, 0x7fffffffu);
        hipLaunchKernelGGL((copy_variant_kernel<1, true, 0>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           (uint4 *)dst, (const uint4 *)src, n_vec);
    }
    if (n_tail > 0)
        hipLaunchKernelGGL(copy_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, (uint4 *)dst, (const uint4 *)src,
                           (size_t)0, (char *)dst + n_vec * 16, (const char *)src + n_vec * 16, n_tail);
    return check_launch("copy_kernel");
}

int mlel_hip_mfma_rate_probe(mlel_ctx *ctx, void *stream, const void *operands, void *out, int blocks, int iters) {
    MLEL_REQUIRE(ctx != nullptr && operands != nullptr && out != nullptr, MLEL_ERR_INVALID, "mfma_rate_probe: null argument");
    MLEL_REQUIRE(blocks > 0 && blocks <= (1 << 20) && iters > 0, MLEL_ERR_INVALID, "mfma_rate_probe: blocks and iters must be positive");
    MLEL_REQUIRE(((uintptr_t)operands % 16) == 0 && ((uintptr_t)out % 4) == 0, MLEL_ERR_INVALID,
                 "mfma_rate_probe: operands must be 16-byte aligned");
    hipLaunchKernelGGL(mfma_rate_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const v4i_probe *)operands, (int32_t *)out, iters);
    return check_launch("mfma_rate_probe");
}

int mlel_hip_issue_probe(mlel_ctx *ctx, void *stream, const void *operands, void *out, int mode, int iters) {
    MLEL_REQUIRE(ctx != nullptr && operands != nullptr && out != nullptr, MLEL_ERR_INVALID, "issue_probe: null argument");
    MLEL_REQUIRE(iters > 0 && mode >= 0 && mode <= 14, MLEL_ERR_INVALID, "issue_probe: mode 0 .. 14, iters positive");
    MLEL_REQUIRE(((uintptr_t)operands % 16) == 0 && ((uintptr_t)out % 4) == 0, MLEL_ERR_INVALID,
                 "issue_probe: operands must be 16-byte aligned");
    const int blocks = ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256;  // one wavefront per SIMD
    const int32_t *ops = (const int32_t *)operands;
    uint32_t *o = (uint32_t *)out;
    hipStream_t st = (hipStream_t)stream;
#define MLEL_ISSUE_CASE(M) case M: hipLaunchKernelGGL(issue_probe_kernel<M>, dim3((unsigned)blocks), dim3(256), 0, st, ops, o, iters); break;
    switch (mode) {
        MLEL_ISSUE_CASE(0) MLEL_ISSUE_CASE(1) MLEL_ISSUE_CASE(2) MLEL_ISSUE_CASE(3) MLEL_ISSUE_CASE(4) MLEL_ISSUE_CASE(5)
        MLEL_ISSUE_CASE(6) MLEL_ISSUE_CASE(7) MLEL_ISSUE_CASE(8) MLEL_ISSUE_CASE(9) MLEL_ISSUE_CASE(10) MLEL_ISSUE_CASE(11)
        MLEL_ISSUE_CASE(12) MLEL_ISSUE_CASE(13) MLEL_ISSUE_CASE(14)
    }
#undef MLEL_ISSUE_CASE
    return check_launch("issue_probe");
}

int mlel_hip_copy_kernel_variant(mlel_ctx *ctx, void *stream, void *dst, const void *src, size_t bytes, int blocks,
                                 int pieces_in_flight, int non_temporal, int mode) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "copy_kernel_variant: null ctx");
    MLEL_REQUIRE(dst && src && bytes >= 16 && bytes % 16 == 0, MLEL_ERR_INVALID,
                 "copy_kernel_variant: pointers and a size in whole 16-byte pieces are required");
    MLEL_REQUIRE(((uintptr_t)dst % 16) == 0 && ((uintptr_t)src % 16) == 0, MLEL_ERR_INVALID,
                 "copy_kernel_variant: pointers must be 16-byte aligned");
    MLEL_REQUIRE(mode >= 0 && mode <= 2, MLEL_ERR_INVALID, "copy_kernel_variant: mode 0 copy, 1 read, 2 write");
    const int u = pieces_in_flight;
    MLEL_REQUIRE(u == 1 || u == 2 || u == 4 || u == 8, MLEL_ERR_INVALID,
                 "copy_kernel_variant: 1, 2, 4 or 8 pieces in flight");
    const size_t n_vec = bytes / 16;
    size_t cover = (n_vec + (size_t)256 * u - 1) / ((size_t)256 * u);  // blocks <= 0: every thread makes one pass
    const unsigned grid = (unsigned)(blocks > 0 ? (size_t)blocks : std::min<size_t>(cover, 0x7fffffffu));
    uint4 *d = (uint4 *)dst;
    const uint4 *sr = (const uint4 *)src;
    hipStream_t st = (hipStream_t)stream;
    if (non_temporal) {
        if (u == 1) launch_copy_variant<1, true>(mode, grid, st, d, sr, n_vec);
        if (u == 2) launch_copy_variant<2, true>(mode, grid, st, d, sr, n_vec);
        if (u == 4) launch_copy_variant<4, true>(mode, grid, st, d, sr, n_vec);
        if (u == 8) launch_copy_variant<8, true>(mode, grid, st, d, sr, n_vec);
    } else {
        if (u == 1) launch_copy_variant<1, false>(mode, grid, st, d, sr, n_vec);
        if (u == 2) launch_copy_variant<2, false>(mode, grid, st, d, sr, n_vec);
        if (u == 4) launch_copy_variant<4, false>(mode, grid, st, d, sr, n_vec);
        if (u == 8) launch_copy_variant<8, false>(mode, grid, st, d, sr, n_vec);
    }
    return check_launch("copy_kernel_variant");
}

}  // extern "C"
