// Scores, softmax and the product with V of an fp16 attention head in one launch:
//     S = CAST_f16( MATMUL(Q, K^T) )                      [NB, M, S]   (fp32 accumulate)
//     P = softmax chain over the last axis of S           ([MUL by a scale,] REDUCE_MAX, SUB, EXP, REDUCE_SUM,
//                                                           RECIPROCAL, MUL: every step rounded to fp16)
//     O = CAST_f16( MATMUL(P, V) )                        [NB, M, 64]  (fp32 accumulate), optionally stored through the
//                                                          six-dimensional view of a head merge
// with every rounding of the three launches it replaces (the fp16 product of gemm_f16.hip, the compiled row program
// of ops_float.hip, the product again), so the result is theirs bit for bit wherever it is a number.  S and P never
// leave the chip: a block owns 64 query rows of one head; four threads share a row and keep its values in registers
// from the scores to P, shared memory holds 256 keys of the 64 rows at a time (where the products leave and fetch
// their operands and where the fold reads: 33 KiB, so that three blocks fit a compute unit and the 768 blocks of
// 96 heads x 512 queries run in one round), K^T and V stream through one 10 KiB chunk buffer 64 keys at a time.
//
// Same arithmetic as the separate kernels, on purpose:
//   * both products use v_mfma_f32_32x32x16_f16 with the K-major operand as the instruction's first operand and walk
//     k in ascending order into one accumulator per output, which is the summation order of gemm_f16_kernel;
//   * the elementwise steps are the shared static_apply<> functions on 16-byte pieces; REDUCE_MAX is exact;
//     REDUCE_SUM is the reference's left-to-right fp16 fold (reduce.comp:24-70), here one lane per row: a single
//     wavefront folds the block's 64 rows at once (32 values per row in flight from shared memory while 32 are
//     added) while the first chunk of V is on its way.
#include "common.hpp"
#include "dispatch.hpp"
#include "float_programs.hpp"

namespace mlel {
namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s lds_v4s;

constexpr uint32_t kOob = 0x80000000u;
constexpr int kBlock = 256;
constexpr int kRows = 64;       // query rows per block
constexpr int kHead = 64;       // head size: K of the first product, N of the second
constexpr int kChunk = 64;      // keys per chunk of K^T / V
constexpr int kChunkPitch = 2 * kChunk + 32;  // bytes per K row of a chunk: 4 rows x 32 B land on distinct banks
constexpr int kMaxKeys = 512;   // 16 pieces of 16 bytes per thread
constexpr int kPassKeys = 256;  // keys of a row that sit in shared memory at a time
constexpr int kPasses = kMaxKeys / kPassKeys;
constexpr int kPassChunks = kPassKeys / kChunk;
constexpr int kPassPieces = kPassKeys / 32;  // 16-byte pieces per thread and pass

struct AttnArgs {
    const char *q, *kt, *v;
    char *out;
    const uint16_t *scale;  // the chain's single-element fp16 input (SCALED), else unused
    int32_t M, S, batches, strips;
    int64_t q_batch, kt_batch, v_batch, o_batch;  // bytes
    uint32_t ldq, ldkt, ldv, ldo;                 // bytes per row
    uint32_t q_bytes, kt_bytes, v_bytes, o_bytes; // per-batch extents (all below 2^31)
    // result written through a six-dimensional view [NB1, NB2, M1, M2, N1, N2] (see gemm_f16.hip); view == 0: plain
    int32_t view, v_nb2, v_m2, v_n2;
    int64_t vs_nb1, vs_nb2;
    uint32_t vs_m1, vs_m2, vs_n1;
    int32_t total, chunk, fold_span;
    DivMagic div_strips;  // block index / strips as a multiplication and a shift
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 load16(__amdgpu_buffer_rsrc_t r, uint32_t off) {
    const v4i v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
    return make_uint4((uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w);
}
__device__ __forceinline__ v8h as_v8h(const uint4 &u) {
    union {
        uint4 u;
        v8h h;
    } c;
    c.u = u;
    return c.h;
}

template <bool SCALED>
__global__ void __launch_bounds__(kBlock) attention_f16_kernel(const AttnArgs g) {
    extern __shared__ __align__(16) char smem[];
    const int SP = min(g.S, kPassKeys) * 2 + 16;  // pitch of a score row (bytes): consecutive rows start four banks apart
    char *st = smem;               // [64][SP]: one pass of S, later of EXP(..), later of P
    char *cb = smem + kRows * SP;  // [64][kChunkPitch]: a chunk of K^T or V; the row sums; the staged result

    // every argument in one batch: left alone the compiler loads all but the exit test's behind the exit, a second
    // trip to memory in a row before the first address
    asm volatile("" ::"s"(g.chunk), "s"(g.total), "s"(g.fold_span), "s"(g.div_strips.m), "s"(g.div_strips.s), "s"(g.q),
                 "s"(g.kt), "s"(g.v), "s"(g.out), "s"(g.scale), "s"(g.M), "s"(g.S), "s"(g.batches), "s"(g.strips),
                 "s"(g.q_batch), "s"(g.kt_batch), "s"(g.v_batch), "s"(g.o_batch), "s"(g.ldq), "s"(g.ldkt), "s"(g.ldv),
                 "s"(g.ldo), "s"(g.q_bytes), "s"(g.kt_bytes), "s"(g.v_bytes), "s"(g.o_bytes), "s"(g.view), "s"(g.v_nb2),
                 "s"(g.v_m2), "s"(g.v_n2), "s"(g.vs_nb1), "s"(g.vs_nb2), "s"(g.vs_m1), "s"(g.vs_m2), "s"(g.vs_n1));
    const int lin = __builtin_amdgcn_readfirstlane((int)(blockIdx.x % 8u) * g.chunk + (int)(blockIdx.x / 8u));
    if (lin >= g.total) return;
    const int batch = div_magic(lin, g.div_strips);
    const int m0 = (lin - batch * g.strips) * kRows;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // the wavefront's 32 x 32 tile of a 64 x 64 product

    const __amdgpu_buffer_rsrc_t qres = rsrc(g.q + (int64_t)batch * g.q_batch, g.q_bytes);
    const __amdgpu_buffer_rsrc_t kres = rsrc(g.kt + (int64_t)batch * g.kt_batch, g.kt_bytes);
    const __amdgpu_buffer_rsrc_t vres = rsrc(g.v + (int64_t)batch * g.v_batch, g.v_bytes);

    // operand addresses inside a tile, as in gemm_f16_kernel: row operand: row = lane % 32, k group = lane / 32 (8 halfs);
    // K-major operand: 16-lane group q = lane / 16 covers columns 16 (q & 1) .., k group q / 2; lane s = lane % 16
    // points at row s / 4, columns 4 (s % 4) of the 4 x 16 block
    const int a_row = lane & 31, a_kg = lane >> 5;
    const int s16 = lane & 15, q16 = lane >> 4;
    const int b_row = 8 * (q16 >> 1) + (s16 >> 2), b_col = 16 * (q16 & 1) + 4 * (s16 & 3);
    const char *b_base = cb + b_row * kChunkPitch + (wn * 32 + b_col) * 2;
    auto b_frag = [&](int kk) {
        const char *p = b_base + kk * 16 * kChunkPitch;
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)p);
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)(p + 4 * kChunkPitch));
        union {
            v4s s[2];
            v8h h;
        } u;
        u.s[0] = lo;
        u.s[1] = hi;
        return u.h;
    };
    // a chunk is 64 rows of 128 bytes: two 16-byte pieces per thread
    const int c_row = tid >> 2, c_piece = (tid & 3) * 2;
    auto chunk_store = [&](const uint4 (&r)[2]) {
        *reinterpret_cast<uint4 *>(cb + c_row * kChunkPitch + c_piece * 16) = r[0];
        *reinterpret_cast<uint4 *>(cb + c_row * kChunkPitch + c_piece * 16 + 16) = r[1];
    };
    const int nchunks = g.S / kChunk;
    uint4 cr[2];
    auto fetch_kt = [&](int c) {  // rows = k (the head dimension), columns = the chunk's keys
        const uint32_t off = (uint32_t)c_row * g.ldkt + (uint32_t)(c * kChunk + c_piece * 8) * 2;
        cr[0] = load16(kres, c < nchunks ? off : kOob);
        cr[1] = load16(kres, c < nchunks ? off + 16 : kOob);
    };
    auto fetch_v = [&](int c) {  // rows = the chunk's keys, columns = the head dimension
        const uint32_t off = (uint32_t)(c * kChunk + c_row) * g.ldv + (uint32_t)(c_piece * 8) * 2;
        cr[0] = load16(vres, c < nchunks ? off : kOob);
        cr[1] = load16(vres, c < nchunks ? off + 16 : kOob);
    };
    // The softmax chain: four threads share a row (pieces quarter, quarter + 4, ...) and keep the row's values in
    // registers from the scores to P.  Shared memory holds one pass (256 keys) of a row at a time: it is where the
    // products leave and fetch their operands and where the fold reads, and a thread always meets its own pieces there.
    const int row = tid >> 2, quarter = tid & 3;
    const int ppt = g.S >> 5;  // pieces per thread: S / 8 / 4, at most 16
    char *myrow = st + row * SP;
    // Which of a row's 16-byte pieces its four threads take in a pass: piece 2 quarter + uu % 2 + 8 (uu / 2), i.e. the
    // four threads of a row are 32 bytes apart and rows 33 pieces: a 128-bit access of the wavefront then runs at
    // full rate (measured: quarter + 4 uu, the threads 16 bytes apart, takes 1.6 times as long).  A pass has an even
    // number of pieces per thread, so this is a bijection onto the row's pieces.
    auto piece_off = [&](int, int uu) { return (2 * quarter + (uu & 1) + 8 * (uu >> 1)) * 16; };
    uint4 val[kMaxKeys / 32];
    uint32_t scale_w = 0;
    if (SCALED) {
        const uint32_t bits = *g.scale;
        scale_w = bits | (bits << 16);
    }
    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
    h2_t m2 = {(_Float16)-65504.f, (_Float16)-65504.f};
    uint32_t special = 0;

    // ---- phase 1: S = fp16(Q K^T), 64 keys at a time.  The query rows of this wavefront are matrix operands in registers.
    v8h qf[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++)
        qf[kk] = as_v8h(load16(qres, (uint32_t)(m0 + wm * 32 + a_row) * g.ldq + (uint32_t)(kk * 16 + a_kg * 8) * 2));
    fetch_kt(0);
#pragma unroll
    for (int h = 0; h < kPasses; h++) {
        if (h * kPassChunks < nchunks) {  // uniform
            const int c_end = min(nchunks, (h + 1) * kPassChunks);
            for (int c = h * kPassChunks; c < c_end; c++) {
                __syncthreads();  // every wavefront has read the previous chunk (and the previous pass its scores)
                chunk_store(cr);
                __syncthreads();
                fetch_kt(c + 1);
                v16f acc;
#pragma unroll
                for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
                for (int kk = 0; kk < 4; kk++) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(b_frag(kk), qf[kk], acc, 0, 0, 0);
                // lane holds row lane % 32 of the tile and, per register quad q, columns 8 q + 4 (lane / 32) .. + 3
                char *srow = st + (wm * 32 + (lane & 31)) * SP + ((c - h * kPassChunks) * kChunk + wn * 32 + 4 * (lane >> 5)) * 2;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    uint2 w;  // CAST: round to nearest even
                    w.x = __builtin_bit_cast(uint32_t, pack_f16(acc[4 * q + 0], acc[4 * q + 1]));
                    w.y = __builtin_bit_cast(uint32_t, pack_f16(acc[4 * q + 2], acc[4 * q + 3]));
                    *reinterpret_cast<uint2 *>(srow + q * 16) = w;
                }
            }
            __syncthreads();
            // this pass's scores into registers, through the scale; the maximum as they pass
            // (all of a pass's pieces are requested before the first is used, also those beyond a short row, which are
            // inside the pass buffer and not used: one shared-memory round trip per pass instead of one per piece)
            uint4 raw[kPassPieces];
#pragma unroll
            for (int uu = 0; uu < kPassPieces; uu++) raw[uu] = *reinterpret_cast<const uint4 *>(myrow + piece_off(h, uu));
#pragma unroll
            for (int uu = 0; uu < kPassPieces; uu++) {
                const int u = h * kPassPieces + uu;
                if (u < ppt) {
                    uint4 x = raw[uu];
                    if (SCALED) {
                        x = static_apply<F_MUL>(x, make_uint4(scale_w, scale_w, scale_w, scale_w));
                        asm volatile("" : "+v"(x.x), "+v"(x.y), "+v"(x.z), "+v"(x.w));
                    }
                    val[u] = x;
                    // REDUCE_MAX: exact; a NaN or an infinity anywhere in the row makes the maximum a NaN (as the row program)
                    special |= (((x.x & 0x7fff7fffu) + 0x03ff03ffu) | ((x.y & 0x7fff7fffu) + 0x03ff03ffu) |
                                ((x.z & 0x7fff7fffu) + 0x03ff03ffu) | ((x.w & 0x7fff7fffu) + 0x03ff03ffu)) & 0x80008000u;
                    const h2_t *p = reinterpret_cast<const h2_t *>(&x);
                    m2 = __builtin_elementwise_max(m2, __builtin_elementwise_max(__builtin_elementwise_max(p[0], p[1]),
                                                                                   __builtin_elementwise_max(p[2], p[3])));
                }
            }
        }
    }

    // ---- phase 2: the rest of the softmax chain
    float mx = (float)(m2.x > m2.y ? m2.x : m2.y);
#pragma unroll
    for (int d = 1; d < 4; d <<= 1) {
        mx = fmaxf(mx, __shfl_xor(mx, d));
        special |= (uint32_t)__shfl_xor((int)special, d);
    }
    const uint32_t mbits = (uint32_t)__half_as_ushort(f2h(special != 0 ? __builtin_nanf("") : mx));
    const uint4 mrow = make_uint4(mbits | (mbits << 16), mbits | (mbits << 16), mbits | (mbits << 16), mbits | (mbits << 16));
#pragma unroll
    for (int u = 0; u < kMaxKeys / 32; u++) {
        if (u < ppt) {
            uint4 d = static_apply<F_SUB>(val[u], mrow);
            asm volatile("" : "+v"(d.x), "+v"(d.y), "+v"(d.z), "+v"(d.w));
            uint4 e = static_apply<F_EXP>(d, d);
            asm volatile("" : "+v"(e.x), "+v"(e.y), "+v"(e.z), "+v"(e.w));
            val[u] = e;
        }
    }
    // REDUCE_SUM: left to right in fp16, one lane per row, a pass of the rows at a time; the first chunk of V is on its
    // way meanwhile
    uint16_t *sums = reinterpret_cast<uint16_t *>(cb);  // [64]
    // The blocks that share a compute unit run in step and fold at the same time; three chains on one SIMD would take
    // turns (a wavefront instruction holds the SIMD for four clocks), so the folding wavefront rotates with the round
    // of blocks (blocks are dealt to a unit one round at a time: g.fold_span = blocks per round and XCD).
    const int fold_wave = (int)((uint32_t)(blockIdx.x / 8u) / (uint32_t)g.fold_span) & 3;
    fetch_v(0);
    __half facc = f2h(0.f);
#pragma unroll
    for (int h = 0; h < kPasses; h++) {
        if (h * kPassChunks < nchunks) {  // uniform
            if (h > 0) __syncthreads();  // the previous pass has been folded
#pragma unroll
            for (int uu = 0; uu < kPassPieces; uu++) {
                const int u = h * kPassPieces + uu;
                if (u < ppt) *reinterpret_cast<uint4 *>(myrow + piece_off(h, uu)) = val[u];
            }
            __syncthreads();
            if (wave == fold_wave) {
                const char *r = st + lane * SP;
                // 64 bytes (32 values) at a time through two register sets: one is folded while the other is on its
                // way (a pass is a multiple of 64 keys, so it has an even number of sets)
                const int sets = (min(g.S - h * kPassKeys, kPassKeys)) >> 5;
                uint4 a[4], b[4];
                auto fetch = [&](uint4 (&x)[4], int set) {
#pragma unroll
                    for (int t = 0; t < 4; t++) x[t] = *reinterpret_cast<const uint4 *>(r + set * 64 + t * 16);
                };
                auto fold = [&](const uint4 (&x)[4]) {
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const __half2 *hp = reinterpret_cast<const __half2 *>(&x[t]);
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            facc = __hadd(facc, __low2half(hp[e]));
                            facc = __hadd(facc, __high2half(hp[e]));
                        }
                    }
                };
                fetch(a, 0);
                for (int set = 0; set < sets; set += 2) {
                    fetch(b, set + 1);
                    __builtin_amdgcn_sched_barrier(0);
                    fold(a);
                    __builtin_amdgcn_sched_barrier(0);
                    fetch(a, min(set + 2, sets - 1));  // unconditional (the last one is not used): the sets keep their registers
                    __builtin_amdgcn_sched_barrier(0);
                    fold(b);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }
    if (wave == fold_wave) sums[lane] = __half_as_ushort(facc);
    __syncthreads();
    uint4 rrow;
    {
        const uint32_t sbits = sums[row];
        const uint32_t sw = sbits | (sbits << 16);
        uint4 rc = static_apply<F_RECIPROCAL>(make_uint4(sw, sw, sw, sw), make_uint4(sw, sw, sw, sw));
        asm volatile("" : "+v"(rc.x));
        rrow = make_uint4(rc.x, rc.x, rc.x, rc.x);
    }

    // ---- phase 3: O = fp16(P V), 64 keys at a time, P a pass at a time
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    const char *p_base = st + (wm * 32 + a_row) * SP + a_kg * 16;
#pragma unroll
    for (int h = 0; h < kPasses; h++) {
        if (h * kPassChunks < nchunks) {  // uniform
            if (h > 0) __syncthreads();  // the previous pass of P has been multiplied
#pragma unroll
            for (int uu = 0; uu < kPassPieces; uu++) {
                const int u = h * kPassPieces + uu;
                if (u < ppt) {
                    uint4 p = static_apply<F_MUL>(val[u], rrow);
                    asm volatile("" : "+v"(p.x), "+v"(p.y), "+v"(p.z), "+v"(p.w));
                    *reinterpret_cast<uint4 *>(myrow + piece_off(h, uu)) = p;
                }
            }
            const int c_end = min(nchunks, (h + 1) * kPassChunks);
            for (int c = h * kPassChunks; c < c_end; c++) {
                __syncthreads();  // the previous chunk (or the row sums) has been read; this pass of P is complete
                chunk_store(cr);
                __syncthreads();
                fetch_v(c + 1);
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {
                    const v8h pf = *reinterpret_cast<const v8h *>(p_base + ((c - h * kPassChunks) * kChunk + kk * 16) * 2);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(b_frag(kk), pf, acc, 0, 0, 0);
                }
            }
        }
    }
    __syncthreads();
    // the 64 x 64 result through shared memory, so that it leaves in 16-byte pieces (whole 128-byte rows)
    constexpr int OP = kHead * 2 + 16;
    {
        char *orow = cb + (wm * 32 + (lane & 31)) * OP + (wn * 32 + 4 * (lane >> 5)) * 2;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            uint2 w;
            w.x = __builtin_bit_cast(uint32_t, pack_f16(acc[4 * q + 0], acc[4 * q + 1]));
            w.y = __builtin_bit_cast(uint32_t, pack_f16(acc[4 * q + 2], acc[4 * q + 3]));
            *reinterpret_cast<uint2 *>(orow + q * 16) = w;
        }
    }
    __syncthreads();
    const int64_t o_base = g.view ? (int64_t)(batch / g.v_nb2) * g.vs_nb1 + (int64_t)(batch % g.v_nb2) * g.vs_nb2
                                  : (int64_t)batch * g.o_batch;
    const __amdgpu_buffer_rsrc_t ores = rsrc(g.out + o_base, g.o_bytes);
    // the view's two divisions per piece as multiplications (the divisors are the same for every piece; exact while
    // index * divisor < 2^32, else the plain division)
    const uint32_t dm = (uint32_t)(g.view ? g.v_m2 : 1), dn = (uint32_t)(g.view ? g.v_n2 : 1);
    const bool fast_m = dm > 1 && (uint64_t)(uint32_t)g.M * dm < (uint64_t(1) << 32), fast_n = dn > 1 && (uint64_t)kHead * dn < (uint64_t(1) << 32);
    const uint32_t magic_m = fast_m ? 0xffffffffu / dm + 1u : 0u, magic_n = fast_n ? 0xffffffffu / dn + 1u : 0u;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int p = i * kBlock + tid, r = p >> 3, c8 = p & 7;
        const int m = m0 + r, n = c8 * 8;
        const uint4 piece = *reinterpret_cast<const uint4 *>(cb + r * OP + c8 * 16);
        uint32_t off = (uint32_t)m * g.ldo + (uint32_t)n * 2;
        if (g.view) {  // uniform
            const uint32_t m1 = fast_m ? __umulhi((uint32_t)m, magic_m) : (dm == 1 ? (uint32_t)m : (uint32_t)m / dm);
            const uint32_t n1 = fast_n ? __umulhi((uint32_t)n, magic_n) : (dn == 1 ? (uint32_t)n : (uint32_t)n / dn);
            off = m1 * g.vs_m1 + ((uint32_t)m - m1 * dm) * g.vs_m2 + n1 * g.vs_n1 + ((uint32_t)n - n1 * dn) * 2;
        }
        v4i v;
        v.x = (int)piece.x, v.y = (int)piece.y, v.z = (int)piece.z, v.w = (int)piece.w;
        __builtin_amdgcn_raw_buffer_store_b128(v, ores, (int)off, 0, kOutAux);
    }
}

bool dense_rows(const mlel_tensor *t) { return t->strides[2] == 2 && t->strides[1] >= t->dims[2] * 2; }
bool aligned16(const mlel_tensor *t, bool with_ptr) {
    return (!with_ptr || ((uintptr_t)t->ptr % 16) == 0) && t->strides[0] % 16 == 0 && t->strides[1] % 16 == 0;
}

// 0: the softmax chain without a scale, 1: with a scale in front, -1: another chain
int softmax_form(const mlel_chain *c) {
    if (c == nullptr) return -1;
    struct Want {
        int kind, selector, a, b;
    };
    static const Want plain[6] = {{MLEL_CHAIN_REDUCE, MLEL_RED_MAX, 0, 0},       {MLEL_CHAIN_BINARY, MLEL_BIN_SUB, 0, 1},
                                  {MLEL_CHAIN_UNARY, MLEL_UN_EXP, 2, 0},         {MLEL_CHAIN_REDUCE, MLEL_RED_SUM, 3, 0},
                                  {MLEL_CHAIN_UNARY, MLEL_UN_RECIPROCAL, 4, 0}, {MLEL_CHAIN_MUL, 0, 3, 5}};
    const int scaled = c->n_inputs == 2 && c->n_steps == 7 ? 1 : (c->n_inputs == 1 && c->n_steps == 6 ? 0 : -1);
    if (scaled < 0) return -1;
    if (scaled) {
        const mlel_chain_step &s = c->steps[0];
        if (s.kind != MLEL_CHAIN_MUL || s.a != 0 || s.b != 1 || s.dtype != MLEL_F16) return -1;
        const mlel_tensor *k = c->inputs[1];
        if (k == nullptr || k->dtype != MLEL_F16 || numel(k) != 1) return -1;
    }
    // with a scale every value index moves up by two: one more input, one more step
    for (int i = 0; i < 6; i++) {
        const mlel_chain_step &s = c->steps[i + scaled];
        const Want &w = plain[i];
        const auto shifted = [&](int v) { return scaled ? v + 2 : v; };
        const bool two = w.kind == MLEL_CHAIN_BINARY || w.kind == MLEL_CHAIN_MUL;
        if (s.kind != w.kind || s.dtype != MLEL_F16 || s.a != shifted(w.a) || (two && s.b != shifted(w.b))) return -1;
        if (w.kind != MLEL_CHAIN_MUL && s.selector != w.selector) return -1;
    }
    return scaled;
}

// 1 when the three operators are a case for the kernel; `with_pointers`: also check the base addresses
int describe(const mlel_tensor *out, const mlel_tensor *q, const mlel_tensor *kt, const mlel_tensor *v,
             const mlel_chain *chain, bool with_pointers, AttnArgs *filled) {
    const int form = softmax_form(chain);
    if (form < 0) return 0;
    if (q->dtype != MLEL_F16 || kt->dtype != MLEL_F16 || v->dtype != MLEL_F16 || out->dtype != MLEL_F16) return 0;
    if (q->rank != 3 || kt->rank != 3 || v->rank != 3 || (out->rank != 3 && out->rank != 6)) return 0;
    const int64_t NB = q->dims[0], M = q->dims[1], S = kt->dims[2];
    if (q->dims[2] != kHead || kt->dims[0] != NB || kt->dims[1] != kHead || v->dims[0] != NB || v->dims[1] != S ||
        v->dims[2] != kHead)
        return 0;
    if (NB <= 0 || M <= 0 || M % kRows != 0 || S < kChunk || S > kMaxKeys || S % kChunk != 0) return 0;
    if (!dense_rows(q) || !dense_rows(kt) || !dense_rows(v)) return 0;
    if (!aligned16(q, with_pointers) || !aligned16(kt, with_pointers) || !aligned16(v, with_pointers)) return 0;
    const int64_t lim = (int64_t(1) << 31) - 64;
    const int64_t qb = M * q->strides[1], kb = kHead * kt->strides[1], vb = S * v->strides[1];
    if (qb >= lim || kb >= lim || vb >= lim || NB * (M / kRows) >= (int64_t(1) << 30)) return 0;
    AttnArgs g{};
    if (out->rank == 3) {
        if (out->dims[0] != NB || out->dims[1] != M || out->dims[2] != kHead || out->strides[2] != 2) return 0;
        if (!aligned16(out, with_pointers) || M * out->strides[1] >= lim || out->strides[1] < kHead * 2) return 0;
        g.o_batch = out->strides[0];
        g.ldo = (uint32_t)out->strides[1];
        g.o_bytes = (uint32_t)(M * out->strides[1]);
    } else {
        // [NB1, NB2, M1, M2, N1, N2] with eight consecutive n2 contiguous
        if (out->dims[0] * out->dims[1] != NB || out->dims[2] * out->dims[3] != M || out->dims[4] * out->dims[5] != kHead) return 0;
        if (out->strides[5] != 2 || out->dims[5] % 8 != 0) return 0;
        if (with_pointers && ((uintptr_t)out->ptr % 16) != 0) return 0;
        int64_t span = 16;
        for (int i = 0; i < 6; i++) {
            if (i != 5 && (out->strides[i] % 16 != 0 || out->strides[i] < 0)) return 0;
            if (i >= 2) span += (out->dims[i] - 1) * out->strides[i];
        }
        if (span >= lim) return 0;
        g.view = 1;
        g.v_nb2 = (int32_t)out->dims[1];
        g.v_m2 = (int32_t)out->dims[3];
        g.v_n2 = (int32_t)out->dims[5];
        g.vs_nb1 = out->strides[0];
        g.vs_nb2 = out->strides[1];
        g.vs_m1 = (uint32_t)out->strides[2];
        g.vs_m2 = (uint32_t)out->strides[3];
        g.vs_n1 = (uint32_t)out->strides[4];
        g.o_bytes = (uint32_t)span;
    }
    g.q = static_cast<const char *>(q->ptr);
    g.kt = static_cast<const char *>(kt->ptr);
    g.v = static_cast<const char *>(v->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.scale = form == 1 ? static_cast<const uint16_t *>(chain->inputs[1]->ptr) : nullptr;
    if (with_pointers && form == 1 && (g.scale == nullptr || ((uintptr_t)g.scale % 2) != 0)) return 0;
    g.M = (int32_t)M;
    g.S = (int32_t)S;
    g.batches = (int32_t)NB;
    g.strips = (int32_t)(M / kRows);
    g.div_strips = make_div_magic((uint32_t)g.strips);
    g.q_batch = q->strides[0];
    g.kt_batch = kt->strides[0];
    g.v_batch = v->strides[0];
    g.ldq = (uint32_t)q->strides[1];
    g.ldkt = (uint32_t)kt->strides[1];
    g.ldv = (uint32_t)v->strides[1];
    g.q_bytes = (uint32_t)qb;
    g.kt_bytes = (uint32_t)kb;
    g.v_bytes = (uint32_t)vb;
    g.total = (int32_t)(NB * (M / kRows));
    g.chunk = (g.total + 7) / 8;
    if (filled != nullptr) *filled = g;
    return form == 1 ? 2 : 1;
}

}  // namespace

bool attention_f16_supported(const mlel_tensor *out, const mlel_tensor *q, const mlel_tensor *kt, const mlel_tensor *v,
                             const mlel_chain *chain) {
    return describe(out, q, kt, v, chain, false, nullptr) != 0;
}

int try_attention_f16(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *q, const mlel_tensor *kt,
                      const mlel_tensor *v, const mlel_chain *chain) {
    AttnArgs g{};
    const int form = describe(out, q, kt, v, chain, true, &g);
    if (form == 0) return 0;
    const size_t sm = (size_t)kRows * (std::min(g.S, kPassKeys) * 2 + 16) + (size_t)kChunk * kChunkPitch;
    const dim3 grid((unsigned)(g.chunk * 8));
    g.fold_span = std::max(1, (ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256) / 8);
    if (form == 2) {
        auto kernel = attention_f16_kernel<true>;
        static const bool raised = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       kRows * (kPassKeys * 2 + 16) + kChunk * kChunkPitch) == hipSuccess;
        (void)raised;
        kernel<<<grid, dim3(kBlock), sm, s>>>(g);
    } else {
        auto kernel = attention_f16_kernel<false>;
        static const bool raised = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       kRows * (kPassKeys * 2 + 16) + kChunk * kChunkPitch) == hipSuccess;
        (void)raised;
        kernel<<<grid, dim3(kBlock), sm, s>>>(g);
    }
    MLEL_TRY(check_launch("attention fp16"));
    return 1;
}

}  // namespace mlel
