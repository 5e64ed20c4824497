// int8 x int8 -> int32 contractions on the gfx950 matrix cores: CONV2D (implicit GEMM over NHWC input and OHWI
// weights) and MATMUL, with the zero-point handling of the reference shaders and an optional fused
// RESCALE(+CLAMP) epilogue.
//
// What is computed.  out[m][n] = sum_k (X[m][k] - zx) * (Wt[n][k] - zw) + bias[n], where
//   CONV2D : m = (image, oy, ox), n = oc, k = (ky, kx, ic); X[m][k] is the input element under tap (ky,kx) or, for
//            a tap that falls into the padding, the value zx itself so that the tap contributes nothing
//            (the reference skips such taps: conv2d.comp:64);
//   MATMUL : per batch, X = A[m][k], Wt[n][k] = B[k][n] (B is stored K-major and transposed while it is staged
//            into LDS) (reference: matmul.comp:30-73).
// The sum is expanded as  sum X*Wt - zw*sum_k X - zx*sum_k Wt + K*zx*zw  so that the matrix cores multiply the raw
// int8 operands (X - zx does not fit in int8).  All arithmetic is int32 with wraparound, as in the shaders, so the
// regrouping is exact.
//
// Kernel shape.  256 threads = 4 wavefronts of 64.  A block owns a BM x BN output tile; K is walked in steps of
// 64 bytes through two LDS buffers (global loads of step i+1 are in flight while step i is multiplied).  Each
// wavefront owns a (32*TM) x (32*TN) sub-tile and issues v_mfma_i32_32x32x32_i8 with the weights as the row
// operand and the activations as the column operand: a lane then holds, for ONE output position m, groups of four
// consecutive output channels n, which is the byte order of the NHWC / [M][N] output, so requantised results are
// packed four to a dword and stored without a transpose.  Per-channel epilogue constants live in LDS.
#pragma once

#include "common.hpp"
#include <mutex>
#include <unordered_set>

#include "dispatch.hpp"

namespace mlel {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2i lds_v2i;

constexpr int BK = 64;            // bytes of K per step
constexpr int kGroupM = 8;        // tile rows per band of the tile walk
constexpr int PITCH = BK + 16;    // LDS row pitch: 80 B keeps 16-lane groups of 128-bit reads on distinct banks

struct GemmArgs {
    // problem
    int32_t M, N, K, batches;
    // X operand (rows m): conv gather over NHWC; the plain [M][K] case is the 1x1 conv with H = W = 1
    const int8_t *x;
    int64_t x_batch, x_sn, x_sy, x_sx;  // byte strides
    int32_t H, W, IC, OHW, OW, KH, KW, sy, sx, dy, dx, pad_t, pad_l;
    int32_t plain;  // 1: m indexes rows of pitch x_sx directly
    int32_t xch;    // bytes per aligned global load of X: 16, 4 or 1
    uint32_t x_bytes, w_bytes;  // per-batch extent of each operand (buffer-load bounds of the fast fetch modes)
    // W operand (rows n)
    const int8_t *w;
    int64_t w_batch, ldw;
    int32_t w_kmajor;  // 0: [N][K] rows of pitch ldw; 1: [K][N] rows of pitch ldw
    int32_t wch;       // bytes per aligned global load of W: 16, 4 or 1
    int32_t zx, zw;
    // bias (int32, length 1 or N) and output
    const int32_t *bias;
    int32_t bias_len;
    char *out;
    int64_t out_batch, ldo;  // ldo in elements
    int32_t out_size;        // bytes per output element: 1, 2 or 4
    int32_t out_vec_ok;      // four consecutive channels may be stored as one aligned unit
    uint32_t o_bytes;        // per-batch extent of the output when it fits 31-bit buffer offsets, else 0
    // fused epilogue
    int32_t fused;
    const char *mult;  // int32 or int16 per channel (or one)
    const int8_t *shift;
    int32_t mult16;
    RescaleParams rp;
    // residual stage (Q8 epilogue only): out = rescale_out(rescale_res(res[m][n]) + rescale_conv(y)), y the int8 result
    // of the fused epilogue above; all three stages per tensor; `res` has the layout of `out`
    const int8_t *res;
    ScaleRef rs_res, rs_conv, rs_out;
    // launch geometry
    int32_t tiles_m, tiles_n, total_tiles, chunk;
    // Divisions of the tile index by numbers that are fixed for the launch (tiles per batch, tiles per row, tiles per
    // band of kGroupM rows, rows of the last band), as a multiplication and a shift: a division costs a wavefront
    // some thirty dependent scalar instructions, and the first operand request waits for three of them.
    DivMagic div_tiles_per_batch, div_tiles_n, div_band, div_last_rows;
    // Split K (register-staged pipeline only): `splits` blocks share one output tile, block s multiplies the K steps
    // [s * split_steps, (s + 1) * split_steps).  Every block writes its int32 partial tile (zero-point terms of its K
    // range already applied, the bias in split 0) to `partials` and bumps the tile's counter; the block that finds
    // the counter at splits - 1 adds the other partials to its own (int32 addition wraps, so the order is
    // immaterial), resets the counter and runs the epilogue.  splits == 1: split_steps = all K steps, no scratch.
    int32_t splits, split_steps;
    int32_t *partials;   // [total_tiles][splits][BM * BN], register-major so that every store is coalesced
    uint32_t *counters;  // [total_tiles], zero before the launch
};

struct ChanParams {  // per output channel, in LDS: 32 bytes = two 128-bit reads
    ChanScale q;
    int32_t bias_adj;
    int32_t pad[1];
};
static_assert(sizeof(ChanParams) == 32, "ChanParams layout");

struct RowState {
    const int8_t *base;
    int32_t iy0, ix0;
    int32_t valid;
};

struct KState {
    int32_t ky, kx, ic;
};

__device__ __forceinline__ void kstate_advance(KState &s, int step, int IC, int KW) {
    s.ic += step;
    while (s.ic >= IC) {
        s.ic -= IC;
        if (++s.kx == KW) {
            s.kx = 0;
            ++s.ky;
        }
    }
}

__device__ __forceinline__ uint32_t splat8(int v) { return (uint32_t)(uint8_t)v * 0x01010101u; }

// One 16-byte piece of row `r` of the X operand starting at k-position `s`.
__device__ __forceinline__ uint4 load_x_chunk(const GemmArgs &g, const RowState &r, KState s) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (!r.valid) return v;
    if (g.xch == 16) {
        if (s.ky >= g.KH) return v;
        const int y = r.iy0 + s.ky * g.dy, x = r.ix0 + s.kx * g.dx;
        if ((unsigned)y >= (unsigned)g.H || (unsigned)x >= (unsigned)g.W) {
            const uint32_t z = splat8(g.zx);
            return make_uint4(z, z, z, z);
        }
        return *reinterpret_cast<const uint4 *>(r.base + (int64_t)y * g.x_sy + (int64_t)x * g.x_sx + s.ic);
    }
    uint32_t d[4];
    if (g.xch == 4) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t val = 0;
            if (s.ky < g.KH) {
                const int y = r.iy0 + s.ky * g.dy, x = r.ix0 + s.kx * g.dx;
                if ((unsigned)y >= (unsigned)g.H || (unsigned)x >= (unsigned)g.W)
                    val = splat8(g.zx);
                else
                    val = *reinterpret_cast<const uint32_t *>(r.base + (int64_t)y * g.x_sy + (int64_t)x * g.x_sx +
                                                              s.ic);
            }
            d[j] = val;
            kstate_advance(s, 4, g.IC, g.KW);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t val = 0;
            for (int b = 0; b < 4; b++) {
                uint32_t byte = 0;
                if (s.ky < g.KH) {
                    const int y = r.iy0 + s.ky * g.dy, x = r.ix0 + s.kx * g.dx;
                    if ((unsigned)y >= (unsigned)g.H || (unsigned)x >= (unsigned)g.W)
                        byte = (uint8_t)g.zx;
                    else
                        byte = (uint8_t)r.base[(int64_t)y * g.x_sy + (int64_t)x * g.x_sx + s.ic];
                }
                val |= byte << (8 * b);
                kstate_advance(s, 1, g.IC, g.KW);
            }
            d[j] = val;
        }
    }
    return make_uint4(d[0], d[1], d[2], d[3]);
}

// One 16-byte piece of row n of the W operand stored as [N][K].
__device__ __forceinline__ uint4 load_w_chunk(const GemmArgs &g, const int8_t *wb, int n, int k) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (n >= g.N || k >= g.K) return v;
    const int8_t *p = wb + (int64_t)n * g.ldw + k;
    if (g.wch == 16) return *reinterpret_cast<const uint4 *>(p);
    uint32_t d[4];
    if (g.wch == 4) {
#pragma unroll
        for (int j = 0; j < 4; j++) d[j] = (k + 4 * j < g.K) ? *reinterpret_cast<const uint32_t *>(p + 4 * j) : 0u;
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t val = 0;
            for (int b = 0; b < 4; b++)
                if (k + 4 * j + b < g.K) val |= (uint32_t)(uint8_t)p[4 * j + b] << (8 * b);
            d[j] = val;
        }
    }
    return make_uint4(d[0], d[1], d[2], d[3]);
}

// A 4(k) x 4(n) byte block of the K-major W operand, returned transposed: d[j] = the four k-bytes of column n+j.
__device__ __forceinline__ uint4 load_w_block_kmajor(const GemmArgs &g, const int8_t *wb, int n, int k) {
    uint32_t r[4] = {0, 0, 0, 0};
    if (n < g.N) {
        if (g.wch >= 4) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (k + i < g.K) r[i] = *reinterpret_cast<const uint32_t *>(wb + (int64_t)(k + i) * g.ldw + n);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (k + i < g.K)
                    for (int b = 0; b < 4; b++)
                        if (n + b < g.N) r[i] |= (uint32_t)(uint8_t)wb[(int64_t)(k + i) * g.ldw + n + b] << (8 * b);
        }
    }
    // 4x4 byte transpose with v_perm_b32 (selector bytes 0-3 pick from the second source, 4-7 from the first)
    const uint32_t t0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
    return make_uint4(__builtin_amdgcn_perm(t2, t0, 0x05040100u), __builtin_amdgcn_perm(t2, t0, 0x07060302u),
                      __builtin_amdgcn_perm(t3, t1, 0x05040100u), __builtin_amdgcn_perm(t3, t1, 0x07060302u));
}

// Buffer-addressed loads: 32-bit offsets, and an offset at or beyond the extent of the resource returns 0
// without touching memory, which removes every bounds branch from the fast fetch modes.
constexpr uint32_t kOobOffset = 0x80000000u;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t off) {
    const v4i v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
    return make_uint4((uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w);
}
__device__ __forceinline__ uint32_t buf_load4(__amdgpu_buffer_rsrc_t r, uint32_t off) {
    return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0);
}

template <int BN>
constexpr int w_buf_bytes() {
    return BN * PITCH > BK * (BN + 16) ? BN * PITCH : BK * (BN + 16);
}

// How the two operands are fetched; fixed at compile time so that the hot loops carry no per-byte logic.
enum XMode {
    X_PLAIN = 0,    // X[m][k] = base + m * pitch + k, 16-byte pieces (MATMUL A; 1x1 stride-1 CONV2D on a dense input)
    X_TAP = 1,      // 16-byte pieces, IC % 64 == 0: one K step lies inside one filter tap (uniform tap state)
    X_GENERIC = 2,  // anything else: per-piece tap tracking, 16 / 4 / 1-byte loads
    X_PLAIN4 = 3,   // as X_PLAIN for rows that are only dword aligned (K % 4 == 0): four dword loads per piece
    X_PLAIN_DL = 4, // as X_PLAIN with K % 16 == 0, fetched straight into LDS (no register staging), deep stage ring
};
enum WMode {
    W_ROWS = 0,     // [N][K], 16-byte pieces
    W_KMAJOR = 1,   // [K][N] kept K-major in LDS; MFMA operands are gathered with ds_read_b64_tr_b8; 16-byte loads
    W_GENERIC = 2,  // either layout, any alignment
    W_KMAJOR4 = 3,  // as W_KMAJOR for rows that are only dword aligned (N % 4 == 0): four dword loads per piece
    W_ROWS4 = 4,    // as W_ROWS for rows that are only dword aligned (K % 4 == 0)
    W_ROWS_DL = 5,  // as W_ROWS, fetched straight into LDS (paired with X_PLAIN_DL)
    W_KMAJOR_DL = 6,  // as W_KMAJOR, fetched straight into LDS (paired with X_PLAIN_DL)
};

// Direct-to-LDS pipeline (X_PLAIN_DL): `buffer_load_dwordx4 ... lds` writes lane l's 16 bytes at base + 16 l, so a
// wavefront instruction fills 1 KiB of LDS and which global piece lands in which 16-byte slot is the lane's choice.
// Tiles are stored unpadded ([rows][64] for row operands, [64][BN] for the K-major operand) with the pieces
// XOR-swizzled so that the 128-bit / transposing 64-bit operand reads stay free of bank conflicts:
//   row operand:  piece p (0..3) of row r sits in slot p ^ ((r >> 2) & 3) of the row;
//   K-major:      the 32-byte unit u of K row k sits in unit u ^ ((k / (256 / BN)) % (BN / 32)).
// STAGES K steps are resident; one barrier per step.
// Four stages; eight (tried on the 128 x 128 tile, 128 KiB) changed nothing: the fetch path, not the number of
// requests in flight, bounds the loop.
template <int BM, int BN>
constexpr int dl_stages() {
    return 4;
}
// One wavefront-wide 16-byte-per-lane load from a buffer resource straight into LDS at `lds_addr` + 16 * lane.
// Written as inline assembly on purpose: the compiler orders every LDS read after ALL outstanding loads of this kind
// (it cannot tell which bytes they write), which would drain the whole stage ring at every step; the loop below does
// its own counting with s_waitcnt vmcnt(N).  M0 holds the LDS address for this one instruction only; nothing else
// in these kernels keeps a value in M0.
__device__ __forceinline__ void load16_to_lds(v4i rsrc, uint32_t lds_addr, uint32_t offset, uint32_t scalar_offset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds_addr), "v"(offset),
                 "s"(rsrc), "s"(scalar_offset)
                 : "memory");
}
__device__ __forceinline__ v4i make_rsrc_words(const void *p, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(p);
    return v4i{(int)(uint32_t)a, (int)(uint32_t)(a >> 32), (int)bytes, 0x00020000};
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // s_waitcnt vmcnt(N) only (expcnt / lgkmcnt untouched)
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int XMODE, int WMODE, bool SUMS, bool Q8, bool RES = false>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64) gemm_i8_kernel(const GemmArgs g) {
    static_assert(!RES || Q8, "the residual stage follows the 8-bit epilogue");
    constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wavefront sub-tile
    constexpr int TM = WM / 32, TN = WN / 32;            // 32x32 MFMA tiles per wavefront
    constexpr int XROWS = BM * 4 / NTHREADS;             // X rows per thread (4 pieces of 16 B per row)
    constexpr int WCHUNKS = (BN * 4 + NTHREADS - 1) / NTHREADS;
    static_assert(WAVES_M * WAVES_N == 4 || WAVES_M * WAVES_N == 8, "four or eight wavefronts per block");
    static_assert((BM * 4) % NTHREADS == 0, "whole X rows per thread");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wavefront tile is a multiple of the 32x32 MFMA tile");

    constexpr int PW = BN + 16;           // W_KMAJOR: LDS pitch of one K row of BN channels (bytes)
    constexpr int WBUF = w_buf_bytes<BN>();  // one W buffer: [BN][PITCH] or [BK][PW], whichever is larger
    constexpr int N16 = BN / 16;          // 16-byte pieces per K row of the K-major tile

    extern __shared__ __align__(16) char smem[];
    constexpr bool DL = XMODE == X_PLAIN_DL;
    static_assert(DL == (WMODE == W_ROWS_DL || WMODE == W_KMAJOR_DL), "the direct-to-LDS modes come as a pair");
    constexpr int DL_S = dl_stages<BM, BN>();
    constexpr int DL_STAGE = (BM + BN) * BK;  // one stage: X tile [BM][64] then W tile
    char *xs = smem;                     // [2][BM][PITCH]
    char *ws = smem + 2 * BM * PITCH;    // [2][WBUF]

    // ---- XCD-aware tile assignment: consecutive block ids land on different XCDs (8 of them, each with its own
    // L2), so block b is given tile (b % 8) * chunk + b / 8: tiles that share operands stay on one XCD.
    // Every argument that the tile assignment and the first operand requests depend on is asked for here, in one
    // batch: left alone the compiler loads arguments where they are first used, behind the early exit and behind each
    // other's results, and a wavefront waits for several trips to memory in a row before its first address.
    asm volatile("" ::"s"(g.chunk), "s"(g.total_tiles), "s"(g.splits), "s"(g.tiles_m), "s"(g.tiles_n),
                 "s"(g.div_tiles_per_batch.m), "s"(g.div_tiles_per_batch.s), "s"(g.div_tiles_n.m), "s"(g.div_tiles_n.s),
                 "s"(g.div_band.m), "s"(g.div_band.s), "s"(g.div_last_rows.m), "s"(g.div_last_rows.s), "s"(g.x), "s"(g.w),
                 "s"(g.x_batch), "s"(g.w_batch), "s"(g.M), "s"(g.N), "s"(g.K), "s"(g.x_sx), "s"(g.ldw), "s"(g.x_bytes),
                 "s"(g.w_bytes));
    // The epilogue's arguments ride along: the compiler asks for them up here in any case, but behind the early exit
    // and in registers that the tile assignment is still writing, so the assignment waited for them to arrive first.
    asm volatile("" ::"s"(g.out), "s"(g.out_batch), "s"(g.ldo), "s"(g.o_bytes), "s"(g.fused), "s"(g.mult), "s"(g.shift),
                 "s"(g.mult16), "s"(g.rp.in_zp), "s"(g.rp.out_zp), "s"(g.rp.out_lo), "s"(g.rp.out_hi),
                 "s"(g.rp.double_round), "s"(g.rp.per_channel), "s"(g.rp.clamp_out), "s"(g.zx), "s"(g.zw), "s"(g.bias),
                 "s"(g.bias_len));
    const int lin_all = (int)(blockIdx.x % 8) * g.chunk + (int)(blockIdx.x / 8);
    if (lin_all >= g.total_tiles * g.splits) return;
    // the splits of one tile are consecutive, so they run on one XCD and exchange their partials through its L2
    int lin = lin_all, split = 0;
    if (XMODE != X_PLAIN_DL && g.splits > 1) {
        lin = __builtin_amdgcn_readfirstlane(lin_all / g.splits);
        split = lin_all - lin * g.splits;
    }
    const int step0 = split * g.split_steps;                                  // first K step of this block
    const int nk_own = min(g.split_steps, (g.K + BK - 1) / BK - step0);       // and how many it multiplies
    const int k_begin = step0 * BK;
    const int k_len = min(g.K, k_begin + nk_own * BK) - k_begin;              // bytes of K in this block's range
    const int tiles_per_batch = g.tiles_m * g.tiles_n;
    const int batch = div_magic(lin, g.div_tiles_per_batch);
    const int t_in = lin - batch * tiles_per_batch;
    // Tiles are walked in bands of GROUP_M tile rows, column by column inside a band: the blocks that run at the
    // same time on one XCD then share a few row panels of X and a few column panels of W in its L2, instead of one
    // row panel and every column panel.
    int tile_m, tile_n;
    if (g.tiles_m >= 2 * kGroupM) {
        const int band = div_magic(t_in, g.div_band);
        const int first = band * kGroupM;
        const int rows = min(kGroupM, g.tiles_m - first);
        const int r = t_in - band * kGroupM * g.tiles_n;
        tile_n = rows == kGroupM ? r / kGroupM : div_magic(r, g.div_last_rows);
        tile_m = first + r - tile_n * rows;
    } else {
        tile_m = div_magic(t_in, g.div_tiles_n);
        tile_n = t_in - tile_m * g.tiles_n;
    }
    const int m_base = tile_m * BM, n_base = tile_n * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;

    const int8_t *xb = g.x + (int64_t)batch * g.x_batch;
    const int8_t *wb = g.w + (int64_t)batch * g.w_batch;

    // ---- per-channel epilogue constants.  The accumulators of a wavefront end up with one output channel per lane
    // (lane % 32 of each 32-channel group j), so every lane loads the bias, multiplier and shift of its own TN
    // channels.  The loads are issued here, ahead of the operand prefetch, but only consumed after the main loop, so
    // their latency is never waited for.
    int32_t chan_bias[TN], chan_mult[TN], chan_shift[TN];
    auto load_chan_constants = [&]() {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int gn = n_base + wave_n * WN + j * 32 + (lane & 31);
            chan_bias[j] = chan_mult[j] = chan_shift[j] = 0;
            if (gn < g.N) {
                chan_bias[j] = (g.bias && split == 0) ? g.bias[g.bias_len == 1 ? 0 : gn] : 0;
                if (g.fused) {
                    const int ci = g.rp.per_channel ? gn : 0;
                    chan_mult[j] = g.mult16 ? (int32_t) reinterpret_cast<const int16_t *>(g.mult)[ci]
                                            : reinterpret_cast<const int32_t *>(g.mult)[ci];
                    chan_shift[j] = (int32_t)g.shift[ci];
                }
            }
        }
    };
    // (the direct-to-LDS form requests its first operand stages before anything else and these constants behind them)
    if constexpr (XMODE != X_PLAIN_DL) load_chan_constants();

    // ---- loader state
    const int x_kc = tid & 3;  // which 16-byte piece of the 64-byte K step this thread stages
    RowState rows[XROWS];      // X_GENERIC: pointers; X_TAP: tap origin
    uint32_t xoff[XROWS];      // fast modes: byte offset of the row (X_PLAIN) / image (X_TAP), or kOobOffset
#pragma unroll
    for (int i = 0; i < XROWS; i++) {
        const int m = m_base + (tid >> 2) + (NTHREADS / 4) * i;
        RowState r{xb, 0, 0, m < g.M};
        xoff[i] = kOobOffset;
        if (r.valid) {
            if (g.plain) {
                r.base = xb + (int64_t)m * g.x_sx;
                xoff[i] = (uint32_t)m * (uint32_t)g.x_sx + x_kc * 16;
            } else {
                const int img = m / g.OHW, rem = m - img * g.OHW;
                const int oy = rem / g.OW, ox = rem - oy * g.OW;
                r.base = xb + (int64_t)img * g.x_sn;
                r.iy0 = oy * g.sy - g.pad_t;
                r.ix0 = ox * g.sx - g.pad_l;
                xoff[i] = (uint32_t)img * (uint32_t)g.x_sn + x_kc * 16;
            }
        }
        rows[i] = r;
    }
    KState ks{0, 0, 0};                      // X_GENERIC: k position of this thread's piece
    if (XMODE == X_GENERIC) kstate_advance(ks, k_begin + x_kc * 16, g.IC, g.KW);
    int tap_ky = 0, tap_kx = 0, tap_ic = 0;  // X_TAP: uniform position of the K step
    if (XMODE == X_TAP && k_begin > 0) {
        const int tap = k_begin / g.IC;
        tap_ic = k_begin - tap * g.IC;
        tap_ky = tap / g.KW;
        tap_kx = tap - tap_ky * g.KW;
    }
    const __amdgpu_buffer_rsrc_t xres = make_rsrc(xb, g.x_bytes), wres = make_rsrc(wb, g.w_bytes);

    uint32_t woff[WCHUNKS];  // fast modes: byte offset of the piece at k = 0, or kOobOffset
#pragma unroll
    for (int i = 0; i < WCHUNKS; i++) {
        const int c = tid + NTHREADS * i;
        woff[i] = kOobOffset;
        if (c < BN * 4) {
            if (WMODE == W_ROWS || WMODE == W_ROWS4) {
                const int n = n_base + (c >> 2);
                if (n < g.N) woff[i] = (uint32_t)n * (uint32_t)g.ldw + (c & 3) * 16;
            } else if (WMODE == W_KMAJOR || WMODE == W_KMAJOR4) {
                // piece c = 16 channels of K row c / N16; rows at or beyond K lie past the end of the buffer
                // resource and read as 0 without a test
                const int n = n_base + (c % N16) * 16;
                if (n < g.N) woff[i] = (uint32_t)(c / N16) * (uint32_t)g.ldw + n;
            }
        }
    }

    // global -> registers for the K step starting at k0 (the steps are requested in increasing order)
    auto prefetch = [&](int k0, uint4 (&xr)[XROWS], uint4 (&wr)[WCHUNKS], uint32_t &xpad) {
        xpad = 0;
        if (XMODE == X_PLAIN) {
            const bool kin = k0 + x_kc * 16 < g.K;
#pragma unroll
            for (int i = 0; i < XROWS; i++) xr[i] = buf_load16(xres, kin ? xoff[i] + (uint32_t)k0 : kOobOffset);
        } else if (XMODE == X_PLAIN4) {
            const int kp = k0 + x_kc * 16;  // K % 4 == 0: a dword lies wholly inside or outside the row
#pragma unroll
            for (int i = 0; i < XROWS; i++) {
                const uint32_t off = xoff[i] + (uint32_t)k0;
                const bool v = xoff[i] != kOobOffset;
                xr[i].x = buf_load4(xres, (v && kp + 0 < g.K) ? off + 0 : kOobOffset);
                xr[i].y = buf_load4(xres, (v && kp + 4 < g.K) ? off + 4 : kOobOffset);
                xr[i].z = buf_load4(xres, (v && kp + 8 < g.K) ? off + 8 : kOobOffset);
                xr[i].w = buf_load4(xres, (v && kp + 12 < g.K) ? off + 12 : kOobOffset);
            }
        } else if (XMODE == X_TAP) {
            const bool kin = tap_ky < g.KH;
            const int oy = tap_ky * g.dy, ox = tap_kx * g.dx;
#pragma unroll
            for (int i = 0; i < XROWS; i++) {
                const int y = rows[i].iy0 + oy, x = rows[i].ix0 + ox;
                const bool inb = (unsigned)y < (unsigned)g.H && (unsigned)x < (unsigned)g.W;
                const uint32_t off = xoff[i] + (uint32_t)y * (uint32_t)g.x_sy + (uint32_t)x * (uint32_t)g.x_sx +
                                     (uint32_t)tap_ic;
                xr[i] = buf_load16(xres, (kin && inb && rows[i].valid) ? off : kOobOffset);
                if (kin && !inb && rows[i].valid) xpad |= 1u << i;  // a padded tap: filled with zx when staged
            }
            tap_ic += BK;
            if (tap_ic >= g.IC) {
                tap_ic = 0;
                if (++tap_kx == g.KW) {
                    tap_kx = 0;
                    ++tap_ky;
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < XROWS; i++) xr[i] = load_x_chunk(g, rows[i], ks);
            kstate_advance(ks, BK, g.IC, g.KW);
        }
        if (WMODE == W_ROWS) {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const int c = tid + NTHREADS * i;
                const bool kin = k0 + (c & 3) * 16 < g.K;
                wr[i] = buf_load16(wres, kin ? woff[i] + (uint32_t)k0 : kOobOffset);
            }
        } else if (WMODE == W_ROWS4) {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const int kp = k0 + ((tid + NTHREADS * i) & 3) * 16;
                const uint32_t off = woff[i] + (uint32_t)k0;
                const bool v = woff[i] != kOobOffset;
                wr[i].x = buf_load4(wres, (v && kp + 0 < g.K) ? off + 0 : kOobOffset);
                wr[i].y = buf_load4(wres, (v && kp + 4 < g.K) ? off + 4 : kOobOffset);
                wr[i].z = buf_load4(wres, (v && kp + 8 < g.K) ? off + 8 : kOobOffset);
                wr[i].w = buf_load4(wres, (v && kp + 12 < g.K) ? off + 12 : kOobOffset);
            }
        } else if (WMODE == W_KMAJOR || WMODE == W_KMAJOR4) {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const uint32_t off = woff[i] + (uint32_t)k0 * (uint32_t)g.ldw;
                if (WMODE == W_KMAJOR) {
                    wr[i] = buf_load16(wres, off);
                } else {  // rows are only dword aligned: four loads, channels at or beyond N masked
                    const int n = n_base + ((tid + NTHREADS * i) % N16) * 16;
                    wr[i].x = buf_load4(wres, n + 0 < g.N ? off + 0 : kOobOffset);
                    wr[i].y = buf_load4(wres, n + 4 < g.N ? off + 4 : kOobOffset);
                    wr[i].z = buf_load4(wres, n + 8 < g.N ? off + 8 : kOobOffset);
                    wr[i].w = buf_load4(wres, n + 12 < g.N ? off + 12 : kOobOffset);
                }
            }
        } else if (!g.w_kmajor) {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const int c = tid + NTHREADS * i;
                if (c < BN * 4) wr[i] = load_w_chunk(g, wb, n_base + (c >> 2), k0 + (c & 3) * 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const int c = tid + NTHREADS * i;
                if (c < BN * 4) wr[i] = load_w_block_kmajor(g, wb, n_base + (c % (BN / 4)) * 4, k0 + (c / (BN / 4)) * 4);
            }
        }
    };
    // registers -> LDS buffer `buf`
    auto stage = [&](int buf, const uint4 (&xr)[XROWS], const uint4 (&wr)[WCHUNKS], uint32_t xpad) {
        char *xd = xs + buf * BM * PITCH;
        char *wd = ws + buf * WBUF;
        const uint32_t z = splat8(g.zx);
#pragma unroll
        for (int i = 0; i < XROWS; i++) {
            uint4 v = xr[i];
            if (XMODE == X_TAP && ((xpad >> i) & 1u)) v = make_uint4(z, z, z, z);
            *reinterpret_cast<uint4 *>(xd + ((tid >> 2) + (NTHREADS / 4) * i) * PITCH + x_kc * 16) = v;
        }
        if (WMODE == W_KMAJOR || WMODE == W_KMAJOR4) {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const int c = tid + NTHREADS * i;
                if (c < BN * 4) *reinterpret_cast<uint4 *>(wd + (c / N16) * PW + (c % N16) * 16) = wr[i];
            }
        } else if (WMODE == W_ROWS || WMODE == W_ROWS4 || !g.w_kmajor) {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const int c = tid + NTHREADS * i;
                if (c < BN * 4) *reinterpret_cast<uint4 *>(wd + (c >> 2) * PITCH + (c & 3) * 16) = wr[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < WCHUNKS; i++) {
                const int c = tid + NTHREADS * i;
                if (c < BN * 4) {
                    const int nl = (c % (BN / 4)) * 4, kl = (c / (BN / 4)) * 4;
                    *reinterpret_cast<uint32_t *>(wd + (nl + 0) * PITCH + kl) = wr[i].x;
                    *reinterpret_cast<uint32_t *>(wd + (nl + 1) * PITCH + kl) = wr[i].y;
                    *reinterpret_cast<uint32_t *>(wd + (nl + 2) * PITCH + kl) = wr[i].z;
                    *reinterpret_cast<uint32_t *>(wd + (nl + 3) * PITCH + kl) = wr[i].w;
                }
            }
        }
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    int32_t xsum[TM], wsum[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) xsum[i] = 0;
#pragma unroll
    for (int j = 0; j < TN; j++) wsum[j] = 0;
    const bool need_xsum = SUMS && g.zw != 0, need_wsum = SUMS && g.zx != 0;

    auto compute = [&](int buf) {
        const char *xd = xs + buf * BM * PITCH + (wave_m * WM + (lane & 31)) * PITCH + (lane >> 5) * 16;
        const char *wd = ws + buf * WBUF + (wave_n * WN + (lane & 31)) * PITCH + (lane >> 5) * 16;
        // K-major tile: a 16-lane group transposes an 8(k) x 16(n) byte block; lane L of the group supplies the
        // address of K row L / 2, channel half L % 2, and receives the 8 k-bytes of channel L.  Groups 0/1 cover
        // channels 0-15 / 16-31 of the tile for k 0-15, groups 2/3 the same channels for k 16-31.
        const char *wt = ws + buf * WBUF + ((lane >> 5) * 16 + ((lane & 15) >> 1)) * PW + wave_n * WN +
                         ((lane >> 4) & 1) * 16 + (lane & 1) * 8;
#pragma unroll
        for (int kk = 0; kk < BK / 32; kk++) {
            v4i xf[TM], wf[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) xf[i] = *reinterpret_cast<const v4i *>(xd + i * 32 * PITCH + kk * 32);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (WMODE == W_KMAJOR || WMODE == W_KMAJOR4) {
                    const char *p = wt + kk * 32 * PW + j * 32;
                    const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)(p));
                    const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)(p + 8 * PW));
                    wf[j] = v4i{lo.x, lo.y, hi.x, hi.y};
                } else {
                    wf[j] = *reinterpret_cast<const v4i *>(wd + j * 32 * PITCH + kk * 32);
                }
            }
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[i], wf[j], acc[i][j], 0, 0, 0);
            if (SUMS) {  // both sums are kept whenever a zero point is non-zero: 16 dot4 beside 8 MFMAs
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int q = 0; q < 4; q++) xsum[i] = __builtin_amdgcn_sdot4(xf[i][q], 0x01010101, xsum[i], false);
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) wsum[j] = __builtin_amdgcn_sdot4(wf[j][q], 0x01010101, wsum[j], false);
            }
        }
    };

    if constexpr (DL) {
        // ---- direct-to-LDS main loop (K % 64 == 0).  The matrix-core instructions and everything else a wavefront
        // does share one issue stream, so what need not be in the loop is kept out of it: the K advance of the
        // requests rides in the scalar offset of the buffer instruction, the stage ring is unrolled so that LDS
        // addresses are lane base + immediate, and the zero-point sums of a K half are taken by one wavefront only
        // (combined through LDS after the loop).
        constexpr int XI = BM * 4 / NTHREADS, WI = BN * 4 / NTHREADS;  // 16-byte pieces per thread and stage
        static_assert((BN * 4) % NTHREADS == 0 && BN % 32 == 0 && BN <= 256, "whole W pieces per thread");
        static_assert((DL_S == 4 || DL_S == 8) && WAVES_M == 2 && WAVES_N >= 2, "ring of four or eight stages, 2 x N wavefronts");
        constexpr int P16 = BN / 16, UN = BN / 32, RP = 256 / BN;  // K-major: pieces / units per row, rows per 256 B
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        uint32_t xo[XI], wo[WI];
#pragma unroll
        for (int i = 0; i < XI; i++) {
            const int q = i * NTHREADS + tid, r = q >> 2, p = (q & 3) ^ ((r >> 2) & 3);
            const int m = m_base + r;
            xo[i] = m < g.M ? (uint32_t)m * (uint32_t)g.x_sx + (uint32_t)(p * 16) : kOobOffset;
        }
#pragma unroll
        for (int i = 0; i < WI; i++) {
            const int q = i * NTHREADS + tid;
            if (WMODE == W_ROWS_DL) {
                const int r = q >> 2, p = (q & 3) ^ ((r >> 2) & 3);
                const int n = n_base + r;
                wo[i] = n < g.N ? (uint32_t)n * (uint32_t)g.ldw + (uint32_t)(p * 16) : kOobOffset;
            } else {
                const int kr = q / P16, c = q % P16;
                const int u = (c >> 1) ^ ((kr / RP) % UN);
                const int n = n_base + u * 32 + (c & 1) * 16;
                wo[i] = n < g.N ? (uint32_t)kr * (uint32_t)g.ldw + (uint32_t)n : kOobOffset;
            }
        }
        const v4i xres4 = make_rsrc_words(xb, g.x_bytes), wres4 = make_rsrc_words(wb, g.w_bytes);
        const uint32_t lds0 = (uint32_t) reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char *)smem) +
                              (uint32_t)(wave_u * 1024);
        const uint32_t w_kstep = WMODE == W_ROWS_DL ? (uint32_t)BK : (uint32_t)BK * (uint32_t)g.ldw;
        // operand addresses inside a stage: lane base (per K half) + compile-time offset
        const int h = lane >> 5;
        const int xswz = ((lane >> 2) & 3);
        const int kfun = WMODE == W_KMAJOR_DL ? (((lane & 15) >> 1) / RP) % UN : 0;
        const char *x_base[2], *w_base[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int slot = ((kk * 2 + h) ^ xswz) * 16;
            x_base[kk] = smem + (wave_m * WM + (lane & 31)) * BK + slot;
            if (WMODE == W_KMAJOR_DL)
                w_base[kk] = smem + BM * BK + (kk * 32 + h * 16 + ((lane & 15) >> 1)) * BN + ((lane >> 4) & 1) * 16 +
                             (lane & 1) * 8;
            else
                w_base[kk] = smem + BM * BK + (wave_n * WN + (lane & 31)) * BK + slot;
        }
        // ---- the loop.  A wavefront issues in order and is alone on its SIMD here, so whatever is not a matrix
        // instruction delays the next one unless it is issued while the matrix core works on the last (35 clocks
        // per instruction on random operands).  Measured on one wavefront per SIMD: shared-memory reads, loads into
        // shared memory and ordinary vector instructions (v_add, v_xor, v_sad_u8) issue in that shadow for free;
        // v_dot4 does not (a dot product and a matrix instruction take turns), and four loads issued back to back
        // hold the wavefront for 3 x 64 clocks (the address path takes a wavefront's kilobyte in 64).  A K half is
        // therefore one straight line: a matrix instruction, then a share of the next half's operand reads, of the
        // requests and of the zero-point sums, then the next matrix instruction.  (Steps of 0.40 us became 0.22 us
        // on 8 x 512 x 1024 x 1024; the requests alone, with the same barrier and waits, take 0.165 us per step.)
        //
        // Zero-point sums on the matrix cores, one small instruction per operand fragment: the 16 bytes a lane holds
        // for v_mfma_i32_32x32x32_i8 (row lane % 32, K bytes 16 (lane / 32) ...) are, read as an operand of
        // v_mfma_i32_16x16x64_i8 (row lane % 16, K block lane / 16), row r of the fragment in K blocks 0 and 2 of row
        // r % 16 when r < 16 and in blocks 1 and 3 when r >= 16.  Against a constant operand that is all ones in
        // blocks 0 and 2 for its first eight columns and in blocks 1 and 3 for the other eight, the 16 x 16 result holds
        // sum_k of row r (< 16) in columns 0 - 7 and of row r + 16 in columns 8 - 15: four accumulator registers and
        // 16 clocks of the matrix core per fragment, where v_dot4 takes four instructions that take turns with the
        // matrix instructions and v_xor + v_sad_u8 eight that crowd the issue stream (measured per K step of a
        // 128 x 128 tile: about 35 clocks against 217 and 142).  Which wavefront sums what in which
        // K half (wave-uniform, fixed for the kernel): with 2 x 2 wavefronts the two that share a row panel take one
        // K half each and so do the two that share a channel panel, arranged so that every wavefront has exactly one
        // of the two duties in every half; otherwise the first two wavefront columns take the row panels' halves
        // and the wavefront rows the channel panels' halves.
        const int sel_w = (((lane & 15) < 8) != (((lane >> 4) & 1) != 0)) ? 0x01010101 : 0;
        const v4i selv = v4i{sel_w, sel_w, sel_w, sel_w};
        v4i sx4[TM], sw4[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) sx4[i] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < TN; j++) sw4[j] = v4i{0, 0, 0, 0};
        const int wave_n_u = __builtin_amdgcn_readfirstlane(wave_n), wave_m_u = __builtin_amdgcn_readfirstlane(wave_m);
        constexpr bool BALANCED = WAVES_M == 2 && WAVES_N == 2;
        bool dx[2], dw[2];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
            dx[hh] = need_xsum && (BALANCED ? wave_n_u == (wave_m_u ^ hh) : wave_n_u == hh);
            dw[hh] = need_wsum && (BALANCED ? wave_n_u != (wave_m_u ^ hh) : wave_m_u == hh);
        }
        constexpr bool KM = WMODE == W_KMAJOR_DL;
        const v4i null4 = v4i{xres4[0], xres4[1], 0, xres4[3]};  // no bytes: a request through it fetches nothing
        const int nk = g.K / BK;
        // one K half: multiplies (xc, wc), reads K half `rkk` of stage `rbuf` into (xn, wn), and -- after the step's
        // barrier -- requests stage `ibuf` (K step `istep`, nothing beyond the last step)
        auto half = [&](auto dx_t, auto dw_t, auto issue_t, auto steady_t, const v4i(&xc)[TM], const v4i(&wc)[TN],
                        v4i(&xn)[TM], v4i(&wn)[TN], int rbuf, int rkk, int ibuf, int istep) {
            // LP: 1 when the stage's requests ride in this half (the one behind the step's barrier), 0 otherwise
            constexpr bool DX = decltype(dx_t)::value, DW = decltype(dw_t)::value;
            constexpr int LP = decltype(issue_t)::value;
            constexpr bool ISSUE = LP != 0;
            constexpr int NM = TM * TN;
            constexpr int NR = TM + TN * (KM ? 2 : 1), RPER = (NR + NM / 2 - 1) / (NM / 2);  // reads early in the half
            constexpr int NS = (DX ? TM : 0) + (DW ? TN : 0), SPER = (NS + NM - 1) / NM;
            constexpr int NLA = XI + WI, L0 = 0, L1 = LP == 1 ? NLA : 0;
            constexpr int NL = L1 - L0, LPER = (NL + NM - 1) / NM;
            // (steady: the caller knows that the requested step exists, and the choice of the resource falls away)
            const bool live = ISSUE && (decltype(steady_t)::value || istep < nk);
            const v4i xr = live ? xres4 : null4, wr = live ? wres4 : null4;
            const uint32_t xd = lds0 + (uint32_t)(ibuf * DL_STAGE), wd = xd + BM * BK;
            const uint32_t xk = (uint32_t)istep * BK, wk = (uint32_t)istep * w_kstep;
#pragma unroll
            for (int t = 0; t < NM; t++) {
                const int i = t / TN, j = t % TN;
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xc[i], wc[j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < RPER; u++) {
                    const int r = t * RPER + u;
                    if (r < TM) {
                        xn[r] = *reinterpret_cast<const v4i *>(x_base[rkk] + rbuf * DL_STAGE + r * 32 * BK);
                    } else if (r < NR) {
                        const int e = r - TM;
                        if (KM) {
                            const int jj = e >> 1;
                            const char *pw = w_base[rkk] + rbuf * DL_STAGE + (((wave_n * WN / 32 + jj) ^ kfun) * 32);
                            const v2i part = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)(pw + (e & 1) * 8 * BN));
                            if (e & 1) {
                                wn[jj][2] = part.x;
                                wn[jj][3] = part.y;
                            } else {
                                wn[jj][0] = part.x;
                                wn[jj][1] = part.y;
                            }
                        } else {
                            wn[e] = *reinterpret_cast<const v4i *>(w_base[rkk] + rbuf * DL_STAGE + e * 32 * BK);
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < LPER; u++) {
                    const int l = L0 + t * LPER + u;
                    if (l < L1) {
                        if (l < XI) load16_to_lds(xr, xd + l * NTHREADS * 16, xo[l], xk);
                        else load16_to_lds(wr, wd + (l - XI) * NTHREADS * 16, wo[l - XI], wk);
                    }
                }
#pragma unroll
                for (int u = 0; u < SPER; u++) {
                    const int f = t * SPER + u;  // fragment of the duty: row tiles first
                    if (f < NS) {
                        if (DX && f < TM) {
                            sx4[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xc[f], selv, sx4[f], 0, 0, 0);
                        } else {
                            const int jj = f - (DX ? TM : 0);
                            sw4[jj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(selv, wc[jj], sw4[jj], 0, 0, 0);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        using T_ = std::true_type;
        using F_ = std::false_type;
        // Stage s lives in buffer s % DL_S; DL_S - 1 stages are requested ahead, every step requests one more (beyond
        // the last step through the empty resource, so that the number of requests in flight is the same at every
        // step and the waits below count exactly).  While the first K half of step s is multiplied the second half
        // is read, and while the second half is multiplied the first half of step s + 1 is read.  In between sits
        // the one barrier of the step: at most DL_S - 3 stages of this thread's requests outstanding means its part
        // of stage s + 1 has landed; the barrier extends that to every thread's part and also says that every
        // wavefront has received its reads of stage s - 1, whose buffer the step's request overwrites.
        v4i xf0[TM], wf0[TN], xf1[TM], wf1[TN];
#pragma unroll
        for (int d = 0; d < DL_S - 1; d++) {
            const v4i xr = d < nk ? xres4 : null4, wr = d < nk ? wres4 : null4;
            const uint32_t xd = lds0 + (uint32_t)(d * DL_STAGE), wd = xd + BM * BK;
#pragma unroll
            for (int l = 0; l < XI + WI; l++) {
                if (l < XI) load16_to_lds(xr, xd + l * NTHREADS * 16, xo[l], (uint32_t)d * BK);
                else load16_to_lds(wr, wd + (l - XI) * NTHREADS * 16, wo[l - XI], (uint32_t)d * w_kstep);
            }
        }
        // the epilogue's per-channel constants: requested behind the first stages, used behind the loop.  They are
        // younger than the first stages and older than every later request, so the counted waits below and in the
        // loop hold with them in flight (how many there are depends on the operator: the waits count none of them,
        // which only makes the first ones wait for a few requests more).
        load_chan_constants();
        wait_vmcnt<(DL_S - 2) * (XI + WI)>();  // stage 0 has landed: what was requested behind it may be in flight
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < TM; i++) xf0[i] = *reinterpret_cast<const v4i *>(x_base[0] + i * 32 * BK);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if (KM) {
                const char *pw = w_base[0] + (((wave_n * WN / 32 + j) ^ kfun) * 32);
                const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)(pw));
                const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)(pw + 8 * BN));
                wf0[j] = v4i{lo.x, lo.y, hi.x, hi.y};
            } else {
                wf0[j] = *reinterpret_cast<const v4i *>(w_base[0] + j * 32 * BK);
            }
        }
        // The loop exists once per combination of duties (a template argument each) and the wavefront picks its copy
        // in front of it: chosen inside the loop, the variants of a half would meet again behind it, and the register
        // allocator then has them leave the accumulators in different registers and copies all 64 at every joint.
        auto loop = [&](auto dx0_t, auto dw0_t, auto dx1_t, auto dw1_t) {
            // groups of DL_S steps that all still have a step to request run without the tests of the general form
            int step = 0;
            for (; step + 2 * DL_S - 1 <= nk; step += DL_S) {
#pragma unroll
                for (int d = 0; d < DL_S; d++) {
                    half(dx0_t, dw0_t, std::integral_constant<int, 0>{}, T_{}, xf0, wf0, xf1, wf1, d, 1, 0, 0);
                    wait_vmcnt<(DL_S - 3) * (XI + WI)>();
                    asm volatile("" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    half(dx1_t, dw1_t, std::integral_constant<int, 1>{}, T_{}, xf1, wf1, xf0, wf0, (d + 1) % DL_S, 0,
                         (d + DL_S - 1) % DL_S, step + d + DL_S - 1);
                }
            }
            for (; step < nk; step += DL_S) {
#pragma unroll
                for (int d = 0; d < DL_S; d++) {
                    if (step + d < nk) {  // uniform
                        half(dx0_t, dw0_t, std::integral_constant<int, 0>{}, F_{}, xf0, wf0, xf1, wf1, d, 1, 0, 0);
                        wait_vmcnt<(DL_S - 3) * (XI + WI)>();
                        asm volatile("" ::: "memory");
                        __builtin_amdgcn_s_barrier();
                        asm volatile("" ::: "memory");
                        half(dx1_t, dw1_t, std::integral_constant<int, 1>{}, F_{}, xf1, wf1, xf0, wf0, (d + 1) % DL_S, 0,
                             (d + DL_S - 1) % DL_S, step + d + DL_S - 1);
                    }
                }
            }
        };
        // a wavefront never has the same duty in both halves, and with balanced duties never both in one half
        const int duties = !SUMS ? 0 : (int)dx[0] | ((int)dw[0] << 1) | ((int)dx[1] << 2) | ((int)dw[1] << 3);
#define MLEL_DUTY_CASE(C)                                                                                          \
    case C:                                                                                                        \
        if constexpr (SUMS && !((C & 5) == 5) && !((C & 10) == 10) && !(BALANCED && ((C & 3) == 3 || (C & 12) == 12)))   \
            loop(std::bool_constant<(C & 1) != 0>{}, std::bool_constant<(C & 2) != 0>{},                           \
                 std::bool_constant<(C & 4) != 0>{}, std::bool_constant<(C & 8) != 0>{});                          \
        break;
        switch (duties) {
            MLEL_DUTY_CASE(1) MLEL_DUTY_CASE(2) MLEL_DUTY_CASE(3) MLEL_DUTY_CASE(4) MLEL_DUTY_CASE(6) MLEL_DUTY_CASE(8)
            MLEL_DUTY_CASE(9) MLEL_DUTY_CASE(12)
        default: loop(F_{}, F_{}, F_{}, F_{}); break;
        }
#undef MLEL_DUTY_CASE
        wait_vmcnt<0>();  // the requests beyond the last step write (zeros) into the ring, which the epilogue reuses
        __syncthreads();
        // ---- combine the split zero-point sums: afterwards every wavefront holds, per lane half, partial sums whose
        // total over the two halves is the full sum of its rows (X) and of its channels (W), as in the other fetch modes
        if (SUMS) {
            int32_t *xs_l = reinterpret_cast<int32_t *>(smem) + BM;      // [2][BM]: by K half
            int32_t *ws_l = reinterpret_cast<int32_t *>(smem) + 3 * BM;  // [2][BN]: by K half
            // a fragment's row sums sit in lanes 16 g (rows 4 g .. 4 g + 3) and 16 g + 8 (rows 16 + 4 g ...), its channel
            // sums in register 0 of lanes 0 - 15 (channels 0 - 15) and 32 - 47 (channels 16 - 31)
            if (need_xsum && wave_n < 2 && (lane & 7) == 0) {
#pragma unroll
                for (int i = 0; i < TM; i++)  // times minus the weight zero point: what the epilogue adds per row
                    *reinterpret_cast<v4i *>(&xs_l[wave_n * BM + wave_m * WM + i * 32 + ((lane >> 3) & 1) * 16 + (lane >> 4) * 4]) =
                        sx4[i] * -g.zw;
            }
            if (need_wsum && (lane & 16) == 0) {
#pragma unroll
                for (int j = 0; j < TN; j++)
                    ws_l[wave_m * BN + wave_n * WN + j * 32 + (lane & 15) + ((lane >> 5) << 4)] = sw4[j][0];
            }
            __syncthreads();
            // every lane takes the whole sum of its channel from the two tables (the other fetch modes leave partial
            // sums in the two lane halves, which the epilogue adds); the row terms stay in their tables, which the
            // epilogue reads
            if (need_wsum) {
                int32_t lo[TN], hi[TN];
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int c = wave_n * WN + j * 32 + (lane & 31);
                    lo[j] = ws_l[c], hi[j] = ws_l[BN + c];
                }
#pragma unroll
                for (int j = 0; j < TN; j++) wsum[j] = lo[j] + hi[j];
            }
        }
    } else {
    // ---- main loop: a ring of DEPTH register sets keeps DEPTH - 1 K steps of global loads in flight while one
    // step is multiplied out of LDS (two LDS buffers).  At the top of sub-iteration s: LDS[s & 1] holds step s and
    // register set (s + j) % DEPTH holds step s + j for j = 1 .. DEPTH - 1; the set of step s is free again.
    // Every prefetch and stage is unconditional: a K step at or beyond K loads nothing (buffer bounds / tap state
    // return zeros) and is never multiplied, and the straight-line body lets the compiler count exactly how many
    // loads may remain in flight at each wait instead of draining them all.
    // the generic fetch state is large, and so are the register sets of the widest tiles
    constexpr int DEPTH = (XMODE == X_GENERIC || WMODE == W_GENERIC || XROWS + WCHUNKS > 4) ? 2 : 4;
    const int nk = nk_own;
    uint4 xr[DEPTH][XROWS], wr[DEPTH][WCHUNKS];
    uint32_t xp[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) prefetch(k_begin + d * BK, xr[d], wr[d], xp[d]);
    stage(0, xr[0], wr[0], xp[0]);
    __syncthreads();
    for (int step = 0; step < nk; step += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            if (step + d < nk) {  // uniform
                prefetch(k_begin + (step + d + DEPTH) * BK, xr[d], wr[d], xp[d]);
                compute(d & 1);
                stage((d + 1) & 1, xr[(d + 1) % DEPTH], wr[(d + 1) % DEPTH], xp[(d + 1) % DEPTH]);
                __syncthreads();
            }
        }
    }

    }

    // ---- after the loop a lane holds, per 32 x 32 accumulator tile (i, j) and register 4q + e, the output of
    // position 32 i + 8 q + 4 (lane / 32) + e and channel 32 j + lane % 32 of the wavefront's sub-tile: one channel per
    // lane and tile column, so everything that depends on the channel only sits in a few registers.
    const int half = lane >> 5, cl = lane & 31;
    int32_t *xs_tab = reinterpret_cast<int32_t *>(smem);  // [BM]: -zw * sum_k X[m][k]; the operand buffers are free now
    int32_t bias_adj[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        bias_adj[j] = chan_bias[j];
        if (need_wsum) {  // -zx * sum_k W[n][k] + K zx zw: the zero-point terms that depend on the channel only
            const int32_t sw = DL ? wsum[j] : wsum[j] + __shfl_xor(wsum[j], 32);
            bias_adj[j] = (int32_t)((uint32_t)bias_adj[j] - (uint32_t)g.zx * (uint32_t)sw +
                                    (uint32_t)k_len * (uint32_t)g.zx * (uint32_t)g.zw);
        }
    }
    if (need_xsum && !DL) {  // the row terms are needed by register index: through a table in shared memory
        if (wave_n == 0) {
#pragma unroll
            for (int i = 0; i < TM; i++) {
                const int32_t sx = xsum[i] + __shfl_xor(xsum[i], 32);
                if (lane < 32) xs_tab[wave_m * WM + i * 32 + lane] = (int32_t)(0u - (uint32_t)sx * (uint32_t)g.zw);
            }
        }
        __syncthreads();
    }
    // minus zw * sum_k X of the four positions of register group q of tile row i (minus, so that accumulator + channel
    // term + row term is one three-operand addition)
    auto row_terms = [&](int i, int q, int32_t (&xc)[4]) {
        if (need_xsum && DL) {  // the two K halves' tables of the direct-to-LDS loop, behind the row table's place
            const int32_t *p0 = xs_tab + BM + wave_m * WM + i * 32 + 8 * q + 4 * half;
            const int4 t = *reinterpret_cast<const int4 *>(p0), u = *reinterpret_cast<const int4 *>(p0 + BM);
            xc[0] = t.x + u.x, xc[1] = t.y + u.y, xc[2] = t.z + u.z, xc[3] = t.w + u.w;
        } else if (need_xsum) {
            const int4 t = *reinterpret_cast<const int4 *>(xs_tab + wave_m * WM + i * 32 + 8 * q + 4 * half);
            xc[0] = t.x, xc[1] = t.y, xc[2] = t.z, xc[3] = t.w;
        } else {
            xc[0] = xc[1] = xc[2] = xc[3] = 0;
        }
    };
    bool rows_done = false;  // split K: the row and channel terms are already inside the accumulators

    if constexpr (XMODE != X_PLAIN_DL) {
        if (g.splits > 1) {
            // ---- split K: this block's partial tile, complete with the bias / zero-point terms of its K range
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int32_t xc[4];
                    row_terms(i, q, xc);
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            acc[i][j][4 * q + e] = (int32_t)((uint32_t)acc[i][j][4 * q + e] + (uint32_t)bias_adj[j] +
                                                             (uint32_t)xc[e]);
                }
#pragma unroll
            for (int j = 0; j < TN; j++) bias_adj[j] = 0;
            rows_done = true;
            // The exchange uses device-scope atomic stores and loads (relaxed): they are coherent across the GPU's
            // eight L2 caches by themselves, so no fence is needed -- a device-scope fence would write back and
            // invalidate the whole L2 (measured: 20 - 50 us per launch).  Order: every thread waits until its own
            // stores have been acknowledged, the block barrier extends that to the block, then one thread counts the
            // arrival; the block that arrives last reads the others' tiles after it has seen the count.
            int32_t *mine = g.partials + ((int64_t)lin * g.splits + split) * (BM * BN) + tid;
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        __hip_atomic_store(&mine[((i * TN + j) * 16 + r) * NTHREADS], acc[i][j][r], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            int *last_flag = reinterpret_cast<int *>(smem) + BM;  // behind the row table
            __syncthreads();
            if (tid == 0) {
                const uint32_t arrived =
                    __hip_atomic_fetch_add(&g.counters[lin], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const int last = arrived == (uint32_t)(g.splits - 1);
                if (last)  // ready for the next launch
                    __hip_atomic_store(&g.counters[lin], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *last_flag = last;
            }
            __syncthreads();
            if (*last_flag == 0) return;
            for (int o = 0; o < g.splits; o++) {
                if (o == split) continue;
                const int32_t *theirs = g.partials + ((int64_t)lin * g.splits + o) * (BM * BN) + tid;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            acc[i][j][r] = (int32_t)((uint32_t)acc[i][j][r] +
                                                     (uint32_t)__hip_atomic_load(&theirs[((i * TN + j) * 16 + r) * NTHREADS],
                                                                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            }
        }
    }

    char *ob = g.out + (int64_t)batch * g.out_batch;
    if (Q8) {
        // ---- fused RESCALE(+CLAMP) to 8-bit outputs, N % 4 == 0, output extent below 2^31.  The requantisation
        // constants of a lane's channels are registers.  The four results of a register group are four consecutive
        // positions of ONE channel; a 4 x 4 byte transpose inside each group of four lanes (two lane exchanges, two
        // byte permutes) turns them into four consecutive channels of one position, which go to a staging tile in
        // shared memory as a dword.  The tile then leaves in 16-byte pieces, so that every store instruction writes
        // whole runs of a row (up to 128 bytes) instead of 8-byte fragments of 32 rows.
        constexpr int OP = BN + 32;                        // pitch of the staging tile (bytes): rows 8 banks apart
        char *so = smem + (3 * BM + 2 * BN) * 4;           // behind the tables of the zero-point sums
        static_assert((3 * BM + 2 * BN) * 4 + BM * OP <= (int)(2 * BM * PITCH + 2 * w_buf_bytes<BN>()),
                      "the staging tile fits the operand buffers");
        // Narrow tiles (fewer than 128 channels) store the dwords directly instead: runs of 32 bytes per row, without
        // the barrier and the trip through shared memory, which is what their few outputs per thread can afford.
        constexpr bool STAGED = BN >= 128;
        const __amdgpu_buffer_rsrc_t ores = make_rsrc(ob, g.o_bytes);
        const __amdgpu_buffer_rsrc_t rres =
            make_rsrc(RES ? reinterpret_cast<const char *>(g.res) + (int64_t)batch * g.out_batch : ob, g.o_bytes);
        ChanScale q_res{}, q_conv{}, q_out{};
        if (RES) {
            q_res = make_chan_scale(load_mult(g.rs_res, 0), g.rs_res.shift[0], g.rs_res.p);
            q_conv = make_chan_scale(load_mult(g.rs_conv, 0), g.rs_conv.shift[0], g.rs_conv.p);
            q_out = make_chan_scale(load_mult(g.rs_out, 0), g.rs_out.shift[0], g.rs_out.p);
        }
        ChanScale cs[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) cs[j] = make_chan_scale(chan_mult[j], chan_shift[j], g.rp);
        const uint32_t sel_a = (lane & 1) ? 0x03070105u : 0x06020400u;  // exchange with lane ^ 1
        const uint32_t sel_b = (lane & 2) ? 0x03020706u : 0x05040100u;  // exchange with lane ^ 2
        char *so_lane = so + (wave_m * WM + 4 * half + (lane & 3)) * OP + wave_n * WN + (cl & ~3);
        // direct stores: where this lane's dwords go, and the residual operand's dwords, requested before the arithmetic
        uint32_t d_off[STAGED ? 1 : TM * 4 * TN], d_res[(STAGED || !RES) ? 1 : TM * 4 * TN];
        if constexpr (!STAGED) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const int m = m_base + wave_m * WM + i * 32 + 8 * q + 4 * half + (lane & 3);
                        const int n0 = n_base + wave_n * WN + j * 32 + (cl & ~3);
                        const int k = (i * 4 + q) * TN + j;
                        d_off[k] = (m < g.M && n0 < g.N) ? (uint32_t)m * (uint32_t)g.ldo + (uint32_t)n0 : kOobOffset;
                        if constexpr (RES) d_res[k] = buf_load4(rres, d_off[k]);
                    }
        }
        // The row terms of every register group are read from their tables up front where the registers allow it: a
        // wavefront alone on its SIMD issues in order, and a read in front of each group's arithmetic made it wait for
        // a trip to shared memory (and for the staging write in front of it) once per group.
        constexpr bool ROWS_AHEAD = TM * 16 <= 32;
        int32_t xca[ROWS_AHEAD ? TM : 1][4][4];
        if constexpr (ROWS_AHEAD) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int q = 0; q < 4; q++) xca[i][q][0] = xca[i][q][1] = xca[i][q][2] = xca[i][q][3] = 0;
            if (need_xsum && !rows_done) {  // uniform: one test around all reads, so that they are issued together
                int4 t[TM][4], u[TM][4];
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int32_t *p0 = xs_tab + (DL ? BM : 0) + wave_m * WM + i * 32 + 8 * q + 4 * half;
                        t[i][q] = *reinterpret_cast<const int4 *>(p0);
                        u[i][q] = DL ? *reinterpret_cast<const int4 *>(p0 + BM) : int4{0, 0, 0, 0};
                    }
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        xca[i][q][0] = t[i][q].x + u[i][q].x, xca[i][q][1] = t[i][q].y + u[i][q].y;
                        xca[i][q][2] = t[i][q].z + u[i][q].z, xca[i][q][3] = t[i][q].w + u[i][q].w;
                    }
            }
        }
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int32_t xc[4];
                if constexpr (ROWS_AHEAD) {
                    xc[0] = xca[i][q][0], xc[1] = xca[i][q][1], xc[2] = xca[i][q][2], xc[3] = xca[i][q][3];
                } else {
                    if (!rows_done) row_terms(i, q, xc); else xc[0] = xc[1] = xc[2] = xc[3] = 0;
                }
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    int32_t v[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int32_t a = (int32_t)((uint32_t)acc[i][j][4 * q + e] + (uint32_t)bias_adj[j] + (uint32_t)xc[e]);
                        v[e] = requant_acc(a, cs[j], g.rp);
                    }
                    // bytes = positions e of this lane's channel
                    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
                    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
                    uint32_t p = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                    uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0xb1, 0xf, 0xf, true);  // lane ^ 1
                    p = __builtin_amdgcn_perm(o, p, sel_a);
                    o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0x4e, 0xf, 0xf, true);           // lane ^ 2
                    p = __builtin_amdgcn_perm(o, p, sel_b);
                    // now: position 8q + 4 half + lane % 4 of tile row i, channels 4 (cl / 4) .. + 3 of tile column j
                    if constexpr (STAGED) {
                        *reinterpret_cast<uint32_t *>(so_lane + (i * 32 + 8 * q) * OP + j * 32) = p;
                    } else {
                        const uint32_t off = d_off[(i * 4 + q) * TN + j];
                        if constexpr (RES) {
                            const uint32_t xw = d_res[(i * 4 + q) * TN + j];
                            uint32_t summed = 0;
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                const int32_t x = (int8_t)(xw >> (8 * e)), y = (int8_t)(p >> (8 * e));
                                const int32_t r1 = requant_chan(x, q_res, g.rs_res.p), r2 = requant_chan(y, q_conv, g.rs_conv.p);
                                const int32_t sum = (int32_t)((uint32_t)r1 + (uint32_t)r2);
                                summed |= ((uint32_t)requant_acc(sum, q_out, g.rs_out.p) & 0xffu) << (8 * e);
                            }
                            p = summed;
                        }
                        __builtin_amdgcn_raw_buffer_store_b32(p, ores, (int)off, 0, 0);
                    }
                }
            }
        }
        if constexpr (!STAGED) return;
        __syncthreads();
        constexpr int PPR = BN / 16;  // 16-byte pieces per tile row
        static_assert((BM * PPR) % NTHREADS == 0, "whole pieces per thread");
        if (!RES && (g.N & 15) == 0) {
            // every piece inside the tensor is whole (uniform): all of a thread's pieces are read first and leave
            // without a test (a piece outside the tensor has an offset beyond the buffer's extent and is dropped)
            constexpr int NP = BM * PPR / NTHREADS;
            uint4 d[NP];
            uint32_t off[NP];
#pragma unroll
            for (int t = 0; t < NP; t++) {
                const int piece = t * NTHREADS + tid;
                const int r = piece / PPR, c16 = (piece % PPR) * 16;
                const int m = m_base + r, n0 = n_base + c16;
                d[t] = *reinterpret_cast<const uint4 *>(so + r * OP + c16);
                off[t] = (m < g.M && n0 < g.N) ? (uint32_t)m * (uint32_t)g.ldo + (uint32_t)n0 : kOobOffset;
            }
#pragma unroll
            for (int t = 0; t < NP; t++)
                __builtin_amdgcn_raw_buffer_store_b128(v4i{(int)d[t].x, (int)d[t].y, (int)d[t].z, (int)d[t].w}, ores, (int)off[t], 0,
                                                       kOutAux);
            return;
        }
#pragma unroll
        for (int t = 0; t < BM * PPR / NTHREADS; t++) {
            const int piece = t * NTHREADS + tid;
            const int r = piece / PPR, c16 = (piece % PPR) * 16;
            const int m = m_base + r, n0 = n_base + c16;
            uint4 d = *reinterpret_cast<const uint4 *>(so + r * OP + c16);
            const uint32_t off = (m < g.M && n0 < g.N) ? (uint32_t)m * (uint32_t)g.ldo + (uint32_t)n0 : kOobOffset;
            const bool whole = n0 + 16 <= g.N;
            if (RES) {
                uint32_t w[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t xw = buf_load4(rres, (whole || n0 + 4 * k < g.N) && off != kOobOffset ? off + 4 * k : kOobOffset);
                    uint32_t summed = 0;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int32_t x = (int8_t)(xw >> (8 * e)), y = (int8_t)(w[k] >> (8 * e));
                        const int32_t r1 = requant_chan(x, q_res, g.rs_res.p), r2 = requant_chan(y, q_conv, g.rs_conv.p);
                        const int32_t sum = (int32_t)((uint32_t)r1 + (uint32_t)r2);
                        summed |= ((uint32_t)requant_acc(sum, q_out, g.rs_out.p) & 0xffu) << (8 * e);
                    }
                    w[k] = summed;
                }
                d = make_uint4(w[0], w[1], w[2], w[3]);
            }
            if (whole) {
                __builtin_amdgcn_raw_buffer_store_b128(v4i{(int)d.x, (int)d.y, (int)d.z, (int)d.w}, ores, (int)off, 0, kOutAux);
            } else if (off != kOobOffset) {  // the last channels of a row whose extent is not a multiple of 16
                const uint32_t w[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
                for (int k = 0; k < 4; k++)
                    if (n0 + 4 * k < g.N) __builtin_amdgcn_raw_buffer_store_b32(w[k], ores, (int)(off + 4 * k), 0, 0);
            }
        }
        return;
    }
    // ---- every other output form: int32 accumulators, or RESCALE to 16- / 32-bit or unaligned 8-bit outputs; a
    // store instruction writes 32 consecutive channels of two positions
    ChanScale cs[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) cs[j] = make_chan_scale(chan_mult[j], chan_shift[j], g.rp);
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int32_t xc[4];
            if (!rows_done) row_terms(i, q, xc); else xc[0] = xc[1] = xc[2] = xc[3] = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int m = m_base + wave_m * WM + i * 32 + 8 * q + 4 * half + e;
                if (m >= g.M) continue;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int n = n_base + wave_n * WN + j * 32 + cl;
                    if (n >= g.N) continue;
                    const int32_t a = (int32_t)((uint32_t)acc[i][j][4 * q + e] + (uint32_t)bias_adj[j] + (uint32_t)xc[e]);
                    const int32_t v = g.fused ? requant_acc(a, cs[j], g.rp) : a;
                    const int64_t off = (int64_t)m * g.ldo + n;
                    if (g.out_size == 1)
                        *reinterpret_cast<int8_t *>(ob + off) = (int8_t)v;
                    else if (g.out_size == 2)
                        *reinterpret_cast<int16_t *>(ob + off * 2) = (int16_t)v;
                    else
                        *reinterpret_cast<int32_t *>(ob + off * 4) = v;
                }
            }
        }
    }
}

template <int BM, int BN>
constexpr size_t smem_bytes() {
    return (size_t)2 * BM * PITCH + (size_t)2 * w_buf_bytes<BN>() + (size_t)BN * sizeof(ChanParams);
}
template <int BM, int BN>
constexpr size_t smem_bytes_dl() {
    return (size_t)dl_stages<BM, BN>() * (BM + BN) * BK + (size_t)BN * sizeof(ChanParams);
}

template <typename Kernel>
void launch_kernel(Kernel kernel, const GemmArgs &g, int threads, size_t sm, dim3 grid, hipStream_t s) {
    if (sm > 48 * 1024) {  // above the default dynamic LDS limit: raise it once per kernel
        static std::mutex lock;
        static std::unordered_set<const void *> raised;
        const void *key = reinterpret_cast<const void *>(kernel);
        std::lock_guard<std::mutex> guard(lock);
        if (raised.insert(key).second)
            (void)hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm);
    }
    kernel<<<grid, dim3(threads), sm, s>>>(g);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool SUMS, bool Q8>
void launch_tile(const GemmArgs &g, int xmode, int wmode, dim3 grid, hipStream_t s) {
    const size_t sm = smem_bytes<BM, BN>();
    if constexpr (BM >= 128 && BN >= 128) {  // the direct-to-LDS pipeline exists for the large tiles only
        if (xmode == X_PLAIN_DL && wmode == W_ROWS_DL)
            return launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_PLAIN_DL, W_ROWS_DL, SUMS, Q8>, g,
                                 WAVES_M * WAVES_N * 64, smem_bytes_dl<BM, BN>(), grid, s);
        if (xmode == X_PLAIN_DL && wmode == W_KMAJOR_DL)
            return launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_PLAIN_DL, W_KMAJOR_DL, SUMS, Q8>, g,
                                 WAVES_M * WAVES_N * 64, smem_bytes_dl<BM, BN>(), grid, s);
    }
    if constexpr (Q8 && BM * BN <= 128 * 128) {  // residual stage: the 1x1 projections (plain rows on both sides)
        if (g.res != nullptr && xmode == X_PLAIN && wmode == W_ROWS)
            return launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_PLAIN, W_ROWS, SUMS, Q8, true>, g,
                                 WAVES_M * WAVES_N * 64, sm, grid, s);
    }
    if (xmode == X_PLAIN && wmode == W_ROWS)
        launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_PLAIN, W_ROWS, SUMS, Q8>, g, WAVES_M * WAVES_N * 64, sm, grid, s);
    else if (xmode == X_TAP && wmode == W_ROWS)
        launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_TAP, W_ROWS, SUMS, Q8>, g, WAVES_M * WAVES_N * 64, sm, grid, s);
    else if (xmode == X_PLAIN && wmode == W_KMAJOR)
        launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_PLAIN, W_KMAJOR, SUMS, Q8>, g, WAVES_M * WAVES_N * 64, sm, grid, s);
    else if (xmode == X_PLAIN && wmode == W_KMAJOR4)
        launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_PLAIN, W_KMAJOR4, SUMS, Q8>, g, WAVES_M * WAVES_N * 64, sm, grid, s);
    else if (xmode == X_PLAIN4 && wmode == W_ROWS4)
        launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_PLAIN4, W_ROWS4, SUMS, Q8>, g, WAVES_M * WAVES_N * 64, sm, grid, s);
    else
        launch_kernel(gemm_i8_kernel<BM, BN, WAVES_M, WAVES_N, X_GENERIC, W_GENERIC, SUMS, Q8>, g, WAVES_M * WAVES_N * 64, sm, grid, s);
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
void launch_tile_zp(const GemmArgs &g, int xmode, int wmode, dim3 grid, hipStream_t s) {
    const bool sums = g.zx != 0 || g.zw != 0;
    const bool q8 = g.fused && g.out_size == 1 && g.out_vec_ok && g.o_bytes != 0;
    if (sums && q8)
        launch_tile<BM, BN, WAVES_M, WAVES_N, true, true>(g, xmode, wmode, grid, s);
    else if (sums)
        launch_tile<BM, BN, WAVES_M, WAVES_N, true, false>(g, xmode, wmode, grid, s);
    else if (q8)
        launch_tile<BM, BN, WAVES_M, WAVES_N, false, true>(g, xmode, wmode, grid, s);
    else
        launch_tile<BM, BN, WAVES_M, WAVES_N, false, false>(g, xmode, wmode, grid, s);
}

}  // namespace

// One function per tile shape, each compiled in its own translation unit (gemm_i8_tile*.hip) so that the tile
// shapes build in parallel.  Tile ids: see kGemmTiles in gemm_i8.hip.
#define MLEL_DECLARE_GEMM_TILE(ID) \
    void launch_gemm_tile##ID(const void *args, int xmode, int wmode, dim3 grid, hipStream_t s)
MLEL_DECLARE_GEMM_TILE(0);
MLEL_DECLARE_GEMM_TILE(1);
MLEL_DECLARE_GEMM_TILE(2);
MLEL_DECLARE_GEMM_TILE(3);
MLEL_DECLARE_GEMM_TILE(4);
MLEL_DECLARE_GEMM_TILE(5);
MLEL_DECLARE_GEMM_TILE(6);
// the LDS-free form for 1x1 convolutions of few tiles (gemm_i8_cols.hip); 1 when launched
int launch_conv_cols_mfma(const void *args, hipStream_t s);
int launch_conv_cols_pool(const void *args, int8_t *pool_out, int images, int positions, int zi, int zo, bool probe,
                          hipStream_t s);
#define MLEL_DEFINE_GEMM_TILE(ID, BM, BN, WAVES_M, WAVES_N)                                          \
    void launch_gemm_tile##ID(const void *args, int xmode, int wmode, dim3 grid, hipStream_t s) {    \
        launch_tile_zp<BM, BN, WAVES_M, WAVES_N>(*static_cast<const GemmArgs *>(args), xmode, wmode, grid, s); \
    }

}  // namespace mlel
