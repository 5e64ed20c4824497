// fp16 x fp16 -> fp32 MATMUL on the gfx950 matrix cores (reference arithmetic: matmul.comp:30-73 with an fp32
// accumulator: out[b][m][n] = sum_k A[b][m][k] * B[b][k][n]; the order of the fp32 additions differs from the
// shader's sequential loop, which is why floating-point graphs are compared within a tolerance).
//
// Kernel shape.  256 threads = 4 wavefronts; a block owns a BM x BN tile of one batch and walks K in steps of 32
// halfs through two LDS buffers, with the global loads of the next step in flight while the current one is
// multiplied (v_mfma_f32_32x32x16_f16).  As in the int8 kernel the B matrix supplies the MFMA row operand and A the
// column operand, so a lane ends up with four consecutive output columns of one output row per register quad and
// stores them as one 128-bit word.
//   A tile: [BM][32 halfs], 80-byte pitch, operands read with ds_read_b128 (8 consecutive k of one row);
//   B tile: kept K-major as in memory, [32][BN halfs]; operands are gathered with ds_read_b64_tr_b16, which hands
//           lane L of a 16-lane group the four k values of column L out of a 4(k) x 16(n) block whose rows are
//           addressed by the group's lanes (lane s points at row s / 4, columns 4 * (s % 4) ..).
// All global loads are buffer loads: an offset at or beyond the extent returns 0, which pads M, N and K tails.
#include <algorithm>

#include "common.hpp"
#include "dispatch.hpp"
#include "float_programs.hpp"

namespace mlel {
namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s lds_v4s;

constexpr uint32_t kOob = 0x80000000u;

struct HGemmArgs {
    const char *a, *b;
    char *out;
    int32_t M, N, K, batches;
    int32_t b_rows;                     // B is laid down row-wise, [N][K]: ldb is then the pitch of a row of K
    int64_t a_batch, b_batch, o_batch;  // bytes
    uint32_t lda, ldb, ldo;             // bytes per row
    uint32_t a_bytes, b_bytes, o_bytes; // per-batch extents (all below 2^31)
    int32_t tiles_m, tiles_n, total_tiles, chunk;
    // the tile index divided by tiles per batch, tiles per row and tiles per product as a multiplication and a shift
    // (set by launch_k from the fields above and tiles_n_group)
    DivMagic div_per_batch, div_tiles_n, div_group;
    // fused epilogue (EPI = 1): out = fp16(acc + bias[n]) with the addition in fp32; bias may be null
    const float *bias;
    int32_t bias_len;  // 1 (broadcast) or N
    // fp16 tensor of the output's shape added to the rounded result (the ADD of a residual connection), or null
    const char *res;
    int64_t r_batch;
    uint32_t ldr, r_bytes;
    // fp16 result written through a six-dimensional view [NB1, NB2, M1, M2, N1, N2] of other strides (a head split
    // or merge behind the product): batch = nb1 * NB2 + nb2, row = m1 * M2 + m2, column = n1 * N2 + n2 with eight
    // consecutive n2 contiguous.  view == 0: the plain [batch][row][column] layout above.
    // view == 2: the same with eight consecutive m2 contiguous instead (the innermost extent of the product ends up
    // somewhere else: a transposing view) and n2 at a stride of vs_n2 bytes
    int32_t view, v_nb2, v_m2, v_n2;
    int64_t vs_nb1, vs_nb2;
    uint32_t vs_m1, vs_m2, vs_n1, vs_n2;
    // Several products of the same A in one launch (the Q, K and V projections): tile columns [k * tiles_n_group,
    // (k + 1) * tiles_n_group) belong to product k, which has a B, a bias and an output of its own; product 0 uses
    // the fields above.  All products have the same extents and operand strides.
    // the tanh form of GELU applied to the rounded result (GeluTanhProgram with the result as its value 0): the
    // program's four single-element fp16 inputs, or null
    const uint16_t *act[4];
    int32_t groups, tiles_n_group;
    struct Extra {
        const char *b;
        const float *bias;
        char *out;
        int64_t o_batch;
        uint32_t ldo, o_bytes;
        int32_t view, v_nb2, v_m2, v_n2;
        int64_t vs_nb1, vs_nb2;
        uint32_t vs_m1, vs_m2, vs_n1, vs_n2;
    } extra[2];
};
// what a block needs of its product: filled from HGemmArgs or from one of its Extra entries
struct HProduct {
    const char *b;
    const float *bias;
    char *out;
    int64_t o_batch;
    uint32_t ldo, o_bytes;
    int32_t view, v_nb2, v_m2, v_n2;
    int64_t vs_nb1, vs_nb2;
    uint32_t vs_m1, vs_m2, vs_n1, vs_n2;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 load16(__amdgpu_buffer_rsrc_t r, uint32_t off) {
    const v4i v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
    return make_uint4((uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w);
}

// One wavefront-wide 16-byte-per-lane load from a buffer resource straight into LDS at `lds_addr` + 16 * lane.
// Inline assembly on purpose: the compiler orders every LDS read after ALL outstanding loads of this kind (it cannot
// tell which bytes they write), which would drain the stage ring at every step; the loop does its own counting with
// s_waitcnt vmcnt(N).  M0 holds the LDS address for this one instruction only.
__device__ __forceinline__ void load16_to_lds(v4i res, uint32_t lds_addr, uint32_t offset, uint32_t scalar_offset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds_addr), "v"(offset),
                 "s"(res), "s"(scalar_offset)
                 : "memory");
}
__device__ __forceinline__ v4i rsrc_words(const void *p, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(p);
    return v4i{(int)(uint32_t)a, (int)(uint32_t)(a >> 32), (int)bytes, 0x00020000};
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // s_waitcnt vmcnt(N) only (expcnt / lgkmcnt untouched)
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Division of the row and column indices of a view by its inner extents, once per 16-byte piece: the extents are the
// same for every piece, so the quotient is one multiplication by floor((2^32 - 1) / d) + 1 (exact while x * d < 2^32,
// which `usable` says for the tile's largest index; otherwise, and for d == 1, the plain division).
struct ViewDiv {
    uint32_t d, magic;
    bool usable;
    __device__ __forceinline__ ViewDiv(int32_t divisor, int32_t largest) {
        d = (uint32_t)divisor;
        usable = d > 1 && (uint64_t)(uint32_t)largest * d < (uint64_t(1) << 32);
        magic = usable ? 0xffffffffu / d + 1u : 0u;
    }
    __device__ __forceinline__ uint32_t quotient(uint32_t x) const { return usable ? __umulhi(x, magic) : (d == 1 ? x : x / d); }
};

// BKH: halfs of K per step (32, or 64 for long contractions: half as many barriers and LDS round trips per K)
// BROWS: B is given row-wise, [N][K] (a weight matrix laid down transposed once, ahead of time): both operands are
// then rows of K, and the main loop is the direct-to-LDS pipeline of the int8 kernel (gemm_i8_kernel.hpp): 64 bytes of
// K per step, `buffer_load ... lds` into a ring of four unpadded stages whose 16-byte pieces are XOR-swizzled (piece p
// of row r in slot p ^ ((r >> 2) & 3)), 128-bit operand reads without bank conflicts and without the transposing
// reads of the K-major tile, one barrier per step, reads of the next half step issued before the multiplies of this one.
template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI, int BKH, bool BROWS = false>
__global__ void __launch_bounds__(64 * WAVES_M * WAVES_N) gemm_f16_kernel(const HGemmArgs g) {
    constexpr int NT = 64 * WAVES_M * WAVES_N;  // four or eight wavefronts
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int XPITCH = BKH * 2 + 16;      // bytes per A row in LDS
    constexpr int XP16 = BKH / 8;             // 16-byte pieces per A row
    constexpr int XPASS = NT / XP16;          // A rows covered by one pass of the block
    constexpr int XROWS = BM / XPASS;         // 16-byte pieces of A per thread and step
    constexpr int WPITCH = 2 * BN + 32;       // bytes per K row of the B tile: 4 rows x 32 B land on distinct banks
    constexpr int WROW16 = BN / 8;            // 16-byte pieces per K row
    constexpr int WCHUNKS = (BKH * WROW16) / NT;
    static_assert((WAVES_M * WAVES_N == 4 || WAVES_M * WAVES_N == 8) && BM % XPASS == 0 && WM % 32 == 0 && WN % 32 == 0 && (BKH * WROW16) % NT == 0, "tile shape");
    constexpr int XBUF = BM * XPITCH, WBUF = BKH * WPITCH;
    extern __shared__ __align__(16) char smem[];
    char *xs = smem;             // [2][BM][XPITCH]
    char *ws = smem + 2 * XBUF;  // [2][BKH][WPITCH]

    // Every argument that the tile assignment and the first operand requests depend on is asked for here, in one
    // batch (every dword of the wide loads that bring them named: a register nobody waits for is given away at once,
    // and whoever gets it waits for the load first).  Left alone the compiler loads arguments where they are first
    // used, behind the early exit, behind three divisions and behind each other: five to nine trips to memory in a
    // row before a wavefront's first address.
    asm volatile("" ::"s"(g.chunk), "s"(g.total_tiles), "s"(g.tiles_m), "s"(g.tiles_n), "s"(g.div_per_batch.m),
                 "s"(g.div_per_batch.s), "s"(g.div_tiles_n.m), "s"(g.div_tiles_n.s), "s"(g.div_group.m), "s"(g.div_group.s),
                 "s"(g.groups), "s"(g.tiles_n_group), "s"(g.a), "s"(g.b), "s"(g.extra[0].b), "s"(g.extra[1].b), "s"(g.out),
                 "s"(g.M), "s"(g.N), "s"(g.K), "s"(g.batches), "s"(g.b_rows), "s"(g.a_batch), "s"(g.b_batch), "s"(g.o_batch),
                 "s"(g.lda), "s"(g.ldb), "s"(g.ldo), "s"(g.a_bytes), "s"(g.b_bytes), "s"(g.o_bytes),
                 // the pointers of the epilogue, which the compiler follows up here already (the activation's scalars)
                 "s"(g.bias), "s"(g.bias_len), "s"(g.res), "s"(g.act[0]), "s"(g.act[1]), "s"(g.act[2]), "s"(g.act[3]));
    // consecutive tiles (sharing operand panels) go to the same XCD; blocks are dealt to XCDs round-robin
    const int lin = __builtin_amdgcn_readfirstlane((int)(blockIdx.x % 8u) * g.chunk + (int)(blockIdx.x / 8u));
    if (lin >= g.total_tiles) return;
    const int per_batch = g.tiles_m * g.tiles_n;
    const int batch = div_magic(lin, g.div_per_batch);
    const int t_in = lin - batch * per_batch;
    const int tile_m = div_magic(t_in, g.div_tiles_n);
    int tile_n = t_in - tile_m * g.tiles_n;
    HProduct o{g.b, g.bias, g.out, g.o_batch, g.ldo, g.o_bytes, g.view, g.v_nb2, g.v_m2, g.v_n2, g.vs_nb1, g.vs_nb2,
               g.vs_m1, g.vs_m2, g.vs_n1, g.vs_n2};
    if (g.groups > 1) {  // uniform
        const int product = div_magic(tile_n, g.div_group);
        tile_n -= product * g.tiles_n_group;
        if (product > 0) {
            const HGemmArgs::Extra &e = product == 1 ? g.extra[0] : g.extra[1];
            o = HProduct{e.b, e.bias, e.out, e.o_batch, e.ldo, e.o_bytes, e.view, e.v_nb2, e.v_m2, e.v_n2, e.vs_nb1, e.vs_nb2,
                         e.vs_m1, e.vs_m2, e.vs_n1, e.vs_n2};
        }
        // the operand pointer is on the way to the first request: picked from registers that are already there
        o.b = product == 0 ? g.b : (product == 1 ? g.extra[0].b : g.extra[1].b);
    }
    const int m_base = tile_m * BM, n_base = tile_n * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;

    const __amdgpu_buffer_rsrc_t ares = rsrc(g.a + (int64_t)batch * g.a_batch, g.a_bytes);
    const __amdgpu_buffer_rsrc_t bres = rsrc(o.b + (int64_t)batch * g.b_batch, g.b_bytes);

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // the bias of this lane's columns (fused form): lane holds, per register quad q, columns 8q + 4 * (lane / 32) ...
    // (where to fetch it: behind the first stages of the direct-to-LDS loop when that costs 16 registers; the wide tile's
    // 32 cost its GELU epilogue more than the trip to memory they hide, 35.5 -> 36.0 us)
    constexpr bool BIAS_AHEAD = BROWS && TN == 1;
    float bias_r[TN][4][4];
    auto fetch_bias = [&]() {
        // through a buffer resource of the bias's extent: a column beyond N (or no bias at all) reads as zero without a test
        const __amdgpu_buffer_rsrc_t bias_res =
            rsrc(o.bias, o.bias != nullptr ? (g.bias_len == 1 ? 4u : (uint32_t)g.N * 4u) : 0u);
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n0 = n_base + wave_n * WN + j * 32 + 8 * q + 4 * (lane >> 5);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    bias_r[j][q][e] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(bias_res, g.bias_len == 1 ? 0 : (n0 + e) * 4, 0, 0));
            }
    };
    if constexpr (BROWS) {
        // ---- direct-to-LDS main loop (K % 32 == 0: whole 64-byte steps)
        constexpr int BK = 64, DL_S = 4, DL_STAGE = (BM + BN) * BK;
        constexpr int XI = BM * 4 / NT, WI = BN * 4 / NT;  // 16-byte pieces per thread and stage
        // (request counts above 15 need the upper bits of the vmcnt field, a path no instance has exercised)
        static_assert((BM * 4) % NT == 0 && (BN * 4) % NT == 0 && (DL_S - 1) * (XI + WI) < 16, "whole pieces per thread");
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        uint32_t xo[XI], wo[WI];
#pragma unroll
        for (int i = 0; i < XI; i++) {
            const int q = i * NT + tid, r = q >> 2, p = (q & 3) ^ ((r >> 2) & 3);
            const int m = m_base + r;
            xo[i] = m < g.M ? (uint32_t)m * g.lda + (uint32_t)(p * 16) : kOob;
        }
#pragma unroll
        for (int i = 0; i < WI; i++) {
            const int q = i * NT + tid, r = q >> 2, p = (q & 3) ^ ((r >> 2) & 3);
            const int n = n_base + r;
            wo[i] = n < g.N ? (uint32_t)n * g.ldb + (uint32_t)(p * 16) : kOob;
        }
        const v4i xres4 = rsrc_words(g.a + (int64_t)batch * g.a_batch, g.a_bytes);
        const v4i wres4 = rsrc_words(o.b + (int64_t)batch * g.b_batch, g.b_bytes);
        const uint32_t lds0 = (uint32_t) reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char *)smem) +
                              (uint32_t)(wave_u * 1024);
        // operand addresses inside a stage: row lane % 32 of a 32-row group, the lane half's eight halfs of K half kk
        const int h = lane >> 5, swz = (lane >> 2) & 3;
        const char *x_base[2], *w_base[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int slot = ((kk * 2 + h) ^ swz) * 16;
            x_base[kk] = smem + (wave_m * WM + (lane & 31)) * BK + slot;
            w_base[kk] = smem + BM * BK + (wave_n * WN + (lane & 31)) * BK + slot;
        }
        // The loop, as in the int8 kernel's direct-to-LDS form: a wavefront issues in order, so a K half is one
        // straight line -- a matrix instruction, then a share of the next half's operand reads and of the requests,
        // which issue while the matrix core works, then the next matrix instruction.  Stage s lives in buffer
        // s % DL_S; a stage's requests ride in the second K half of a step, behind the step's barrier, which frees the
        // buffer (spread over both halves of a step they arrive a step later, which the long contractions whose
        // operands come from memory rather than from the L2 pay for: 4096 x 3072 x 768 ran 5 % slower).  Beyond the last step they go through an
        // empty resource and fetch nothing, so every step has the same requests in flight and the waits count exactly:
        // at most DL_S - 3 stages outstanding at the barrier of step s means this thread's part of stage s + 1 has
        // landed; the barrier extends that to every thread's part and says that every wavefront has received its
        // reads of stage s - 1, whose buffer the step's requests overwrite.
        const int nk = g.K / 32;
        const v4i null4 = v4i{xres4[0], xres4[1], 0, xres4[3]};
        constexpr int NLA = XI + WI;
        auto half = [&](auto lp_t, const v8h(&xc)[TM], const v8h(&wc)[TN], v8h(&xn)[TM], v8h(&wn)[TN], int rbuf, int rkk,
                        int ibuf, int istep) {
            constexpr int LP = decltype(lp_t)::value;  // 1: the stage's requests ride in this half, 0: none
            constexpr int NM = TM * TN, NR = TM + TN;
            constexpr int L0 = 0, L1 = LP == 1 ? NLA : 0, NL = L1 - L0, LPER = (NL + NM - 1) / NM;
            const bool live = istep < nk;
            const v4i xr = live ? xres4 : null4, wr = live ? wres4 : null4;
            const uint32_t xd = lds0 + (uint32_t)(ibuf * DL_STAGE), wd = xd + BM * BK;
            const uint32_t kb = (uint32_t)istep * BK;
            // (two wavefronts share a SIMD here and fill each other's gaps: the reads go first, so that their data
            // is there when the next half starts; only the requests are dealt out behind the matrix instructions)
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if (r < TM) xn[r] = *reinterpret_cast<const v8h *>(x_base[rkk] + rbuf * DL_STAGE + r * 32 * BK);
                else wn[r - TM] = *reinterpret_cast<const v8h *>(w_base[rkk] + rbuf * DL_STAGE + (r - TM) * 32 * BK);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < NM; t++) {
                const int i = t / TN, j = t % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wc[j], xc[i], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < LPER; u++) {
                    const int l = L0 + t * LPER + u;
                    if (l < L1) {
                        if (l < XI) load16_to_lds(xr, xd + l * NT * 16, xo[l], kb);
                        else load16_to_lds(wr, wd + (l - XI) * NT * 16, wo[l - XI], kb);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        v8h xf0[TM], wf0[TN], xf1[TM], wf1[TN];
#pragma unroll
        for (int d = 0; d < DL_S - 1; d++) {
            const v4i xr = d < nk ? xres4 : null4, wr = d < nk ? wres4 : null4;
            const uint32_t xd = lds0 + (uint32_t)(d * DL_STAGE), wd = xd + BM * BK;
#pragma unroll
            for (int l = 0; l < NLA; l++) {
                if (l < XI) load16_to_lds(xr, xd + l * NT * 16, xo[l], (uint32_t)d * BK);
                else load16_to_lds(wr, wd + (l - XI) * NT * 16, wo[l - XI], (uint32_t)d * BK);
            }
        }
        // The bias is asked for behind the first stages and used behind the loop (asked for there, its trip to memory
        // was waited out by every wavefront in front of the first store).  These loads are younger than the first
        // stages and older than every later request, so the counted waits hold with them in flight: the first ones
        // only wait for a few requests more.
        if (EPI == 1 && BIAS_AHEAD) fetch_bias();
        wait_vmcnt<(DL_S - 2) * NLA>();  // stage 0 has landed: what was requested behind it may be in flight
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < TM; i++) xf0[i] = *reinterpret_cast<const v8h *>(x_base[0] + i * 32 * BK);
#pragma unroll
        for (int j = 0; j < TN; j++) wf0[j] = *reinterpret_cast<const v8h *>(w_base[0] + j * 32 * BK);
        for (int step = 0; step < nk; step += DL_S) {
#pragma unroll
            for (int d = 0; d < DL_S; d++) {
                if (step + d < nk) {  // uniform
                    half(std::integral_constant<int, 0>{}, xf0, wf0, xf1, wf1, d, 1, 0, 0);
                    wait_vmcnt<(DL_S - 3) * NLA>();
                    asm volatile("" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    half(std::integral_constant<int, 1>{}, xf1, wf1, xf0, wf0, (d + 1) % DL_S, 0, (d + DL_S - 1) % DL_S,
                         step + d + DL_S - 1);
                }
            }
        }
        wait_vmcnt<0>();  // the requests beyond the last step write (zeros) into the ring, which the epilogue reuses
        __syncthreads();
    } else {
    uint32_t xoff[XROWS], woff[WCHUNKS];
#pragma unroll
    for (int i = 0; i < XROWS; i++) {
        const int m = m_base + tid / XP16 + XPASS * i;
        xoff[i] = m < g.M ? (uint32_t)m * g.lda + (tid % XP16) * 16 : kOob;
    }
#pragma unroll
    for (int i = 0; i < WCHUNKS; i++) {
        const int c = tid + NT * i;
        const int n = n_base + (c % WROW16) * 8;
        woff[i] = n < g.N ? (uint32_t)(c / WROW16) * g.ldb + (uint32_t)n * 2 : kOob;
    }
    auto prefetch = [&](int k0, uint4 (&xr)[XROWS], uint4 (&wr)[WCHUNKS]) {
        const bool kin = k0 + (tid % XP16) * 8 < g.K;  // K % 8 == 0: a piece lies wholly inside or outside
#pragma unroll
        for (int i = 0; i < XROWS; i++) xr[i] = load16(ares, (kin && xoff[i] != kOob) ? xoff[i] + (uint32_t)k0 * 2 : kOob);
#pragma unroll
        for (int i = 0; i < WCHUNKS; i++) {
            const int row = (tid + NT * i) / WROW16;
            wr[i] = load16(bres, (k0 + row < g.K && woff[i] != kOob) ? woff[i] + (uint32_t)k0 * g.ldb : kOob);
        }
    };
    auto stage = [&](int buf, const uint4 (&xr)[XROWS], const uint4 (&wr)[WCHUNKS]) {
#pragma unroll
        for (int i = 0; i < XROWS; i++)
            *reinterpret_cast<uint4 *>(xs + buf * XBUF + (tid / XP16 + XPASS * i) * XPITCH + (tid % XP16) * 16) = xr[i];
#pragma unroll
        for (int i = 0; i < WCHUNKS; i++) {
            const int c = tid + NT * i;
            *reinterpret_cast<uint4 *>(ws + buf * WBUF + (c / WROW16) * WPITCH + (c % WROW16) * 16) = wr[i];
        }
    };

    // operand addresses inside a tile: A row = lane % 32, k group = lane / 32 (8 halfs each);
    // B: 16-lane group q = lane / 16 covers columns 16 * (q & 1) .., k group q / 2; lane s = lane % 16 points at
    // row s / 4, columns 4 * (s % 4) of the 4 x 16 block
    const int a_row = lane & 31, a_kg = lane >> 5;
    const int s16 = lane & 15, q16 = lane >> 4;
    const int b_row = 8 * (q16 >> 1) + (s16 >> 2), b_col = 16 * (q16 & 1) + 4 * (s16 & 3);
    auto compute = [&](int buf) {
        const char *xt = xs + buf * XBUF;
        const char *wt = ws + buf * WBUF;
#pragma unroll
        for (int kk = 0; kk < BKH / 16; kk++) {
            v8h af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                af[i] = *reinterpret_cast<const v8h *>(xt + (wave_m * WM + i * 32 + a_row) * XPITCH + kk * 32 + a_kg * 16);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const char *p = wt + (kk * 16 + b_row) * WPITCH + (wave_n * WN + j * 32 + b_col) * 2;
                const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)p);
                const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)(p + 4 * WPITCH));
                union {
                    v4s s[2];
                    v8h h;
                } u;
                u.s[0] = lo;
                u.s[1] = hi;
                bf[j] = u.h;
            }
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
    };

    // ring of DEPTH register sets: DEPTH - 1 steps of global loads in flight while one step is multiplied
    constexpr int DEPTH = BKH == 32 ? 4 : 3;
    const int nk = (g.K + BKH - 1) / BKH;
    uint4 xr[DEPTH][XROWS], wr[DEPTH][WCHUNKS];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) prefetch(d * BKH, xr[d], wr[d]);
    stage(0, xr[0], wr[0]);
    __syncthreads();
    for (int step = 0; step < nk; step += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            if (step + d < nk) {  // uniform
                const int cur = (step + d) & 1;  // LDS buffer of this step
                prefetch((step + d + DEPTH) * BKH, xr[d], wr[d]);
                compute(cur);
                stage(cur ^ 1, xr[(d + 1) % DEPTH], wr[(d + 1) % DEPTH]);
                __syncthreads();
            }
        }
    }
    }

    // ---- store: lane holds row m = lane % 32 of each sub-tile and, per register quad q, columns 8q + 4 * (lane / 32)
    const int64_t o_base = o.view ? (int64_t)(batch / o.v_nb2) * o.vs_nb1 + (int64_t)(batch % o.v_nb2) * o.vs_nb2
                                  : (int64_t)batch * o.o_batch;
    const __amdgpu_buffer_rsrc_t ores = rsrc(o.out + o_base, o.o_bytes);
    // otherwise fetched here, in one batch before any store (a load after a store would have to wait for it: the
    // compiler cannot tell that the two do not alias)
    if (EPI == 1 && !BIAS_AHEAD) fetch_bias();
    if (EPI == 1) {
        // fp16 result: a lane's four values are only eight bytes of a row, and a store instruction would touch 32 rows.
        // The tile goes through shared memory instead (the operand buffers are free: the loop ended with a barrier)
        // and leaves in 16-byte pieces, consecutive lanes along a row, so that every instruction writes whole lines.
        constexpr int OPITCH = BN * 2 + 16;
        constexpr int TPITCH = BM * 2 + 16;  // a column of the tile, for transposing views
        // the launch sizes shared memory for the larger of the operand buffers and the result tile
#pragma unroll
        for (int i = 0; i < TM; i++) {
            char *orow = smem + (wave_m * WM + i * 32 + (lane & 31)) * OPITCH;
#pragma unroll
            for (int j = 0; j < TN; j++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    // ADD in fp32 (one rounding), then CAST to fp16 (round to nearest even): the two operators that
                    // follow the MATMUL in the unfused graph
                    _Float16 h[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float sum = o.bias != nullptr ? acc[i][j][4 * q + e] + bias_r[j][q][e] : acc[i][j][4 * q + e];
                        h[e] = (_Float16)sum;
                    }
                    const int col = wave_n * WN + j * 32 + 8 * q + 4 * (lane >> 5);
                    if (o.view == 2) {  // uniform; transposing view: the tile is laid down column by column
                        const int trow = wave_m * WM + i * 32 + (lane & 31);
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            *reinterpret_cast<_Float16 *>(smem + (col + e) * TPITCH + trow * 2) = h[e];
                        continue;
                    }
                    uint2 v;
                    v.x = (uint32_t)__builtin_bit_cast(unsigned short, h[0]) | ((uint32_t)__builtin_bit_cast(unsigned short, h[1]) << 16);
                    v.y = (uint32_t)__builtin_bit_cast(unsigned short, h[2]) | ((uint32_t)__builtin_bit_cast(unsigned short, h[3]) << 16);
                    *reinterpret_cast<uint2 *>(orow + col * 2) = v;
                }
            }
        }
        const __amdgpu_buffer_rsrc_t rres = rsrc(g.res != nullptr ? g.res + (int64_t)batch * g.r_batch : o.out, g.res != nullptr ? g.r_bytes : 0);
        // the residual's pieces of this thread, requested before the barrier and before any store (a load behind a
        // store waits for it, and one fetch per piece in the store loop would expose its latency four times over)
        constexpr int PIECES = BM * (BN / 8) / NT;
        constexpr bool RES_AHEAD = PIECES <= 4;
        uint4 res_r[RES_AHEAD ? PIECES : 1];
        if (RES_AHEAD && g.res != nullptr && o.view != 2) {  // uniform
#pragma unroll
            for (int i = 0; i < (RES_AHEAD ? PIECES : 1); i++) {
                const int p = i * NT + tid, r = p / (BN / 8), c = p % (BN / 8);
                const int m = m_base + r, n = n_base + c * 8;
                res_r[i] = load16(rres, (m < g.M && n < g.N) ? (uint32_t)m * g.ldr + (uint32_t)n * 2 : kOob);
            }
        }
        __syncthreads();
        const ViewDiv by_m2(o.view ? o.v_m2 : 1, g.M), by_n2(o.view ? o.v_n2 : 1, g.N);
        if (o.view == 2) {
            // transposing view: a piece is eight consecutive rows of one column (tile rows start at multiples of
            // eight and M2 is one, so a piece never straddles two m1)
            for (int p = tid; p < BN * (BM / 8); p += NT) {
                const int c = p / (BM / 8), r8 = p - c * (BM / 8);
                const int m = m_base + r8 * 8, n = n_base + c;
                if (m >= g.M || n >= g.N) continue;
                const uint4 piece = *reinterpret_cast<const uint4 *>(smem + c * TPITCH + r8 * 16);
                const uint32_t w[4] = {piece.x, piece.y, piece.z, piece.w};
                const uint32_t m1 = by_m2.quotient((uint32_t)m), n1 = by_n2.quotient((uint32_t)n);
                const uint32_t off = m1 * o.vs_m1 + ((uint32_t)m - m1 * (uint32_t)o.v_m2) * 2 + n1 * o.vs_n1 +
                                     ((uint32_t)n - n1 * (uint32_t)o.v_n2) * o.vs_n2;
                v4i v;
                v.x = (int)w[0], v.y = (int)w[1], v.z = (int)w[2], v.w = (int)w[3];
                __builtin_amdgcn_raw_buffer_store_b128(v, ores, (int)off, 0, kOutAux);
            }
            return;
        }
        constexpr int PPR = BN / 8;  // 16-byte pieces per row of the tile
        uint32_t act_c[4] = {0, 0, 0, 0};
        if (g.act[0] != nullptr) {  // uniform
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t bits = *g.act[k];
                act_c[k] = bits | (bits << 16);
            }
        }
#pragma unroll
        for (int p0 = 0; p0 < BM * PPR; p0 += NT) {
            const int p = p0 + tid, r = p / PPR, c = p % PPR;
            const int m = m_base + r, n = n_base + c * 8;
            uint4 piece = *reinterpret_cast<const uint4 *>(smem + r * OPITCH + c * 16);
            const bool inside = m < g.M && n < g.N;
            uint32_t off = inside ? (uint32_t)m * o.ldo + (uint32_t)n * 2 : kOob;
            if (o.view && inside) {  // uniform
                const uint32_t m1 = by_m2.quotient((uint32_t)m), n1 = by_n2.quotient((uint32_t)n);
                off = m1 * o.vs_m1 + ((uint32_t)m - m1 * (uint32_t)o.v_m2) * o.vs_m2 + n1 * o.vs_n1 +
                      ((uint32_t)n - n1 * (uint32_t)o.v_n2) * 2;
            }
            if (g.act[0] != nullptr) piece = gelu_tanh_piece(piece, act_c);  // uniform
            if (g.res != nullptr) {  // uniform; ADD of two fp16 tensors: one rounding of the exact sum
                const uint4 other = RES_AHEAD ? res_r[RES_AHEAD ? p0 / NT : 0]
                                              : load16(rres, inside ? (uint32_t)m * g.ldr + (uint32_t)n * 2 : kOob);
                typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
                h2_t *ph = reinterpret_cast<h2_t *>(&piece);
                const h2_t *oh = reinterpret_cast<const h2_t *>(&other);
#pragma unroll
                for (int e = 0; e < 4; e++) ph[e] = ph[e] + oh[e];
            }
            v4i v;
            v.x = (int)piece.x, v.y = (int)piece.y, v.z = (int)piece.z, v.w = (int)piece.w;
            __builtin_amdgcn_raw_buffer_store_b128(v, ores, (int)off, 0, kOutAux);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m_base + wave_m * WM + i * 32 + (lane & 31);
        const uint32_t row_off = m < g.M ? (uint32_t)m * o.ldo : kOob;
#pragma unroll
        for (int j = 0; j < TN; j++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n0 = n_base + wave_n * WN + j * 32 + 8 * q + 4 * (lane >> 5);
                const uint32_t off = (row_off != kOob && n0 < g.N) ? row_off + (uint32_t)n0 * 4 : kOob;
                v4i v;
                v.x = __float_as_int(acc[i][j][4 * q + 0]);
                v.y = __float_as_int(acc[i][j][4 * q + 1]);
                v.z = __float_as_int(acc[i][j][4 * q + 2]);
                v.w = __float_as_int(acc[i][j][4 * q + 3]);
                __builtin_amdgcn_raw_buffer_store_b128(v, ores, (int)off, 0, kOutAux);
            }
        }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int BKH, bool BROWS = false>
void launch_k(const HGemmArgs &args, bool cast_epilogue, dim3 grid, hipStream_t s) {
    HGemmArgs g = args;
    g.div_per_batch = make_div_magic((uint32_t)(g.tiles_m * g.tiles_n));
    g.div_tiles_n = make_div_magic((uint32_t)g.tiles_n);
    g.div_group = make_div_magic((uint32_t)(g.tiles_n_group > 0 ? g.tiles_n_group : 1));
    constexpr size_t operands = BROWS ? (size_t)4 * (BM + BN) * 64
                                      : (size_t)2 * BM * (BKH * 2 + 16) + (size_t)2 * BKH * (2 * BN + 32);
    constexpr size_t result = std::max((size_t)BM * (BN * 2 + 16), (size_t)BN * (BM * 2 + 16));
    constexpr size_t sm = std::max(operands, result);
    static_assert(sm <= 160 * 1024, "shared memory of a compute unit");
    // above the default dynamic shared-memory limit the limit is raised once per kernel (thread-safe static)
    if (cast_epilogue) {
        auto kernel = gemm_f16_kernel<BM, BN, WAVES_M, WAVES_N, 1, BKH, BROWS>;
        static const bool raised = sm <= 48 * 1024 || hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm) == hipSuccess;
        (void)raised;
        kernel<<<grid, dim3(64 * WAVES_M * WAVES_N), sm, s>>>(g);
    } else {
        auto kernel = gemm_f16_kernel<BM, BN, WAVES_M, WAVES_N, 0, BKH, BROWS>;
        static const bool raised = sm <= 48 * 1024 || hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm) == hipSuccess;
        (void)raised;
        kernel<<<grid, dim3(64 * WAVES_M * WAVES_N), sm, s>>>(g);
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
void launch(const HGemmArgs &g, bool cast_epilogue, dim3 grid, hipStream_t s) {
    if (g.K >= 256)
        launch_k<BM, BN, WAVES_M, WAVES_N, 64>(g, cast_epilogue, grid, s);
    else
        launch_k<BM, BN, WAVES_M, WAVES_N, 32>(g, cast_epilogue, grid, s);
}

bool dense_rows(const mlel_tensor *t) { return t->strides[2] == 2 && t->strides[1] >= t->dims[2] * 2; }

// Checks one product against what the kernel's indexing assumes and describes it.  1: described, 0: not a case for
// this kernel, 2: nothing to compute.
int fill_args(const mlel_tensor *out, const mlel_tensor *a, const mlel_tensor *b, const mlel_matmul_attr *attr,
              bool bias_cast, const mlel_tensor *bias, const mlel_tensor *residual, HGemmArgs *filled,
              const mlel_tensor *const *act = nullptr) {
    if (act != nullptr) {
        if (!bias_cast || residual != nullptr || out->rank != 3) return 0;
        for (int k = 0; k < 4; k++)
            if (act[k] == nullptr || act[k]->dtype != MLEL_F16 || numel(act[k]) != 1 || ((uintptr_t)act[k]->ptr % 2) != 0) return 0;
    }
    if (residual != nullptr) {
        if (!bias_cast || residual->dtype != MLEL_F16 || residual->rank != 3 || !same_shape(residual, out)) return 0;
        if (residual->strides[2] != 2 || ((uintptr_t)residual->ptr % 16) != 0 || residual->strides[0] % 16 != 0 ||
            residual->strides[1] % 16 != 0)
            return 0;
        const int64_t rb = residual->dims[1] * residual->strides[1];
        if (rb >= (int64_t(1) << 31) - 64 || residual->strides[1] < residual->dims[2] * 2) return 0;
    }
    if (a->dtype != MLEL_F16 || b->dtype != MLEL_F16 || out->dtype != (bias_cast ? MLEL_F16 : MLEL_F32)) return 0;
    // a six-dimensional output is a strided view [NB1, NB2, M1, M2, N1, N2] of the product (fused fp16 form only)
    mlel_tensor plain_out;
    const mlel_tensor *view = nullptr;
    if (out->rank == 6) {
        if (!bias_cast || residual != nullptr) return 0;
        view = out;
        plain_out = *out;
        plain_out.rank = 3;
        plain_out.dims[0] = out->dims[0] * out->dims[1];
        plain_out.dims[1] = out->dims[2] * out->dims[3];
        plain_out.dims[2] = out->dims[4] * out->dims[5];
        plain_out.strides[2] = 2;
        plain_out.strides[1] = plain_out.dims[2] * 2;
        plain_out.strides[0] = plain_out.dims[1] * plain_out.strides[1];
        out = &plain_out;  // extents for the checks below; the addresses come from the view
        // eight contiguous elements along n2 (strides[5] == 2) or, transposing, along m2 (strides[3] == 2)
        const int inner = view->strides[5] == 2 ? 5 : 3;
        if (view->strides[inner] != 2 || view->dims[inner] % 8 != 0) return 0;
        int64_t span = 16;
        for (int i = 0; i < 6; i++) {
            if (i != inner && (view->strides[i] % 16 != 0 || view->strides[i] < 0)) return 0;
            if (i >= 2) span += (view->dims[i] - 1) * view->strides[i];
        }
        if (span >= (int64_t(1) << 31) - 64) return 0;
    }
    const int osize = bias_cast ? 2 : 4;
    if (bias_cast && bias != nullptr) {
        const int64_t n = numel(bias);
        const bool last_axis = bias->dims[bias->rank - 1] == n && bias->strides[bias->rank - 1] == 4;
        if (bias->dtype != MLEL_F32 || !last_axis || (n != 1 && n != out->dims[2]) || ((uintptr_t)bias->ptr % 4) != 0)
            return 0;
    }
    if (attr->a_zp != 0 || attr->b_zp != 0) return 0;
    const int64_t NB = out->dims[0], M = out->dims[1], N = out->dims[2], K = a->dims[2];
    // what the kernel's indexing assumes: element-contiguous rows, 16-byte aligned rows and bases, K and N in
    // multiples of 8, per-batch extents below 2^31, operands at least as large as the output implies
    if (a->dims[0] < NB || b->dims[0] < NB || a->dims[1] < M || b->dims[1] < K || b->dims[2] < N) return 0;
    // B row-wise: element (k, n) at n * pitch + 2 k, i.e. a [K][N] view of a matrix stored as [N][K] (K > 1, so the
    // two layouts cannot be confused); the direct-to-LDS loop then wants whole 64-byte steps of K
    const bool b_rows = K > 1 && b->strides[1] == 2 && b->strides[2] >= b->dims[1] * 2;
    if (!dense_rows(a) || !(b_rows || dense_rows(b)) || out->strides[2] != osize) return 0;
    if (K % 8 != 0 || N % 8 != 0 || K <= 0 || (b_rows && K % 32 != 0)) return 0;
    auto aligned = [](const mlel_tensor *t) {
        return ((uintptr_t)t->ptr % 16) == 0 && t->strides[0] % 16 == 0 && t->strides[1] % 16 == 0;
    };
    if (!aligned(a) || !aligned(out) || (b_rows ? ((uintptr_t)b->ptr % 16) != 0 || b->strides[0] % 16 != 0 || b->strides[2] % 16 != 0
                                                : !aligned(b)))
        return 0;
    const int64_t lim = (int64_t(1) << 31) - 64;
    const int64_t b_pitch = b_rows ? b->strides[2] : b->strides[1];
    const int64_t ab = a->dims[1] * a->strides[1], bb = (b_rows ? b->dims[2] : b->dims[1]) * b_pitch, ob = M * out->strides[1];
    if (ab >= lim || bb >= lim || ob >= lim || a->strides[1] >= lim || b_pitch >= lim) return 0;
    if (M >= (1 << 24) || N >= (1 << 24) || K >= (1 << 24)) return 0;
    if (NB <= 0 || M <= 0 || N <= 0) return 2;

    HGemmArgs g{};
    g.a = static_cast<const char *>(a->ptr);
    g.b = static_cast<const char *>(b->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.M = (int)M;
    g.N = (int)N;
    g.K = (int)K;
    g.batches = (int)NB;
    g.a_batch = a->strides[0];
    g.b_batch = b->strides[0];
    g.o_batch = out->strides[0];
    g.lda = (uint32_t)a->strides[1];
    g.ldb = (uint32_t)b_pitch;
    g.b_rows = b_rows ? 1 : 0;
    g.ldo = (uint32_t)out->strides[1];
    g.a_bytes = (uint32_t)ab;
    g.b_bytes = (uint32_t)bb;
    g.o_bytes = (uint32_t)ob;
    g.bias = bias_cast && bias != nullptr ? static_cast<const float *>(bias->ptr) : nullptr;
    g.bias_len = bias_cast && bias != nullptr ? (int)numel(bias) : 0;
    if (view != nullptr) {
        g.view = 1;
        g.v_nb2 = (int32_t)view->dims[1];
        g.v_m2 = (int32_t)view->dims[3];
        g.v_n2 = (int32_t)view->dims[5];
        g.vs_nb1 = view->strides[0];
        g.vs_nb2 = view->strides[1];
        g.vs_m1 = (uint32_t)view->strides[2];
        g.vs_m2 = (uint32_t)view->strides[3];
        g.vs_n1 = (uint32_t)view->strides[4];
        g.vs_n2 = (uint32_t)view->strides[5];
        if (view->strides[5] != 2) g.view = 2;
        int64_t span = 16;
        for (int i = 2; i < 6; i++) span += (view->dims[i] - 1) * view->strides[i];
        g.o_bytes = (uint32_t)span;
    }
    if (residual != nullptr) {
        g.res = static_cast<const char *>(residual->ptr);
        g.r_batch = residual->strides[0];
        g.ldr = (uint32_t)residual->strides[1];
        g.r_bytes = (uint32_t)(residual->dims[1] * residual->strides[1]);
    }
    if (act != nullptr)
        for (int k = 0; k < 4; k++) g.act[k] = static_cast<const uint16_t *>(act[k]->ptr);
    g.groups = 1;
    *filled = g;
    return 1;
}

// Tile choice and launch of a described product (or group of products).
int launch_args(mlel_ctx *ctx, hipStream_t s, HGemmArgs &g, bool bias_cast) {
    const int64_t M = g.M, N = g.N, K = g.K, NB = g.batches;
    // tile choice: the width with the least padding of N; the tall tile when it still gives every compute unit two
    // blocks and the contraction is long enough to matter (a K of a few steps is bound by the stores, which the
    // short tile spreads over more blocks), otherwise the short one
    const int BN = ((N + 127) / 128) * 128 <= ((N + 63) / 64) * 64 ? 128 : 64;
    const int cus = ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256;
    g.tiles_n_group = (int)((N + BN - 1) / BN);
    const int64_t tiles_n = (int64_t)g.tiles_n_group * g.groups;
    const bool tall = K > 128 && ((M + 127) / 128) * tiles_n * NB >= 2 * (int64_t)cus;
    const int BM = tall ? 128 : 64;
    g.tiles_m = (int)((M + BM - 1) / BM);
    g.tiles_n = (int)tiles_n;
    const int64_t total = (int64_t)g.tiles_m * g.tiles_n * NB;
    MLEL_REQUIRE(total < (int64_t(1) << 30), MLEL_ERR_LIMIT, "matmul: %lld tiles", (long long)total);
    g.total_tiles = (int)total;
    g.chunk = (int)((total + 7) / 8);
    const dim3 grid((unsigned)(g.chunk * 8));
    // Eight wavefronts on the 128 x 128 tile when a compute unit gets at most three tiles: with so few blocks
    // resident nothing else hides the per-step barrier and LDS round trip (4096 x 768 x 3072: 36.4 -> 33.3 us); with
    // more tiles the four-wavefront blocks overlap each other and the larger wavefront tile wins.
    // A contraction of some length over few tiles (4096 x 3072 x 768 and 4096 x 768 x 768: 192 tiles of 128 x 128):
    // the eight-wavefront tile even when it leaves a quarter of the compute units idle, 43.1 -> 38.4 us and
    // 15.5 -> 13.7 us against 384 short tiles
    const int64_t tiles128 = ((M + 127) / 128) * tiles_n * NB;
    // The 256 x 256 tile of eight wavefronts (128 x 64 each: a third fewer operand reads from shared memory per
    // multiply) when it still occupies three quarters of the compute units: 4096 x 768 x 3072 in 192 tiles,
    // 37.7 -> 34.7 us.  With fewer tiles the idle compute units cost more than the reads (144 tiles: no gain;
    // 48 tiles: twice the time).  With the K-major loop an activation in the epilogue loses too, its arithmetic
    // running on three quarters of the machine (the same product with the tanh GELU: 40.9 -> 44.1 us); with the
    // direct-to-LDS loop it gains a little (38.4 -> 37.3 us inside the encoder block), so that path takes the large
    // tile with or without one.
    const int64_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256) * NB;
    if (g.b_rows) {
        // row-wise B: the direct-to-LDS loop; the 256 x 256 tile under the same condition as below, else 128 x 128 of
        // eight wavefronts, whatever the extents (rows beyond M or N are fetched as zeros)
        const int64_t tn128 = (N + 127) / 128;
        if (g.groups == 1 && g.K >= 256 && tiles256 * 4 >= 3 * (int64_t)cus && tiles256 <= 2 * (int64_t)cus) {
            g.tiles_m = (int)((M + 255) / 256);
            g.tiles_n_group = (int)((N + 255) / 256);
            g.tiles_n = g.tiles_n_group;
            g.total_tiles = (int)tiles256;
            g.chunk = (int)((tiles256 + 7) / 8);
            launch_k<256, 256, 2, 4, 32, true>(g, bias_cast, dim3((unsigned)(g.chunk * 8)), s);
        } else {
            g.tiles_m = (int)((M + 127) / 128);
            g.tiles_n_group = (int)tn128;
            g.tiles_n = (int)(tn128 * g.groups);
            const int64_t t = (int64_t)g.tiles_m * g.tiles_n * NB;
            MLEL_REQUIRE(t < (int64_t(1) << 30), MLEL_ERR_LIMIT, "matmul: %lld tiles", (long long)t);
            g.total_tiles = (int)t;
            g.chunk = (int)((t + 7) / 8);
            launch_k<128, 128, 2, 4, 32, true>(g, bias_cast, dim3((unsigned)(g.chunk * 8)), s);
        }
        MLEL_TRY(check_launch("matmul fp16, row-wise B"));
        return 1;
    }
    if (BN == 128 && g.groups == 1 && g.act[0] == nullptr && g.K >= 256 && tiles256 * 4 >= 3 * (int64_t)cus && tiles256 <= 2 * (int64_t)cus) {
        g.tiles_m = (int)((M + 255) / 256);
        g.tiles_n_group = (int)((N + 255) / 256);
        g.tiles_n = g.tiles_n_group;
        g.total_tiles = (int)tiles256;
        g.chunk = (int)((tiles256 + 7) / 8);
        launch_k<256, 256, 2, 4, 32>(g, bias_cast, dim3((unsigned)(g.chunk * 8)), s);
    } else if (BN == 128 && !tall && g.K >= 512 && tiles128 * 5 >= 3 * (int64_t)cus) {
        g.tiles_m = (int)((M + 127) / 128);
        g.total_tiles = (int)tiles128;
        g.chunk = (int)((tiles128 + 7) / 8);
        launch_k<128, 128, 2, 4, 64>(g, bias_cast, dim3((unsigned)(g.chunk * 8)), s);
    } else if (BN == 128 && tall && g.K >= 256 && total <= 3 * (int64_t)cus)
        launch_k<128, 128, 2, 4, 64>(g, bias_cast, grid, s);
    else if (BN == 128 && tall)
        launch<128, 128, 2, 2>(g, bias_cast, grid, s);
    else if (BN == 128)
        launch<64, 128, 1, 4>(g, bias_cast, grid, s);
    else if (tall)
        launch<128, 64, 2, 2>(g, bias_cast, grid, s);
    else
        launch<64, 64, 2, 2>(g, bias_cast, grid, s);
    MLEL_TRY(check_launch("matmul fp16"));
    return 1;
}

}  // namespace

// `bias_cast` set: the fused form out(fp16) = CAST(MATMUL + bias) with an fp32 bias of length 1 or N (or none)
int try_matmul_f16_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *a,
                        const mlel_tensor *b, const mlel_matmul_attr *attr, bool bias_cast, const mlel_tensor *bias,
                        const mlel_tensor *residual, const mlel_tensor *const *gelu_inputs) {
    HGemmArgs g{};
    const int rc = fill_args(out, a, b, attr, bias_cast, bias, residual, &g, gelu_inputs);
    if (rc != 1) return rc == 2 ? 1 : 0;
    return launch_args(ctx, s, g, bias_cast);
}

// Up to three fused products of one A in a single launch; 0 unless every product is a case for the kernel and they
// agree in everything but their B, bias and output.
int try_matmul_f16_group(mlel_ctx *ctx, hipStream_t s, int n, const mlel_tensor *const *outs, const mlel_tensor *a,
                         const mlel_tensor *const *bs, const mlel_tensor *const *biases, const mlel_matmul_attr *attr) {
    if (n < 2 || n > 3) return 0;
    HGemmArgs g[3];
    for (int i = 0; i < n; i++) {
        if (fill_args(outs[i], a, bs[i], attr, true, biases[i], nullptr, &g[i]) != 1) return 0;
        const HGemmArgs &x = g[i], &y = g[0];
        if (x.M != y.M || x.N != y.N || x.K != y.K || x.batches != y.batches || x.ldb != y.ldb || x.b_rows != y.b_rows || x.b_bytes != y.b_bytes ||
            (x.batches > 1 && x.b_batch != y.b_batch) || x.bias_len != y.bias_len || (x.bias == nullptr) != (y.bias == nullptr))
            return 0;
    }
    for (int i = 1; i < n; i++) {
        const HGemmArgs &x = g[i];
        g[0].extra[i - 1] = HGemmArgs::Extra{x.b, x.bias, x.out, x.o_batch, x.ldo, x.o_bytes, x.view, x.v_nb2, x.v_m2, x.v_n2,
                                             x.vs_nb1, x.vs_nb2, x.vs_m1, x.vs_m2, x.vs_n1, x.vs_n2};
    }
    g[0].groups = n;
    return launch_args(ctx, s, g[0], true);
}

}  // namespace mlel
