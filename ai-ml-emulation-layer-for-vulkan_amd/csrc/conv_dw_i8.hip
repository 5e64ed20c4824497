// 1x1 CONV2D + RESCALE (+CLAMP) followed by 3x3 DEPTHWISE_CONV2D + RESCALE (+CLAMP), int8, in one launch: the
// expansion and the depthwise stage of an inverted-residual block whose image is small enough (at most 32 x 32
// positions) that a block of 256 or 512 threads can keep the expanded activations of 32 channels of a band of image rows in
// shared memory.  The expanded tensor (the largest of such a network) then never travels to memory, and the pair costs one
// launch.  Arithmetic as the two operators one after the other (reference: graph/shaders/graph_op/tosa/conv2d.comp:
// 40-116, depthwise_conv2d.comp, rescale.comp:28-63, clamp.comp:18-31): the bytes the first operator would have
// stored are the bytes held in shared memory.
//
// A block owns one image, one slice of 32 expanded channels and one band of at most eight output rows (bands
// recompute the input rows they share with a neighbour: the two phases are chains of dependent work, and a block's
// life is as long as its longest wavefront's).
//   Fill    the tile [TH][TW] positions x 32 channels (pitch YP bytes) is filled with the depthwise input zero point:
//           the positions around the image are the padding, whose taps then contribute nothing (see the expansion of
//           sum (x - zi) w in ops_fast.hip), so the second phase needs no bounds test.
//   Expand  the wavefronts walk the image in groups of 32 positions: v_mfma_i32_32x32x32_i8 with the positions as
//           rows and the slice's weights (registers) as columns, accumulators started from the bias with the input
//           zero point folded in.  A lane holds one channel and 16 positions: it requantises with that channel's
//           constants, a 4 x 4 byte transpose inside each lane quad turns four positions of one channel into four
//           channels of one position, and the dword goes to the tile.
//   Depthwise  work item = 4 channels x 4 output columns x TY output rows (2, or 1 when that still leaves no more
//           items than threads), as the stand-alone kernel: rows
//           transposed with v_perm_b32 into three taps per dword, v_dot4_i32_i8 against the weight columns,
//           requantise, one dword store per position.
// ---------------------------------------------------------------------------------------------------------------
#include <algorithm>

#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {
namespace {

constexpr int kSliceCh = 32;  // expanded channels per block

typedef int v16i32 __attribute__((ext_vector_type(16)));
typedef int v4i32 __attribute__((ext_vector_type(4)));

struct ConvDwArgs {
    const int8_t *x, *w1, *w2;
    const int32_t *b1, *b2;
    char *out;
    int32_t N, H, W, IC, C, OH, OW, P;  // P = H * W positions of an image, C expanded channels
    int32_t zx, b1_len;                 // 1x1 convolution: input zero point
    int32_t zi, b2_len, pad_t, pad_l;   // depthwise: input zero point, padding before the image
    uint32_t x_bytes, o_bytes;
    ScaleRef s1, s2;
    int32_t slices;                      // C / 32
    int32_t bands, band_out;             // bands of `band_out` output rows per image
    int32_t th, tw;                      // tile extent in positions
    int32_t strips, row_groups, items;   // depthwise work items of a block: 8 channel quads x strips x row groups
    uint32_t strips_magic, w_magic;      // floor(2^32 / d) + 1 for d = strips, W: x / d == umulhi(x, magic) for
                                         // x < 2^16 and 1 < d < 2^16
    int32_t blocks, chunk;               // `chunk` consecutive blocks per XCD
    DivMagic div_slices, div_bands;      // block index / slices, / bands as a multiplication and a shift
};

struct DwConst {  // per channel of the slice, in shared memory: 48 bytes
    ChanScale q;
    int32_t bias_adj;
    uint32_t wcol[3];  // column kx: bytes = the taps (0, kx), (1, kx), (2, kx), 0
    uint32_t pad[2];
};
static_assert(sizeof(DwConst) == 48, "DwConst layout");

// 3 rows x 4 channels (bytes) -> 4 channels x (3 taps, 0)
__device__ __forceinline__ void rows_to_taps(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t (&col)[4]) {
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    col[0] = __builtin_amdgcn_perm(r2, t0, 0x0c040100u);
    col[1] = __builtin_amdgcn_perm(r2, t0, 0x0c050302u);
    col[2] = __builtin_amdgcn_perm(r2, t1, 0x0c060100u);
    col[3] = __builtin_amdgcn_perm(r2, t1, 0x0c070302u);
}

// pitch of a position in the tile: 4 output columns further (4 SX positions) is 8 dwords further modulo 32, so the
// 8 quads x 4 strips that a half wavefront reads at once fall into 32 different banks
template <int SX>
constexpr int tile_pitch() {
    return SX == 1 ? 40 : 36;
}

template <int KC, int SX, int TY, int NT>
__global__ void __launch_bounds__(NT) conv1x1_dw3x3_i8_kernel(const ConvDwArgs a) {
    constexpr int kBlock = NT;
    constexpr int YP = tile_pitch<SX>();
    constexpr int TX = 4;
    extern __shared__ __align__(16) char smem[];
    DwConst *dwc = reinterpret_cast<DwConst *>(smem);  // [4][8]: [channel of the quad][quad]
    char *tile = smem + kSliceCh * sizeof(DwConst);

    // Every argument that the first requests depend on is asked for here, in one batch: left alone the compiler loads
    // arguments where they are first used, behind the early exit and behind each other's results, and a wavefront
    // waits for four trips to memory in a row before it has computed its first address.
    asm volatile("" ::"s"(a.chunk), "s"(a.blocks), "s"(a.slices), "s"(a.bands), "s"(a.band_out), "s"(a.OH), "s"(a.pad_t),
                 "s"(a.th), "s"(a.H), "s"(a.W), "s"(a.x), "s"(a.x_bytes), "s"(a.P), "s"(a.IC), "s"(a.w1), "s"(a.div_slices.m),
                 "s"(a.div_slices.s), "s"(a.div_bands.m), "s"(a.div_bands.s));
    // the rest of what the kernel reads before its first request, and every dword of the wide loads that bring it (a
    // register that nobody waits for is given away at once, and whoever gets it waits for the load to land first)
    asm volatile("" ::"s"(a.o_bytes), "s"(a.tw), "s"(a.strips), "s"(a.row_groups), "s"(a.items), "s"(a.strips_magic),
                 "s"(a.w_magic), "s"(a.zx), "s"(a.zi), "s"(a.b1_len), "s"(a.b2_len), "s"(a.pad_l), "s"(a.C), "s"(a.OW),
                 "s"(a.N), "s"(a.w2), "s"(a.b1), "s"(a.b2), "s"(a.out), "s"(a.s1.mult), "s"(a.s1.shift), "s"(a.s1.mult16),
                 "s"(a.s1.p.in_zp), "s"(a.s1.p.out_zp), "s"(a.s1.p.out_lo), "s"(a.s1.p.out_hi), "s"(a.s1.p.double_round),
                 "s"(a.s1.p.per_channel), "s"(a.s1.p.clamp_out), "s"(a.s2.mult), "s"(a.s2.shift), "s"(a.s2.mult16),
                 "s"(a.s2.p.in_zp), "s"(a.s2.p.out_zp), "s"(a.s2.p.out_lo), "s"(a.s2.p.out_hi), "s"(a.s2.p.double_round),
                 "s"(a.s2.p.per_channel), "s"(a.s2.p.clamp_out));
    const int bid = (int)(blockIdx.x % 8u) * a.chunk + (int)(blockIdx.x / 8u);
    if (bid >= a.blocks) return;
    const int rest_b = div_magic(bid, a.div_slices), slice = bid - rest_b * a.slices;
    const int n = div_magic(rest_b, a.div_bands), band = rest_b - n * a.bands;
    const int c0 = slice * kSliceCh;
    // the band's output rows [ob0, ob1) read the input rows y_base .. y_base + th - 1 (tile row r = input row
    // y_base + r); the rows of the image among them are [y_lo, y_hi)
    const int ob0 = band * a.band_out, ob1 = min(ob0 + a.band_out, a.OH);
    const int y_base = ob0 * SX - a.pad_t;
    const int y_lo = max(y_base, 0), y_hi = min(y_base + a.th, a.H);
    const int p_lo = y_lo * a.W, p_count = (y_hi - y_lo) * a.W;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 31, half = lane >> 5;
    const int32_t hi1_v = pin_vgpr(a.s1.p.out_hi), hi2_v = pin_vgpr(a.s2.p.out_hi);

    // ---- requests first: the slice's weights (matrix B operand: lane = channel lane % 32, 16 bytes of K from
    // 32 kc + 16 (lane / 32)) and the wavefront's first position group
    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);
    const uint32_t kOob = 0x80000000u;
    const int groups = (p_count + 31) >> 5;
    auto fetch = [&](int g, v4i32 (&xf)[KC]) {  // matrix A operand: lane = position lane % 32 of the group
        const int p = g * 32 + cl;
        const uint32_t off = (g < groups && p < p_count)
                                 ? ((uint32_t)n * (uint32_t)a.P + (uint32_t)(p_lo + p)) * (uint32_t)a.IC + (uint32_t)half * 16u
                                 : kOob;
#pragma unroll
        for (int kc = 0; kc < KC; kc++) xf[kc] = __builtin_amdgcn_raw_buffer_load_b128(xres, (int)(off + (uint32_t)kc * 32u), 0, 0);
    };
    v4i32 xf[KC], xn[KC], wf[KC];
    int g = wave;
    fetch(g, xf);
    {
        const int8_t *wp = a.w1 + (int64_t)(c0 + cl) * a.IC + half * 16;
#pragma unroll
        for (int kc = 0; kc < KC; kc++) wf[kc] = *reinterpret_cast<const v4i32 *>(wp + kc * 32);
    }

    // ---- fill the tile with the depthwise zero point (16-byte stores; the tile's size is a multiple of 16)
    const uint32_t zsplat = (uint32_t)(uint8_t)a.zi * 0x01010101u;
    {
        const int pieces = (a.th * a.tw * YP + 15) >> 4;  // the host rounds the tile's size up likewise
        const uint4 z = make_uint4(zsplat, zsplat, zsplat, zsplat);
        for (int i = tid; i < pieces; i += kBlock) reinterpret_cast<uint4 *>(tile)[i] = z;
    }
    // ---- depthwise constants of the slice: one channel per thread of the first half wavefront
    if (tid < kSliceCh) {
        const int ch = c0 + tid;
        DwConst d{};
        int32_t wsum = 0;
#pragma unroll
        for (int kx = 0; kx < 3; kx++) {
            const uint32_t w0 = (uint8_t)a.w2[(0 * 3 + kx) * a.C + ch], w1 = (uint8_t)a.w2[(1 * 3 + kx) * a.C + ch],
                           w2 = (uint8_t)a.w2[(2 * 3 + kx) * a.C + ch];
            d.wcol[kx] = w0 | (w1 << 8) | (w2 << 16);
            wsum = __builtin_amdgcn_sdot4((int)d.wcol[kx], 0x00010101, wsum, false);
        }
        const int32_t bias = a.b2[a.b2_len == 1 ? 0 : ch];
        d.bias_adj = (int32_t)((uint32_t)bias - (uint32_t)a.zi * (uint32_t)wsum);
        const int ci = a.s2.p.per_channel ? ch : 0;
        d.q = make_chan_scale(load_mult(a.s2, ci), (int32_t)a.s2.shift[ci], a.s2.p);
        dwc[(tid & 3) * 8 + (tid >> 2)] = d;
    }
    // ---- the 1x1 convolution's constants of this lane's channel: every lane holds half of the channel's weights
    int32_t bias_adj1;
    ChanScale q1;
    {
        int32_t wsum = 0;
#pragma unroll
        for (int kc = 0; kc < KC; kc++)
#pragma unroll
            for (int e = 0; e < 4; e++) wsum = __builtin_amdgcn_sdot4(wf[kc][e], 0x01010101, wsum, false);
        wsum += __shfl_xor(wsum, 32);
        const int ch = c0 + cl;
        const int32_t bias = a.b1[a.b1_len == 1 ? 0 : ch];
        bias_adj1 = (int32_t)((uint32_t)bias - (uint32_t)a.zx * (uint32_t)wsum);
        const int ci = a.s1.p.per_channel ? ch : 0;
        q1 = make_chan_scale(load_mult(a.s1, ci), (int32_t)a.s1.shift[ci], a.s1.p);
    }
    __syncthreads();  // the fill is complete before any position is written

    // ---- expand: 32 positions x 32 channels per step
    const uint32_t sel_a = (lane & 1) ? 0x03070105u : 0x06020400u;  // exchange with lane ^ 1
    const uint32_t sel_b = (lane & 2) ? 0x03020706u : 0x05040100u;  // exchange with lane ^ 2
    for (; g < groups; g += kBlock / 64) {
        fetch(g + kBlock / 64, xn);
        v16i32 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = bias_adj1;
#pragma unroll
        for (int kc = 0; kc < KC; kc++) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[kc], wf[kc], acc, 0, 0, 0);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int32_t v[4];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = requant_acc(acc[4 * q + e], q1, a.s1.p, hi1_v);
            const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
            uint32_t p = __builtin_amdgcn_perm(hi, lo, 0x05040100u);  // bytes = positions e of this lane's channel
            uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0xb1, 0xf, 0xf, true);
            p = __builtin_amdgcn_perm(o, p, sel_a);
            o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0x4e, 0xf, 0xf, true);
            p = __builtin_amdgcn_perm(o, p, sel_b);
            // now: position 32 g + 8 q + 4 (lane / 32) + lane % 4 of the band's rows, channels 4 (lane % 32 / 4) .. + 3
            const int pos = g * 32 + 8 * q + 4 * half + (lane & 3);
            if (pos < p_count) {
                const int ly = a.W == 1 ? pos : (int)__umulhi((uint32_t)pos, a.w_magic), x = pos - ly * a.W;
                *reinterpret_cast<uint32_t *>(tile + ((y_lo - y_base + ly) * a.tw + x + a.pad_l) * YP + (cl & ~3)) = p;
            }
        }
#pragma unroll
        for (int kc = 0; kc < KC; kc++) xf[kc] = xn[kc];
    }
    __syncthreads();

    // ---- depthwise over the tile
    const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(a.out, 0, (int)a.o_bytes, 0x00020000);
    const int cq = tid & 7;  // channel quad of the slice: the same for every item of a thread (kBlock % 8 == 0)
    uint32_t wc[3][4];
    int32_t bias_adj[4];
    ChanScale q2[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const DwConst d = dwc[e * 8 + cq];
        wc[0][e] = d.wcol[0], wc[1][e] = d.wcol[1], wc[2][e] = d.wcol[2];
        bias_adj[e] = d.bias_adj;
        q2[e] = d.q;
    }
    constexpr int NCOL = SX * (TX - 1) + 3, NROW = SX * (TY - 1) + 3;
    uint32_t wc1[3][4];  // the weight columns one byte up (second output row of a 4 x 4 transpose)
#pragma unroll
    for (int kx = 0; kx < 3; kx++)
#pragma unroll
        for (int e = 0; e < 4; e++) wc1[kx][e] = wc[kx][e] << 8;
    const uint32_t c = (uint32_t)(c0 + cq * 4);
    for (int item = tid; item < a.items; item += kBlock) {
        const uint32_t sp = (uint32_t)item >> 3;
        const int rg = a.strips == 1 ? (int)sp : (int)__umulhi(sp, a.strips_magic);
        const int strip = (int)sp - rg * a.strips;
        const int ox0 = strip * TX, ry0 = rg * TY;  // ry0: output row within the band
        const char *tp = tile + ((ry0 * SX) * a.tw + ox0 * SX) * YP + cq * 4;
        uint32_t raw[NROW][NCOL];
#pragma unroll
        for (int r = 0; r < NROW; r++) {
            const char *rp = tp + r * a.tw * YP;
#pragma unroll
            for (int j = 0; j < NCOL; j++) raw[r][j] = *reinterpret_cast<const uint32_t *>(rp + j * YP);
        }
        int32_t acc[TY][TX][4];  // tap kx == 0 of an output starts its accumulator from the bias term
        if constexpr (TY == 2 && SX == 1) {
            // both output rows from one 4 x 4 transpose per column: row 1 uses the weights one byte up
#pragma unroll
            for (int j = 0; j < NCOL; j++) {
                uint32_t col[4];
                transpose_4x4(raw[0][j], raw[1][j], raw[2][j], raw[3][j], col);
#pragma unroll
                for (int t = 0; t < TX; t++) {
                    const int kx = j - t;
                    if (kx < 0 || kx > 2) continue;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (kx == 0) {
                            acc[0][t][e] = dot4_from(col[e], wc[0][e], bias_adj[e]);
                            acc[1][t][e] = dot4_from(col[e], wc1[0][e], bias_adj[e]);
                        } else {
                            acc[0][t][e] = __builtin_amdgcn_sdot4((int)col[e], (int)wc[kx][e], acc[0][t][e], false);
                            acc[1][t][e] = __builtin_amdgcn_sdot4((int)col[e], (int)wc1[kx][e], acc[1][t][e], false);
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int ty = 0; ty < TY; ty++) {
#pragma unroll
                for (int j = 0; j < NCOL; j++) {
                    uint32_t col[4];
                    rows_to_taps(raw[ty * SX][j], raw[ty * SX + 1][j], raw[ty * SX + 2][j], col);
#pragma unroll
                    for (int t = 0; t < TX; t++) {
                        const int kx = j - t * SX;
                        if (kx < 0 || kx > 2) continue;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            if (kx == 0)
                                acc[ty][t][e] = dot4_from(col[e], wc[0][e], bias_adj[e]);
                            else
                                acc[ty][t][e] = __builtin_amdgcn_sdot4((int)col[e], (int)wc[kx][e], acc[ty][t][e], false);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int ty = 0; ty < TY; ty++) {
            const int oy = ob0 + ry0 + ty;
            if (oy >= ob1) break;
            const uint32_t orow = ((uint32_t)n * (uint32_t)a.OH + (uint32_t)oy) * (uint32_t)a.OW;
#pragma unroll
            for (int t = 0; t < TX; t++) {
                const int ox = ox0 + t;
                if (ox >= a.OW) break;
                int32_t v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = requant_acc(acc[ty][t][e], q2[e], a.s2.p, hi2_v);
                const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
                const uint32_t off = (orow + (uint32_t)ox) * (uint32_t)a.C + c;
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_amdgcn_perm(hi, lo, 0x05040100u), ores, (int)off, 0, kOutAux);
            }
        }
    }
}

template <int KC, int SX, int TY, int NT>
void launch_conv_dw_v(const ConvDwArgs &g, dim3 grid, size_t sm, hipStream_t s) {
    if (sm > 48 * 1024)
        (void)hipFuncSetAttribute((const void *)conv1x1_dw3x3_i8_kernel<KC, SX, TY, NT>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm);
    conv1x1_dw3x3_i8_kernel<KC, SX, TY, NT><<<grid, dim3(NT), sm, s>>>(g);
}

template <int KC, int NT>
void launch_conv_dw(const ConvDwArgs &g, int sx, int ty, dim3 grid, size_t sm, hipStream_t s) {
    if (sx == 1) {
        if (ty == 1)
            launch_conv_dw_v<KC, 1, 1, NT>(g, grid, sm, s);
        else
            launch_conv_dw_v<KC, 1, 2, NT>(g, grid, sm, s);
    } else {
        if (ty == 1)
            launch_conv_dw_v<KC, 2, 1, NT>(g, grid, sm, s);
        else
            launch_conv_dw_v<KC, 2, 2, NT>(g, grid, sm, s);
    }
}

template <int NT>
void launch_conv_dw_k(const ConvDwArgs &g, int kc, int sx, int ty, dim3 grid, size_t sm, hipStream_t s) {
    switch (kc) {
    case 1: launch_conv_dw<1, NT>(g, sx, ty, grid, sm, s); break;
    case 2: launch_conv_dw<2, NT>(g, sx, ty, grid, sm, s); break;
    case 3: launch_conv_dw<3, NT>(g, sx, ty, grid, sm, s); break;
    case 4: launch_conv_dw<4, NT>(g, sx, ty, grid, sm, s); break;
    default: launch_conv_dw<5, NT>(g, sx, ty, grid, sm, s); break;
    }
}

bool dense(const mlel_tensor *t) { return is_packed(t); }

}  // namespace

// What the kernel's indexing assumes is checked here; `launch` false only answers whether the case is covered.
// Returns 1 when taken (or covered), 0 when not, < 0 on a launch error.
int try_conv2d_dwconv_i8(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                         const mlel_tensor *w1, const mlel_tensor *b1, const mlel_conv2d_attr *a1,
                         const FusedEpilogue *e1, const mlel_tensor *w2, const mlel_tensor *b2,
                         const mlel_conv2d_attr *a2, const FusedEpilogue *e2, bool launch) {
    if (in->rank != 4 || out->rank != 4 || w1->rank != 4 || w2->rank != 4 || b1->rank != 1 || b2->rank != 1) return 0;
    if (in->dtype != MLEL_I8 || w1->dtype != MLEL_I8 || w2->dtype != MLEL_I8 || out->dtype != MLEL_I8) return 0;
    if (b1->dtype != MLEL_I32 || b2->dtype != MLEL_I32) return 0;
    if (a1->acc_type != MLEL_ACC_I32 || a2->acc_type != MLEL_ACC_I32) return 0;
    const int64_t N = in->dims[0], H = in->dims[1], W = in->dims[2], IC = in->dims[3];
    const int64_t C = w1->dims[0], OH = out->dims[1], OW = out->dims[2];
    // the 1x1 convolution: unit stride, no padding, symmetric weights, dense operands
    if (w1->dims[1] != 1 || w1->dims[2] != 1 || w1->dims[3] != IC) return 0;
    if (a1->stride[0] != 1 || a1->stride[1] != 1 || a1->dilation[0] != 1 || a1->dilation[1] != 1) return 0;
    if (a1->pad[0] || a1->pad[1] || a1->pad[2] || a1->pad[3] || a1->weight_zp != 0) return 0;
    if (IC % 32 != 0 || IC < 32 || IC > 160 || C % kSliceCh != 0 || C <= 0 || C >= (1 << 20)) return 0;
    if (!dense(in) || !dense(w1) || !dense(w2) || !dense(out)) return 0;
    if (!(b1->dims[0] == 1 || b1->dims[0] >= C) || b1->strides[0] != 4) return 0;
    if (!(b2->dims[0] == 1 || b2->dims[0] >= C) || b2->strides[0] != 4) return 0;
    // the depthwise convolution: 3x3 taps, multiplier 1, equal stride 1 or 2, symmetric weights
    if (w2->dims[0] != 3 || w2->dims[1] != 3 || w2->dims[2] != C || w2->dims[3] != 1) return 0;
    if (a2->dilation[0] != 1 || a2->dilation[1] != 1 || a2->weight_zp != 0) return 0;
    if (a2->stride[0] != a2->stride[1] || a2->stride[0] < 1 || a2->stride[0] > 2) return 0;
    const int sx = a2->stride[0];
    for (int i = 0; i < 4; i++)
        if (a2->pad[i] < 0 || a2->pad[i] > 2) return 0;
    if (out->dims[0] != N || out->dims[3] != C || N <= 0 || H <= 0 || W <= 0 || OH <= 0 || OW <= 0) return 0;
    // output extent as the operator defines it: every tap of every output lies inside the padded image
    if ((OH - 1) * sx + 3 > H + a2->pad[0] + a2->pad[1] || (OW - 1) * sx + 3 > W + a2->pad[2] + a2->pad[3]) return 0;
    if (e1 == nullptr || e2 == nullptr) return 0;
    // image small enough for the tile, 32-bit offsets
    if (H > 32 || W > 32) return 0;
    if (N * H * W * IC >= (int64_t(1) << 31) || N * OH * OW * C >= (int64_t(1) << 31)) return 0;

    ConvDwArgs g{};
    const int cus = ctx != nullptr && ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256;
    // bands of eight output rows (measured on 7 x 7 to 28 x 28 images: a longer band leaves its block's wavefronts
    // with chains of work too long to hide, a shorter one recomputes too many shared rows); shorter bands only when
    // the launch would otherwise leave compute units without a block
    g.strips = (int)((OW + 3) / 4);
    int band_out = (int)std::min<int64_t>(8, (OH + 1) & ~int64_t(1));
    while (band_out > 4 && N * (C / kSliceCh) * ((OH + band_out - 1) / band_out) < (int64_t)cus * 3 / 2) band_out -= 2;
    g.bands = (int)((OH + band_out - 1) / band_out);
    g.band_out = band_out;
    // 512 threads when the band has more than twelve groups of 32 input positions, else 256; two output rows per
    // work item, one when that still leaves threads without an item
    const int64_t band_in = std::min<int64_t>((band_out - 1) * sx + 3, H) * W;
    const int nt = band_in > 12 * 32 ? 512 : 256;
    const int ty = 8 * g.strips * (band_out / 2) * 2 <= nt ? 1 : 2;
    g.row_groups = band_out / ty;
    // the tile covers every tap of every work item, also of the columns beyond the output's edge
    g.th = (band_out - 1) * sx + 3;
    g.tw = (int)std::max<int64_t>((g.strips * 4 - 1) * sx + 3, W + a2->pad[2]);
    const int yp = sx == 1 ? tile_pitch<1>() : tile_pitch<2>();
    size_t tile_bytes = (size_t)g.th * g.tw * yp;
    tile_bytes = (tile_bytes + 15) & ~size_t(15);
    const size_t sm = kSliceCh * sizeof(DwConst) + tile_bytes;
    if (sm > 64 * 1024) return 0;
    if (!launch) return 1;
    // requant_acc: both RESCALEs read int32 accumulators, whose input_zp TOSA fixes at 0
    if (e1->p.in_zp != 0 || e2->p.in_zp != 0) return 0;
    if (((uintptr_t)in->ptr % 16) != 0 || ((uintptr_t)w1->ptr % 16) != 0 || ((uintptr_t)out->ptr % 4) != 0) return 0;
    if (((uintptr_t)b1->ptr % 4) != 0 || ((uintptr_t)b2->ptr % 4) != 0) return 0;

    g.x = static_cast<const int8_t *>(in->ptr);
    g.w1 = static_cast<const int8_t *>(w1->ptr);
    g.w2 = static_cast<const int8_t *>(w2->ptr);
    g.b1 = static_cast<const int32_t *>(b1->ptr);
    g.b2 = static_cast<const int32_t *>(b2->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.N = (int)N, g.H = (int)H, g.W = (int)W, g.IC = (int)IC, g.C = (int)C, g.OH = (int)OH, g.OW = (int)OW;
    g.P = (int)(H * W);
    g.zx = a1->input_zp;
    g.b1_len = (int)b1->dims[0];
    g.zi = a2->input_zp;
    g.b2_len = (int)b2->dims[0];
    g.pad_t = a2->pad[0];
    g.pad_l = a2->pad[2];
    g.x_bytes = (uint32_t)(N * H * W * IC);
    g.o_bytes = (uint32_t)(N * OH * OW * C);
    g.s1 = make_ref(*e1);
    g.s2 = make_ref(*e2);
    g.slices = (int)(C / kSliceCh);
    g.items = 8 * g.strips * g.row_groups;
    g.strips_magic = (uint32_t)((uint64_t(1) << 32) / (uint64_t)g.strips + 1);
    g.w_magic = (uint32_t)((uint64_t(1) << 32) / (uint64_t)W + 1);
    const int64_t blocks = N * g.slices * g.bands;
    if (blocks >= (int64_t(1) << 31) - 8) return 0;
    g.blocks = (int)blocks;
    g.chunk = (int)((blocks + 7) / 8);
    g.div_slices = make_div_magic((uint32_t)g.slices);
    g.div_bands = make_div_magic((uint32_t)g.bands);
    const dim3 grid((unsigned)(g.chunk * 8));
    if (nt == 512)
        launch_conv_dw_k<512>(g, (int)(IC / 32), sx, ty, grid, sm, s);
    else
        launch_conv_dw_k<256>(g, (int)(IC / 32), sx, ty, grid, sm, s);
    MLEL_TRY(check_launch("conv2d 1x1 + depthwise 3x3 int8"));
    return 1;
}

}  // namespace mlel
