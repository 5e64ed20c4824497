// Direct int8 CONV2D for contractions too short to feed the matrix cores: K = KH*KW*IC of a few dozen bytes.
//
// Two shapes are covered (reference arithmetic: graph/shaders/graph_op/tosa/conv2d.comp:40-116):
//   STEM   3x3 taps, 1..4 input channels, any stride and padding, unit dilation (an image stem: K = 27 for RGB)
//   ROWS   1x1 stride-1 convolution over a dense image whose pixels are 16 / 24 / 32 bytes (K = IC)
// One thread owns one output position and OCB (16 or 32) consecutive output channels.  It gathers its K input bytes into KD
// dwords once, then for every channel runs KD v_dot4_i32_i8 against the channel's weights (broadcast reads from
// shared memory), requantises and stores OCB bytes with 128-bit stores.  There is no K loop, no barrier after the
// prologue and no padding of K to a matrix tile: the kernel is bound by the requantisation arithmetic and the
// output stream, not by the multiply-adds.
//
// Zero points follow the same expansion as the matrix kernel: taps that fall into the padding are filled with the
// input zero point (they then contribute exactly nothing), and
//   sum (x - zx)(w - zw) = sum x*w - zw * sum x - zx * sum w + K * zx * zw.
#include <algorithm>

#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {
namespace {

constexpr int kBlock = 256;

struct DirectArgs {
    const int8_t *x, *w;
    const int32_t *bias;
    char *out;
    int32_t M, OHW, OW, H, W, IC, OC;
    uint32_t x_sn, x_sy, x_sx;  // byte strides (the input extent is below 2^31)
    uint32_t x_bytes;
    int64_t ldw;  // bytes between the weights of consecutive output channels
    int32_t sy, sx, pad_t, pad_l, zx, zw, bias_len;
    int32_t fused, out_size;  // out_size 1 (fused, 8-bit) or 4 (int32 accumulators)
    ScaleRef scale;
    int32_t blocks, chunk;  // blocks over M; `chunk` consecutive blocks per XCD
    int32_t ocb;            // output channels per block (grid.y blocks cover OC)
};

struct ChanConst {  // per output channel, in shared memory.  48 bytes: lane l reads entry l with 128-bit accesses, and
                    // entries 32 bytes apart put two lanes of every group of sixteen on the same banks
    ChanScale q;
    int32_t bias_adj;
    int32_t pad[5];
};
static_assert(sizeof(ChanConst) == 48, "ChanConst layout");

enum { STEM = 0, ROWS = 1 };

// STEM: which bytes of dword `d` of a 3-pixel row segment belong to pixel `p` (pixels are IC bytes each)
template <int IC>
__host__ __device__ constexpr uint32_t pixel_mask(int p, int d) {
    uint32_t m = 0;
    for (int b = 0; b < 4; b++) {
        const int byte = 4 * d + b;
        if (byte / IC == p && byte < 3 * IC) m |= 0xffu << (8 * b);
    }
    return m;
}

// KD = dwords of gathered input per position; STEM: 3 rows x 3 dwords (IC = ICS), ROWS: IC / 4
template <int MODE, int ICS, int KD, int OCB, int P, bool Q8, bool ZW>
__global__ void __launch_bounds__(kBlock) conv_direct_i8_kernel(const DirectArgs a) {
    __shared__ __align__(16) uint32_t wl[OCB][KD];
    __shared__ __align__(16) ChanConst cc[OCB];
    const int oc0 = blockIdx.y * OCB;
    const int tid = threadIdx.x;

    // ---- prologue: this block's weights (in the gathered layout) and per-channel constants
    for (int i = tid; i < OCB * KD; i += kBlock) {
        const int oc = i / KD, j = i - oc * KD;
        const int8_t *wp = a.w + (int64_t)(oc0 + oc) * a.ldw;
        uint32_t v = 0;
        if (MODE == ROWS) {
            v = *reinterpret_cast<const uint32_t *>(wp + 4 * j);
        } else {
            const int ky = j / 3, d = j - ky * 3;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int byte = 4 * d + b;  // position inside the row segment of 3 * ICS bytes
                if (byte < 3 * ICS) v |= (uint32_t)(uint8_t)wp[ky * 3 * ICS + byte] << (8 * b);
            }
        }
        wl[oc][j] = v;
    }
    __syncthreads();
    const int kreal = MODE == ROWS ? 4 * KD : 27 * ICS / 3;
    for (int oc = tid; oc < OCB; oc += kBlock) {
        int32_t wsum = 0;
#pragma unroll
        for (int j = 0; j < KD; j++) wsum = __builtin_amdgcn_sdot4((int)wl[oc][j], 0x01010101, wsum, false);
        ChanConst c{};
        const int32_t bias = a.bias[a.bias_len == 1 ? 0 : oc0 + oc];
        c.bias_adj = (int32_t)((uint32_t)bias - (uint32_t)a.zx * (uint32_t)wsum +
                               (uint32_t)kreal * (uint32_t)a.zx * (uint32_t)a.zw);
        if (Q8) {
            const int ci = a.scale.p.per_channel ? oc0 + oc : 0;
            c.q = make_chan_scale(load_mult(a.scale, ci), (int32_t)a.scale.shift[ci], a.scale.p);
        }
        cc[oc] = c;
    }
    __syncthreads();

    // ---- this thread's P output positions (consecutive lanes take consecutive positions); blocks are dealt
    // round-robin to the XCDs, so hand XCD k the k-th contiguous run of positions (neighbouring output rows share
    // input rows in one L2)
    const int bid = (int)(blockIdx.x % 8u) * a.chunk + (int)(blockIdx.x / 8u);
    if (bid >= a.blocks) return;
    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);

    // ---- gather
    uint32_t xd[P][KD];
    int32_t xcorr[P];
    int mpos[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
        const int m = (bid * P + p) * kBlock + tid;
        mpos[p] = m;
        const bool live = m < a.M;
        if (MODE == ROWS) {
            const uint32_t off = (uint32_t)m * a.x_sx;
#pragma unroll
            for (int j = 0; j < KD; j++)
                xd[p][j] = live ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(xres, (int)(off + 4 * j), 0, 0) : 0u;
        } else {
            const int img = m / a.OHW, rem = m - img * a.OHW;
            const int oy = rem / a.OW, ox = rem - oy * a.OW;
            const int iy0 = oy * a.sy - a.pad_t, ix0 = ox * a.sx - a.pad_l;
            const uint32_t zs = (uint32_t)(uint8_t)a.zx * 0x01010101u;
            bool px[3];
#pragma unroll
            for (int q = 0; q < 3; q++) px[q] = (unsigned)(ix0 + q) < (unsigned)a.W;
#pragma unroll
            for (int ky = 0; ky < 3; ky++) {
                const int y = iy0 + ky;
                const bool rowok = live && (unsigned)y < (unsigned)a.H;
                // byte address of the segment; it may start before the tensor (left padding): such offsets wrap to
                // values beyond the extent and read as 0, and those bytes are replaced below anyway
                const int32_t addr = (int32_t)((uint32_t)img * a.x_sn + (uint32_t)y * a.x_sy) + ix0 * ICS;
                const int sh = addr & 3;
                const uint32_t base = (uint32_t)(addr - sh);
                uint32_t d[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    // 3 * ICS bytes starting at byte `sh` of the window: dword 3 is only touched for 4-byte pixels
                    const bool need = i * 4 < 3 * ICS + 3;
                    d[i] = (need && rowok)
                               ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(xres, (int)(base + 4 * i), 0, 0)
                               : 0u;
                }
#pragma unroll
                for (int i = 0; i < 3; i++) {
                    const uint32_t v = __builtin_amdgcn_alignbyte(d[i + 1], d[i], (uint32_t)sh);
                    uint32_t mask = 0;
#pragma unroll
                    for (int q = 0; q < 3; q++) mask |= (rowok && px[q]) ? pixel_mask<ICS>(q, i) : 0u;
                    const uint32_t segmask = pixel_mask<ICS>(0, i) | pixel_mask<ICS>(1, i) | pixel_mask<ICS>(2, i);
                    xd[p][ky * 3 + i] = ((v & mask) | (zs & ~mask)) & segmask;
                }
            }
        }
        xcorr[p] = 0;
        if (ZW) {
            int32_t xsum = 0;
#pragma unroll
            for (int j = 0; j < KD; j++) xsum = __builtin_amdgcn_sdot4((int)xd[p][j], 0x01010101, xsum, false);
            xcorr[p] = (int32_t)((uint32_t)a.zw * (uint32_t)xsum);
        }
    }

    // ---- multiply, requantise, store: the channel's weights and constants are read once for the P positions
#pragma unroll
    for (int g = 0; g < OCB / 16; g++) {
        uint32_t packed[P][4];
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int i = 0; i < 4; i++) packed[p][i] = 0;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int oc = g * 16 + e;
            uint32_t wv[KD];
#pragma unroll
            for (int j = 0; j < KD; j++) wv[j] = wl[oc][j];
            const ChanConst c = cc[oc];
#pragma unroll
            for (int p = 0; p < P; p++) {
                // the dot products accumulate on top of the bias term (and the weight zero-point term, if any)
                int32_t v = ZW ? (int32_t)((uint32_t)c.bias_adj - (uint32_t)xcorr[p]) : c.bias_adj;
#pragma unroll
                for (int j = 0; j < KD; j++) v = __builtin_amdgcn_sdot4((int)xd[p][j], (int)wv[j], v, false);
                if (Q8) {
                    packed[p][e / 4] |= ((uint32_t)requant_acc(v, c.q, a.scale.p) & 0xffu) << (8 * (e % 4));
                } else {
                    packed[p][e % 4] = (uint32_t)v;
                    if (e % 4 == 3 && mpos[p] < a.M)
                        *reinterpret_cast<uint4 *>(a.out + ((int64_t)mpos[p] * a.OC + oc0 + g * 16 + e - 3) * 4) =
                            make_uint4(packed[p][0], packed[p][1], packed[p][2], packed[p][3]);
                }
            }
        }
        if (Q8) {
#pragma unroll
            for (int p = 0; p < P; p++)
                if (mpos[p] < a.M)
                    *reinterpret_cast<uint4 *>(a.out + (int64_t)mpos[p] * a.OC + oc0 + g * 16) =
                        make_uint4(packed[p][0], packed[p][1], packed[p][2], packed[p][3]);
        }
    }
}

template <int MODE, int ICS, int KD, int P>
void launch_direct_p(const DirectArgs &g, dim3 grid, hipStream_t s) {
    // fused 8-bit epilogue or int32 accumulators, weight zero point or none: compile-time choices, so that the unrolled
    // channel loop is one basic block and the requantisation chains of neighbouring channels interleave
    const bool q8 = g.out_size == 1, zw = g.zw != 0;
#define MLEL_DIRECT(OCBV, Q8V, ZWV) conv_direct_i8_kernel<MODE, ICS, KD, OCBV, P, Q8V, ZWV><<<grid, dim3(kBlock), 0, s>>>(g)
    if (g.ocb == 32) {
        if (q8 && !zw) MLEL_DIRECT(32, true, false);
        else if (q8) MLEL_DIRECT(32, true, true);
        else if (!zw) MLEL_DIRECT(32, false, false);
        else MLEL_DIRECT(32, false, true);
    } else {
        if (q8 && !zw) MLEL_DIRECT(16, true, false);
        else if (q8) MLEL_DIRECT(16, true, true);
        else if (!zw) MLEL_DIRECT(16, false, false);
        else MLEL_DIRECT(16, false, true);
    }
#undef MLEL_DIRECT
}

// Positions per thread: every channel's weights and constants are broadcast from shared memory once per thread, so
// two positions per thread halve that traffic.  It pays for the shortest rows only (16-byte pixels, 32 channels per
// block, measured); longer rows lose more to the registers the second position holds.
template <int MODE, int ICS, int KD>
void launch_direct(DirectArgs &g, int splits, int cus, hipStream_t s) {
    int p = 1;
    if (MODE == ROWS && KD == 4 && g.ocb == 32 && g.out_size == 1) {
        const int64_t blocks = (g.M + (int64_t)kBlock * 2 - 1) / ((int64_t)kBlock * 2);
        if (blocks * splits >= 2 * (int64_t)cus) p = 2;  // still two blocks per compute unit
    }
    g.blocks = (int)((g.M + (int64_t)kBlock * p - 1) / ((int64_t)kBlock * p));
    g.chunk = (g.blocks + 7) / 8;
    const dim3 grid((unsigned)(g.chunk * 8), (unsigned)splits);
    if (p == 2) {
        if constexpr (MODE == ROWS && KD == 4) launch_direct_p<MODE, ICS, KD, 2>(g, grid, s);
    } else {
        launch_direct_p<MODE, ICS, KD, 1>(g, grid, s);
    }
}


// ---------------------------------------------------------------------------------------------------------------
// ROWS on the matrix cores: 1x1 stride-1 CONV2D + RESCALE (+CLAMP) to 8 bits over a dense image with 8..32-byte
// pixels and at most 192 output channels (MobileNetV2's expansions 16 -> 96, 24 -> 144, 32 -> 192 and 32 -> 16).
// The contraction is one or two v_mfma_i32_32x32x16_i8 per 32 positions x 32 channels, so the multiply-adds cost
// next to nothing; the kernel is built around the two things that do cost: the requantisation arithmetic and the
// output stream.
//   * A wavefront owns 32 consecutive positions and ALL output channels; it walks position groups in a grid-stride
//     loop with the weights (matrix B operand) in registers.  Its output tile is therefore one contiguous run of
//     32 * OC bytes of the NHWC tensor.
//   * After the multiply a lane holds one channel per 32-channel column (lane % 32) and 16 positions: the channel's
//     requantisation constants are read once per column from shared memory (32 bytes per lane) and used 16 times.
//   * The four results of a register group are four consecutive positions of one channel; a 4 x 4 byte transpose
//     inside each lane quad turns them into four consecutive channels of one position, which go to the wavefront's
//     own staging tile in shared memory as a dword.  The tile leaves in 16-byte pieces in memory order: every store
//     instruction writes one kilobyte of consecutive bytes.  No block-wide barrier after the prologue.
// ---------------------------------------------------------------------------------------------------------------
struct RowsMfmaArgs {
    const int8_t *x, *w;
    const int32_t *bias;
    char *out;
    int32_t M, IC, OC, zx, bias_len;
    int32_t groups;  // ceil(M / 32)
    int32_t op;      // pitch of a staging row (bytes): OC + padding, chosen so that four consecutive rows start in
                     // different bank octets
    uint32_t x_bytes, o_bytes;
    ScaleRef scale;
};

typedef int v16i32 __attribute__((ext_vector_type(16)));
typedef int v4i32 __attribute__((ext_vector_type(4)));

template <int NJ, int KC>
__global__ void __launch_bounds__(kBlock) conv_rows_mfma_i8_kernel(const RowsMfmaArgs a) {
    const int32_t hi_v = pin_vgpr(a.scale.p.out_hi);
    extern __shared__ __align__(16) char smem[];
    ChanConst *cc = reinterpret_cast<ChanConst *>(smem);  // [NJ * 32], channels at or beyond OC hold zeros
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 31, half = lane >> 5;

    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(a.out, 0, (int)a.o_bytes, 0x00020000);
    const uint32_t kOob = 0x80000000u;
    auto fetch = [&](int g, long (&xf)[KC]) {  // matrix A operand: lane = position lane % 32 of the group
        const int m = g * 32 + cl;
#pragma unroll
        for (int c = 0; c < KC; c++) {
            const int k0 = c * 16 + half * 8;
            const uint32_t off = (g < a.groups && m < a.M && k0 < a.IC) ? (uint32_t)m * (uint32_t)a.IC + (uint32_t)k0 : kOob;
            const auto v = __builtin_amdgcn_raw_buffer_load_b64(xres, (int)off, 0, 0);
            xf[c] = (long)(((uint64_t)v[1] << 32) | (uint64_t)v[0]);
        }
    };
    // the first group's pixels and the weights are requested before the constants are worked out, so that the
    // prologue waits for memory once
    const int nwaves = (int)gridDim.x * (kBlock / 64);
    int g = (int)blockIdx.x * (kBlock / 64) + wave;
    long xf[KC], xn[KC];
    fetch(g, xf);
    // ---- the weights as matrix B operand: lane = channel lane % 32 of column j, 8 bytes of K from 16 c + 8 (lane / 32)
    long wf[NJ][KC];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int c = 0; c < KC; c++) {
            const int oc = j * 32 + cl, k0 = c * 16 + half * 8;
            wf[j][c] = (oc < a.OC && k0 < a.IC) ? *reinterpret_cast<const long *>(a.w + (int64_t)oc * a.IC + k0) : 0;
        }
    // ---- per-channel constants (the input zero point folded into the bias term)
    for (int oc = tid; oc < NJ * 32; oc += kBlock) {
        ChanConst c{};
        if (oc < a.OC) {
            int32_t wsum = 0;
            const uint32_t *wp = reinterpret_cast<const uint32_t *>(a.w + (int64_t)oc * a.IC);
            for (int j = 0; j < a.IC / 4; j++) wsum = __builtin_amdgcn_sdot4((int)wp[j], 0x01010101, wsum, false);
            const int32_t bias = a.bias[a.bias_len == 1 ? 0 : oc];
            c.bias_adj = (int32_t)((uint32_t)bias - (uint32_t)a.zx * (uint32_t)wsum);
            const int ci = a.scale.p.per_channel ? oc : 0;
            c.q = make_chan_scale(load_mult(a.scale, ci), (int32_t)a.scale.shift[ci], a.scale.p);
        }
        cc[oc] = c;
    }
    __syncthreads();

    int32_t bias_adj[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) bias_adj[j] = cc[j * 32 + cl].bias_adj;
    char *so = smem + NJ * 32 * sizeof(ChanConst) + wave * 32 * a.op;  // this wavefront's staging tile [32][op]
    // The tile leaves in 16-byte pieces.  Lanes walk the staging tile itself, padding included: slot s = 64 t + lane
    // is bytes 16 s .. 16 s + 15 of the tile, so a 128-bit read of the wavefront covers one kilobyte of consecutive
    // shared memory (no bank is asked twice); a slot that falls into a row's padding moves nothing.  Slot s is row
    // s / (op / 16), 16-byte column s % (op / 16).
    constexpr int NP = NJ + 1;  // op <= OC + 48 and OC > 32 (NJ - 1): at most NJ + 1 rounds of 64 slots
    const int spr = a.op >> 4, ppr = a.OC >> 4, nslots = 32 * spr;
    uint32_t piece_row[NP], piece_out[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) {
        const int sl = t * 64 + lane;
        const int r = sl / spr, c = sl - r * spr;
        const bool live = sl < nslots && c < ppr;
        piece_row[t] = live ? (uint32_t)r : 0xffffu;  // a dead slot: never below a row count
        piece_out[t] = (uint32_t)(r * a.OC + c * 16);
    }
    const int rounds = (nslots + 63) >> 6;
    const uint32_t sel_a = (lane & 1) ? 0x03070105u : 0x06020400u;  // exchange with lane ^ 1
    const uint32_t sel_b = (lane & 2) ? 0x03020706u : 0x05040100u;  // exchange with lane ^ 2
    char *so_lane = so + (4 * half + (lane & 3)) * a.op + (cl & ~3);
    for (; g < a.groups; g += nwaves) {
        fetch(g + nwaves, xn);  // the next group's pixels travel while this one is requantised
        // the accumulators start from the channel's bias term (every register of a lane is the same channel)
        v16i32 accs[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++) {
#pragma unroll
            for (int r = 0; r < 16; r++) accs[j][r] = bias_adj[j];
#pragma unroll
            for (int kc = 0; kc < KC; kc++)
                accs[j] = __builtin_amdgcn_mfma_i32_32x32x16_i8(xf[kc], wf[j][kc], accs[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const ChanConst c = cc[j * 32 + cl];
            const bool col_live = j * 32 + (cl & ~3) < a.OC;  // OC is a multiple of 16: whole dwords are in or out
            const v16i32 acc = accs[j];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int32_t v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[e] = requant_acc(acc[4 * q + e], c.q, a.scale.p, hi_v);
                }
                const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
                uint32_t p = __builtin_amdgcn_perm(hi, lo, 0x05040100u);  // bytes = positions e of this lane's channel
                uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0xb1, 0xf, 0xf, true);
                p = __builtin_amdgcn_perm(o, p, sel_a);
                o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0x4e, 0xf, 0xf, true);
                p = __builtin_amdgcn_perm(o, p, sel_b);
                // now: position 8 q + 4 (lane / 32) + lane % 4, channels 32 j + 4 (lane % 32 / 4) .. + 3
                if (col_live) *reinterpret_cast<uint32_t *>(so_lane + 8 * q * a.op + j * 32) = p;
            }
        }
        // the wavefront's own writes and reads of its tile execute in order; the compiler must keep that order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint32_t rows = (uint32_t)min(32, a.M - g * 32);
        const uint32_t obase = (uint32_t)g * 32u * (uint32_t)a.OC;
#pragma unroll
        for (int t = 0; t < NP; t++) {
            if (t < rounds) {  // uniform
                const uint4 d = *reinterpret_cast<const uint4 *>(so + (t * 64 + lane) * 16);
                const uint32_t off = piece_row[t] < rows ? obase + piece_out[t] : kOob;
                __builtin_amdgcn_raw_buffer_store_b128(v4i32{(int)d.x, (int)d.y, (int)d.z, (int)d.w}, ores, (int)off, 0, kOutAux);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int c = 0; c < KC; c++) xf[c] = xn[c];
    }
}

template <int NJ>
void launch_rows_mfma(const RowsMfmaArgs &g, int kc, dim3 grid, size_t sm, hipStream_t s) {
    if (kc == 1)
        conv_rows_mfma_i8_kernel<NJ, 1><<<grid, dim3(kBlock), sm, s>>>(g);
    else
        conv_rows_mfma_i8_kernel<NJ, 2><<<grid, dim3(kBlock), sm, s>>>(g);
}

// returns 1 when the case was taken
int try_rows_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                  const mlel_tensor *bias, const mlel_conv2d_attr *a, const FusedEpilogue *epi, int64_t M, int64_t IC,
                  int64_t OC, int64_t xbytes) {
    if (epi == nullptr || a->weight_zp != 0) return 0;
    if (IC % 8 != 0 || IC > 32 || OC % 16 != 0 || OC > 192) return 0;
    if (((uintptr_t)in->ptr % 8) != 0 || ((uintptr_t)w->ptr % 8) != 0) return 0;
    if (M * OC >= (int64_t(1) << 31) || M * IC >= (int64_t(1) << 31)) return 0;
    RowsMfmaArgs g{};
    g.x = static_cast<const int8_t *>(in->ptr);
    g.w = static_cast<const int8_t *>(w->ptr);
    g.bias = static_cast<const int32_t *>(bias->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.M = (int)M;
    g.IC = (int)IC;
    g.OC = (int)OC;
    g.zx = a->input_zp;
    g.bias_len = (int)bias->dims[0];
    g.groups = (int)((M + 31) / 32);
    int op = (int)OC;
    while (op % 128 != 32 && op % 128 != 96) op += 16;
    g.op = op;
    g.x_bytes = (uint32_t)xbytes;
    g.o_bytes = (uint32_t)(M * OC);
    g.scale = make_ref(*epi);
    const int nj = (int)((OC + 31) / 32), kc = IC > 16 ? 2 : 1;
    // (the last round of slots may read up to 512 bytes past the last wavefront's tile: they are part of the allocation)
    const size_t sm = (size_t)nj * 32 * sizeof(ChanConst) + (size_t)(kBlock / 64) * 32 * op + 512;
    const int cus = ctx != nullptr && ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256;
    // Sixteen position groups per block (four per wavefront) amortise the prologue (weights, channel constants);
    // between two and three blocks per compute unit, never more blocks than a group per wavefront needs.  Measured:
    // 16 -> 96 channels on 112 x 112 images is flat from two to four blocks per compute unit, 24 -> 144 on 56 x 56
    // (a quarter of the groups) loses 15 % at three.
    const int64_t per_wave = (g.groups + kBlock / 64 - 1) / (kBlock / 64);
    const int64_t want =
        std::min<int64_t>(per_wave, std::min<int64_t>((int64_t)cus * 3, std::max<int64_t>((int64_t)cus * 2, (g.groups + 15) / 16)));
    const dim3 grid((unsigned)std::max<int64_t>(want, 1));
    switch (nj) {
    case 1: launch_rows_mfma<1>(g, kc, grid, sm, s); break;
    case 2: launch_rows_mfma<2>(g, kc, grid, sm, s); break;
    case 3: launch_rows_mfma<3>(g, kc, grid, sm, s); break;
    case 4: launch_rows_mfma<4>(g, kc, grid, sm, s); break;
    case 5: launch_rows_mfma<5>(g, kc, grid, sm, s); break;
    default: launch_rows_mfma<6>(g, kc, grid, sm, s); break;
    }
    return 1;
}

// ---------------------------------------------------------------------------------------------------------------
// Two 1x1 CONV2D + RESCALE (+CLAMP) in a row in one launch: a projection to at most 32 channels followed by the
// expansion that reads it (MobileNetV2: 32 -> 16 -> 96 at 112 x 112, 96 -> 24 -> 144 at 56 x 56).  Both operators
// treat positions independently, so the wavefront that owns 32 positions runs the first product (K = IC0 in steps of
// 16 on v_mfma_i32_32x32x16_i8, rows straight from memory, weights in registers), requantises its 32 x OC0 bytes into
// a tile of its own in shared memory -- the bytes the first operator would have stored -- and reads them back as the
// row operand of conv_rows_mfma_i8_kernel's loop.  When another operator reads the intermediate tensor as well (a
// residual connection further on) the tile is also written to memory, as consecutive bytes; otherwise it never
// leaves the chip.  Reference arithmetic: conv2d.comp:40-116, rescale.comp:28-63, clamp.comp:18-31, twice.
// ---------------------------------------------------------------------------------------------------------------
struct Rows2Args {
    RowsMfmaArgs r;          // the second operator; r.x is unused, r.IC = OC0
    const int8_t *x0, *w0;   // the first operator's input [M][IC0] and weights [OC0][IC0]
    const int32_t *bias0;
    char *mid;               // where the intermediate tensor [M][OC0] is stored as well, or nullptr
    int32_t IC0, zx0, bias0_len;
    uint32_t x0_bytes, mid_bytes;
    ScaleRef scale0;
};

template <int NJ, int KC, int KC0>
__global__ void __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(NJ <= 3 ? 3 : 2, NJ <= 3 ? 3 : 2)))
conv_rows2_mfma_i8_kernel(const Rows2Args b) {
    const RowsMfmaArgs &a = b.r;
    const int32_t hi_v = pin_vgpr(a.scale.p.out_hi), hi0_v = pin_vgpr(b.scale0.p.out_hi);
    extern __shared__ __align__(16) char smem[];
    ChanConst *cc = reinterpret_cast<ChanConst *>(smem);  // [NJ * 32] second operator, then [32] first operator
    ChanConst *cc0 = cc + NJ * 32;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 31, half = lane >> 5;
    const int OC0 = a.IC;

    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(b.x0), 0, (int)b.x0_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(a.out, 0, (int)a.o_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t mres =
        __builtin_amdgcn_make_buffer_rsrc(b.mid != nullptr ? b.mid : a.out, 0, (int)(b.mid != nullptr ? b.mid_bytes : 0u), 0x00020000);
    const uint32_t kOob = 0x80000000u;
    auto fetch = [&](int g, long (&xf)[KC0]) {  // first product's row operand: lane = position lane % 32 of the group
        const int m = g * 32 + cl;
#pragma unroll
        for (int c = 0; c < KC0; c++) {
            const int k0 = c * 16 + half * 8;
            const uint32_t off = (g < a.groups && m < a.M && k0 < b.IC0) ? (uint32_t)m * (uint32_t)b.IC0 + (uint32_t)k0 : kOob;
            const auto v = __builtin_amdgcn_raw_buffer_load_b64(xres, (int)off, 0, 0);
            xf[c] = (long)(((uint64_t)v[1] << 32) | (uint64_t)v[0]);
        }
    };
    const int nwaves = (int)gridDim.x * (kBlock / 64);
    int g = (int)blockIdx.x * (kBlock / 64) + wave;
    long xf0[KC0], xn0[KC0];
    fetch(g, xf0);
    // ---- both weight sets as matrix B operands: lane = channel lane % 32 (of column j), 8 bytes of K per lane half
    long wf0[KC0];
#pragma unroll
    for (int c = 0; c < KC0; c++) {
        const int k0 = c * 16 + half * 8;
        wf0[c] = (cl < OC0 && k0 < b.IC0) ? *reinterpret_cast<const long *>(b.w0 + (int64_t)cl * b.IC0 + k0) : 0;
    }
    long wf[NJ][KC];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int c = 0; c < KC; c++) {
            const int oc = j * 32 + cl, k0 = c * 16 + half * 8;
            wf[j][c] = (oc < a.OC && k0 < OC0) ? *reinterpret_cast<const long *>(a.w + (int64_t)oc * OC0 + k0) : 0;
        }
    // ---- per-channel constants of both operators (each input zero point folded into its bias term)
    for (int oc = tid; oc < NJ * 32 + 32; oc += kBlock) {
        ChanConst c{};
        const bool first = oc >= NJ * 32;
        const int ch = first ? oc - NJ * 32 : oc;
        const int chans = first ? OC0 : a.OC, kk = first ? b.IC0 : OC0;
        if (ch < chans) {
            int32_t wsum = 0;
            const uint32_t *wp = reinterpret_cast<const uint32_t *>((first ? b.w0 : a.w) + (int64_t)ch * kk);
            for (int j = 0; j < kk / 4; j++) wsum = __builtin_amdgcn_sdot4((int)wp[j], 0x01010101, wsum, false);
            const int32_t bias = first ? b.bias0[b.bias0_len == 1 ? 0 : ch] : a.bias[a.bias_len == 1 ? 0 : ch];
            c.bias_adj = (int32_t)((uint32_t)bias - (uint32_t)(first ? b.zx0 : a.zx) * (uint32_t)wsum);
            const ScaleRef &sc = first ? b.scale0 : a.scale;
            const int ci = sc.p.per_channel ? ch : 0;
            c.q = make_chan_scale(load_mult(sc, ci), (int32_t)sc.shift[ci], sc.p);
        }
        cc[oc] = c;
    }
    __syncthreads();

    int32_t bias_adj[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) bias_adj[j] = cc[j * 32 + cl].bias_adj;
    const ChanConst c0 = cc0[cl];  // the first operator's constants of this lane's channel stay in registers
    // this wavefront's tiles: the intermediate [32][OC0] (+ 16 bytes that the last row's second K piece may read),
    // then the staging tile [32][op] of the result
    const int mid_tile = 32 * OC0 + 16;
    char *mt = smem + (NJ * 32 + 32) * sizeof(ChanConst) + wave * (mid_tile + 32 * a.op);
    char *so = mt + mid_tile;
    constexpr int NP = NJ + 1;
    const int spr = a.op >> 4, ppr = a.OC >> 4, nslots = 32 * spr;
    uint32_t piece_row[NP], piece_out[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) {
        const int sl = t * 64 + lane;
        const int r = sl / spr, c = sl - r * spr;
        const bool live = sl < nslots && c < ppr;
        piece_row[t] = live ? (uint32_t)r : 0xffffu;
        piece_out[t] = (uint32_t)(r * a.OC + c * 16);
    }
    const int rounds = (nslots + 63) >> 6;
    const uint32_t sel_a = (lane & 1) ? 0x03070105u : 0x06020400u;  // exchange with lane ^ 1
    const uint32_t sel_b = (lane & 2) ? 0x03020706u : 0x05040100u;  // exchange with lane ^ 2
    char *so_lane = so + (4 * half + (lane & 3)) * a.op + (cl & ~3);
    char *mt_lane = mt + (4 * half + (lane & 3)) * OC0 + (cl & ~3);
    const bool mid_col_live = (cl & ~3) < OC0;  // OC0 is a multiple of 8: whole dwords are in or out
    const int mid_pieces = 2 * OC0;             // 16-byte pieces of the intermediate tile: 32 * OC0 / 16
    auto pack4 = [&](const int32_t (&v)[4]) {
        const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
        const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
        uint32_t p = __builtin_amdgcn_perm(hi, lo, 0x05040100u);  // bytes = positions e of this lane's channel
        uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0xb1, 0xf, 0xf, true);
        p = __builtin_amdgcn_perm(o, p, sel_a);
        o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0x4e, 0xf, 0xf, true);
        return __builtin_amdgcn_perm(o, p, sel_b);  // position 8 q + 4 (lane / 32) + lane % 4, four channels
    };
    auto wave_sync = [] {
        // the wavefront's own writes and reads of its tiles execute in order; the compiler must keep that order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    for (; g < a.groups; g += nwaves) {
        fetch(g + nwaves, xn0);  // the next group's pixels travel while this one is worked on
        const uint32_t rows = (uint32_t)min(32, a.M - g * 32);
        // ---- first operator: 32 positions x OC0 channels into the intermediate tile
        {
            v16i32 acc0;
#pragma unroll
            for (int r = 0; r < 16; r++) acc0[r] = c0.bias_adj;
#pragma unroll
            for (int kc = 0; kc < KC0; kc++) acc0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(xf0[kc], wf0[kc], acc0, 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int32_t v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = requant_acc(acc0[4 * q + e], c0.q, b.scale0.p, hi0_v);
                const uint32_t p = pack4(v);
                if (mid_col_live) *reinterpret_cast<uint32_t *>(mt_lane + 8 * q * OC0) = p;
            }
        }
        wave_sync();
        if (b.mid != nullptr && lane < mid_pieces) {  // the intermediate tensor's 32 rows are consecutive in memory
            const uint4 d = *reinterpret_cast<const uint4 *>(mt + lane * 16);
            const uint32_t off = (uint32_t)(lane * 16) < rows * (uint32_t)OC0 ? (uint32_t)g * 32u * (uint32_t)OC0 + (uint32_t)lane * 16u : kOob;
            __builtin_amdgcn_raw_buffer_store_b128(v4i32{(int)d.x, (int)d.y, (int)d.z, (int)d.w}, mres, (int)off, 0, kOutAux);
        }
        long xf[KC];
#pragma unroll
        for (int c = 0; c < KC; c++) xf[c] = *reinterpret_cast<const long *>(mt + cl * OC0 + c * 16 + half * 8);
        // ---- second operator, as conv_rows_mfma_i8_kernel, one 32-channel column after the other: only two
        // accumulator tiles are alive at a time (the next column's product runs while this one is requantised), which
        // keeps the register count low enough for several wavefronts per SIMD
        auto column = [&](int j) {
            v16i32 acc;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = bias_adj[j];
#pragma unroll
            for (int kc = 0; kc < KC; kc++) acc = __builtin_amdgcn_mfma_i32_32x32x16_i8(xf[kc], wf[j][kc], acc, 0, 0, 0);
            return acc;
        };
        v16i32 acc = column(0);
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            v16i32 next = acc;
            if (j + 1 < NJ) next = column(j + 1);
            const ChanConst c = cc[j * 32 + cl];
            const bool col_live = j * 32 + (cl & ~3) < a.OC;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int32_t v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = requant_acc(acc[4 * q + e], c.q, a.scale.p, hi_v);
                const uint32_t p = pack4(v);
                if (col_live) *reinterpret_cast<uint32_t *>(so_lane + 8 * q * a.op + j * 32) = p;
            }
            acc = next;
            __builtin_amdgcn_sched_barrier(0);  // (the scheduler would otherwise start every column's product first)
        }
        wave_sync();
        const uint32_t obase = (uint32_t)g * 32u * (uint32_t)a.OC;
#pragma unroll
        for (int t = 0; t < NP; t++) {
            if (t < rounds) {  // uniform
                const uint4 d = *reinterpret_cast<const uint4 *>(so + (t * 64 + lane) * 16);
                const uint32_t off = piece_row[t] < rows ? obase + piece_out[t] : kOob;
                __builtin_amdgcn_raw_buffer_store_b128(v4i32{(int)d.x, (int)d.y, (int)d.z, (int)d.w}, ores, (int)off, 0, kOutAux);
            }
        }
        wave_sync();
#pragma unroll
        for (int c = 0; c < KC0; c++) xf0[c] = xn0[c];
    }
}

// The shapes the two-operator kernel exists for (each is its own kernel): second operator's 32-channel columns,
// 16-byte K pieces of the second and of the first operator.
template <int NJ, int KC, int KC0>
void launch_rows2(const Rows2Args &g, dim3 grid, size_t sm, hipStream_t s) {
    auto kernel = conv_rows2_mfma_i8_kernel<NJ, KC, KC0>;
    if (sm > 48 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm);
    kernel<<<grid, dim3(kBlock), sm, s>>>(g);
}

bool rows2_shape(int64_t IC0, int64_t OC0, int64_t OC, int *nj, int *kc, int *kc0) {
    if (IC0 % 16 != 0 || OC0 % 8 != 0 || OC0 > 32 || OC0 <= 0 || OC % 16 != 0 || OC > 192 || OC <= 0) return false;
    *nj = (int)((OC + 31) / 32);
    *kc = OC0 > 16 ? 2 : 1;
    *kc0 = (int)(IC0 / 16);
    // the instantiated combinations: 32 -> 16 -> 96, 96 -> 24 -> 144 (MobileNetV2) and their neighbours
    const bool known = (*nj == 3 && *kc == 1 && *kc0 == 2) || (*nj == 5 && *kc == 2 && *kc0 == 6) ||
                       (*nj == 6 && *kc == 2 && *kc0 == 2) || (*nj == 6 && *kc == 2 && *kc0 == 6);
    return known;
}

// ---------------------------------------------------------------------------------------------------------------
// STEM on the matrix cores: 3x3 CONV2D over 3-byte pixels (an RGB image stem, K = 27) + RESCALE (+CLAMP) to 8 bits
// with 16 or 32 output channels.  The structure of conv_rows_mfma_i8_kernel (a wavefront owns 32 consecutive output
// positions and all channels, weights in registers, per-wavefront staging tile), with one v_mfma_i32_32x32x32_i8 per
// group and an operand fetch that gathers the patch: k = 9 ky + 3 kx + c, so a patch row is 9 consecutive bytes of
// the image.  Lane (position, half) supplies k = 16 half .. 16 half + 15: it loads the two patch rows it needs
// (half 0: rows 0 and 1, half 1: rows 1 and 2) as three dwords each around the unaligned 9 bytes, shifts them into
// place (v_alignbyte_b32), replaces the bytes of pixels outside the image by the input zero point (such taps then
// contribute nothing) and takes 16 bytes of the stream [row a, row b, zeros] from byte 0 or 7.  The weights of
// k = 27 .. 31 are zero.
// ---------------------------------------------------------------------------------------------------------------
struct StemMfmaArgs {
    const int8_t *x, *w;
    const int32_t *bias;
    char *out;
    int32_t M, OC, H, W, OW, OHW, zx, bias_len;
    int32_t sy, sx, pad_t, pad_l;
    uint32_t ow_magic;  // floor(2^32 / OW) + 1: x / OW == umulhi(x, magic) while x * OW < 2^32 (the host checks)
    int32_t groups, op;
    uint32_t x_bytes, o_bytes;
    ScaleRef scale;
};

__global__ void __launch_bounds__(kBlock) conv_stem_mfma_i8_kernel(const StemMfmaArgs a) {
    const int32_t hi_v = pin_vgpr(a.scale.p.out_hi);
    extern __shared__ __align__(16) char smem[];
    ChanConst *cc = reinterpret_cast<ChanConst *>(smem);  // [32], channels at or beyond OC hold zeros
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 31, half = lane >> 5;
    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(a.out, 0, (int)a.o_bytes, 0x00020000);
    const uint32_t kOob = 0x80000000u;
    const uint32_t zsplat = (uint32_t)(uint8_t)a.zx * 0x01010101u;

    // the six dwords around the lane's two patch rows, and what is needed to put them in place afterwards
    struct Patch {
        uint32_t d[2][3];
        uint32_t shift;       // byte offset of the patch row inside its first dword
        uint32_t m0, m1, m2;  // which bytes of a row are inside the image (by pixel), per dword of the shifted row
        bool row_in[2];
    };
    auto fetch = [&](int g, Patch &p) {
        const int m = g * 32 + cl;
        const bool live = g < a.groups && m < a.M;
        // image and position inside it: the group's first position is divided on the scalar side (g is uniform),
        // a lane is at most one image further (an image has at least 32 positions)
        const uint32_t m0 = (uint32_t)__builtin_amdgcn_readfirstlane(g) * 32u;
        uint32_t n = m0 / (uint32_t)a.OHW;
        uint32_t rem = m0 - n * (uint32_t)a.OHW + (uint32_t)cl;
        if (rem >= (uint32_t)a.OHW) rem -= (uint32_t)a.OHW, n++;
        const uint32_t oy = __umulhi(rem, a.ow_magic), ox = rem - oy * (uint32_t)a.OW;
        const int iy0 = (int)oy * a.sy - a.pad_t + half, ix0 = (int)ox * a.sx - a.pad_l;
        const bool px0 = (unsigned)ix0 < (unsigned)a.W, px1 = (unsigned)(ix0 + 1) < (unsigned)a.W,
                   px2 = (unsigned)(ix0 + 2) < (unsigned)a.W;
        p.m0 = (px0 ? 0x00ffffffu : 0u) | (px1 ? 0xff000000u : 0u);
        p.m1 = (px1 ? 0x0000ffffu : 0u) | (px2 ? 0xffff0000u : 0u);
        p.m2 = px2 ? 0x000000ffu : 0u;
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const int iy = iy0 + r;
            p.row_in[r] = live && (unsigned)iy < (unsigned)a.H;
            // byte address of pixel (iy, ix0); a negative ix0 names bytes before the row, which the masks discard
            const int32_t addr = (int32_t)((n * (uint32_t)a.H + (uint32_t)iy) * (uint32_t)a.W) * 3 + ix0 * 3;
            const int32_t base = addr & ~3;
            if (r == 0) p.shift = (uint32_t)addr & 3u;
#pragma unroll
            for (int k = 0; k < 3; k++) {
                const int32_t off = base + 4 * k;
                p.d[r][k] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(xres, (p.row_in[r] && off >= 0) ? off : (int)kOob, 0, 0);
            }
        }
    };
    // rows of a lane start at the same column, and consecutive rows are W * 3 bytes apart: the shift of row 1 is
    // (shift of row 0 + 3 W) & 3, worked out in place below
    auto operand = [&](const Patch &p) -> v4i32 {
        uint32_t q[2][3];
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const uint32_t sh = (p.shift + (uint32_t)(r * 3 * a.W)) & 3u;
            const uint32_t q0 = __builtin_amdgcn_alignbyte(p.d[r][1], p.d[r][0], sh);
            const uint32_t q1 = __builtin_amdgcn_alignbyte(p.d[r][2], p.d[r][1], sh);
            const uint32_t q2 = __builtin_amdgcn_alignbyte(0u, p.d[r][2], sh);
            const uint32_t m0 = p.row_in[r] ? p.m0 : 0u, m1 = p.row_in[r] ? p.m1 : 0u, m2 = p.row_in[r] ? p.m2 : 0u;
            q[r][0] = (q0 & m0) | (zsplat & ~m0);
            q[r][1] = (q1 & m1) | (zsplat & ~m1);
            q[r][2] = (q2 & m2) | (zsplat & ~m2);  // byte 0 = byte 8 of the row
        }
        // the stream [a0 .. a8, b0 .. b8, 0 ...] as dwords
        const uint32_t s0 = q[0][0], s1 = q[0][1];
        const uint32_t s2 = __builtin_amdgcn_perm(q[1][0], q[0][2], 0x06050400u);      // a8 b0 b1 b2
        const uint32_t s3 = __builtin_amdgcn_alignbyte(q[1][1], q[1][0], 3u);           // b3 b4 b5 b6
        const uint32_t s4 = __builtin_amdgcn_perm(q[1][2], q[1][1], 0x0c0c0403u);      // b7 b8 0 0
        // half 0 takes bytes 0 .. 15, half 1 bytes 7 .. 22
        v4i32 f;
        if (half == 0) {
            f = v4i32{(int)s0, (int)s1, (int)s2, (int)s3};
        } else {
            f = v4i32{(int)__builtin_amdgcn_alignbyte(s2, s1, 3u), (int)__builtin_amdgcn_alignbyte(s3, s2, 3u),
                      (int)__builtin_amdgcn_alignbyte(s4, s3, 3u), (int)__builtin_amdgcn_alignbyte(0u, s4, 3u)};
        }
        return f;
    };

    const int nwaves = (int)gridDim.x * (kBlock / 64);
    int g = (int)blockIdx.x * (kBlock / 64) + wave;
    Patch cur, nxt;
    fetch(g, cur);
    // ---- the weights as matrix B operand: lane = channel lane % 32, bytes k = 16 half .. 16 half + 15 (k < 27)
    v4i32 wf;
    {
        uint32_t wd[4] = {0, 0, 0, 0};
        if (cl < a.OC) {
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const int kk = 16 * half + k;
                if (kk < 27) wd[k >> 2] |= (uint32_t)(uint8_t)a.w[cl * 27 + kk] << (8 * (k & 3));
            }
        }
        wf = v4i32{(int)wd[0], (int)wd[1], (int)wd[2], (int)wd[3]};
    }
    // ---- per-channel constants (the input zero point folded into the bias term)
    if (tid < 32) {
        ChanConst c{};
        if (tid < a.OC) {
            int32_t wsum = 0;
            for (int k = 0; k < 27; k++) wsum += (int32_t)a.w[tid * 27 + k];
            const int32_t bias = a.bias[a.bias_len == 1 ? 0 : tid];
            c.bias_adj = (int32_t)((uint32_t)bias - (uint32_t)a.zx * (uint32_t)wsum);
            const int ci = a.scale.p.per_channel ? tid : 0;
            c.q = make_chan_scale(load_mult(a.scale, ci), (int32_t)a.scale.shift[ci], a.scale.p);
        }
        cc[tid] = c;
    }
    __syncthreads();
    const ChanConst c = cc[cl];
    char *so = smem + 32 * sizeof(ChanConst) + wave * 32 * a.op;  // this wavefront's staging tile [32][op]
    const int ppr = a.OC >> 4, npieces = 32 * ppr;                 // 16-byte pieces per row / per tile (at most 64)
    const int prow = lane / ppr;
    const uint32_t piece_row = lane < npieces ? (uint32_t)prow : 0xffffu;
    const uint32_t piece_lds = lane < npieces ? (uint32_t)(prow * a.op + (lane - prow * ppr) * 16) : 0u;
    const uint32_t sel_a = (lane & 1) ? 0x03070105u : 0x06020400u;  // exchange with lane ^ 1
    const uint32_t sel_b = (lane & 2) ? 0x03020706u : 0x05040100u;  // exchange with lane ^ 2
    char *so_lane = so + (4 * half + (lane & 3)) * a.op + (cl & ~3);
    const bool col_live = (cl & ~3) < a.OC;
    for (; g < a.groups; g += nwaves) {
        fetch(g + nwaves, nxt);
        const v4i32 xf = operand(cur);
        v16i32 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = c.bias_adj;
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf, wf, acc, 0, 0, 0);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int32_t v[4];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = requant_acc(acc[4 * q + e], c.q, a.scale.p, hi_v);
            const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
            uint32_t p = __builtin_amdgcn_perm(hi, lo, 0x05040100u);  // bytes = positions e of this lane's channel
            uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0xb1, 0xf, 0xf, true);
            p = __builtin_amdgcn_perm(o, p, sel_a);
            o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0x4e, 0xf, 0xf, true);
            p = __builtin_amdgcn_perm(o, p, sel_b);
            // now: position 8 q + 4 (lane / 32) + lane % 4, channels 4 (lane % 32 / 4) .. + 3
            if (col_live) *reinterpret_cast<uint32_t *>(so_lane + 8 * q * a.op) = p;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint32_t rows = (uint32_t)min(32, a.M - g * 32);
        const uint4 d = *reinterpret_cast<const uint4 *>(so + piece_lds);
        const uint32_t off = piece_row < rows ? (uint32_t)g * 32u * (uint32_t)a.OC + (uint32_t)lane * 16u : kOob;
        __builtin_amdgcn_raw_buffer_store_b128(v4i32{(int)d.x, (int)d.y, (int)d.z, (int)d.w}, ores, (int)off, 0, kOutAux);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        cur = nxt;
    }
}

// returns 1 when the case was taken
int try_stem_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                  const mlel_tensor *bias, const mlel_conv2d_attr *a, const FusedEpilogue *epi, int64_t M, int64_t xbytes) {
    const int64_t OH = out->dims[1], OW = out->dims[2], OC = out->dims[3], H = in->dims[1], W = in->dims[2];
    if (epi == nullptr || a->weight_zp != 0 || in->dims[3] != 3 || w->dims[1] != 3 || w->dims[2] != 3) return 0;
    if ((OC != 16 && OC != 32) || ((uintptr_t)in->ptr % 4) != 0) return 0;
    // dense image: rows of W * 3 bytes, images of H rows
    if (in->strides[2] != 3 || in->strides[1] != W * 3 || in->strides[0] != H * W * 3) return 0;
    if (a->stride[0] < 1 || a->stride[0] > 4 || a->stride[1] < 1 || a->stride[1] > 4) return 0;
    if (a->pad[0] < 0 || a->pad[0] > 4 || a->pad[2] < 0 || a->pad[2] > 4) return 0;
    // the quotient by the magic number is exact while dividend * divisor < 2^32; an image holds at least one group
    if (OH * OW * OW >= (int64_t(1) << 32) || OH * OW < 32 || OW < 2) return 0;
    if (xbytes >= (int64_t(1) << 31) - 16 || M * OC >= (int64_t(1) << 31)) return 0;
    StemMfmaArgs g{};
    g.x = static_cast<const int8_t *>(in->ptr);
    g.w = static_cast<const int8_t *>(w->ptr);
    g.bias = static_cast<const int32_t *>(bias->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.M = (int)M, g.OC = (int)OC, g.H = (int)H, g.W = (int)W, g.OW = (int)OW, g.OHW = (int)(OH * OW);
    g.zx = a->input_zp;
    g.bias_len = (int)bias->dims[0];
    g.sy = a->stride[0], g.sx = a->stride[1], g.pad_t = a->pad[0], g.pad_l = a->pad[2];
    g.ow_magic = (uint32_t)((uint64_t(1) << 32) / (uint64_t)g.OW + 1);
    g.groups = (int)((M + 31) / 32);
    int op = (int)OC;
    while (op % 128 != 32 && op % 128 != 96) op += 16;  // as in the rows kernel
    g.op = op;
    g.x_bytes = (uint32_t)((xbytes + 3) & ~int64_t(3));
    g.o_bytes = (uint32_t)(M * OC);
    g.scale = make_ref(*epi);
    const size_t sm = 32 * sizeof(ChanConst) + (size_t)(kBlock / 64) * 32 * g.op;
    const int cus = ctx != nullptr && ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256;
    const int64_t per_wave = (g.groups + kBlock / 64 - 1) / (kBlock / 64);
    const int64_t want =
        std::min<int64_t>(per_wave, std::min<int64_t>((int64_t)cus * 3, std::max<int64_t>((int64_t)cus * 2, (g.groups + 15) / 16)));
    conv_stem_mfma_i8_kernel<<<dim3((unsigned)std::max<int64_t>(want, 1)), dim3(kBlock), sm, s>>>(g);
    return 1;
}

}  // namespace

int try_conv2d_i8_direct(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                         const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                         const FusedEpilogue *epi) {
    if (in->dtype != MLEL_I8 || w->dtype != MLEL_I8 || bias->dtype != MLEL_I32 || a->acc_type != MLEL_ACC_I32) return 0;
    if (epi == nullptr && out->dtype != MLEL_I32) return 0;
    if (epi != nullptr && dt_size(out->dtype) != 1) return 0;
    // the kernels' requantisation assumes the int32 accumulator's RESCALE has input_zp == 0 (requant_acc); an
    // operator that names another runs as the general operator sequence
    if (epi != nullptr && epi->p.in_zp != 0) return 0;
    const int64_t N = out->dims[0], OH = out->dims[1], OW = out->dims[2], OC = out->dims[3];
    const int64_t H = in->dims[1], W = in->dims[2], IC = in->dims[3];
    const int64_t KH = w->dims[1], KW = w->dims[2];
    // what the kernel's indexing assumes, checked here: dense weights and output, pixels contiguous in the input,
    // 31-bit input extent, output channels in groups of 16, 16-byte aligned output
    if (w->dims[0] != OC || w->dims[3] != IC || in->dims[0] < N) return 0;
    if (!is_packed(w) || !is_packed(out) || in->strides[3] != 1 || in->strides[2] != IC) return 0;
    if (OC % 16 != 0 || ((uintptr_t)out->ptr % 16) != 0 || ((uintptr_t)bias->ptr % 4) != 0) return 0;
    if (!(bias->dims[0] == 1 || bias->dims[0] >= OC) || bias->strides[0] != 4) return 0;
    if (a->dilation[0] != 1 || a->dilation[1] != 1) return 0;
    const int64_t xbytes = in->dims[0] * in->strides[0];
    if (xbytes <= 0 || xbytes >= (int64_t(1) << 31) - 4 || in->strides[0] < 0 || in->strides[1] < 0) return 0;
    if (((uintptr_t)in->ptr % 4) != 0) return 0;
    const int64_t M = N * OH * OW;
    if (M >= (int64_t(1) << 31) - 4 * kBlock || OC >= (1 << 24)) return 0;

    int mode = -1;
    if (KH == 3 && KW == 3 && (IC == 1 || IC == 3 || IC == 4)) {
        if (a->stride[0] < 1 || a->stride[1] < 1 || a->stride[0] > 64 || a->stride[1] > 64) return 0;
        if (a->pad[0] < 0 || a->pad[2] < 0 || a->pad[0] > 64 || a->pad[2] > 64) return 0;
        if (H >= (1 << 24) || W >= (1 << 24) || OH >= (1 << 24) || OW >= (1 << 24)) return 0;
        mode = STEM;
    } else if (KH == 1 && KW == 1 && (IC == 16 || IC == 24 || IC == 32) && a->stride[0] == 1 && a->stride[1] == 1 &&
               a->pad[0] == 0 && a->pad[2] == 0 && OH == H && OW == W && in->strides[1] == W * in->strides[2] &&
               in->strides[0] == H * in->strides[1] && ((uintptr_t)in->ptr % 4) == 0 && ((uintptr_t)w->ptr % 4) == 0) {
        mode = ROWS;
    }
    if (M <= 0 && mode >= 0) return 1;
    const bool rows_shape = KH == 1 && KW == 1 && a->stride[0] == 1 && a->stride[1] == 1 && a->pad[0] == 0 &&
                            a->pad[2] == 0 && OH == H && OW == W && in->strides[1] == W * in->strides[2] &&
                            in->strides[0] == H * in->strides[1];
    if (rows_shape && M > 0 && try_rows_mfma(ctx, s, out, in, w, bias, a, epi, M, IC, OC, xbytes)) {
        MLEL_TRY(check_launch("conv2d rows int8"));
        return 1;
    }
    if (mode < 0) return 0;
    if (mode == STEM && IC == 3 && M > 0 && try_stem_mfma(ctx, s, out, in, w, bias, a, epi, M, xbytes)) {
        MLEL_TRY(check_launch("conv2d stem int8"));
        return 1;
    }

    DirectArgs g{};
    g.x = static_cast<const int8_t *>(in->ptr);
    g.w = static_cast<const int8_t *>(w->ptr);
    g.bias = static_cast<const int32_t *>(bias->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.M = (int)M;
    g.OHW = (int)(OH * OW);
    g.OW = (int)OW;
    g.H = (int)H;
    g.W = (int)W;
    g.IC = (int)IC;
    g.OC = (int)OC;
    g.x_sn = (uint32_t)in->strides[0];
    g.x_sy = (uint32_t)in->strides[1];
    g.x_sx = (uint32_t)in->strides[2];
    // dword loads: the last dword of the tensor may hold 1-3 bytes past its end.  With a 4-byte aligned base that
    // dword lies inside the same page as the last valid byte, and the surplus bytes are masked out in the kernel.
    g.x_bytes = (uint32_t)((xbytes + 3) & ~int64_t(3));
    g.ldw = w->strides[0];
    g.sy = a->stride[0];
    g.sx = a->stride[1];
    g.pad_t = a->pad[0];
    g.pad_l = a->pad[2];
    g.zx = a->input_zp;
    g.zw = a->weight_zp;
    g.bias_len = (int)bias->dims[0];
    g.fused = epi != nullptr;
    g.out_size = dt_size(out->dtype);
    if (epi) g.scale = make_ref(*epi);
    // 32 (or 16) output channels per block; grid.y walks the channel blocks
    const int ocb = OC % 32 == 0 ? 32 : 16;
    const int splits = (int)(OC / ocb);
    if (splits > 65535) return 0;
    g.ocb = ocb;
    const int cus = ctx != nullptr ? ctx->props.multiProcessorCount : 256;
    if (mode == STEM) {
        if (IC == 1)
            launch_direct<STEM, 1, 9>(g, splits, cus, s);
        else if (IC == 3)
            launch_direct<STEM, 3, 9>(g, splits, cus, s);
        else
            launch_direct<STEM, 4, 9>(g, splits, cus, s);
    } else {
        if (IC == 16)
            launch_direct<ROWS, 4, 4>(g, splits, cus, s);
        else if (IC == 24)
            launch_direct<ROWS, 4, 6>(g, splits, cus, s);
        else
            launch_direct<ROWS, 4, 8>(g, splits, cus, s);
    }
    MLEL_TRY(check_launch("conv2d direct int8"));
    return 1;
}

// Two 1x1 CONV2D + RESCALE (+CLAMP) in a row (conv_rows2_mfma_i8_kernel).  `mid`: the intermediate tensor when something
// else reads it too, else nullptr.  Returns 1 when launched, 0 to decline; `probe`: judge only, launch nothing.
int try_conv2d_pair_rows(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *mid,
                         const mlel_tensor *in, const mlel_tensor *w1, const mlel_tensor *b1, const mlel_conv2d_attr *a1,
                         const FusedEpilogue *e1, int mid_dtype, const mlel_tensor *w2, const mlel_tensor *b2,
                         const mlel_conv2d_attr *a2, const FusedEpilogue *e2, bool probe) {
    if (in->dtype != MLEL_I8 || w1->dtype != MLEL_I8 || w2->dtype != MLEL_I8 || b1->dtype != MLEL_I32 ||
        b2->dtype != MLEL_I32 || out->dtype != MLEL_I8 || mid_dtype != MLEL_I8)
        return 0;
    if (a1->acc_type != MLEL_ACC_I32 || a2->acc_type != MLEL_ACC_I32 || a1->weight_zp != 0 || a2->weight_zp != 0) return 0;
    if (e1 == nullptr || e2 == nullptr || e1->p.in_zp != 0 || e2->p.in_zp != 0) return 0;
    if (in->rank != 4 || out->rank != 4 || w1->rank != 4 || w2->rank != 4) return 0;
    const int64_t N = out->dims[0], H = out->dims[1], W = out->dims[2], OC = out->dims[3];
    const int64_t IC0 = in->dims[3], OC0 = w1->dims[0];
    for (const mlel_conv2d_attr *a : {a1, a2})
        if (a->stride[0] != 1 || a->stride[1] != 1 || a->dilation[0] != 1 || a->dilation[1] != 1 || a->pad[0] != 0 ||
            a->pad[1] != 0 || a->pad[2] != 0 || a->pad[3] != 0)
            return 0;
    if (w1->dims[1] != 1 || w1->dims[2] != 1 || w1->dims[3] != IC0 || w2->dims[0] != OC || w2->dims[1] != 1 ||
        w2->dims[2] != 1 || w2->dims[3] != OC0)
        return 0;
    if (in->dims[0] != N || in->dims[1] != H || in->dims[2] != W) return 0;
    if (!is_packed(in) || !is_packed(out) || !is_packed(w1) || !is_packed(w2)) return 0;
    if (mid != nullptr && (!is_packed(mid) || mid->dtype != MLEL_I8 || mid->rank != 4 || mid->dims[0] != N ||
                           mid->dims[1] != H || mid->dims[2] != W || mid->dims[3] != OC0))
        return 0;
    for (const mlel_tensor *bt : {b1, b2})
        if (bt->rank != 1 || bt->strides[0] != 4 || ((uintptr_t)bt->ptr % 4) != 0) return 0;
    if (!(b1->dims[0] == 1 || b1->dims[0] >= OC0) || !(b2->dims[0] == 1 || b2->dims[0] >= OC)) return 0;
    int nj = 0, kc = 0, kc0 = 0;
    if (!rows2_shape(IC0, OC0, OC, &nj, &kc, &kc0)) return 0;
    const int64_t M = N * H * W;
    if (M <= 0) return probe ? 1 : 1;
    if (M * OC >= (int64_t(1) << 31) || M * IC0 >= (int64_t(1) << 31)) return 0;
    // the intermediate tensor leaves in 16-byte pieces: its extent must be whole pieces (a probe does not know whether
    // it will be stored, so it asks for this as well)
    if ((M * OC0) % 16 != 0) return 0;
    if (probe) return 1;  // (alignment is a property of the bound memory: checked at launch, the caller then falls back)
    if (((uintptr_t)in->ptr % 8) != 0 || ((uintptr_t)w1->ptr % 8) != 0 || ((uintptr_t)w2->ptr % 8) != 0 ||
        ((uintptr_t)out->ptr % 16) != 0 || (mid != nullptr && ((uintptr_t)mid->ptr % 16) != 0))
        return 0;
    Rows2Args g{};
    g.r.w = static_cast<const int8_t *>(w2->ptr);
    g.r.bias = static_cast<const int32_t *>(b2->ptr);
    g.r.out = static_cast<char *>(out->ptr);
    g.r.M = (int)M;
    g.r.IC = (int)OC0;
    g.r.OC = (int)OC;
    g.r.zx = a2->input_zp;
    g.r.bias_len = (int)b2->dims[0];
    g.r.groups = (int)((M + 31) / 32);
    int op = (int)OC;
    while (op % 128 != 32 && op % 128 != 96) op += 16;
    g.r.op = op;
    g.r.o_bytes = (uint32_t)(M * OC);
    g.r.scale = make_ref(*e2);
    g.x0 = static_cast<const int8_t *>(in->ptr);
    g.w0 = static_cast<const int8_t *>(w1->ptr);
    g.bias0 = static_cast<const int32_t *>(b1->ptr);
    g.mid = mid != nullptr ? static_cast<char *>(mid->ptr) : nullptr;
    g.IC0 = (int)IC0;
    g.zx0 = a1->input_zp;
    g.bias0_len = (int)b1->dims[0];
    g.x0_bytes = (uint32_t)(M * IC0);
    g.mid_bytes = (uint32_t)(M * OC0);
    g.scale0 = make_ref(*e1);
    const size_t sm = (size_t)(nj * 32 + 32) * sizeof(ChanConst) +
                      (size_t)(kBlock / 64) * (32 * (size_t)OC0 + 16 + 32 * (size_t)op) + 512;
    const int cus = ctx != nullptr && ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256;
    const int64_t per_wave = (g.r.groups + kBlock / 64 - 1) / (kBlock / 64);
    const int64_t want = std::min<int64_t>(
        per_wave, std::min<int64_t>((int64_t)cus * 3, std::max<int64_t>((int64_t)cus * 2, (g.r.groups + 15) / 16)));
    const dim3 grid((unsigned)std::max<int64_t>(want, 1));
    if (nj == 3 && kc == 1 && kc0 == 2)
        launch_rows2<3, 1, 2>(g, grid, sm, s);
    else if (nj == 5 && kc == 2 && kc0 == 6)
        launch_rows2<5, 2, 6>(g, grid, sm, s);
    else if (nj == 6 && kc == 2 && kc0 == 2)
        launch_rows2<6, 2, 2>(g, grid, sm, s);
    else
        launch_rows2<6, 2, 6>(g, grid, sm, s);
    MLEL_TRY(check_launch("conv2d pair rows int8"));
    return 1;
}

}  // namespace mlel
