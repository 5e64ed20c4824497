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

struct ChanConst {  // per output channel, in shared memory: 32 bytes
    ChanScale q;
    int32_t bias_adj;
    int32_t pad;
};

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
                    packed[p][e / 4] |= ((uint32_t)requant_chan(v, c.q, a.scale.p) & 0xffu) << (8 * (e % 4));
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

}  // namespace

int try_conv2d_i8_direct(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                         const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                         const FusedEpilogue *epi) {
    if (in->dtype != MLEL_I8 || w->dtype != MLEL_I8 || bias->dtype != MLEL_I32 || a->acc_type != MLEL_ACC_I32) return 0;
    if (epi == nullptr && out->dtype != MLEL_I32) return 0;
    if (epi != nullptr && dt_size(out->dtype) != 1) return 0;
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
    if (mode < 0) return 0;
    if (M <= 0) return 1;

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

}  // namespace mlel
