// Bandwidth-bound specialisations for the int8 NHWC hot path: 128-bit coalesced accesses, per-channel constants
// held in registers, RESCALE/CLAMP applied in the producing kernel.  Every function here is an optimisation of a
// case the generic kernels (ops_generic.hip) also compute; `try_*` returns 0 to decline a case.
#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {
namespace {

constexpr int kBlock = 256;

struct ScaleRef {
    const char *mult;
    const int8_t *shift;
    int32_t mult16;
    RescaleParams p;
};

ScaleRef make_ref(const FusedEpilogue &f) {
    ScaleRef r;
    r.mult = static_cast<const char *>(f.mult->ptr);
    r.shift = static_cast<const int8_t *>(f.shift->ptr);
    r.mult16 = f.scale32 ? 0 : 1;
    r.p = f.p;
    return r;
}

__device__ __forceinline__ int32_t load_mult(const ScaleRef &s, int64_t c) {
    return s.mult16 ? (int32_t) reinterpret_cast<const int16_t *>(s.mult)[c]
                    : reinterpret_cast<const int32_t *>(s.mult)[c];
}

// out = RESCALE_o(RESCALE_1(in1) + RESCALE_2(in2)), any integer storage types, any strides
__global__ void __launch_bounds__(kBlock) rescale_add_rescale_kernel(TV out, TV in1, TV in2, ScaleRef s1, ScaleRef s2,
                                                                     ScaleRef so, int in1_dt, int in2_dt,
                                                                     int64_t total) {
    const int64_t flat = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t ch = o[out.rank - 1];
    TV a = in1, b = in2;
    a.dtype = in1_dt;
    b.dtype = in2_dt;
    const int64_t c1 = s1.p.per_channel ? ch : 0, c2 = s2.p.per_channel ? ch : 0, co = so.p.per_channel ? ch : 0;
    int32_t r1 = apply_scale(ld_i(a, o) - (int64_t)s1.p.in_zp, load_mult(s1, c1), s1.shift[c1], s1.p.double_round != 0);
    r1 = (int32_t)((uint32_t)r1 + (uint32_t)s1.p.out_zp);
    int32_t r2 = apply_scale(ld_i(b, o) - (int64_t)s2.p.in_zp, load_mult(s2, c2), s2.shift[c2], s2.p.double_round != 0);
    r2 = (int32_t)((uint32_t)r2 + (uint32_t)s2.p.out_zp);
    const int32_t sum = (int32_t)((uint32_t)r1 + (uint32_t)r2);
    st_i(out, o, requant_i32(sum, load_mult(so, co), so.shift[co], so.p));
}


// Per-tensor scales, int8 in / int8 out, dense tensors: 16 elements per thread with 128-bit accesses.
__global__ void __launch_bounds__(kBlock) rescale_add_rescale_i8x16_kernel(uint4 *__restrict__ out,
                                                                           const uint4 *__restrict__ in1,
                                                                           const uint4 *__restrict__ in2, ScaleRef s1,
                                                                           ScaleRef s2, ScaleRef so, int64_t n_vec) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_vec) return;
    const ChanScale q1 = make_chan_scale(load_mult(s1, 0), s1.shift[0], s1.p);
    const ChanScale q2 = make_chan_scale(load_mult(s2, 0), s2.shift[0], s2.p);
    const ChanScale qo = make_chan_scale(load_mult(so, 0), so.shift[0], so.p);
    const uint4 a = in1[i], b = in2[i];
    const uint32_t av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
    uint32_t ov[4];
#pragma unroll
    for (int d = 0; d < 4; d++) {
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int32_t x1 = (int8_t)(av[d] >> (8 * e)), x2 = (int8_t)(bv[d] >> (8 * e));
            const int32_t r1 = requant_chan(x1, q1, s1.p), r2 = requant_chan(x2, q2, s2.p);
            const int32_t sum = (int32_t)((uint32_t)r1 + (uint32_t)r2);
            const int32_t r = requant_chan(sum, qo, so.p);
            packed |= (uint32_t)(uint8_t)r << (8 * e);
        }
        ov[d] = packed;
    }
    out[i] = make_uint4(ov[0], ov[1], ov[2], ov[3]);
}

}  // namespace

int rescale_add_rescale_launch(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1,
                               const FusedEpilogue &f1, const mlel_tensor *in2, const FusedEpilogue &f2,
                               const FusedEpilogue &fo) {
    (void)ctx;
    const int64_t total = numel(out);
    if (total == 0) return 0;
    const bool dense_i8 = in1->dtype == MLEL_I8 && in2->dtype == MLEL_I8 && out->dtype == MLEL_I8 && f1.in_dt == MLEL_I8 &&
                          f2.in_dt == MLEL_I8 && is_packed(in1) && is_packed(in2) && is_packed(out) && total % 16 == 0 &&
                          !f1.p.per_channel && !f2.p.per_channel && !fo.p.per_channel &&
                          ((uintptr_t)in1->ptr % 16) == 0 && ((uintptr_t)in2->ptr % 16) == 0 &&
                          ((uintptr_t)out->ptr % 16) == 0;
    if (dense_i8) {
        const int64_t n_vec = total / 16;
        hipLaunchKernelGGL(rescale_add_rescale_i8x16_kernel, grid_1d(n_vec, kBlock), dim3(kBlock), 0, s,
                           (uint4 *)out->ptr, (const uint4 *)in1->ptr, (const uint4 *)in2->ptr, make_ref(f1),
                           make_ref(f2), make_ref(fo), n_vec);
        return check_launch("rescale_add_rescale");
    }
    // the stage-1/2 zero points were narrowed against the (un)signed twin of each input type; loads use the twin too
    const int in1_dt = f1.in_dt, in2_dt = f2.in_dt;
    hipLaunchKernelGGL(rescale_add_rescale_kernel, grid_1d(total, kBlock), dim3(kBlock), 0, s, make_tv(out),
                       make_tv(in1), make_tv(in2), make_ref(f1), make_ref(f2), make_ref(fo), in1_dt, in2_dt, total);
    return check_launch("rescale_add_rescale");
}

namespace {

// ---------------------------------------------------------------------------------------------------------------
// DEPTHWISE_CONV2D 3x3, int8 NHWC, channel multiplier 1, fused RESCALE (+CLAMP) or int32 output.
//
// Work item = 4 consecutive channels x TX consecutive output positions of one output row.  Lanes run over the
// channel quads first, so every load and store instruction of a wavefront covers consecutive dwords of a pixel.
// For each input column the three rows are transposed (v_perm_b32) into one dword per channel holding the three
// vertical taps; a v_dot4_i32_i8 against the matching weight column then adds three taps at once, and a column is
// shared by up to three neighbouring outputs.  Padded taps are filled with the input zero point, so the expansion
//   sum (x - zi)(w - zw) = sum x*w - zw * sum x - zi * sum w + 9 * zi * zw
// gives exactly the reference's result (padded taps contribute nothing).  Weight columns and per-channel
// requantisation constants are prepared once per block in LDS.
// ---------------------------------------------------------------------------------------------------------------
struct DwArgs {
    const int8_t *x, *w;
    const int32_t *bias;
    char *out;
    int32_t N, H, W, C, OH, OW;
    int64_t x_sn, x_sy, x_sx;  // input byte strides (channel stride 1)
    int32_t sy, sx, pad_t, pad_l, zi, zw, bias_len;
    int32_t fused, out_size;
    ScaleRef scale;
    int64_t items;  // N * OH * strips * C/4
    int32_t strips;
};

struct DwChan {  // per channel, in LDS (32 bytes)
    ChanScale q;
    int32_t bias_adj;
    int32_t pad;
};

template <int TX, int SX, bool ZW>
__global__ void __launch_bounds__(kBlock) dwconv3x3_i8_kernel(const DwArgs a) {
    extern __shared__ __align__(16) char smem[];
    uint32_t *wcol = reinterpret_cast<uint32_t *>(smem);                // [3][C]: bytes (w[0][kx][c], w[1].., w[2].., 0)
    DwChan *chan = reinterpret_cast<DwChan *>(smem + (size_t)3 * a.C * 4);  // [C]
    for (int i = threadIdx.x; i < 3 * a.C; i += kBlock) {
        const int kx = i / a.C, c = i - kx * a.C;
        const uint32_t b0 = (uint8_t)a.w[(0 * 3 + kx) * a.C + c], b1 = (uint8_t)a.w[(1 * 3 + kx) * a.C + c],
                       b2 = (uint8_t)a.w[(2 * 3 + kx) * a.C + c];
        wcol[i] = b0 | (b1 << 8) | (b2 << 16);
    }
    for (int c = threadIdx.x; c < a.C; c += kBlock) {
        int32_t wsum = 0;
        for (int t = 0; t < 9; t++) wsum += a.w[t * a.C + c];
        DwChan d{};
        const int32_t bias = a.bias[a.bias_len == 1 ? 0 : c];
        d.bias_adj = (int32_t)((uint32_t)bias - (uint32_t)a.zi * (uint32_t)wsum + 9u * (uint32_t)a.zi * (uint32_t)a.zw);
        if (a.fused) {
            const int ci = a.scale.p.per_channel ? c : 0;
            d.q = make_chan_scale(load_mult(a.scale, ci), (int32_t)a.scale.shift[ci], a.scale.p);
        }
        chan[c] = d;
    }
    __syncthreads();

    const int64_t item = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (item >= a.items) return;
    const int c4n = a.C >> 2;
    const int c4 = (int)(item % c4n);
    int64_t rest = item / c4n;
    const int strip = (int)(rest % a.strips);
    rest /= a.strips;
    const int oy = (int)(rest % a.OH);
    const int n = (int)(rest / a.OH);
    const int c = c4 * 4;
    const int ox0 = strip * TX;

    // ---- input columns ix0 .. ix0 + NCOL - 1, three rows each, transposed to one dword per channel
    constexpr int NCOL = SX * (TX - 1) + 3;
    const int iy0 = oy * a.sy - a.pad_t, ix0 = ox0 * SX - a.pad_l;
    const uint32_t zsplat = (uint32_t)(uint8_t)a.zi * 0x01010101u;
    const int8_t *xb = a.x + (int64_t)n * a.x_sn + c;
    uint32_t raw[3][NCOL];
#pragma unroll
    for (int r = 0; r < 3; r++) {
        const int y = iy0 + r;
        const bool yin = (unsigned)y < (unsigned)a.H;
#pragma unroll
        for (int j = 0; j < NCOL; j++) {
            const int x = ix0 + j;
            uint32_t v = zsplat;
            if (yin && (unsigned)x < (unsigned)a.W)
                v = *reinterpret_cast<const uint32_t *>(xb + (int64_t)y * a.x_sy + (int64_t)x * a.x_sx);
            raw[r][j] = v;
        }
    }
    uint32_t wc[3][4];
#pragma unroll
    for (int kx = 0; kx < 3; kx++) {
        const uint4 t = *reinterpret_cast<const uint4 *>(wcol + kx * a.C + c);
        wc[kx][0] = t.x;
        wc[kx][1] = t.y;
        wc[kx][2] = t.z;
        wc[kx][3] = t.w;
    }
    int32_t acc[TX][4], xs[TX][4];
#pragma unroll
    for (int t = 0; t < TX; t++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[t][e] = xs[t][e] = 0;
#pragma unroll
    for (int j = 0; j < NCOL; j++) {
        // 3 rows x 4 channels (bytes) -> 4 channels x (3 taps, 0): selector bytes 0-3 pick from the 2nd operand
        const uint32_t r0 = raw[0][j], r1 = raw[1][j], r2 = raw[2][j];
        const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // [r0.b0 r1.b0 r0.b1 r1.b1]
        const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // [r0.b2 r1.b2 r0.b3 r1.b3]
        uint32_t col[4];
        col[0] = __builtin_amdgcn_perm(r2, t0, 0x0c040100u);  // [t0.b0 t0.b1 r2.b0 0]
        col[1] = __builtin_amdgcn_perm(r2, t0, 0x0c050302u);  // [t0.b2 t0.b3 r2.b1 0]
        col[2] = __builtin_amdgcn_perm(r2, t1, 0x0c060100u);  // [t1.b0 t1.b1 r2.b2 0]
        col[3] = __builtin_amdgcn_perm(r2, t1, 0x0c070302u);  // [t1.b2 t1.b3 r2.b3 0]
#pragma unroll
        for (int t = 0; t < TX; t++) {
            const int kx = j - t * SX;  // this column is tap kx of output t (compile-time after unrolling)
            if (kx < 0 || kx > 2) continue;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t w = wc[kx][e];
                acc[t][e] = __builtin_amdgcn_sdot4((int)col[e], (int)w, acc[t][e], false);
                if (ZW) xs[t][e] = __builtin_amdgcn_sdot4((int)col[e], 0x00010101, xs[t][e], false);
            }
        }
    }

    // ---- epilogue
    DwChan ch[4];
#pragma unroll
    for (int e = 0; e < 4; e++) ch[e] = chan[c + e];
    const int64_t orow = ((int64_t)n * a.OH + oy) * a.OW;
#pragma unroll
    for (int t = 0; t < TX; t++) {
        const int ox = ox0 + t;
        if (ox >= a.OW) break;
        int32_t v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int32_t s = (int32_t)((uint32_t)acc[t][e] + (uint32_t)ch[e].bias_adj);
            if (ZW) s = (int32_t)((uint32_t)s - (uint32_t)a.zw * (uint32_t)xs[t][e]);
            if (a.fused) s = requant_chan(s, ch[e].q, a.scale.p);
            v[e] = s;
        }
        const int64_t off = (orow + ox) * a.C + c;
        if (a.out_size == 1) {
            *reinterpret_cast<uint32_t *>(a.out + off) = (uint32_t)(uint8_t)v[0] | ((uint32_t)(uint8_t)v[1] << 8) |
                                                         ((uint32_t)(uint8_t)v[2] << 16) | ((uint32_t)(uint8_t)v[3] << 24);
        } else if (a.out_size == 2) {
            *reinterpret_cast<uint2 *>(a.out + off * 2) =
                make_uint2((uint32_t)(uint16_t)v[0] | ((uint32_t)(uint16_t)v[1] << 16),
                           (uint32_t)(uint16_t)v[2] | ((uint32_t)(uint16_t)v[3] << 16));
        } else {
            *reinterpret_cast<int4 *>(a.out + off * 4) = make_int4(v[0], v[1], v[2], v[3]);
        }
    }
}

}  // namespace

int try_dwconv_i8_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                       const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                       const FusedEpilogue *epi) {
    (void)ctx;
    if (in->dtype != MLEL_I8 || w->dtype != MLEL_I8 || bias->dtype != MLEL_I32 || a->acc_type != MLEL_ACC_I32) return 0;
    if (epi == nullptr && out->dtype != MLEL_I32) return 0;
    if (epi != nullptr && (dt_size(out->dtype) > 4 || out->dtype == MLEL_BOOL)) return 0;
    const int64_t N = out->dims[0], OH = out->dims[1], OW = out->dims[2], C = out->dims[3];
    // the kernel's indexing assumes: 3x3 taps, multiplier 1, unit dilation, stride 1 or 2, channels in quads, dense
    // weights [3][3][C][1], packed output, channel-contiguous 4-byte aligned input
    if (w->dims[0] != 3 || w->dims[1] != 3 || w->dims[3] != 1 || w->dims[2] != C || in->dims[3] != C) return 0;
    if (a->dilation[0] != 1 || a->dilation[1] != 1) return 0;
    if (a->stride[0] < 1 || a->stride[0] > 2 || a->stride[1] < 1 || a->stride[1] > 2) return 0;
    if (C % 4 != 0 || C <= 0 || C > 2048 || in->dims[0] < N) return 0;
    if (!is_packed(w) || !is_packed(out) || in->strides[3] != 1) return 0;
    if (!(bias->dims[0] == 1 || bias->dims[0] >= C) || bias->strides[0] != 4) return 0;
    if (((uintptr_t)in->ptr % 4) || in->strides[0] % 4 || in->strides[1] % 4 || in->strides[2] % 4) return 0;
    if (((uintptr_t)out->ptr % 16) != 0) return 0;
    if (N <= 0 || OH <= 0 || OW <= 0) return 1;
    if (in->dims[1] >= (1 << 30) || in->dims[2] >= (1 << 30) || OH >= (1 << 30) || OW >= (1 << 30)) return 0;

    constexpr int TX = 4;
    DwArgs g{};
    g.x = static_cast<const int8_t *>(in->ptr);
    g.w = static_cast<const int8_t *>(w->ptr);
    g.bias = static_cast<const int32_t *>(bias->ptr);
    g.out = static_cast<char *>(out->ptr);
    g.N = (int)N;
    g.H = (int)in->dims[1];
    g.W = (int)in->dims[2];
    g.C = (int)C;
    g.OH = (int)OH;
    g.OW = (int)OW;
    g.x_sn = in->strides[0];
    g.x_sy = in->strides[1];
    g.x_sx = in->strides[2];
    g.sy = a->stride[0];
    g.sx = a->stride[1];
    g.pad_t = a->pad[0];
    g.pad_l = a->pad[2];
    g.zi = a->input_zp;
    g.zw = a->weight_zp;
    g.bias_len = (int)bias->dims[0];
    g.fused = epi != nullptr;
    g.out_size = dt_size(out->dtype);
    if (epi) g.scale = make_ref(*epi);
    g.strips = (int)((OW + TX - 1) / TX);
    g.items = N * OH * g.strips * (C / 4);
    const size_t smem = (size_t)3 * C * 4 + (size_t)C * sizeof(DwChan);
    const int64_t blocks = (g.items + kBlock - 1) / kBlock;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "depthwise_conv2d: too many work items");
    const dim3 grid((unsigned)blocks), block(kBlock);
    if (g.sx == 1 && g.zw == 0)
        dwconv3x3_i8_kernel<TX, 1, false><<<grid, block, smem, s>>>(g);
    else if (g.sx == 1)
        dwconv3x3_i8_kernel<TX, 1, true><<<grid, block, smem, s>>>(g);
    else if (g.zw == 0)
        dwconv3x3_i8_kernel<TX, 2, false><<<grid, block, smem, s>>>(g);
    else
        dwconv3x3_i8_kernel<TX, 2, true><<<grid, block, smem, s>>>(g);
    MLEL_TRY(check_launch("depthwise_conv2d 3x3 int8"));
    return 1;
}

int try_rescale_fast(mlel_ctx *, hipStream_t, const mlel_tensor *, const mlel_tensor *, const mlel_tensor *,
                     const mlel_tensor *, const mlel_rescale_attr *, const RescaleParams &) {
    return 0;
}
int try_clamp_fast(mlel_ctx *, hipStream_t, const mlel_tensor *, const mlel_tensor *, const mlel_clamp_attr *) {
    return 0;
}
int try_binary_fast(mlel_ctx *, hipStream_t, int, const mlel_tensor *, const mlel_tensor *, const mlel_tensor *) {
    return 0;
}
int try_avgpool_fast(mlel_ctx *, hipStream_t, const mlel_tensor *, const mlel_tensor *, const mlel_pool2d_attr *) {
    return 0;
}

}  // namespace mlel
