// Bandwidth-bound specialisations for the int8 NHWC hot path: 128-bit coalesced accesses, per-channel constants
// held in registers, RESCALE/CLAMP applied in the producing kernel.  Every function here is an optimisation of a
// case the generic kernels (ops_generic.hip) also compute; `try_*` returns 0 to decline a case.
#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {
namespace {

constexpr int kBlock = 256;

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
    store16_result(out + i, make_uint4(ov[0], ov[1], ov[2], ov[3]));
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
// Work item = 4 consecutive channels x TX consecutive output columns x TY consecutive output rows.  Lanes run over
// the channel quads first, so every load and store instruction of a wavefront covers consecutive dwords of a pixel.
// For each input column the rows are transposed (v_perm_b32) into one dword per channel holding three vertical
// taps; a v_dot4_i32_i8 against the matching weight column then adds three taps at once, and a column is shared by
// up to three neighbouring outputs.  Padded taps are filled with the input zero point, so the expansion
//   sum (x - zi)(w - zw) = sum x*w - zw * sum x - zi * sum w + 9 * zi * zw
// gives exactly the reference's result (padded taps contribute nothing).  A block covers CB channel quads x SPB
// spatial items of one image; its first 4 CB threads work out one channel each (three weight columns, the bias with
// the zero-point terms folded in, the requantisation constants) into shared memory, and after one barrier every
// thread reads the 48 bytes of each of its four channels.  (Every thread preparing its own four channels cost
// 8 of 25 vector instructions per output, three runtime divisions for its position among them.)  Consecutive
// blocks are dealt to the XCDs in contiguous runs, so rows shared by vertically adjacent items are fetched into
// one L2 only.
// ---------------------------------------------------------------------------------------------------------------
struct DwArgs {
    const int8_t *x, *w;
    const int32_t *bias;
    char *out;
    int32_t N, H, W, C, OH, OW;
    uint32_t x_sn, x_sy, x_sx;  // input byte strides (channel stride 1); input and output extents are below 2^31
    uint32_t x_bytes, o_bytes;
    int32_t sy, sx, pad_t, pad_l, zi, zw, bias_len;
    int32_t fused, out_size;
    ScaleRef scale;
    int32_t strips, row_groups;
    // block = cb_size channel quads x spb spatial items (row group, strip) of one image; blocks are ordered
    // [image][spatial block][channel block]
    int32_t cb_size, cb_count, spb, sb_count;
    uint32_t cb_magic, strips_magic;  // floor(2^32 / d) + 1: x / d == umulhi(x, magic) for x < 2^16, 1 < d < 2^16
    int32_t blocks, chunk;  // launch geometry: `chunk` consecutive blocks per XCD
    DivMagic div_cb, div_sb;  // block index / cb_count, / sb_count as a multiplication and a shift
};

struct DwChan {  // per channel, in shared memory: 48 bytes
    ChanScale q;
    int32_t bias_adj;
    uint32_t wcol[3];  // column kx: bytes = the taps (0, kx), (1, kx), (2, kx), 0
    uint32_t pad[2];
};
static_assert(sizeof(DwChan) == 48, "DwChan layout");

// 3 rows x 4 channels (bytes) -> 4 channels x (3 taps, 0)
__device__ __forceinline__ void transpose_3x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t (&col)[4]) {
    // selector bytes 0-3 pick from the second operand, 4-7 from the first, 0x0c gives zero
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // [r0.b0 r1.b0 r0.b1 r1.b1]
    const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // [r0.b2 r1.b2 r0.b3 r1.b3]
    col[0] = __builtin_amdgcn_perm(r2, t0, 0x0c040100u);             // [t0.b0 t0.b1 r2.b0 0]
    col[1] = __builtin_amdgcn_perm(r2, t0, 0x0c050302u);             // [t0.b2 t0.b3 r2.b1 0]
    col[2] = __builtin_amdgcn_perm(r2, t1, 0x0c060100u);             // [t1.b0 t1.b1 r2.b2 0]
    col[3] = __builtin_amdgcn_perm(r2, t1, 0x0c070302u);             // [t1.b2 t1.b3 r2.b3 0]
}

// Q8: fused epilogue with 8-bit output (a compile-time choice keeps the unrolled epilogue free of branches).  All
// index arithmetic is 32-bit (the host checks the extents); loads and stores are buffer instructions with 32-bit
// offsets, so an address costs one add.
template <int TX, int TY, int SX, bool ZW, bool Q8>
__global__ void __launch_bounds__(kBlock) dwconv3x3_i8_kernel(const DwArgs a) {
    __shared__ __align__(16) DwChan chan[kBlock];
    // Every argument asked for in one batch (left alone the compiler loads them in three trips to memory in a row:
    // behind the early exit, and again where a register of a wide load that nobody was waiting for had been given
    // away), every dword of the wide loads named for that reason.
    asm volatile("" ::"s"(a.chunk), "s"(a.blocks), "s"(a.div_cb.m), "s"(a.div_cb.s), "s"(a.div_sb.m), "s"(a.div_sb.s),
                 "s"(a.cb_size), "s"(a.cb_count), "s"(a.spb), "s"(a.sb_count), "s"(a.cb_magic), "s"(a.strips_magic),
                 "s"(a.strips), "s"(a.row_groups), "s"(a.x), "s"(a.w), "s"(a.bias), "s"(a.out), "s"(a.N), "s"(a.H), "s"(a.W),
                 "s"(a.C), "s"(a.OH), "s"(a.OW), "s"(a.x_sn), "s"(a.x_sy), "s"(a.x_sx), "s"(a.x_bytes), "s"(a.o_bytes),
                 "s"(a.sy), "s"(a.sx), "s"(a.pad_t), "s"(a.pad_l), "s"(a.zi), "s"(a.zw), "s"(a.bias_len), "s"(a.fused),
                 "s"(a.out_size), "s"(a.scale.mult), "s"(a.scale.shift), "s"(a.scale.mult16), "s"(a.scale.p.in_zp),
                 "s"(a.scale.p.out_zp), "s"(a.scale.p.out_lo), "s"(a.scale.p.out_hi), "s"(a.scale.p.double_round),
                 "s"(a.scale.p.per_channel), "s"(a.scale.p.clamp_out));
    // blocks are dealt round-robin to the XCDs: give XCD k the k-th contiguous run of blocks
    const int bid = (int)(blockIdx.x % 8u) * a.chunk + (int)(blockIdx.x / 8u);
    if (bid >= a.blocks) return;
    // block -> (image, spatial block, channel block): uniform, on the scalar unit
    const int rest_b = div_magic(bid, a.div_cb);
    const int cb = bid - rest_b * a.cb_count;
    const int n = div_magic(rest_b, a.div_sb);
    const int sb = rest_b - n * a.sb_count;
    const int tid = threadIdx.x;

    // ---- one channel per thread: weight columns, bias with the zero-point terms folded in, scales
    if (tid < 4 * a.cb_size) {
        const int ch = cb * a.cb_size * 4 + tid;
        DwChan d{};
        if (ch < a.C) {
            int32_t wsum = 0;
#pragma unroll
            for (int kx = 0; kx < 3; kx++) {
                const uint32_t w0 = (uint8_t)a.w[(0 * 3 + kx) * a.C + ch], w1 = (uint8_t)a.w[(1 * 3 + kx) * a.C + ch],
                               w2 = (uint8_t)a.w[(2 * 3 + kx) * a.C + ch];
                d.wcol[kx] = w0 | (w1 << 8) | (w2 << 16);
                wsum = __builtin_amdgcn_sdot4((int)d.wcol[kx], 0x00010101, wsum, false);
            }
            const int32_t bias = a.bias[a.bias_len == 1 ? 0 : ch];
            d.bias_adj = (int32_t)((uint32_t)bias - (uint32_t)a.zi * (uint32_t)wsum + 9u * (uint32_t)a.zi * (uint32_t)a.zw);
            if (Q8 || a.fused) {
                const int ci = a.scale.p.per_channel ? ch : 0;
                d.q = make_chan_scale(load_mult(a.scale, ci), (int32_t)a.scale.shift[ci], a.scale.p);
            }
        }
        chan[(tid & 3) * 64 + (tid >> 2)] = d;  // [channel of the quad][quad]: a lane's reads are 48 bytes apart
    }
    __syncthreads();

    // ---- thread -> (channel quad, spatial item) of the block
    const uint32_t sl = a.cb_size == 1 ? (uint32_t)tid : __umulhi((uint32_t)tid, a.cb_magic);  // tid / cb_size
    const int cl = tid - (int)sl * a.cb_size;
    const int c4 = cb * a.cb_size + cl;
    const uint32_t sp = (uint32_t)sb * (uint32_t)a.spb + sl;  // spatial item of the image: row group * strips + strip
    if ((int)sl >= a.spb || c4 * 4 >= a.C || sp >= (uint32_t)(a.row_groups * a.strips)) return;
    const int rg = a.strips == 1 ? (int)sp : (int)__umulhi(sp, a.strips_magic);
    const int strip = (int)sp - rg * a.strips;
    const int c = c4 * 4;
    const int ox0 = strip * TX, oy0 = rg * TY;

    uint32_t wc[3][4];
    int32_t bias_adj[4];
    ChanScale q[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const DwChan d = chan[e * 64 + cl];
        wc[0][e] = d.wcol[0], wc[1][e] = d.wcol[1], wc[2][e] = d.wcol[2];
        bias_adj[e] = d.bias_adj;
        q[e] = d.q;
    }

    // ---- input columns ix0 .. ix0 + NCOL - 1 of rows iy0 .. iy0 + NROW - 1
    constexpr int NCOL = SX * (TX - 1) + 3;
    constexpr int sy = SX;  // the host only sends equal strides here
    const int iy0 = oy0 * sy - a.pad_t, ix0 = ox0 * SX - a.pad_l;
    const uint32_t zsplat = (uint32_t)(uint8_t)a.zi * 0x01010101u;
    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);
    // offsets of taps outside the image wrap to values beyond the extent (such loads return 0) or name another
    // pixel; either way the value is replaced by the zero point below
    const uint32_t xbase = (uint32_t)n * a.x_sn + (uint32_t)c + (uint32_t)iy0 * a.x_sy + (uint32_t)ix0 * a.x_sx;
    int32_t acc[TY][TX][4], xs[TY][TX][4];  // tap kx == 0 of an output starts its accumulator from the bias term
#pragma unroll
    for (int ty = 0; ty < TY; ty++)
#pragma unroll
        for (int t = 0; t < TX; t++)
#pragma unroll
            for (int e = 0; e < 4; e++) xs[ty][t][e] = 0;

    constexpr int NROW_MAX = SX * (TY - 1) + 3;
    uint32_t raw[NROW_MAX][NCOL];
    bool xin[NCOL];
#pragma unroll
    for (int j = 0; j < NCOL; j++) xin[j] = (unsigned)(ix0 + j) < (unsigned)a.W;
#pragma unroll
    for (int r = 0; r < NROW_MAX; r++) {
        const bool yin = (unsigned)(iy0 + r) < (unsigned)a.H;
        const uint32_t rowoff = xbase + (uint32_t)r * a.x_sy;
#pragma unroll
        for (int j = 0; j < NCOL; j++) {
            const uint32_t v =
                (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(xres, (int)(rowoff + (uint32_t)j * a.x_sx), 0, 0);
            raw[r][j] = (yin && xin[j]) ? v : zsplat;
        }
    }
    if constexpr (TY == 2 && SX == 1) {
        // both output rows from one 4 x 4 transpose per column: row 1 uses the weights one byte up
        uint32_t wc1[3][4];
#pragma unroll
        for (int kx = 0; kx < 3; kx++)
#pragma unroll
            for (int e = 0; e < 4; e++) wc1[kx][e] = wc[kx][e] << 8;
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
                    if (ZW) {
                        xs[0][t][e] = __builtin_amdgcn_sdot4((int)col[e], 0x00010101, xs[0][t][e], false);
                        xs[1][t][e] = __builtin_amdgcn_sdot4((int)col[e], 0x01010100, xs[1][t][e], false);
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
                transpose_3x4(raw[ty * SX][j], raw[ty * SX + 1][j], raw[ty * SX + 2][j], col);
#pragma unroll
                for (int t = 0; t < TX; t++) {
                    const int kx = j - t * SX;  // this column is tap kx of output t (compile-time after unrolling)
                    if (kx < 0 || kx > 2) continue;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (kx == 0)
                            acc[ty][t][e] = dot4_from(col[e], wc[0][e], bias_adj[e]);
                        else
                            acc[ty][t][e] = __builtin_amdgcn_sdot4((int)col[e], (int)wc[kx][e], acc[ty][t][e], false);
                        if (ZW) xs[ty][t][e] = __builtin_amdgcn_sdot4((int)col[e], 0x00010101, xs[ty][t][e], false);
                    }
                }
            }
        }
    }

    // ---- epilogue
    const int32_t hi_v = pin_vgpr(a.scale.p.out_hi);
    const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(a.out, 0, (int)a.o_bytes, 0x00020000);
    const uint32_t esz = Q8 ? 1u : (uint32_t)a.out_size;
#pragma unroll
    for (int ty = 0; ty < TY; ty++) {
        const int oy = oy0 + ty;
        if (oy >= a.OH) break;
        const uint32_t orow = ((uint32_t)n * (uint32_t)a.OH + (uint32_t)oy) * (uint32_t)a.OW;
#pragma unroll
        for (int t = 0; t < TX; t++) {
            const int ox = ox0 + t;
            if (ox >= a.OW) break;
            int32_t v[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                int32_t s = acc[ty][t][e];
                if (ZW) s = (int32_t)((uint32_t)s - (uint32_t)a.zw * (uint32_t)xs[ty][t][e]);
                if (Q8 || a.fused) s = requant_acc(s, q[e], a.scale.p, hi_v);
                v[e] = s;
            }
            const uint32_t off = ((orow + (uint32_t)ox) * (uint32_t)a.C + (uint32_t)c) * esz;
            if (Q8 || a.out_size == 1) {
                // the low bytes of the four results, by three byte permutes
                const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
                const uint32_t packed = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                __builtin_amdgcn_raw_buffer_store_b32(packed, ores, (int)off, 0, kOutAux);
            } else if (a.out_size == 2) {
                __builtin_amdgcn_raw_buffer_store_b32((uint32_t)(uint16_t)v[0] | ((uint32_t)(uint16_t)v[1] << 16), ores, (int)off, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b32((uint32_t)(uint16_t)v[2] | ((uint32_t)(uint16_t)v[3] << 16), ores, (int)off + 4, 0, 0);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) __builtin_amdgcn_raw_buffer_store_b32((uint32_t)v[e], ores, (int)off + 4 * e, 0, 0);
            }
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
    // the kernels' requantisation assumes the int32 accumulator's RESCALE has input_zp == 0 (requant_acc); an
    // operator that names another runs as the general operator sequence
    if (epi != nullptr && epi->p.in_zp != 0) return 0;
    const int64_t N = out->dims[0], OH = out->dims[1], OW = out->dims[2], C = out->dims[3];
    // the kernel's indexing assumes: 3x3 taps, multiplier 1, unit dilation, stride 1 or 2, channels in quads, dense
    // weights [3][3][C][1], packed output, channel-contiguous 4-byte aligned input
    if (w->dims[0] != 3 || w->dims[1] != 3 || w->dims[3] != 1 || w->dims[2] != C || in->dims[3] != C) return 0;
    if (a->dilation[0] != 1 || a->dilation[1] != 1) return 0;
    if (a->stride[0] < 1 || a->stride[0] > 2 || a->stride[1] < 1 || a->stride[1] > 2) return 0;
    if (C % 4 != 0 || C <= 0 || C >= (1 << 24) || in->dims[0] < N) return 0;
    if (a->stride[0] != a->stride[1]) return 0;
    if (((uintptr_t)w->ptr % 4) != 0 || ((uintptr_t)bias->ptr % 4) != 0) return 0;
    if (!is_packed(w) || !is_packed(out) || in->strides[3] != 1) return 0;
    if (!(bias->dims[0] == 1 || bias->dims[0] >= C) || bias->strides[0] != 4) return 0;
    if (((uintptr_t)in->ptr % 4) || in->strides[0] % 4 || in->strides[1] % 4 || in->strides[2] % 4) return 0;
    if (((uintptr_t)out->ptr % 16) != 0) return 0;
    if (N <= 0 || OH <= 0 || OW <= 0) return 1;
    if (in->dims[1] >= (1 << 30) || in->dims[2] >= (1 << 30) || OH >= (1 << 30) || OW >= (1 << 30)) return 0;

    // 32-bit offsets: both extents and the item count stay below 2^31
    if (in->strides[0] < 0 || in->strides[1] < 0 || in->strides[2] < 0) return 0;
    const int64_t x_extent = in->dims[0] * in->strides[0], o_extent = N * OH * OW * C * dt_size(out->dtype);
    if (x_extent <= 0 || x_extent >= (int64_t(1) << 31) || o_extent >= (int64_t(1) << 31)) return 0;
    constexpr int TX = 4;
    const int TY = OH >= 2 ? 2 : 1;
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
    g.x_sn = (uint32_t)in->strides[0];
    g.x_sy = (uint32_t)in->strides[1];
    g.x_sx = (uint32_t)in->strides[2];
    g.x_bytes = (uint32_t)x_extent;
    g.o_bytes = (uint32_t)o_extent;
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
    g.row_groups = (int)((OH + TY - 1) / TY);
    // channel quads per block: all of them up to 64, else the even split into the fewest chunks of at most 64
    const int c4n = (int)(C / 4);
    const int chunks = (c4n + 63) / 64;
    g.cb_size = (c4n + chunks - 1) / chunks;
    g.cb_count = (c4n + g.cb_size - 1) / g.cb_size;
    g.spb = kBlock / g.cb_size;
    const int64_t spatial = (int64_t)g.row_groups * g.strips;
    if (spatial >= (1 << 16)) return 0;  // the magic-number divisions hold below 2^16
    g.sb_count = (int)((spatial + g.spb - 1) / g.spb);
    g.cb_magic = (uint32_t)((uint64_t(1) << 32) / (uint64_t)g.cb_size + 1);
    g.strips_magic = (uint32_t)((uint64_t(1) << 32) / (uint64_t)g.strips + 1);
    const int64_t blocks = N * g.sb_count * g.cb_count;
    if (blocks >= (int64_t(1) << 31) - 8) return 0;
    g.blocks = (int)blocks;
    g.chunk = (int)((blocks + 7) / 8);
    g.div_cb = make_div_magic((uint32_t)g.cb_count);
    g.div_sb = make_div_magic((uint32_t)g.sb_count);
    const dim3 grid((unsigned)(g.chunk * 8)), block(kBlock);
    const bool q8 = g.fused && g.out_size == 1;
    const int variant = (TY == 2 ? 4 : 0) + (g.sx == 2 ? 2 : 0) + (g.zw != 0 ? 1 : 0);
#define MLEL_DW_CASE(ID, TYV, SXV, ZWV)                                                  \
    case ID:                                                                             \
        if (q8)                                                                          \
            dwconv3x3_i8_kernel<TX, TYV, SXV, ZWV, true><<<grid, block, 0, s>>>(g);      \
        else                                                                             \
            dwconv3x3_i8_kernel<TX, TYV, SXV, ZWV, false><<<grid, block, 0, s>>>(g);     \
        break;
    switch (variant) {
        MLEL_DW_CASE(0, 1, 1, false)
        MLEL_DW_CASE(1, 1, 1, true)
        MLEL_DW_CASE(2, 1, 2, false)
        MLEL_DW_CASE(3, 1, 2, true)
        MLEL_DW_CASE(4, 2, 1, false)
        MLEL_DW_CASE(5, 2, 1, true)
        MLEL_DW_CASE(6, 2, 2, false)
    default:
        if (q8)
            dwconv3x3_i8_kernel<TX, 2, 2, true, true><<<grid, block, 0, s>>>(g);
        else
            dwconv3x3_i8_kernel<TX, 2, 2, true, false><<<grid, block, 0, s>>>(g);
        break;
    }
#undef MLEL_DW_CASE
    MLEL_TRY(check_launch("depthwise_conv2d 3x3 int8"));
    return 1;
}

namespace {

// ---------------------------------------------------------------------------------------------------------------
// AVG_POOL2D, int8 NHWC, int32 accumulator.  Work item = 4 consecutive channels of one output position; lanes run
// over the channel quads, so a wavefront reads consecutive dwords of each input pixel.  The bytes of a dword are
// widened and accumulated with v_dot4_i32_i8 against a one-hot byte vector.  Arithmetic as avgpool2d.comp:27-75:
// sum of (x - input_zp) over the in-bounds taps, divided by their count with rounding half away from zero,
// output zero point added, clamped to the output type.
// ---------------------------------------------------------------------------------------------------------------
struct AvgArgs {
    const int8_t *x;
    int8_t *out;
    int32_t H, W, C, OH, OW;
    int64_t x_sn, x_sy, x_sx, o_sn, o_sy, o_sx;
    int32_t kh, kw, sy, sx, pad_t, pad_l, zi, zo;
    int64_t items;  // N * OH * OW * C/4
};

// SPLIT threads share the window of one work item (taps dealt round-robin) and combine through shared memory:
// used when there are too few outputs to fill the machine and the window is large (global average pooling).
template <int SPLIT>
__global__ void __launch_bounds__(kBlock) avgpool_i8x4_kernel(const AvgArgs a) {
    constexpr int ITEMS = kBlock / SPLIT;
    __shared__ int32_t partial[SPLIT > 1 ? SPLIT : 1][ITEMS][4];
    const int slot = threadIdx.x % ITEMS, part = threadIdx.x / ITEMS;
    const int64_t item = (int64_t)blockIdx.x * ITEMS + slot;
    const bool live = item < a.items;
    const int c4n = a.C >> 2;
    const int c = live ? (int)(item % c4n) * 4 : 0;
    int64_t rest = live ? item / c4n : 0;
    const int ox = (int)(rest % a.OW);
    rest /= a.OW;
    const int oy = (int)(rest % a.OH);
    const int n = (int)(rest / a.OH);
    const int y0 = max(0, oy * a.sy - a.pad_t), y1 = min(a.H, oy * a.sy - a.pad_t + a.kh);
    const int x0 = max(0, ox * a.sx - a.pad_l), x1 = min(a.W, ox * a.sx - a.pad_l + a.kw);
    const int nx = x1 - x0;
    const int count = (live && y1 > y0 && nx > 0) ? (y1 - y0) * nx : 0;
    int32_t acc[4] = {0, 0, 0, 0};
    const int8_t *xb = a.x + (int64_t)n * a.x_sn + c;
    // taps part, part + SPLIT, ... in batches of four independent loads
    int ty = y0, tx = x0 + part;
    for (int t = part; t < count; t += 4 * SPLIT) {
        int v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            while (tx >= x1) {
                tx -= nx;
                ty++;
            }
            v[k] = (t + k * SPLIT < count)
                       ? *reinterpret_cast<const int32_t *>(xb + (int64_t)ty * a.x_sy + (int64_t)tx * a.x_sx)
                       : 0;
            tx += SPLIT;
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            acc[0] = __builtin_amdgcn_sdot4(v[k], 0x00000001, acc[0], false);
            acc[1] = __builtin_amdgcn_sdot4(v[k], 0x00000100, acc[1], false);
            acc[2] = __builtin_amdgcn_sdot4(v[k], 0x00010000, acc[2], false);
            acc[3] = __builtin_amdgcn_sdot4(v[k], 0x01000000, acc[3], false);
        }
    }
    if (SPLIT > 1) {
#pragma unroll
        for (int e = 0; e < 4; e++) partial[part][slot][e] = acc[e];
        __syncthreads();
        if (part != 0) return;
#pragma unroll
        for (int p = 1; p < SPLIT; p++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[e] += partial[p][slot][e];
    }
    if (!live) return;
    uint32_t packed = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        int32_t r = 0;
        if (count > 0) {
            const int32_t s = (int32_t)((uint32_t)acc[e] - (uint32_t)a.zi * (uint32_t)count);
            r = (s + (s < 0 ? -(count >> 1) : (count >> 1))) / count;
        }
        r = min(max(r + a.zo, -128), 127);
        packed |= ((uint32_t)r & 0xffu) << (8 * e);
    }
    *reinterpret_cast<uint32_t *>(a.out + (int64_t)n * a.o_sn + (int64_t)oy * a.o_sy + (int64_t)ox * a.o_sx + c) = packed;
}

}  // namespace

int try_avgpool_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                     const mlel_pool2d_attr *attr) {
    (void)ctx;
    if (in->dtype != MLEL_I8 || out->dtype != MLEL_I8 || attr->acc_type != MLEL_ACC_I32) return 0;
    const int64_t N = out->dims[0], OH = out->dims[1], OW = out->dims[2], C = out->dims[3];
    // the kernel's indexing assumes: channel quads contiguous and dword aligned on both sides, 32-bit coordinates,
    // a window small enough that the rounded sum stays inside int32
    if (C % 4 != 0 || in->dims[3] != C || in->dims[0] < N) return 0;
    if (in->strides[3] != 1 || out->strides[3] != 1) return 0;
    for (int i = 0; i < 3; i++)
        if (in->strides[i] % 4 != 0 || out->strides[i] % 4 != 0) return 0;
    if (((uintptr_t)in->ptr % 4) != 0 || ((uintptr_t)out->ptr % 4) != 0) return 0;
    if (attr->kernel[0] < 1 || attr->kernel[1] < 1 || (int64_t)attr->kernel[0] * attr->kernel[1] > 65536) return 0;
    if (attr->stride[0] < 1 || attr->stride[1] < 1) return 0;
    if (attr->input_zp < -128 || attr->input_zp > 127 || attr->output_zp < -128 || attr->output_zp > 127) return 0;
    const int64_t lim = int64_t(1) << 24;
    if (in->dims[1] >= lim || in->dims[2] >= lim || OH >= lim || OW >= lim || C >= lim) return 0;
    if ((int64_t)attr->stride[0] >= lim || (int64_t)attr->stride[1] >= lim || (int64_t)attr->pad[0] >= lim ||
        (int64_t)attr->pad[2] >= lim || attr->pad[0] < 0 || attr->pad[2] < 0)
        return 0;
    if (N <= 0 || OH <= 0 || OW <= 0 || C <= 0) return 1;
    AvgArgs g{};
    g.x = static_cast<const int8_t *>(in->ptr);
    g.out = static_cast<int8_t *>(out->ptr);
    g.H = (int)in->dims[1];
    g.W = (int)in->dims[2];
    g.C = (int)C;
    g.OH = (int)OH;
    g.OW = (int)OW;
    g.x_sn = in->strides[0];
    g.x_sy = in->strides[1];
    g.x_sx = in->strides[2];
    g.o_sn = out->strides[0];
    g.o_sy = out->strides[1];
    g.o_sx = out->strides[2];
    g.kh = attr->kernel[0];
    g.kw = attr->kernel[1];
    g.sy = attr->stride[0];
    g.sx = attr->stride[1];
    g.pad_t = attr->pad[0];
    g.pad_l = attr->pad[2];
    g.zi = attr->input_zp;
    g.zo = attr->output_zp;
    g.items = N * OH * OW * (C / 4);
    const bool split = g.items < 256 * 1024 && (int64_t)g.kh * g.kw >= 16;
    const int per_block = split ? kBlock / 8 : kBlock;
    const int64_t blocks = (g.items + per_block - 1) / per_block;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "avg_pool2d: too many work items");
    if (split)
        avgpool_i8x4_kernel<8><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(g);
    else
        avgpool_i8x4_kernel<1><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(g);
    MLEL_TRY(check_launch("avg_pool2d int8"));
    return 1;
}


namespace {

// ---------------------------------------------------------------------------------------------------------------
// TRANSPOSE of dense tensors (transpose.comp:19-32: out[o] = in[i] with i[perms[k]] = o[k]).
//   rows : the last axis stays last: whole rows are moved with 128-bit accesses;
//   tiles: the last axis moves: 64 x 64 element tiles go through shared memory so that both the reads (along the
//          input's last axis) and the writes (along the output's last axis) are contiguous.
// ---------------------------------------------------------------------------------------------------------------
struct TransposeArgs {
    const char *in;
    char *out;
    int32_t rank;
    int64_t odims[MLEL_MAX_RANK];     // output extents
    int64_t istride[MLEL_MAX_RANK];   // byte stride of the input axis that feeds output axis k
    int64_t ostride[MLEL_MAX_RANK];   // byte strides of the output
    int64_t vecs;                     // rows kernel: 16-byte pieces in total
    int32_t segs;                     // rows kernel: 16-byte pieces per row
    int32_t q;                        // tiles kernel: output axis fed by the input's last axis
    int64_t tiles_i, tiles_j, batches;
};

__global__ void __launch_bounds__(kBlock) transpose_rows_kernel(const TransposeArgs a) {
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v >= a.vecs) return;
    int64_t row = v / a.segs;
    const int64_t seg = v - row * a.segs;
    int64_t src = seg * 16;
    for (int k = a.rank - 2; k >= 0; k--) {
        const int64_t d = a.odims[k];
        const int64_t o = row % d;
        row /= d;
        src += o * a.istride[k];
    }
    *reinterpret_cast<uint4 *>(a.out + v * 16) = *reinterpret_cast<const uint4 *>(a.in + src);
}

template <typename T>
__global__ void __launch_bounds__(kBlock) transpose_tiles_kernel(const TransposeArgs a) {
    __shared__ T tile[64][65];
    int64_t b = blockIdx.x;
    const int64_t tj = b % a.tiles_j;
    b /= a.tiles_j;
    const int64_t ti = b % a.tiles_i;
    int64_t batch = b / a.tiles_i;
    const int last = a.rank - 1;
    int64_t src = 0, dst = 0;
    for (int k = last - 1; k >= 0; k--) {  // the remaining output axes enumerate the batch
        if (k == a.q) continue;
        const int64_t d = a.odims[k];
        const int64_t o = batch % d;
        batch /= d;
        src += o * a.istride[k];
        dst += o * a.ostride[k];
    }
    const int64_t i0 = ti * 64, j0 = tj * 64;  // i: output axis q = input last axis; j: output last axis
    const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
    for (int r = ly; r < 64; r += 4) {
        const int64_t j = j0 + r, i = i0 + lx;
        if (j < a.odims[last] && i < a.odims[a.q])
            tile[r][lx] = *reinterpret_cast<const T *>(a.in + src + j * a.istride[last] + i * (int64_t)sizeof(T));
    }
    __syncthreads();
    for (int r = ly; r < 64; r += 4) {
        const int64_t i = i0 + r, j = j0 + lx;
        if (i < a.odims[a.q] && j < a.odims[last])
            *reinterpret_cast<T *>(a.out + dst + i * a.ostride[a.q] + j * (int64_t)sizeof(T)) = tile[lx][r];
    }
}

// The same for 2-byte elements when both moving extents are multiples of 8 and everything is 16-byte aligned: the
// tile enters and leaves in 16-byte pieces (eight elements), the transposition happens in shared memory, where the
// second phase gathers its eight elements from eight rows.
__global__ void __launch_bounds__(kBlock) transpose_tiles_u16x8_kernel(const TransposeArgs a) {
    constexpr int kPitch = 136;  // bytes per tile row: 8-byte aligned, eight rows apart land 16 banks apart
    __shared__ __align__(16) char tile[64 * kPitch];
    int64_t b = blockIdx.x;
    const int64_t tj = b % a.tiles_j;
    b /= a.tiles_j;
    const int64_t ti = b % a.tiles_i;
    int64_t batch = b / a.tiles_i;
    const int last = a.rank - 1;
    int64_t src = 0, dst = 0;
    for (int k = last - 1; k >= 0; k--) {
        if (k == a.q) continue;
        const int64_t d = a.odims[k];
        const int64_t o = batch % d;
        batch /= d;
        src += o * a.istride[k];
        dst += o * a.ostride[k];
    }
    const int64_t i0 = ti * 64, j0 = tj * 64;  // i: output axis q = input last axis; j: output last axis
    const int tid = threadIdx.x;
    uint4 v[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {  // tile row j (an input row), piece c of eight elements along i
        const int p = tid + kBlock * k, j = p >> 3, c = p & 7;
        v[k] = make_uint4(0, 0, 0, 0);
        if (j0 + j < a.odims[last] && i0 + c * 8 < a.odims[a.q])
            v[k] = *reinterpret_cast<const uint4 *>(a.in + src + (j0 + j) * a.istride[last] + (i0 + c * 8) * 2);
    }
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int p = tid + kBlock * k, j = p >> 3, c = p & 7;
        *reinterpret_cast<uint2 *>(tile + j * kPitch + c * 16) = make_uint2(v[k].x, v[k].y);
        *reinterpret_cast<uint2 *>(tile + j * kPitch + c * 16 + 8) = make_uint2(v[k].z, v[k].w);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 2; k++) {  // output row i, piece c of eight elements along j
        const int p = tid + kBlock * k, i = p >> 3, c = p & 7;
        if (i0 + i >= a.odims[a.q] || j0 + c * 8 >= a.odims[last]) continue;
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t lo = *reinterpret_cast<const uint16_t *>(tile + (c * 8 + 2 * e) * kPitch + i * 2);
            const uint32_t hi = *reinterpret_cast<const uint16_t *>(tile + (c * 8 + 2 * e + 1) * kPitch + i * 2);
            w[e] = lo | (hi << 16);
        }
        *reinterpret_cast<uint4 *>(a.out + dst + (i0 + i) * a.ostride[a.q] + (j0 + c * 8) * 2) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

}  // namespace

int try_transpose_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                       const uint32_t *perms) {
    (void)ctx;
    const int rank = out->rank;
    const int esize = dt_size(out->dtype);
    if (rank < 2 || !is_packed(in) || !is_packed(out)) return 0;
    uint32_t seen = 0;
    for (int k = 0; k < rank; k++) {
        if (perms[k] >= (uint32_t)rank || out->dims[k] != in->dims[perms[k]]) return 0;
        seen |= 1u << perms[k];
    }
    if (seen != (1u << rank) - 1) return 0;
    if (numel(out) <= 0) return 1;
    TransposeArgs a{};
    a.in = static_cast<const char *>(in->ptr);
    a.out = static_cast<char *>(out->ptr);
    a.rank = rank;
    int64_t stride = esize;
    for (int k = rank - 1; k >= 0; k--) {  // dense strides computed here (a packed tensor may carry any stride on
        a.ostride[k] = stride;             // an axis of extent 1)
        stride *= out->dims[k];
    }
    int64_t in_dense[MLEL_MAX_RANK];
    stride = esize;
    for (int k = rank - 1; k >= 0; k--) {
        in_dense[k] = stride;
        stride *= in->dims[k];
    }
    for (int k = 0; k < rank; k++) {
        a.odims[k] = out->dims[k];
        a.istride[k] = in_dense[perms[k]];
    }
    const int last = rank - 1;
    if (perms[last] == (uint32_t)last) {
        const int64_t row_bytes = out->dims[last] * esize;
        if (row_bytes % 16 != 0 || ((uintptr_t)in->ptr % 16) != 0 || ((uintptr_t)out->ptr % 16) != 0) return 0;
        if (row_bytes / 16 >= (int64_t(1) << 31)) return 0;
        a.segs = (int32_t)(row_bytes / 16);
        a.vecs = numel(out) * esize / 16;
        const int64_t blocks = (a.vecs + kBlock - 1) / kBlock;
        MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "transpose: too many work items");
        transpose_rows_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(a);
        MLEL_TRY(check_launch("transpose rows"));
        return 1;
    }
    if (esize != 1 && esize != 2 && esize != 4) return 0;
    if (((uintptr_t)in->ptr % esize) != 0 || ((uintptr_t)out->ptr % esize) != 0) return 0;
    int q = -1;
    for (int k = 0; k < rank; k++)
        if (perms[k] == (uint32_t)last) q = k;
    a.q = q;
    a.tiles_i = (out->dims[q] + 63) / 64;
    a.tiles_j = (out->dims[last] + 63) / 64;
    a.batches = numel(out) / (out->dims[q] * out->dims[last]);
    const int64_t blocks = a.tiles_i * a.tiles_j * a.batches;
    MLEL_REQUIRE(blocks < (int64_t(1) << 31), MLEL_ERR_LIMIT, "transpose: too many tiles");
    const dim3 grid((unsigned)blocks), block(kBlock);
    const bool pieces = esize == 2 && out->dims[q] % 8 == 0 && out->dims[last] % 8 == 0 && in->dims[last] % 8 == 0 &&
                        ((uintptr_t)in->ptr % 16) == 0 && ((uintptr_t)out->ptr % 16) == 0;
    if (pieces)
        transpose_tiles_u16x8_kernel<<<grid, block, 0, s>>>(a);
    else if (esize == 1)
        transpose_tiles_kernel<uint8_t><<<grid, block, 0, s>>>(a);
    else if (esize == 2)
        transpose_tiles_kernel<uint16_t><<<grid, block, 0, s>>>(a);
    else
        transpose_tiles_kernel<uint32_t><<<grid, block, 0, s>>>(a);
    MLEL_TRY(check_launch("transpose tiles"));
    return 1;
}

}  // namespace mlel
