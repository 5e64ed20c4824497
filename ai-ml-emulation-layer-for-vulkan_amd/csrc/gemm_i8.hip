// Host side of the int8 matrix-core contractions: operand analysis, fetch-mode and tile choice, launch.
// The kernel itself is in gemm_i8_kernel.hpp; every tile shape is instantiated in its own gemm_i8_tile*.hip.
#include "gemm_i8_kernel.hpp"

#include <algorithm>

namespace mlel {
namespace {

// Where the split-K mode may keep its partial tiles and counters: the context's workspace of the launch stream, or a
// caller-chosen region (the statically allocated scratch).  `partial_bytes` == 0: never split.
struct SplitScratch {
    char *partials = nullptr;
    uint32_t *counters = nullptr;
    size_t partial_bytes = 0;
    bool from_ctx = true;  // look the workspace up in the context when a split is wanted
};

int launch_gemm(mlel_ctx *ctx, hipStream_t s, GemmArgs &g, const SplitScratch &scratch) {
    // operand fetch modes
    int xmode = X_GENERIC, wmode = W_GENERIC;
    const bool small = g.x_bytes != 0 && g.w_bytes != 0;  // both operand extents fit 31-bit buffer offsets
    if (g.xch == 16 && small) {
        if (g.plain)
            xmode = X_PLAIN;
        else if (g.IC % BK == 0)
            xmode = X_TAP;
    }
    if (g.xch == 4 && small && g.plain && g.K % 4 == 0) xmode = X_PLAIN4;
    if (!g.w_kmajor && g.wch == 16 && small) wmode = W_ROWS;
    if (!g.w_kmajor && g.wch == 4 && small && g.K % 4 == 0) wmode = W_ROWS4;
    if (xmode == X_PLAIN4 && wmode == W_ROWS) wmode = W_ROWS4;  // the dword forms also serve 16-byte aligned rows
    if (xmode == X_PLAIN && wmode == W_ROWS4) xmode = X_PLAIN4;
    if (g.w_kmajor && g.wch >= 4 && small) wmode = g.wch == 16 ? W_KMAJOR : W_KMAJOR4;
    const bool fast = (xmode == X_PLAIN && wmode == W_ROWS) || (xmode == X_TAP && wmode == W_ROWS) ||
                      (xmode == X_PLAIN && (wmode == W_KMAJOR || wmode == W_KMAJOR4)) ||
                      (xmode == X_PLAIN4 && wmode == W_ROWS4);
    if (!fast) {
        xmode = X_GENERIC;
        wmode = W_GENERIC;
    }
    // tile choice: least padded channel extent, larger tile on ties
    const int bn_opts[3] = {128, 64, 32};
    int best = 0;
    int64_t best_pad = INT64_MAX;
    for (int i = 0; i < 3; i++) {
        const int64_t padded = (int64_t)((g.N + bn_opts[i] - 1) / bn_opts[i]) * bn_opts[i];
        if (padded < best_pad) {
            best_pad = padded;
            best = i;
        }
    }
    int BN = bn_opts[best];
    // a problem of very few rows (a fully connected layer over a small batch): narrower tiles on a tie, so that the
    // K loop of a handful of blocks is shared by four times as many
    if (BN == 128 && g.M <= 64 && (int64_t)((g.N + 127) / 128) * g.batches < 32 && (g.N + 31) / 32 * 32 == best_pad) BN = 32;
    // Two tile heights per width: the tall one when there are enough tiles to give every compute unit at least two
    // blocks, otherwise the short one, so that small problems still spread over the machine and several independent
    // blocks per compute unit hide each other's LDS and barrier latency.
    struct Tile {
        int id, bm;
    };
    const Tile tall = BN == 128 ? Tile{0, 128} : (BN == 64 ? Tile{1, 256} : Tile{2, 256});
    const Tile low = BN == 128 ? Tile{3, 64} : (BN == 64 ? Tile{4, 64} : Tile{5, 128});
    int64_t tiles_n = (g.N + BN - 1) / BN;
    const int64_t tall_total = (int64_t)((g.M + tall.bm - 1) / tall.bm) * tiles_n * g.batches;
    const int cus = ctx->props.multiProcessorCount > 0 ? ctx->props.multiProcessorCount : 256;
    Tile tile = tall_total >= 2 * (int64_t)cus ? tall : low;
    // Direct-to-LDS pipeline (dense 16-byte aligned rows on both sides or a K-major W, K in whole 64-byte steps):
    // the 256 x 256 tile when that still gives every compute unit a block, else the 128 x 128 tile when that does
    // (one block per compute unit of this pipeline beats two of the register-staged one: 13.3 against 13.9 us on
    // 8 x 512 x 1024 x 1024).  Smaller problems keep the short tiles of the register-staged pipeline.
    const bool dl_ok = xmode == X_PLAIN && (wmode == W_ROWS || wmode == W_KMAJOR) && g.K % BK == 0 && BN == 128;
    if (dl_ok && g.res == nullptr) {
        const int64_t total256 = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256) * g.batches;
        const bool big = total256 >= cus, mid = tall_total >= (int64_t)cus;
        if (big || mid) {
            tile = big ? Tile{6, 256} : Tile{0, 128};
            xmode = X_PLAIN_DL;
            wmode = wmode == W_ROWS ? W_ROWS_DL : W_KMAJOR_DL;
        }
    }
    if (tile.id == 6) tiles_n = (g.N + 255) / 256;
    g.tiles_m = (g.M + tile.bm - 1) / tile.bm;
    g.tiles_n = (int)tiles_n;
    const int64_t total = (int64_t)g.tiles_m * g.tiles_n * g.batches;
    MLEL_REQUIRE(total > 0 && total < (int64_t(1) << 30), MLEL_ERR_LIMIT, "contraction: %lld tiles", (long long)total);
    g.total_tiles = (int)total;
    // Split K only when the tiles fill less than half of the machine and the K loop is very long.  Measured on
    // MobileNetV2's 7 x 7 layers (75 - 125 tiles, 9 - 15 K steps): a split removes about 0.3 us per K step from a
    // block but the exchange of partial tiles through memory (write-through stores, one atomic, loads) costs 4 - 5 us
    // of latency, so those layers ran 1.5 - 2.5 us SLOWER split; the mode pays from about 24 removed steps on.
    // At least three K steps per block, at most eight splits.
    const int steps = (g.K + BK - 1) / BK;
    g.splits = 1;
    g.split_steps = steps;
    g.partials = nullptr;
    g.counters = nullptr;
    if (ctx->split_k > 1 && xmode != X_PLAIN_DL && total * 2 <= cus && total <= kSplitCounters && steps >= 32) {
        int want = (int)std::min<int64_t>(std::min(8, ctx->split_k), (cus + total - 1) / total);
        int per = std::max(3, (steps + want - 1) / want);
        const int splits = (steps + per - 1) / per;
        const size_t need = (size_t)total * splits * tile.bm * BN * sizeof(int32_t);
        if (splits > 1 && steps - per >= 24) {
            SplitScratch sc = scratch;
            if (sc.from_ctx) {
                SplitWorkspace w;
                if (split_workspace(ctx, s, &w)) {
                    sc.partials = w.partials;
                    sc.counters = w.counters;
                    sc.partial_bytes = kSplitPartialBytes;
                }
            }
            if (sc.partials != nullptr && need <= sc.partial_bytes) {
                g.splits = splits;
                g.split_steps = per;
                g.partials = reinterpret_cast<int32_t *>(sc.partials);
                g.counters = sc.counters;
                // the context's workspaces start at zero and every launch leaves its counters at zero; the shared
                // static region is cleared by a small kernel instead of trusting what the last call left there
                if (!sc.from_ctx) MLEL_TRY(static_scratch_clear_counters(ctx, s));
            }
        }
    }
    const int64_t blocks = total * g.splits;
    g.chunk = (int)((blocks + 7) / 8);
    g.div_tiles_per_batch = make_div_magic((uint32_t)(g.tiles_m * g.tiles_n));
    g.div_tiles_n = make_div_magic((uint32_t)g.tiles_n);
    g.div_band = make_div_magic((uint32_t)(kGroupM * g.tiles_n));
    g.div_last_rows = make_div_magic((uint32_t)(g.tiles_m % kGroupM == 0 ? kGroupM : g.tiles_m % kGroupM));
    const dim3 grid((unsigned)(g.chunk * 8));
    switch (tile.id) {
    case 0: launch_gemm_tile0(&g, xmode, wmode, grid, s); break;
    case 1: launch_gemm_tile1(&g, xmode, wmode, grid, s); break;
    case 2: launch_gemm_tile2(&g, xmode, wmode, grid, s); break;
    case 3: launch_gemm_tile3(&g, xmode, wmode, grid, s); break;
    case 4: launch_gemm_tile4(&g, xmode, wmode, grid, s); break;
    case 6: launch_gemm_tile6(&g, xmode, wmode, grid, s); break;
    default: launch_gemm_tile5(&g, xmode, wmode, grid, s); break;
    }
    return check_launch("int8 contraction");
}

int align_of(const void *p, int64_t a, int64_t b = 16, int64_t c = 16, int64_t d = 16) {
    auto ok = [&](int64_t n) { return ((uintptr_t)p % n) == 0 && a % n == 0 && b % n == 0 && c % n == 0 && d % n == 0; };
    return ok(16) ? 16 : (ok(4) ? 4 : 1);
}

int fill_epilogue(GemmArgs &g, const mlel_tensor *out, const FusedEpilogue *epi) {
    g.out = static_cast<char *>(out->ptr);
    g.out_size = dt_size(out->dtype);
    g.fused = epi != nullptr;
    if (epi) {
        g.mult = static_cast<const char *>(epi->mult->ptr);
        g.shift = static_cast<const int8_t *>(epi->shift->ptr);
        g.mult16 = epi->scale32 ? 0 : 1;
        g.rp = epi->p;
    }
    const int64_t unit = 4 * g.out_size;
    g.out_vec_ok = (g.N % 4 == 0) && ((g.ldo * g.out_size) % unit == 0) && ((uintptr_t)out->ptr % unit == 0) &&
                   ((g.out_batch) % unit == 0);
    const int64_t ob = ((int64_t)(g.M - 1) * g.ldo + g.N) * g.out_size;
    g.o_bytes = ob < (int64_t(1) << 31) ? (uint32_t)ob : 0;
    return 0;
}

bool packed_tail(const mlel_tensor *t, int from) {
    // dims[from..] are laid out contiguously (row-major, no gaps)
    int64_t s = dt_size(t->dtype);
    for (int i = t->rank - 1; i >= from; i--) {
        if (t->strides[i] != s) return false;
        s *= t->dims[i];
    }
    return true;
}

}  // namespace

// `residual`: the fused residual stage (see GemmArgs::res); the case is declined unless the kernel variant that
// carries it applies (plain rows, 8-bit epilogue, not the direct-to-LDS tiles)
int try_conv2d_i8_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                       const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                       const FusedEpilogue *epi, const ConvResidual *residual, const GemmScratch *static_scratch) {
    if (in->dtype != MLEL_I8 || w->dtype != MLEL_I8 || bias->dtype != MLEL_I32 || a->acc_type != MLEL_ACC_I32) return 0;
    if (residual != nullptr && (epi == nullptr || out->dtype != MLEL_I8)) return 0;
    // the kernels' requantisation assumes the int32 accumulator's RESCALE has input_zp == 0 (requant_acc); an
    // operator that names another runs as the general operator sequence
    if (epi != nullptr && epi->p.in_zp != 0) return 0;
    if (epi == nullptr && out->dtype != MLEL_I32) return 0;
    if (epi != nullptr && dt_size(out->dtype) > 4) return 0;
    const int64_t N = out->dims[0], OH = out->dims[1], OW = out->dims[2], OC = out->dims[3];
    const int64_t H = in->dims[1], W = in->dims[2], IC = in->dims[3];
    const int64_t KH = w->dims[1], KW = w->dims[2];
    // shapes the kernel's indexing assumes; anything else goes to the generic path
    if (in->dims[0] < N || w->dims[0] < OC || w->dims[3] != IC || IC <= 0 || KH <= 0 || KW <= 0) return 0;
    if (!(bias->dims[0] == 1 || bias->dims[0] >= OC) || bias->strides[0] != 4) return 0;
    if (in->strides[3] != 1 || !packed_tail(w, 1) || !is_packed(out)) return 0;
    if (a->stride[0] <= 0 || a->stride[1] <= 0 || a->dilation[0] <= 0 || a->dilation[1] <= 0) return 0;
    const int64_t M = N * OH * OW, K = KH * KW * IC;
    if (M <= 0 || OC <= 0) return 1;  // nothing to do
    if (M >= (int64_t(1) << 31) || K >= (int64_t(1) << 30) || OC >= (int64_t(1) << 30)) return 0;
    if (H >= (1 << 30) || W >= (1 << 30)) return 0;

    GemmArgs g{};
    g.M = (int)M;
    g.N = (int)OC;
    g.K = (int)K;
    g.batches = 1;
    g.x = static_cast<const int8_t *>(in->ptr);
    g.x_sn = in->strides[0];
    g.x_sy = in->strides[1];
    g.x_sx = in->strides[2];
    g.H = (int)H;
    g.W = (int)W;
    g.IC = (int)IC;
    g.OHW = (int)(OH * OW);
    g.OW = (int)OW;
    g.KH = (int)KH;
    g.KW = (int)KW;
    g.sy = a->stride[0];
    g.sx = a->stride[1];
    g.dy = a->dilation[0];
    g.dx = a->dilation[1];
    g.pad_t = a->pad[0];
    g.pad_l = a->pad[2];
    g.plain = 0;
    g.xch = align_of(in->ptr, IC, in->strides[0], in->strides[1], in->strides[2]);
    // a 1x1, stride-1, unpadded convolution over a dense image is a plain [M][K] operand with the pixel pitch
    if (KH == 1 && KW == 1 && a->stride[0] == 1 && a->stride[1] == 1 && a->pad[0] == 0 && a->pad[2] == 0 && OH == H &&
        OW == W && in->strides[1] == W * in->strides[2] && in->strides[0] == H * in->strides[1]) {
        g.plain = 1;
        g.H = g.W = 1;
        g.OHW = g.OW = 1;
    }
    {
        const int64_t xb = in->dims[0] * in->strides[0], wbytes = (OC - 1) * w->strides[0] + K;
        g.x_bytes = xb < (int64_t(1) << 31) ? (uint32_t)xb : 0;
        g.w_bytes = wbytes < (int64_t(1) << 31) ? (uint32_t)wbytes : 0;
    }
    g.w = static_cast<const int8_t *>(w->ptr);
    g.ldw = w->strides[0];
    g.w_kmajor = 0;
    g.wch = align_of(w->ptr, K, w->strides[0]);
    g.zx = a->input_zp;
    g.zw = a->weight_zp;
    g.bias = static_cast<const int32_t *>(bias->ptr);
    g.bias_len = (int)bias->dims[0];
    g.ldo = OC;
    g.out_batch = 0;
    MLEL_TRY(fill_epilogue(g, out, epi));
    if (residual != nullptr) {
        const bool q8 = g.fused && g.out_size == 1 && g.out_vec_ok && g.o_bytes != 0;
        const bool rows = g.plain && g.xch == 16 && g.wch == 16 && g.x_bytes != 0 && g.w_bytes != 0;
        if (!q8 || !rows || ((uintptr_t)residual->res->ptr % 4) != 0) return 0;
        g.res = static_cast<const int8_t *>(residual->res->ptr);
        g.rs_res = make_ref(residual->f_res);
        g.rs_conv = make_ref(residual->f_conv);
        g.rs_out = make_ref(residual->f_out);
    }
    {
        // Few tiles of a 1x1 convolution (the projections of an inverted-residual network below 56 x 56): one
        // 32 x 32 tile per wavefront with both operands straight from memory, no LDS and no barrier (gemm_i8_cols.hip).
        // Its operand traffic is 64 K bytes per tile, all of it from L2, so it is bounded: 64 MiB.  Measured on
        // MobileNetV2 b32: 7.1 -> 4.6 us (96 -> 24 at 56 x 56), 5.3 -> 3.7 (144 -> 32 at 28 x 28), 9.0 -> 6.2
        // (960 -> 160 at 7 x 7 with the residual addition), 17 launches, 19 us in all.
        const bool q8 = g.fused && g.out_size == 1 && g.out_vec_ok && g.o_bytes != 0;
        const bool rows = g.plain && g.xch == 16 && g.wch == 16 && g.x_bytes != 0 && g.w_bytes != 0;
        const int64_t tiles = ((M + 31) / 32) * ((OC + 31) / 32);
        if (q8 && rows && tiles <= 8192 && tiles * K <= (int64_t(1) << 20) && launch_conv_cols_mfma(&g, s)) {
            MLEL_TRY(check_launch("conv2d 1x1 int8, one tile per wavefront"));
            return 1;
        }
    }
    SplitScratch sc;
    if (static_scratch != nullptr) {  // the caller's region instead of the context's workspace
        sc.from_ctx = false;
        sc.partials = static_scratch->partials;
        sc.counters = static_scratch->counters;
        sc.partial_bytes = static_scratch->partial_bytes;
    }
    MLEL_TRY(launch_gemm(ctx, s, g, sc));
    if (static_scratch != nullptr && static_scratch->used_split != nullptr) *static_scratch->used_split = g.splits > 1;
    return 1;
}

int try_matmul_i8_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *A,
                       const mlel_tensor *B, const mlel_matmul_attr *attr, const FusedEpilogue *epi) {
    if (A->dtype != MLEL_I8 || B->dtype != MLEL_I8) return 0;
    // the kernels' requantisation assumes the int32 accumulator's RESCALE has input_zp == 0 (requant_acc); an
    // operator that names another runs as the general operator sequence
    if (epi != nullptr && epi->p.in_zp != 0) return 0;
    if (epi == nullptr && out->dtype != MLEL_I32) return 0;
    if (epi != nullptr && dt_size(out->dtype) > 4) return 0;
    const int64_t NB = out->dims[0], M = out->dims[1], N = out->dims[2], K = A->dims[2];
    if (A->dims[0] < NB || B->dims[0] < NB || A->dims[1] < M || B->dims[1] != K || B->dims[2] < N) return 0;
    // B row-wise: element (k, n) at n * pitch + k, i.e. the operator's [K][N] tensor described over a matrix stored as
    // [N][K] (what a graph does once with a constant weight matrix): the weights are then rows of K as a convolution's
    const bool b_rows = K > 1 && N > 1 && B->strides[1] == 1 && B->strides[2] >= K;
    if (A->strides[2] != 1 || (B->strides[2] != 1 && !b_rows) || !is_packed(out)) return 0;
    if (M <= 0 || N <= 0 || NB <= 0) return 1;
    if (K <= 0) return 0;
    if (M >= (int64_t(1) << 30) || N >= (int64_t(1) << 30) || K >= (int64_t(1) << 30) || NB >= (1 << 20)) return 0;

    GemmArgs g{};
    g.M = (int)M;
    g.N = (int)N;
    g.K = (int)K;
    g.batches = (int)NB;
    g.x = static_cast<const int8_t *>(A->ptr);
    g.x_batch = A->strides[0];
    g.x_sx = A->strides[1];
    g.H = 1;
    g.W = 1;
    g.IC = (int)K;
    g.OHW = 1;
    g.OW = 1;
    g.KH = 1;
    g.KW = 1;
    g.sy = g.sx = g.dy = g.dx = 1;
    g.plain = 1;
    g.xch = align_of(A->ptr, K, A->strides[0], A->strides[1]);
    {
        const int64_t xb = (M - 1) * A->strides[1] + K;
        const int64_t wbytes = b_rows ? (N - 1) * B->strides[2] + K : (K - 1) * B->strides[1] + N;
        g.x_bytes = xb < (int64_t(1) << 31) ? (uint32_t)xb : 0;
        g.w_bytes = wbytes < (int64_t(1) << 31) ? (uint32_t)wbytes : 0;
    }
    g.w = static_cast<const int8_t *>(B->ptr);
    g.w_batch = B->strides[0];
    g.ldw = b_rows ? B->strides[2] : B->strides[1];
    g.w_kmajor = b_rows ? 0 : 1;
    g.wch = b_rows ? align_of(B->ptr, K, B->strides[0], B->strides[2]) : align_of(B->ptr, N, B->strides[0], B->strides[1]);
    g.zx = attr->a_zp;
    g.zw = attr->b_zp;
    g.bias = nullptr;
    g.bias_len = 0;
    g.ldo = N;
    g.out_batch = out->strides[0];
    MLEL_TRY(fill_epilogue(g, out, epi));
    if (b_rows) {  // few tiles (a fully connected layer over a batch of rows): one tile per wavefront, as for 1x1 convolutions
        const bool q8 = g.fused && g.out_size == 1 && g.out_vec_ok && g.o_bytes != 0;
        const bool rows = g.xch == 16 && g.wch == 16 && g.x_bytes != 0 && g.w_bytes != 0;
        const int64_t tiles = ((M + 31) / 32) * ((N + 31) / 32);
        if (q8 && rows && tiles <= 8192 && tiles * K <= (int64_t(1) << 20) && launch_conv_cols_mfma(&g, s)) {
            MLEL_TRY(check_launch("matmul int8, one tile per wavefront"));
            return 1;
        }
    }
    MLEL_TRY(launch_gemm(ctx, s, g, SplitScratch{}));
    return 1;
}

// 1x1 CONV2D + RESCALE (+CLAMP) to int8 whose only reader is a global AVG_POOL2D, in one launch
// (conv_cols_pool_i8_kernel).  `conv_out` carries the convolution's result shape and type, its memory is not touched.
// Returns 1 when launched (or, with `probe`, when the shapes are the kernel's), 0 to decline.
int try_conv2d_avgpool_cols(hipStream_t s, const mlel_tensor *pool_out, const mlel_tensor *conv_out, const mlel_tensor *in,
                            const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                            const FusedEpilogue *epi, const mlel_pool2d_attr *pool, bool probe) {
    if (in->dtype != MLEL_I8 || w->dtype != MLEL_I8 || bias->dtype != MLEL_I32 || a->acc_type != MLEL_ACC_I32) return 0;
    if (conv_out->dtype != MLEL_I8 || pool_out->dtype != MLEL_I8 || epi == nullptr) return 0;
    if (!probe && epi->p.in_zp != 0) return 0;
    if (conv_out->rank != 4 || pool_out->rank != 4 || in->rank != 4 || w->rank != 4) return 0;
    const int64_t N = conv_out->dims[0], H = conv_out->dims[1], W = conv_out->dims[2], OC = conv_out->dims[3];
    const int64_t IC = in->dims[3];
    if (in->dims[0] != N || in->dims[1] != H || in->dims[2] != W || w->dims[0] != OC || w->dims[1] != 1 || w->dims[2] != 1 ||
        w->dims[3] != IC)
        return 0;
    if (a->stride[0] != 1 || a->stride[1] != 1 || a->pad[0] != 0 || a->pad[1] != 0 || a->pad[2] != 0 || a->pad[3] != 0 ||
        a->weight_zp != 0)
        return 0;
    if (!(bias->dims[0] == 1 || bias->dims[0] >= OC) || bias->strides[0] != 4) return 0;
    if (!is_packed(in) || !is_packed(w) || !is_packed(pool_out)) return 0;
    // the pooling takes every position of an image into one value per channel
    if (pool->kernel[0] != H || pool->kernel[1] != W || pool->pad[0] != 0 || pool->pad[1] != 0 || pool->pad[2] != 0 ||
        pool->pad[3] != 0 || pool->acc_type != MLEL_ACC_I32)
        return 0;
    if (pool_out->dims[0] != N || pool_out->dims[1] != 1 || pool_out->dims[2] != 1 || pool_out->dims[3] != OC) return 0;
    const int64_t P = H * W, M = N * P;
    if (P <= 0 || P > 64 || N <= 0 || OC <= 0 || IC <= 0 || IC % 16 != 0 || M >= (int64_t(1) << 24)) return 0;
    if (M * IC >= (int64_t(1) << 31) || OC * IC >= (int64_t(1) << 31)) return 0;
    GemmArgs g{};
    g.M = (int)M, g.N = (int)OC, g.K = (int)IC, g.batches = 1;
    g.plain = 1;
    g.x_sx = IC;
    g.x_bytes = (uint32_t)(M * IC);
    g.ldw = IC;
    g.w_bytes = (uint32_t)(OC * IC);
    g.zx = a->input_zp, g.zw = 0;
    g.bias_len = (int)bias->dims[0];
    if (probe) return launch_conv_cols_pool(&g, nullptr, (int)N, (int)P, 0, 0, true, s);
    if (((uintptr_t)in->ptr % 16) != 0 || ((uintptr_t)w->ptr % 16) != 0 || ((uintptr_t)bias->ptr % 4) != 0) return 0;
    g.x = static_cast<const int8_t *>(in->ptr);
    g.w = static_cast<const int8_t *>(w->ptr);
    g.bias = static_cast<const int32_t *>(bias->ptr);
    g.ldo = OC;
    MLEL_TRY(fill_epilogue(g, conv_out, epi));
    if (!launch_conv_cols_pool(&g, static_cast<int8_t *>(pool_out->ptr), (int)N, (int)P, pool->input_zp, pool->output_zp,
                               false, s))
        return 0;
    MLEL_TRY(check_launch("conv2d 1x1 int8 + global avg_pool2d"));
    return 1;
}

}  // namespace mlel
