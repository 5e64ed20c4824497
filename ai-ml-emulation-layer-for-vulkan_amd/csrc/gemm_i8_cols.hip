// int8 1x1 CONV2D + RESCALE (+CLAMP) (+ residual ADD) for contractions whose operands can stay out of shared memory:
// every wavefront owns one 32 x 32 output tile (32 consecutive positions x 32 consecutive channels) and streams its
// 32 pixel rows and its 32 weight rows straight from memory into the operands of v_mfma_i32_32x32x32_i8 (lane =
// row lane % 32, 16 bytes of K from 32 c + 16 (lane / 32)), four K chunks per round with the next round's loads in
// flight.  No LDS, no barrier, no tile shared between wavefronts: the layers this serves (the projections of an
// inverted-residual network below 56 x 56: a few thousand tiles of K = 144 .. 960) are chains of latencies in the
// staged kernel (fetch, LDS round trip and barrier per 64 bytes of K), not throughput.  Arithmetic as
// gemm_i8_kernel with a zero weight zero point: sum x w - zx * sum w + bias, requantised (reference:
// conv2d.comp:40-116, rescale.comp:28-63, clamp.comp:18-31), then the residual stage of that kernel.
#include "gemm_i8_kernel.hpp"

namespace mlel {
namespace {

constexpr int kColsBlock = 256;
constexpr int KR = 4;  // 32-byte K chunks per round

// table[byte e of w]: the byte is scaled to a dword offset by one SDWA shift
template <int E>
__device__ __forceinline__ uint32_t byte_times_4(uint32_t w) {
    uint32_t r;
    const uint32_t two = 2;
    if constexpr (E == 0)
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(two), "v"(w));
    else if constexpr (E == 1)
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(two), "v"(w));
    else if constexpr (E == 2)
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(two), "v"(w));
    else
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(two), "v"(w));
    return r;
}
__device__ __forceinline__ int32_t lds_entry(const int32_t *table, uint32_t w, int e) {
    const uint32_t off = e == 0 ? byte_times_4<0>(w) : e == 1 ? byte_times_4<1>(w) : e == 2 ? byte_times_4<2>(w) : byte_times_4<3>(w);
    return *reinterpret_cast<const int32_t *>(reinterpret_cast<const char *>(table) + off);
}

// KS == 1: a wavefront per tile.  KS == 4 (few tiles): the four wavefronts of a block share a tile, each takes a
// quarter of the K chunks, the partial tiles are added through shared memory (int32 addition wraps: the order is
// immaterial) and each wavefront requantises and stores a quarter of the tile (eight of its 32 positions).
template <bool RES, int KS>
__global__ void __launch_bounds__(kColsBlock) conv_cols_mfma_i8_kernel(const GemmArgs g, int groups_n, int total_waves,
                                                                         const DivMagic div_groups_n, int chunk) {
    // every argument that the tile assignment, the first operand requests and the epilogue depend on, asked for in one
    // batch: left alone the compiler loads most of them behind the early exit, a second trip to memory in a row
    asm volatile("" ::"s"(total_waves), "s"(groups_n), "s"(div_groups_n.m), "s"(div_groups_n.s), "s"(chunk), "s"(g.x), "s"(g.w),
                 "s"(g.x_bytes), "s"(g.w_bytes), "s"(g.M), "s"(g.N), "s"(g.K), "s"(g.batches), "s"(g.x_sx), "s"(g.ldw), "s"(g.ldo),
                 "s"(g.o_bytes), "s"(g.out), "s"(g.bias), "s"(g.bias_len), "s"(g.zx), "s"(g.mult), "s"(g.shift),
                 "s"(g.mult16), "s"(g.rp.out_zp), "s"(g.rp.out_lo), "s"(g.rp.out_hi), "s"(g.rp.double_round),
                 "s"(g.rp.per_channel));
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // blocks are dealt round-robin to the XCDs: XCD k gets the k-th contiguous run of blocks, so the tiles of a
    // pixel row group (which read the same 32 pixel rows) fetch them into one L2
    // (`chunk`: an eighth of the grid, which is a multiple of eight blocks)
    const int bid = (int)(blockIdx.x % 8u) * chunk + (int)(blockIdx.x / 8u);
    const int wid = KS == 1 ? bid * (kColsBlock / 64) + wave : bid;
    // whole wavefronts (KS == 1) or whole blocks (KS == 4) have nothing to do; with the residual stage a wavefront
    // stays for the block's table and its barrier and leaves behind it
    if (!(RES && KS == 1) && wid >= total_waves) return;
    const int mg = div_magic(wid, div_groups_n), ng = wid - mg * groups_n;
    const int cl = lane & 31, half = lane >> 5;
    const int m = mg * 32 + cl, n = ng * 32 + cl;
    const __amdgpu_buffer_rsrc_t xres = make_rsrc(g.x, g.x_bytes), wres = make_rsrc(g.w, g.w_bytes);
    const uint32_t xoff = m < g.M ? (uint32_t)m * (uint32_t)g.x_sx + (uint32_t)half * 16u : kOobOffset;
    const uint32_t woff = n < g.N ? (uint32_t)n * (uint32_t)g.ldw + (uint32_t)half * 16u : kOobOffset;
    auto fetch = [&](int round, v4i (&xf)[KR], v4i (&wf)[KR]) {
        // a round wholly inside K needs no test: the offset of a row outside the tensor stays beyond the buffer's
        // extent when k is added to it (kOobOffset + k < 2^32), and such loads return zeros
        const bool whole = (round + 1) * KR * 32 <= g.K;  // uniform
#pragma unroll
        for (int c = 0; c < KR; c++) {
            const int k = (round * KR + c) * 32;
            const bool in = whole || k + half * 16 < g.K;  // K % 16 == 0: a piece lies wholly inside or outside the row
            const uint4 xv = buf_load16(xres, in ? xoff + (uint32_t)k : kOobOffset);
            const uint4 wv = buf_load16(wres, in ? woff + (uint32_t)k : kOobOffset);
            xf[c] = v4i{(int)xv.x, (int)xv.y, (int)xv.z, (int)xv.w};
            wf[c] = v4i{(int)wv.x, (int)wv.y, (int)wv.z, (int)wv.w};
        }
    };
    // rounds of this wavefront: all of them, or its quarter [first, first + rounds)
    const int all_rounds = (g.K + KR * 32 - 1) / (KR * 32);
    const int per = KS == 1 ? all_rounds : (all_rounds + KS - 1) / KS;
    const int first = KS == 1 ? 0 : wave * per;
    const int rounds = max(0, min(per, all_rounds - first));
    v4i xa[KR], wa[KR], xb[KR], wb[KR];
    fetch(first, xa, wa);

    // ---- where this lane's results go: position 8 q + 4 half + lane % 4 of the tile, channels 4 (cl / 4) .. + 3
    char *ob = g.out;
    const __amdgpu_buffer_rsrc_t ores = make_rsrc(ob, g.o_bytes);
    const __amdgpu_buffer_rsrc_t rres = make_rsrc(RES ? reinterpret_cast<const char *>(g.res) : ob, g.o_bytes);
    // KS == 4: the four wavefronts share the epilogue as well, wavefront w takes register group q = w
    constexpr int NQ = KS == 1 ? 4 : 1;
    uint32_t d_off[NQ], d_res[RES ? NQ : 1];
#pragma unroll
    for (int i = 0; i < NQ; i++) {
        const int q = KS == 1 ? i : wave;
        const int pm = mg * 32 + 8 * q + 4 * half + (lane & 3), pn = ng * 32 + (cl & ~3);
        d_off[i] = (pm < g.M && pn < g.N) ? (uint32_t)pm * (uint32_t)g.ldo + (uint32_t)pn : kOobOffset;
        if constexpr (RES) d_res[i] = buf_load4(rres, d_off[i]);
    }
    // ---- this lane's channel: bias, requantisation constants
    int32_t bias = 0, mult = 0, shift = 0;
    if (n < g.N) {
        bias = g.bias ? g.bias[g.bias_len == 1 ? 0 : n] : 0;
        const int ci = g.rp.per_channel ? n : 0;
        mult = g.mult16 ? (int32_t) reinterpret_cast<const int16_t *>(g.mult)[ci] : reinterpret_cast<const int32_t *>(g.mult)[ci];
        shift = (int32_t)g.shift[ci];
    }

    // The residual stage rescales two 8-bit values per output with per-tensor constants: both are functions of a
    // byte, so the block tabulates them once (256 dwords each, one entry of either table per thread, while the first
    // operands travel) and an output costs two lookups instead of two requantisations.
    ChanScale q_out{};
    __shared__ int32_t res_tab[RES ? 2 : 1][256];
    if constexpr (RES) {
        const ChanScale q_res = make_chan_scale(load_mult(g.rs_res, 0), g.rs_res.shift[0], g.rs_res.p);
        const ChanScale q_conv = make_chan_scale(load_mult(g.rs_conv, 0), g.rs_conv.shift[0], g.rs_conv.p);
        q_out = make_chan_scale(load_mult(g.rs_out, 0), g.rs_out.shift[0], g.rs_out.p);
        // entry `tid`: the byte as stored; its value is (int8_t)tid
        res_tab[0][tid] = requant_chan((int32_t)(int8_t)tid, q_res, g.rs_res.p);
        res_tab[1][tid] = requant_chan((int32_t)(int8_t)tid, q_conv, g.rs_conv.p);
        __syncthreads();
    }
    if (RES && KS == 1 && wid >= total_waves) return;
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    int32_t wsum = 0;
    const bool need_wsum = g.zx != 0;
    auto multiply = [&](const v4i (&xf)[KR], const v4i (&wf)[KR]) {
#pragma unroll
        for (int c = 0; c < KR; c++) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[c], wf[c], acc, 0, 0, 0);
        if (need_wsum) {  // uniform
#pragma unroll
            for (int c = 0; c < KR; c++)
#pragma unroll
                for (int e = 0; e < 4; e++) wsum = __builtin_amdgcn_sdot4(wf[c][e], 0x01010101, wsum, false);
        }
    };
    for (int r = 0; r < rounds; r += 2) {
        if (r + 1 < rounds) fetch(first + r + 1, xb, wb);
        multiply(xa, wa);
        if (r + 1 < rounds) {
            if (r + 2 < rounds) fetch(first + r + 2, xa, wa);
            multiply(xb, wb);
        }
    }
    int32_t own[4 * NQ];  // the accumulators this wavefront requantises
    if constexpr (KS > 1) {
        // every wavefront leaves its partial tile in shared memory and picks up, summed over the four, the register
        // group it requantises (int32 addition wraps: the order is immaterial) and the weight sum
        __shared__ int32_t part[KS][17][64];  // [wavefront][register, then the weight sum][lane]
#pragma unroll
        for (int r = 0; r < 16; r++) part[wave][r][lane] = acc[r];
        part[wave][16][lane] = wsum;
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 4; e++) {
            uint32_t t = 0;
#pragma unroll
            for (int o = 0; o < KS; o++) t += (uint32_t)part[o][4 * wave + e][lane];
            own[e] = (int32_t)t;
        }
        uint32_t t = 0;
#pragma unroll
        for (int o = 0; o < KS; o++) t += (uint32_t)part[o][16][lane];
        wsum = (int32_t)t;
    } else {
#pragma unroll
        for (int r = 0; r < 16; r++) own[r] = acc[r];
    }

    // ---- epilogue: the channel's constants are registers; a 4 x 4 byte transpose inside lane quads turns four
    // positions of one channel into four channels of one position, stored as a dword
    const int32_t sw = wsum + __shfl_xor(wsum, 32);
    const int32_t bias_adj = (int32_t)((uint32_t)bias - (uint32_t)g.zx * (uint32_t)sw);
    const ChanScale cs = make_chan_scale(mult, shift, g.rp);
    const int32_t hi_v = pin_vgpr(g.rp.out_hi), hi_out_v = RES ? pin_vgpr(g.rs_out.p.out_hi) : 0;
    (void)hi_out_v;
    const uint32_t sel_a = (lane & 1) ? 0x03070105u : 0x06020400u;  // exchange with lane ^ 1
    const uint32_t sel_b = (lane & 2) ? 0x03020706u : 0x05040100u;  // exchange with lane ^ 2
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        int32_t v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = requant_acc((int32_t)((uint32_t)own[4 * q + e] + (uint32_t)bias_adj), cs, g.rp, hi_v);
        const uint32_t lo = __builtin_amdgcn_perm((uint32_t)v[1], (uint32_t)v[0], 0x0c0c0400u);
        const uint32_t hi = __builtin_amdgcn_perm((uint32_t)v[3], (uint32_t)v[2], 0x0c0c0400u);
        uint32_t p = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0xb1, 0xf, 0xf, true);
        p = __builtin_amdgcn_perm(o, p, sel_a);
        o = (uint32_t)__builtin_amdgcn_mov_dpp((int)p, 0x4e, 0xf, 0xf, true);
        p = __builtin_amdgcn_perm(o, p, sel_b);
        if constexpr (RES) {
            // the sum is an int32 accumulator rescaled with input_zp 0 (checked by the host): requant_acc
            const uint32_t xw = d_res[q];
            int32_t o4[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int32_t r1 = lds_entry(res_tab[0], xw, e), r2 = lds_entry(res_tab[1], p, e);
                o4[e] = requant_acc((int32_t)((uint32_t)r1 + (uint32_t)r2), q_out, g.rs_out.p, hi_out_v);
            }
            const uint32_t l2 = __builtin_amdgcn_perm((uint32_t)o4[1], (uint32_t)o4[0], 0x0c0c0400u);
            const uint32_t h2 = __builtin_amdgcn_perm((uint32_t)o4[3], (uint32_t)o4[2], 0x0c0c0400u);
            p = __builtin_amdgcn_perm(h2, l2, 0x05040100u);
        }
        __builtin_amdgcn_raw_buffer_store_b32(p, ores, (int)d_off[q], 0, 0);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// 1x1 CONV2D + RESCALE (+CLAMP) to int8 followed by a global AVG_POOL2D (the head of a classification network: the
// last expansion of MobileNetV2 and the pooling over its 7 x 7 positions): the convolution's result never leaves the
// registers.  A block owns one image and two groups of 32 channels; a wavefront owns one group and the positions
// 0 .. 31 or 32 .. 63 of the image (at most 64 positions, those beyond the image multiply zeros and are not summed).
// Loop and requantisation as conv_cols_mfma_i8_kernel; then every lane adds up the int8 results of its positions, the
// two lane halves and the two wavefronts of a group are combined (a shuffle, then shared memory), and the pooling
// arithmetic of avgpool2d.comp:27-75 is applied to the sum: minus count * input_zp, divided by the count with
// rounding half away from zero, plus output_zp, clamped to int8.
// ---------------------------------------------------------------------------------------------------------------
struct ColsPoolArgs {
    int8_t *out;       // [images][channels]
    int32_t positions; // per image (H * W <= 64)
    int32_t images, pairs, total_blocks;
    int32_t zi, zo;
    DivMagic div_pairs;  // block index / pairs
    int32_t chunk;       // an eighth of the grid
};

__global__ void __launch_bounds__(kColsBlock) conv_cols_pool_i8_kernel(const GemmArgs g, const ColsPoolArgs pa) {
    asm volatile("" ::"s"(pa.total_blocks), "s"(pa.pairs), "s"(pa.div_pairs.m), "s"(pa.div_pairs.s), "s"(pa.chunk), "s"(pa.positions),
                 "s"(pa.out), "s"(pa.zi), "s"(pa.zo), "s"(g.x), "s"(g.w), "s"(g.x_bytes), "s"(g.w_bytes), "s"(g.M), "s"(g.N), "s"(g.K),
                 "s"(g.batches), "s"(g.x_sx), "s"(g.ldw), "s"(g.bias), "s"(g.bias_len), "s"(g.zx), "s"(g.mult), "s"(g.shift), "s"(g.mult16),
                 "s"(g.rp.out_zp), "s"(g.rp.out_lo), "s"(g.rp.out_hi), "s"(g.rp.double_round), "s"(g.rp.per_channel),
                 "s"(g.rp.clamp_out));  // (every dword of a wide load named: a register nobody waits for is given away at once)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bid = (int)(blockIdx.x % 8u) * pa.chunk + (int)(blockIdx.x / 8u);
    if (bid >= pa.total_blocks) return;
    const int image = div_magic(bid, pa.div_pairs), pair = bid - image * pa.pairs;
    const int t = wave & 1, ng = pair * 2 + (wave >> 1);
    const int cl = lane & 31, half = lane >> 5;
    const int pos = 32 * t + cl;  // this lane's pixel row of the image
    const int n = ng * 32 + cl;   // and its channel
    const __amdgpu_buffer_rsrc_t xres = make_rsrc(g.x, g.x_bytes), wres = make_rsrc(g.w, g.w_bytes);
    const uint32_t xoff = pos < pa.positions
                              ? (uint32_t)(image * pa.positions + pos) * (uint32_t)g.x_sx + (uint32_t)half * 16u
                              : kOobOffset;
    const uint32_t woff = n < g.N ? (uint32_t)n * (uint32_t)g.ldw + (uint32_t)half * 16u : kOobOffset;
    auto fetch = [&](int round, v4i (&xf)[KR], v4i (&wf)[KR]) {
#pragma unroll
        for (int c = 0; c < KR; c++) {
            const int k = (round * KR + c) * 32;
            const bool in = k + half * 16 < g.K;  // (a row outside the tensor: kOobOffset + k stays beyond the extent)
            const uint4 xv = buf_load16(xres, in ? xoff + (uint32_t)k : kOobOffset);
            const uint4 wv = buf_load16(wres, in ? woff + (uint32_t)k : kOobOffset);
            xf[c] = v4i{(int)xv.x, (int)xv.y, (int)xv.z, (int)xv.w};
            wf[c] = v4i{(int)wv.x, (int)wv.y, (int)wv.z, (int)wv.w};
        }
    };
    const int rounds = (g.K + KR * 32 - 1) / (KR * 32);
    v4i xa[KR], wa[KR], xb[KR], wb[KR];
    fetch(0, xa, wa);
    int32_t bias = 0, mult = 0, shift = 0;
    if (n < g.N) {
        bias = g.bias ? g.bias[g.bias_len == 1 ? 0 : n] : 0;
        const int ci = g.rp.per_channel ? n : 0;
        mult = g.mult16 ? (int32_t) reinterpret_cast<const int16_t *>(g.mult)[ci] : reinterpret_cast<const int32_t *>(g.mult)[ci];
        shift = (int32_t)g.shift[ci];
    }
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    int32_t wsum = 0;
    const bool need_wsum = g.zx != 0;
    auto multiply = [&](const v4i (&xf)[KR], const v4i (&wf)[KR]) {
#pragma unroll
        for (int c = 0; c < KR; c++) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[c], wf[c], acc, 0, 0, 0);
        if (need_wsum) {  // uniform
#pragma unroll
            for (int c = 0; c < KR; c++)
#pragma unroll
                for (int e = 0; e < 4; e++) wsum = __builtin_amdgcn_sdot4(wf[c][e], 0x01010101, wsum, false);
        }
    };
    for (int r = 0; r < rounds; r += 2) {
        if (r + 1 < rounds) fetch(r + 1, xb, wb);
        multiply(xa, wa);
        if (r + 1 < rounds) {
            if (r + 2 < rounds) fetch(r + 2, xa, wa);
            multiply(xb, wb);
        }
    }
    // register 4 q + e of a lane: position 32 t + 8 q + 4 half + e of the image, channel n
    const int32_t sw = wsum + __shfl_xor(wsum, 32);
    const int32_t bias_adj = (int32_t)((uint32_t)bias - (uint32_t)g.zx * (uint32_t)sw);
    const ChanScale cs = make_chan_scale(mult, shift, g.rp);
    const int32_t hi_v = pin_vgpr(g.rp.out_hi);
    int32_t sum = 0;
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int32_t v = requant_acc((int32_t)((uint32_t)acc[4 * q + e] + (uint32_t)bias_adj), cs, g.rp, hi_v);
            sum += (32 * t + 8 * q + 4 * half + e < pa.positions) ? v : 0;
        }
    sum += __shfl_xor(sum, 32);
    __shared__ int32_t part[2][32];  // [group of the block][channel]: the sum over positions 32 .. 63
    if (t == 1 && half == 0) part[wave >> 1][cl] = sum;
    __syncthreads();
    if (t == 1 || half != 0 || n >= g.N) return;
    const int32_t count = pa.positions;
    const int32_t total = (int32_t)((uint32_t)sum + (uint32_t)part[wave >> 1][cl] - (uint32_t)pa.zi * (uint32_t)count);
    int32_t r = (total + (total < 0 ? -(count >> 1) : (count >> 1))) / count;
    r = (int32_t)((uint32_t)r + (uint32_t)pa.zo);
    r = r < -128 ? -128 : (r > 127 ? 127 : r);
    pa.out[(int64_t)image * g.N + n] = (int8_t)r;
}

}  // namespace

// The pooled form: `g` describes the plain 1x1 convolution over images * positions rows (its output pointer is not
// used), `pool_out` is [images][g.N] int8.  Returns 1 when launched (or when `probe` and it would be).
int launch_conv_cols_pool(const void *args, int8_t *pool_out, int images, int positions, int zi, int zo, bool probe,
                          hipStream_t s) {
    const GemmArgs &g = *static_cast<const GemmArgs *>(args);
    if (g.zw != 0 || g.K % 16 != 0 || g.batches != 1 || !g.plain || positions <= 0 || positions > 64 || images <= 0) return 0;
    if ((int64_t)images * positions != g.M) return 0;
    const int64_t groups_n = (g.N + 31) / 32, pairs = (groups_n + 1) / 2;
    const int64_t blocks = (int64_t)images * pairs;
    if (blocks >= (int64_t(1) << 24)) return 0;
    if (probe) return 1;
    const dim3 grid((unsigned)((blocks + 7) / 8 * 8));
    ColsPoolArgs pa{pool_out, positions, images, (int)pairs, (int)blocks, zi, zo, make_div_magic((uint32_t)pairs), (int)(grid.x / 8)};
    conv_cols_pool_i8_kernel<<<grid, dim3(kColsBlock), 0, s>>>(g, pa);
    return 1;
}

// What the kernel's indexing assumes is checked by the caller (plain rows on both sides in 16-byte pieces, 8-bit
// fused epilogue with dword stores, 31-bit extents) and here (zero weight zero point, K in 16-byte pieces).
// Returns 1 when launched.
int launch_conv_cols_mfma(const void *args, hipStream_t s) {
    const GemmArgs &g = *static_cast<const GemmArgs *>(args);
    if (g.zw != 0 || g.K % 16 != 0 || g.batches != 1 || !g.plain) return 0;
    const int64_t groups_m = (g.M + 31) / 32, groups_n = (g.N + 31) / 32;
    const int64_t waves = groups_m * groups_n;
    if (waves >= (int64_t(1) << 30)) return 0;
    const DivMagic div_n = make_div_magic((uint32_t)groups_n);
    // At most 700 tiles of at least eight K chunks: the four wavefronts of a block share a tile (384 -> 64 at
    // 14 x 14 with the residual: 7.2 -> 6.3 us, 960 -> 160 at 7 x 7: 8.3 -> 6.2 us; 1960 tiles of 320 -> 1280 lose)
    if (waves <= 700 && g.K >= 2 * KR * 32) {
        const dim3 grid((unsigned)((waves + 7) / 8 * 8));
        if (g.res != nullptr)
            conv_cols_mfma_i8_kernel<true, 4><<<grid, dim3(kColsBlock), 0, s>>>(g, (int)groups_n, (int)waves, div_n, (int)(grid.x / 8));
        else
            conv_cols_mfma_i8_kernel<false, 4><<<grid, dim3(kColsBlock), 0, s>>>(g, (int)groups_n, (int)waves, div_n, (int)(grid.x / 8));
        return 1;
    }
    const dim3 grid((unsigned)(((waves + kColsBlock / 64 - 1) / (kColsBlock / 64) + 7) / 8 * 8));
    if (g.res != nullptr)
        conv_cols_mfma_i8_kernel<true, 1><<<grid, dim3(kColsBlock), 0, s>>>(g, (int)groups_n, (int)waves, div_n, (int)(grid.x / 8));
    else
        conv_cols_mfma_i8_kernel<false, 1><<<grid, dim3(kColsBlock), 0, s>>>(g, (int)groups_n, (int)waves, div_n, (int)(grid.x / 8));
    return 1;
}

}  // namespace mlel
