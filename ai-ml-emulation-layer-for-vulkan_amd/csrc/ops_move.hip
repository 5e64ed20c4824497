// Data movement on packed tensors in whole pieces: SLICE, CONCAT, PAD, TILE, REVERSE and GATHER (reference results:
// slice.comp, concat.comp, pad.comp, tile.comp, reverse.comp, gather.comp: one invocation per element, index arithmetic
// over every dimension).  Here the trailing dimensions an operator leaves alone form a run of consecutive bytes in both
// tensors; a thread moves one piece of a run (16 bytes when every offset involved is a multiple of 16, else 8, 4, 2 or
// 1), and only the dimensions in front of the run go through the operator's index rule:
//     identity (SLICE and CONCAT: their shift is a constant byte offset), modulo (TILE), mirror (REVERSE),
//     shift with a fill value outside (PAD), row looked up in the index tensor (GATHER).
// At most three such dimensions: the two outer ones are the grid's z and y (decoded on the scalar unit), the inner one
// shares the grid's x with the pieces of a run (one division per thread).  Anything else -- strides, index ranges that
// leave a tensor (the reference's out-of-bounds rules then apply), more dimensions -- stays with the generic kernels.
#include "common.hpp"
#include "dispatch.hpp"

#include <algorithm>
#include <vector>

namespace mlel {
namespace {

constexpr int kBlock = 256;
enum { kIdentity = 0, kModulo = 1, kMirror = 2, kPadShift = 3, kIndexed = 4 };

struct MoveDim {
    int32_t extent;   // iterations
    int32_t kind;
    int32_t in_dim;   // extent of the source in this dimension (modulo, mirror, shift, indexed)
    int32_t param;    // kPadShift: the dimension's position in the padding tensor (the shift is padding[2 * param])
    int64_t s_stride, d_stride;  // bytes
};

struct MoveArgs {
    const char *src;
    char *dst;
    MoveDim dim[3];        // outer to inner; unused leading dimensions have extent 1 and identity
    uint32_t pieces;       // pieces per run
    uint32_t piece_bytes;  // 16, 8, 4, 2 or 1
    uint32_t x_extent;     // dim[2].extent * pieces
    uint32_t pieces_magic; // floor(2^32 / pieces) + 1 when x_extent < 2^16, else 0: plain division
    int64_t src_base, dst_base;
    // PAD's fill value and its padding tensor (int32 [2 * rank], device memory: the shifts are read here, not on the
    // host), GATHER's index tensor [dim[1].extent][dim[2].extent] of int32
    int32_t fill_dtype, pad_const_int;
    double pad_const;
    const int32_t *padding;
    const int32_t *indices;
};

__device__ __forceinline__ bool map_index(const MoveDim &d, int32_t it, int64_t &src_off, const int32_t *padding) {
    int32_t s = it;
    switch (d.kind) {
    case kModulo: s = it % d.in_dim; break;
    case kMirror: s = d.in_dim - 1 - it; break;
    case kPadShift:
        s = it - padding[2 * d.param];  // a uniform address: one scalar load
        if ((uint32_t)s >= (uint32_t)d.in_dim) return false;
        break;
    default: break;
    }
    src_off += (int64_t)s * d.s_stride;
    return true;
}

template <typename T>
__device__ __forceinline__ void move_piece(char *dst, const char *src, bool live, uint64_t fill_lo, uint64_t fill_hi) {
    if constexpr (sizeof(T) == 16) {
        uint4 v = make_uint4((uint32_t)fill_lo, (uint32_t)(fill_lo >> 32), (uint32_t)fill_hi, (uint32_t)(fill_hi >> 32));
        if (live) v = *reinterpret_cast<const uint4 *>(src);
        *reinterpret_cast<uint4 *>(dst) = v;
    } else {
        T v = (T)fill_lo;
        if (live) v = *reinterpret_cast<const T *>(src);
        *reinterpret_cast<T *>(dst) = v;
    }
}

__global__ void __launch_bounds__(kBlock) move_pieces_kernel(const MoveArgs a) {
    const uint32_t x = blockIdx.x * kBlock + threadIdx.x;
    if (x >= a.x_extent) return;
    const uint32_t i2 = a.pieces == 1 ? x : (a.pieces_magic ? __umulhi(x, a.pieces_magic) : x / a.pieces);
    const uint32_t p = x - i2 * a.pieces;
    const int32_t i1 = (int32_t)blockIdx.y, i0 = (int32_t)blockIdx.z;
    int64_t src_off = a.src_base + (int64_t)p * a.piece_bytes;
    const int64_t dst_off = a.dst_base + (int64_t)i0 * a.dim[0].d_stride + (int64_t)i1 * a.dim[1].d_stride +
                            (int64_t)i2 * a.dim[2].d_stride + (int64_t)p * a.piece_bytes;
    bool live = map_index(a.dim[0], i0, src_off, a.padding);
    live = map_index(a.dim[1], i1, src_off, a.padding) && live;
    if (a.dim[2].kind == kIndexed) {
        // GATHER: the row of the source comes from the index tensor; a row outside the source reads as zeros
        const uint32_t rowi = (uint32_t)a.indices[(int64_t)i1 * a.dim[2].extent + (int64_t)i2];
        live = live && rowi < (uint32_t)a.dim[2].in_dim;
        src_off += (int64_t)rowi * a.dim[2].s_stride;
    } else {
        live = map_index(a.dim[2], (int32_t)i2, src_off, a.padding) && live;
    }
    uint64_t fill_lo = 0, fill_hi = 0;
    if (!live && a.fill_dtype >= 0) {  // PAD: the constant as the generic kernel stores it, repeated over the piece
        char buf[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        const int dt = a.fill_dtype;
        if (dt == MLEL_I32)
            raw_st_i(buf, dt, a.pad_const_int);
        else if (dt_is_float(dt))
            raw_st_f(buf, dt, (float)a.pad_const);
        else
            raw_st_i(buf, dt, (int64_t)a.pad_const);
        uint64_t e = 0;
        for (int k = 0; k < 8; k++) e |= (uint64_t)(uint8_t)buf[k] << (8 * k);
        const int sz = dt_size(dt);
        for (int k = sz; k < 8; k *= 2) e |= e << (8 * k);
        fill_lo = fill_hi = e;
    }
    char *dst = a.dst + dst_off;
    const char *src = a.src + src_off;
    switch (a.piece_bytes) {
    case 16: move_piece<uint4>(dst, src, live, fill_lo, fill_hi); break;
    case 8: move_piece<uint64_t>(dst, src, live, fill_lo, fill_hi); break;
    case 4: move_piece<uint32_t>(dst, src, live, fill_lo, fill_hi); break;
    case 2: move_piece<uint16_t>(dst, src, live, fill_lo, fill_hi); break;
    default: move_piece<uint8_t>(dst, src, live, fill_lo, fill_hi); break;
    }
}

// One dimension of the iteration space as the operators describe it, before runs are formed.
struct DimSpec {
    int64_t extent;              // iterations
    int kind;
    int64_t in_dim, param;
    int64_t s_stride, d_stride;  // bytes per step in the source / destination
    bool s_full, d_full;         // the iterations cover the whole extent of the source / destination tensor here
};

int64_t pow2_divisor(int64_t v) { return v == 0 ? 16 : (v & -v); }

// Forms the run and the (at most three) dimensions in front of it and launches; 0 when the case is declined.
int launch_move(hipStream_t s, const void *src, void *dst, int esize, std::vector<DimSpec> dims, int64_t src_base,
                int64_t dst_base, int fill_dtype, double pad_const, int32_t pad_const_int, const int32_t *padding,
                const int32_t *indices) {
    int64_t run = esize;
    // trailing dimensions that are copied as they are and are whole on both sides extend the run ...
    while (!dims.empty() && dims.back().kind == kIdentity && dims.back().s_full && dims.back().d_full) {
        run *= dims.back().extent;
        dims.pop_back();
    }
    // ... and so does one more identity dimension (a SLICE or CONCAT range: consecutive on both sides)
    if (!dims.empty() && dims.back().kind == kIdentity) {
        run *= dims.back().extent;
        dims.pop_back();
    }
    // dimensions of one iteration contribute nothing; neighbours that are whole identities merge
    std::vector<DimSpec> outer;
    for (const DimSpec &d : dims) {
        if (d.extent == 1 && d.kind != kIndexed) {
            // a single iteration still has to pass its index rule: only the plain ones can be dropped
            if (d.kind == kIdentity || d.kind == kModulo) continue;
            if (d.kind == kMirror) {
                src_base += (d.in_dim - 1) * d.s_stride;
                continue;
            }
        }
        if (!outer.empty() && outer.back().kind == kIdentity && d.kind == kIdentity && d.s_full && d.d_full &&
            outer.back().s_stride == d.s_stride * d.extent && outer.back().d_stride == d.d_stride * d.extent) {
            outer.back().extent *= d.extent;
            outer.back().s_stride = d.s_stride;
            outer.back().d_stride = d.d_stride;
            continue;
        }
        outer.push_back(d);
    }
    if (outer.size() > 3) return 0;
    if (indices != nullptr && (outer.empty() || outer.back().kind != kIndexed)) return 0;
    while (outer.size() < 3) outer.insert(outer.begin(), DimSpec{1, kIdentity, 1, 0, 0, 0, true, true});
    // the piece: the largest power of two up to 16 that divides the run, both base offsets, both pointers and every
    // stride in front of the run
    int64_t align = pow2_divisor(run) | pow2_divisor(src_base) | pow2_divisor(dst_base) |
                    pow2_divisor((int64_t)(uintptr_t)src) | pow2_divisor((int64_t)(uintptr_t)dst);
    for (const DimSpec &d : outer) align |= pow2_divisor(d.s_stride) | pow2_divisor(d.d_stride);
    const int64_t piece = std::min<int64_t>(16, align & -align);
    const int64_t pieces = run / piece;
    if (pieces <= 0 || pieces >= (int64_t(1) << 31)) return 0;
    const int64_t x_extent = outer[2].extent * pieces;
    if (x_extent <= 0) return 1;  // nothing to move
    if (x_extent >= (int64_t(1) << 31) || outer[0].extent > 65535 || outer[1].extent > 65535) return 0;
    if (outer[0].extent <= 0 || outer[1].extent <= 0) return 1;
    MoveArgs a{};
    a.src = static_cast<const char *>(src);
    a.dst = static_cast<char *>(dst);
    for (int k = 0; k < 3; k++) {
        const DimSpec &d = outer[(size_t)k];
        if (d.extent >= (int64_t(1) << 31) || d.in_dim >= (int64_t(1) << 31) || d.param >= (int64_t(1) << 31) ||
            d.param <= -(int64_t(1) << 31))
            return 0;
        a.dim[k] = MoveDim{(int32_t)d.extent, d.kind, (int32_t)std::max<int64_t>(d.in_dim, 1), (int32_t)d.param,
                           d.s_stride, d.d_stride};
    }
    a.pieces = (uint32_t)pieces;
    a.piece_bytes = (uint32_t)piece;
    a.x_extent = (uint32_t)x_extent;
    a.pieces_magic = x_extent < 65536 && pieces > 1 ? (uint32_t)((uint64_t(1) << 32) / (uint64_t)pieces + 1) : 0u;
    a.src_base = src_base;
    a.dst_base = dst_base;
    a.fill_dtype = fill_dtype;
    a.pad_const = pad_const;
    a.pad_const_int = pad_const_int;
    a.padding = padding;
    a.indices = indices;
    const dim3 grid((unsigned)((x_extent + kBlock - 1) / kBlock), (unsigned)outer[1].extent, (unsigned)outer[0].extent);
    move_pieces_kernel<<<grid, dim3(kBlock), 0, s>>>(a);
    return check_launch("data movement (pieces)") == 0 ? 1 : -1;
}

bool movable(const mlel_tensor *out, const mlel_tensor *in) {
    return in->rank == out->rank && dt_size(in->dtype) == dt_size(out->dtype) && is_packed(in) && is_packed(out) &&
           numel(out) > 0 && numel(in) > 0;
}

}  // namespace

// Each returns 1 when the operator was launched here, 0 when the generic kernel has to take it, < 0 on a launch error.

int try_slice_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const uint32_t *start) {
    if (!movable(out, in)) return 0;
    const int es = dt_size(out->dtype);
    std::vector<DimSpec> dims;
    int64_t src_base = 0;
    for (int i = 0; i < out->rank; i++) {
        if ((int64_t)start[i] + out->dims[i] > in->dims[i]) return 0;  // reads outside the input: zeros, generic rule
        src_base += (int64_t)start[i] * in->strides[i];
        dims.push_back({out->dims[i], kIdentity, in->dims[i], 0, in->strides[i], out->strides[i],
                        out->dims[i] == in->dims[i], true});
    }
    return launch_move(s, in->ptr, out->ptr, es, dims, src_base, 0, -1, 0.0, 0, nullptr, nullptr);
}

int try_concat_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t offset) {
    if (!movable(out, in)) return 0;
    const int es = dt_size(out->dtype);
    std::vector<DimSpec> dims;  // the iteration space is the INPUT
    for (int i = 0; i < out->rank; i++) {
        const int64_t shift = i == (int)axis ? (int64_t)offset : 0;
        if (in->dims[i] + shift > out->dims[i]) return 0;  // writes outside the output are dropped: generic rule
        dims.push_back({in->dims[i], kIdentity, in->dims[i], 0, in->strides[i], out->strides[i], true,
                        in->dims[i] == out->dims[i]});
    }
    return launch_move(s, in->ptr, out->ptr, es, dims, 0, (int64_t)offset * out->strides[axis], -1, 0.0, 0, nullptr, nullptr);
}

// The padding tensor stays in device memory: which dimensions are padded is read off the extents (TOSA requires
// padding >= 0, so equal extents mean no padding there), the amounts are read by the kernel.
int try_pad_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *padding,
                 double pad_const, int32_t pad_const_int) {
    if (!movable(out, in) || in->dtype != out->dtype) return 0;
    if (padding->dtype != MLEL_I32 || !is_packed(padding) || ((uintptr_t)padding->ptr % 4) != 0) return 0;
    const int es = dt_size(out->dtype);
    std::vector<DimSpec> dims;
    for (int i = 0; i < out->rank; i++) {
        if (out->dims[i] < in->dims[i]) return 0;  // a crop: not what TOSA's PAD describes, generic rule
        const bool plain = out->dims[i] == in->dims[i];
        dims.push_back({out->dims[i], plain ? kIdentity : kPadShift, in->dims[i], i, in->strides[i], out->strides[i], plain,
                        true});
    }
    return launch_move(s, in->ptr, out->ptr, es, dims, 0, 0, out->dtype, pad_const, pad_const_int,
                       static_cast<const int32_t *>(padding->ptr), nullptr);
}

int try_tile_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in) {
    if (!movable(out, in)) return 0;
    const int es = dt_size(out->dtype);
    std::vector<DimSpec> dims;
    for (int i = 0; i < out->rank; i++) {
        const bool plain = out->dims[i] == in->dims[i];
        dims.push_back({out->dims[i], plain ? kIdentity : kModulo, in->dims[i], 0, in->strides[i], out->strides[i], plain,
                        true});
    }
    return launch_move(s, in->ptr, out->ptr, es, dims, 0, 0, -1, 0.0, 0, nullptr, nullptr);
}

int try_reverse_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis) {
    if (!movable(out, in) || !same_shape(out, in)) return 0;
    const int es = dt_size(out->dtype);
    std::vector<DimSpec> dims;
    for (int i = 0; i < out->rank; i++)
        dims.push_back({out->dims[i], i == (int)axis ? kMirror : kIdentity, in->dims[i], 0, in->strides[i], out->strides[i],
                        true, true});
    return launch_move(s, in->ptr, out->ptr, es, dims, 0, 0, -1, 0.0, 0, nullptr, nullptr);
}

int try_gather_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *values, const mlel_tensor *indices) {
    if (!movable(out, values) || indices->dtype != MLEL_I32 || !is_packed(indices)) return 0;
    if (out->rank != 3 || indices->rank != 2) return 0;
    const int64_t N = out->dims[0], W = out->dims[1], C = out->dims[2];
    if (values->dims[0] < N || values->dims[2] != C || indices->dims[0] < N || indices->dims[1] != W) return 0;
    if (((uintptr_t)indices->ptr % 4) != 0) return 0;
    const int es = dt_size(out->dtype);
    std::vector<DimSpec> dims;
    dims.push_back({1, kIdentity, 1, 0, 0, 0, true, true});
    dims.push_back({N, kIdentity, values->dims[0], 0, values->strides[0], out->strides[0], false, false});
    dims.push_back({W, kIndexed, values->dims[1], 0, values->strides[1], out->strides[1], false, false});
    dims.push_back({C, kIdentity, C, 0, values->strides[2], out->strides[2], true, true});
    return launch_move(s, values->ptr, out->ptr, es, dims, 0, 0, -1, 0.0, 0, nullptr,
                       static_cast<const int32_t *>(indices->ptr));
}

// ---------------------------------------------------------------------------------------------------------------
// CONV3D as CONV2D: the KD depth taps of an output slice are laid side by side along the channels,
//   x2[n * OD + od][h][w][kd * IC + c] = in[n][od * sd + kd * dd - pad_front][h][w][c]   (the input zero point where
//   that depth lies outside the tensor: such taps then contribute nothing, as in conv3d.comp:37-104),
//   w2[oc][ky][kx][kd * IC + c] = w[oc][kd][ky][kx][c],
// after which out[n * OD + od] = CONV2D(x2, w2) with the height / width attributes.  One thread moves one piece of
// 16, 4 or 1 bytes of a pixel.
// ---------------------------------------------------------------------------------------------------------------
namespace {

struct DepthGatherArgs {
    const char *in;
    char *x2;
    int64_t pieces;            // N * OD * HW * KD * (IC / piece)
    int32_t D, OD, KD, sd, dd, pad_d, piece, ppp;  // ppp: pieces per pixel (IC / piece)
    int64_t HW, in_sn, in_sd;  // positions per slice; byte strides of the dense input: image, depth slice
    uint32_t zsplat;
};

template <typename T>
__global__ void __launch_bounds__(kBlock) conv3d_depth_gather_kernel(const DepthGatherArgs a) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.pieces) return;
    const int64_t c = i % a.ppp;
    int64_t r = i / a.ppp;
    const int64_t kd = r % a.KD;
    r /= a.KD;
    const int64_t hw = r % a.HW;
    r /= a.HW;
    const int64_t od = r % a.OD, n = r / a.OD;
    const int64_t d = od * a.sd + kd * a.dd - a.pad_d;
    T v;
    if (d >= 0 && d < a.D) {
        v = *reinterpret_cast<const T *>(a.in + n * a.in_sn + d * a.in_sd + (hw * a.ppp + c) * a.piece);
    } else {
        if constexpr (sizeof(T) == 16) v = make_uint4(a.zsplat, a.zsplat, a.zsplat, a.zsplat);
        else v = (T)a.zsplat;
    }
    *reinterpret_cast<T *>(a.x2 + i * a.piece) = v;
}

struct WeightRegroupArgs {
    const char *w;
    char *w2;
    int64_t pieces;  // OC * KHW * KD * (IC / piece)
    int32_t KD, KHW, piece, ppp;
};

template <typename T>
__global__ void __launch_bounds__(kBlock) conv3d_weight_regroup_kernel(const WeightRegroupArgs a) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.pieces) return;
    const int64_t c = i % a.ppp;
    int64_t r = i / a.ppp;
    const int64_t kd = r % a.KD;
    r /= a.KD;
    const int64_t khw = r % a.KHW, oc = r / a.KHW;
    *reinterpret_cast<T *>(a.w2 + i * a.piece) =
        *reinterpret_cast<const T *>(a.w + (((oc * a.KD + kd) * a.KHW + khw) * a.ppp + c) * a.piece);
}

int piece_of(int64_t ic, const void *p0, const void *p1) {
    const uintptr_t bits = (uintptr_t)ic | (uintptr_t)p0 | (uintptr_t)p1;
    return (bits % 16) == 0 ? 16 : (bits % 4) == 0 ? 4 : 1;
}

}  // namespace

// x2 / w2: dense device buffers of N*OD*H*W*KD*IC resp. OC*KH*KW*KD*IC bytes (int8 operands)
int launch_conv3d_regroup(hipStream_t s, void *x2, void *w2, const mlel_tensor *in, const mlel_tensor *w, int64_t OD,
                          const mlel_conv3d_attr *a) {
    const int64_t N = in->dims[0], D = in->dims[1], H = in->dims[2], W = in->dims[3], IC = in->dims[4];
    const int64_t OC = w->dims[0], KD = w->dims[1], KHW = w->dims[2] * w->dims[3];
    {
        const int piece = piece_of(IC, in->ptr, x2);
        DepthGatherArgs g{};
        g.in = static_cast<const char *>(in->ptr);
        g.x2 = static_cast<char *>(x2);
        g.piece = piece;
        g.ppp = (int32_t)(IC / piece);
        g.pieces = N * OD * H * W * KD * g.ppp;
        g.D = (int32_t)D, g.OD = (int32_t)OD, g.KD = (int32_t)KD;
        g.sd = a->stride[0], g.dd = a->dilation[0], g.pad_d = a->pad[0];
        g.HW = H * W;
        g.in_sn = in->strides[0], g.in_sd = in->strides[1];
        g.zsplat = (uint32_t)(uint8_t)a->input_zp * 0x01010101u;
        if (g.pieces > 0) {
            const dim3 grid = grid_1d(g.pieces, kBlock);
            if (piece == 16) hipLaunchKernelGGL(conv3d_depth_gather_kernel<uint4>, grid, dim3(kBlock), 0, s, g);
            else if (piece == 4) hipLaunchKernelGGL(conv3d_depth_gather_kernel<uint32_t>, grid, dim3(kBlock), 0, s, g);
            else hipLaunchKernelGGL(conv3d_depth_gather_kernel<uint8_t>, grid, dim3(kBlock), 0, s, g);
            MLEL_TRY(check_launch("conv3d depth gather"));
        }
    }
    {
        const int piece = piece_of(IC, w->ptr, w2);
        WeightRegroupArgs g{};
        g.w = static_cast<const char *>(w->ptr);
        g.w2 = static_cast<char *>(w2);
        g.piece = piece;
        g.ppp = (int32_t)(IC / piece);
        g.KD = (int32_t)KD, g.KHW = (int32_t)KHW;
        g.pieces = OC * KHW * KD * g.ppp;
        if (g.pieces > 0) {
            const dim3 grid = grid_1d(g.pieces, kBlock);
            if (piece == 16) hipLaunchKernelGGL(conv3d_weight_regroup_kernel<uint4>, grid, dim3(kBlock), 0, s, g);
            else if (piece == 4) hipLaunchKernelGGL(conv3d_weight_regroup_kernel<uint32_t>, grid, dim3(kBlock), 0, s, g);
            else hipLaunchKernelGGL(conv3d_weight_regroup_kernel<uint8_t>, grid, dim3(kBlock), 0, s, g);
            MLEL_TRY(check_launch("conv3d weight regroup"));
        }
    }
    return 0;
}

}  // namespace mlel
