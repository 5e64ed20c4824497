// The TOSA operators outside the benchmark graphs: ARGMAX, ARITHMETIC_RIGHT_SHIFT, CONV3D, TRANSPOSE_CONV2D, FFT2D,
// RFFT2D, GATHER, SCATTER, RESIZE, REVERSE, TILE, SELECT.  One thread per output element, any rank <= 6 and any byte
// strides, like the generic kernels of ops_generic.hip; each kernel names the reference shader whose results it
// reproduces.
#include "common.hpp"
#include "dispatch.hpp"

namespace mlel {

namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ int64_t global_flat() { return (int64_t)blockIdx.x * blockDim.x + threadIdx.x; }
__device__ __forceinline__ int32_t wadd32(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
__device__ __forceinline__ int32_t wmul32(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }
__device__ __forceinline__ int64_t wadd64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a + (uint64_t)b); }
__device__ __forceinline__ int64_t wmul64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a * (uint64_t)b); }

__device__ inline void broadcast(const TV &t, const int64_t *o, int64_t *idx) {
    for (int i = 0; i < t.rank; i++) idx[i] = t.dims[i] == 1 ? 0 : o[i];
}

__device__ inline void copy_elem(const TV &out, const int64_t *oi, const TV &in, const int64_t *ii) {
    int64_t so, si;
    if (!elem_off(out, oi, &so)) return;  // writes outside the tensor are dropped, reads outside give 0
    const bool ok = elem_off(in, ii, &si);
    switch (dt_size(out.dtype)) {
    case 1: *(uint8_t *)(out.ptr + so) = ok ? *(const uint8_t *)(in.ptr + si) : (uint8_t)0; break;
    case 2: *(uint16_t *)(out.ptr + so) = ok ? *(const uint16_t *)(in.ptr + si) : (uint16_t)0; break;
    case 4: *(uint32_t *)(out.ptr + so) = ok ? *(const uint32_t *)(in.ptr + si) : 0u; break;
    default: *(uint64_t *)(out.ptr + so) = ok ? *(const uint64_t *)(in.ptr + si) : 0ull; break;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// convolutions: one multiply-accumulate in the accumulator type (as conv2d_generic)
// ---------------------------------------------------------------------------------------------------------------
struct Acc {
    int64_t i;
    float f;
};

__device__ __forceinline__ void conv_mac(uint32_t acc_type, Acc &acc, const TV &in, const int64_t *xi, const TV &w,
                                         const int64_t *wi, int32_t zi, int32_t zw) {
    if (acc_type == MLEL_ACC_I32 || acc_type == MLEL_ACC_I64) {
        const int64_t v = ld_acc_i(in, xi) - zi, ww = ld_acc_i(w, wi) - zw;
        acc.i = acc_type == MLEL_ACC_I32 ? (int64_t)wadd32((int32_t)acc.i, wmul32((int32_t)v, (int32_t)ww))
                                         : wadd64(acc.i, wmul64(v, ww));
    } else {
        const float p = (ld_f(in, xi) - (float)zi) * (ld_f(w, wi) - (float)zw);
        acc.f = acc_type == MLEL_ACC_F16 ? rnd_f16(acc.f + rnd_f16(p)) : acc.f + p;
    }
}

// CONV3D (reference results: conv3d.comp:37-104)
struct Conv3dArgs {
    int32_t zi, zw, pad_d, pad_t, pad_l, sd, sy, sx, dd, dy, dx;
    uint32_t acc;
};

__global__ void __launch_bounds__(kBlock) conv3d_kernel(TV out, TV in, TV w, TV bias, Conv3dArgs a, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t D = in.dims[1], H = in.dims[2], W = in.dims[3], IC = w.dims[4];
    Acc acc{0, 0.f};
    for (int64_t kd = 0; kd < w.dims[1]; kd++) {
        const int64_t d = o[1] * a.sd - a.pad_d + kd * a.dd;
        if (d < 0 || d >= D) continue;
        for (int64_t ky = 0; ky < w.dims[2]; ky++) {
            const int64_t y = o[2] * a.sy - a.pad_t + ky * a.dy;
            if (y < 0 || y >= H) continue;
            for (int64_t kx = 0; kx < w.dims[3]; kx++) {
                const int64_t x = o[3] * a.sx - a.pad_l + kx * a.dx;
                if (x < 0 || x >= W) continue;
                for (int64_t ic = 0; ic < IC; ic++) {
                    const int64_t xi[5] = {o[0], d, y, x, ic};
                    const int64_t wi[5] = {o[4], kd, ky, kx, ic};
                    conv_mac(a.acc, acc, in, xi, w, wi, a.zi, a.zw);
                }
            }
        }
    }
    const int64_t bi[1] = {bias.dims[0] == 1 ? 0 : o[4]};
    if (a.acc == MLEL_ACC_I32 || a.acc == MLEL_ACC_I64) {
        const int64_t b = ld_acc_i(bias, bi);
        st_acc_i(out, o, a.acc == MLEL_ACC_I32 ? (int64_t)wadd32((int32_t)acc.i, (int32_t)b) : wadd64(acc.i, b));
    } else {
        const float b = ld_f(bias, bi);
        st_f(out, o, a.acc == MLEL_ACC_F16 ? rnd_f16(acc.f + rnd_f16(b)) : acc.f + b, ST_ACC);
    }
}

// TRANSPOSE_CONV2D (reference results: transpose_conv2d.comp:31-70): the accumulator starts from the bias
struct TconvArgs {
    int32_t zi, zw, pad_t, pad_l, sy, sx;
    uint32_t acc;
};

__global__ void __launch_bounds__(kBlock) tconv2d_kernel(TV out, TV in, TV w, TV bias, TconvArgs a, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t H = in.dims[1], W = in.dims[2], IC = in.dims[3];
    const bool integer = a.acc == MLEL_ACC_I32 || a.acc == MLEL_ACC_I64;
    const int64_t bi[1] = {bias.dims[0] == 1 ? 0 : o[3]};
    Acc acc{0, 0.f};
    if (integer)
        acc.i = a.acc == MLEL_ACC_I32 ? (int64_t)(int32_t)ld_acc_i(bias, bi) : ld_acc_i(bias, bi);
    else
        acc.f = a.acc == MLEL_ACC_F16 ? rnd_f16(ld_f(bias, bi)) : ld_f(bias, bi);
    for (int64_t ky = 0; ky < w.dims[1]; ky++) {
        for (int64_t kx = 0; kx < w.dims[2]; kx++) {
            int64_t iy = o[1] - a.pad_t - ky, ix = o[2] - a.pad_l - kx;
            if (iy % a.sy != 0 || ix % a.sx != 0) continue;  // truncating remainder, as in the shader
            iy /= a.sy;
            ix /= a.sx;
            if (iy < 0 || ix < 0 || iy >= H || ix >= W) continue;
            for (int64_t ic = 0; ic < IC; ic++) {
                const int64_t xi[4] = {o[0], iy, ix, ic};
                const int64_t wi[4] = {o[3], ky, kx, ic};
                conv_mac(a.acc, acc, in, xi, w, wi, a.zi, a.zw);
            }
        }
    }
    if (integer)
        st_acc_i(out, o, acc.i);
    else
        st_f(out, o, acc.f, ST_ACC);
}

// ---------------------------------------------------------------------------------------------------------------
// ARGMAX (reference results: argmax.comp:26-66)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) argmax_kernel(TV out, TV in, uint32_t axis, uint32_t nan_mode, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    for (uint32_t i = 0; i < axis; i++) ii[i] = o[i];
    for (int i = (int)axis; i < out.rank; i++) ii[i + 1] = o[i];
    const int64_t len = in.dims[axis];
    int64_t best = 0;
    if (dt_is_float(in.dtype)) {
        float mx = dt_lowest_f(in.dtype);  // lowest finite value of the type
        for (int64_t i = 0; i < len; i++) {
            ii[axis] = i;
            const float v = ld_f(in, ii);
            if (isnan(v)) {
                if (nan_mode == MLEL_NAN_IGNORE) continue;
                best = i;
                break;
            }
            if (v > mx) {
                mx = v;
                best = i;
            }
        }
    } else {
        int64_t mx = dt_lowest(in.dtype);
        for (int64_t i = 0; i < len; i++) {
            ii[axis] = i;
            const int64_t v = ld_i(in, ii);
            if (v > mx) {
                mx = v;
                best = i;
            }
        }
    }
    st_i(out, o, best);
}

// ---------------------------------------------------------------------------------------------------------------
// ARITHMETIC_RIGHT_SHIFT (reference results: arithmetic_right_shift.comp:22-48)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) arshift_kernel(TV out, TV in1, TV in2, uint32_t round, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], a[MLEL_MAX_RANK], b[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    broadcast(in1, o, a);
    broadcast(in2, o, b);
    const int bits = 8 * dt_size(out.dtype);
    const int64_t v = ld_i(in1, a), s = ld_i(in2, b);
    int64_t r = v >> (int)(s & (bits - 1));
    if (round && s > 0 && ((v >> (int)((s - 1) & (bits - 1))) & 1) != 0) r++;
    st_i(out, o, narrow_to(out.dtype, r));
}

// ---------------------------------------------------------------------------------------------------------------
// GATHER / SCATTER / REVERSE / TILE / SELECT (reference results: gather.comp:13-25, scatter.comp:14-34,
// reverse.comp:14-30, tile.comp:12-30, select.comp:15-41)
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) gather_kernel(TV out, TV values, TV indices, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t xi[2] = {o[0], o[1]};
    const int64_t vi[3] = {o[0], (int64_t)(uint32_t)ld_i(indices, xi), o[2]};
    copy_elem(out, o, values, vi);
}

__global__ void __launch_bounds__(kBlock) scatter_kernel(TV out, TV values_in, TV indices, TV input, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    const int64_t W = indices.dims[1];
    for (int64_t wv = 0; wv < W; wv++) {
        const int64_t xi[2] = {o[0], wv};
        if ((int64_t)(uint32_t)ld_i(indices, xi) == o[1]) {  // the first matching row wins
            const int64_t ii[3] = {o[0], wv, o[2]};
            copy_elem(out, o, input, ii);
            return;
        }
    }
    copy_elem(out, o, values_in, o);
}

enum { kReverse = 0, kTile = 1 };
__global__ void __launch_bounds__(kBlock) rearrange_kernel(int kind, TV out, TV in, uint32_t axis, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    for (int i = 0; i < out.rank; i++) ii[i] = kind == kTile ? o[i] % in.dims[i] : o[i];
    if (kind == kReverse) {  // the shader reads the input at the grid position and writes the mirrored position
        const int64_t mirrored = out.dims[axis] - 1 - o[axis];
        o[axis] = mirrored;
    }
    copy_elem(out, o, in, ii);
}

__global__ void __launch_bounds__(kBlock) select_kernel(TV out, TV cond, TV a, TV b, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK], c[MLEL_MAX_RANK], ii[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    broadcast(cond, o, c);
    const bool pick = ld_i(cond, c) != 0;
    broadcast(pick ? a : b, o, ii);
    copy_elem(out, o, pick ? a : b, ii);
}

// ---------------------------------------------------------------------------------------------------------------
// RESIZE (reference results: resize.comp:57-134)
// ---------------------------------------------------------------------------------------------------------------
struct ResizeArgs {
    int32_t yn, yd, xn, xd, off_y, off_x;
    uint32_t mode;
};

__device__ __forceinline__ int32_t idiv_floor(int32_t n, int32_t d) {
    int32_t r = n / d;
    if ((int64_t)r * d > n) r--;
    return r;
}

__global__ void __launch_bounds__(kBlock) resize_kernel(TV out, TV in, ResizeArgs a, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out, flat, o);
    // int32 coordinates narrowed to int16 exactly where the shader narrows them
    const int32_t y = (int32_t)((uint32_t)o[1] * (uint32_t)a.yd + (uint32_t)a.off_y);
    const int16_t iy = (int16_t)idiv_floor(y, a.yn);
    const int16_t ry = (int16_t)(y - iy * a.yn);
    const int32_t x = (int32_t)((uint32_t)o[2] * (uint32_t)a.xd + (uint32_t)a.off_x);
    const int16_t ix = (int16_t)idiv_floor(x, a.xn);
    const int16_t rx = (int16_t)(x - ix * a.xn);
    const int16_t iy0 = (int16_t)(iy > 0 ? iy : 0), ix0 = (int16_t)(ix > 0 ? ix : 0);
    const uint32_t uy1 = (uint32_t)(int32_t)(iy + 1), ux1 = (uint32_t)(int32_t)(ix + 1);  // unsigned min, as there
    const uint32_t hy = (uint32_t)in.dims[1] - 1u, hx = (uint32_t)in.dims[2] - 1u;
    const int16_t iy1 = (int16_t)(uy1 < hy ? uy1 : hy), ix1 = (int16_t)(ux1 < hx ? ux1 : hx);
    const int64_t p00[4] = {o[0], iy0, ix0, o[3]}, p01[4] = {o[0], iy0, ix1, o[3]};
    const int64_t p10[4] = {o[0], iy1, ix0, o[3]}, p11[4] = {o[0], iy1, ix1, o[3]};
    const int dt = out.dtype;
    if (dt_is_float(dt)) {
        const float dy = round_to(dt, round_to(dt, (float)ry) / round_to(dt, (float)a.yn));
        const float dx = round_to(dt, round_to(dt, (float)rx) / round_to(dt, (float)a.xn));
        float acc;
        if (a.mode == MLEL_RESIZE_BILINEAR) {
            const float wy0 = round_to(dt, 1.f - dy), wx0 = round_to(dt, 1.f - dx);
            acc = round_to(dt, round_to(dt, round_to(dt, ld_f(in, p00)) * wy0) * wx0);
            acc = round_to(dt, acc + round_to(dt, round_to(dt, round_to(dt, ld_f(in, p01)) * wy0) * dx));
            acc = round_to(dt, acc + round_to(dt, round_to(dt, round_to(dt, ld_f(in, p10)) * dy) * wx0));
            acc = round_to(dt, acc + round_to(dt, round_to(dt, round_to(dt, ld_f(in, p11)) * dy) * dx));
        } else {
            const int64_t p[4] = {o[0], dy >= 0.5f ? iy1 : iy0, dx >= 0.5f ? ix1 : ix0, o[3]};
            acc = ld_f(in, p);
        }
        st_f(out, o, acc);
    } else {
        const bool wide = dt_size(dt) == 8;  // the computation type is the output's: int32 or int64
        int64_t acc = 0;
        if (a.mode == MLEL_RESIZE_BILINEAR) {
            const int64_t wy0 = (int16_t)a.yn - ry, wx0 = (int16_t)a.xn - rx, wy1 = ry, wx1 = rx;
            const int64_t v[4] = {ld_i(in, p00), ld_i(in, p01), ld_i(in, p10), ld_i(in, p11)};
            const int64_t wy[4] = {wy0, wy0, wy1, wy1}, wx[4] = {wx0, wx1, wx0, wx1};
#pragma unroll
            for (int t = 0; t < 4; t++)
                acc = wide ? wadd64(acc, wmul64(wmul64(v[t], wy[t]), wx[t]))
                           : (int64_t)wadd32((int32_t)acc, wmul32(wmul32((int32_t)v[t], (int32_t)wy[t]), (int32_t)wx[t]));
        } else {
            const int64_t p[4] = {o[0], 2 * (int32_t)ry >= a.yn ? iy1 : iy0, 2 * (int32_t)rx >= a.xn ? ix1 : ix0, o[3]};
            acc = ld_i(in, p);
        }
        st_i(out, o, narrow_to(dt, acc));
    }
}

// ---------------------------------------------------------------------------------------------------------------
// FFT2D / RFFT2D (reference results: fft2d.comp:17-52, rfft2d.comp:13-71): the transform sums evaluated directly;
// FFT2D accumulates in double with float angles, RFFT2D reduces the angle numerator modulo W * H first
// ---------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) fft2d_kernel(TV out_r, TV out_i, TV in_r, TV in_i, float sign, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out_r, flat, o);
    const int64_t H = out_r.dims[1], W = out_r.dims[2];
    double sr = 0.0, si = 0.0;
    for (int64_t iy = 0; iy < H; iy++) {
        for (int64_t ix = 0; ix < W; ix++) {
            const int64_t ii[3] = {o[0], iy, ix};
            const float re = ld_f(in_r, ii), im = ld_f(in_i, ii);
            const float frac = (float)(uint32_t)(iy * o[1]) / (float)H + ((float)ix * (float)o[2]) / (float)W;
            const float angle = sign * 2.0f * 3.14159265358979323846f * frac;
            const float c = cosf(angle), s = sinf(angle);
            sr += (double)(re * c) + (double)(im * s);
            si += (double)(-(re * s)) + (double)(im * c);
        }
    }
    st_f(out_r, o, (float)sr);
    st_f(out_i, o, (float)si);
}

__global__ void __launch_bounds__(kBlock) rfft2d_kernel(TV out_r, TV out_i, TV in, int64_t total) {
    const int64_t flat = global_flat();
    if (flat >= total) return;
    int64_t o[MLEL_MAX_RANK];
    unflatten(out_r, flat, o);
    const int64_t H = in.dims[1], W = in.dims[2], oy = o[1], ox = o[2];
    const bool skip_imag = (oy == 0 || oy == H / 2) && (ox == 0 || ox == W / 2);  // purely real bins stay exactly 0
    double sr = 0.0, si = 0.0;
    for (int64_t iy = 0; iy < H; iy++) {
        for (int64_t ix = 0; ix < W; ix++) {
            const int64_t ii[3] = {o[0], iy, ix};
            const double v = (double)ld_f(in, ii);
            const double num = (double)((iy * oy * W + ix * ox * H) % (W * H));
            const double angle = 2.0 * 3.14159265358979323846 * num / (double)(W * H);
            sr += v * cos(angle);
            if (!skip_imag) si -= v * sin(angle);
        }
    }
    st_f(out_r, o, (float)sr);
    st_f(out_i, o, (float)si);
}

template <typename... KArgs, typename... Args>
int launch(const char *what, void (*kernel)(KArgs...), int64_t total, hipStream_t stream, Args... args) {
    if (total <= 0) return 0;
    MLEL_REQUIRE(total < (int64_t(1) << 31) * kBlock, MLEL_ERR_LIMIT, "%s: too many elements", what);
    hipLaunchKernelGGL(kernel, grid_1d(total, kBlock), dim3(kBlock), 0, stream, args...);
    return check_launch(what);
}

}  // namespace

int conv3d_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                  const mlel_tensor *bias, const mlel_conv3d_attr *a) {
    const Conv3dArgs args{a->input_zp, a->weight_zp, a->pad[0], a->pad[2], a->pad[4], a->stride[0], a->stride[1],
                          a->stride[2], a->dilation[0], a->dilation[1], a->dilation[2], a->acc_type};
    return launch("conv3d", conv3d_kernel, numel(out), s, make_tv(out), make_tv(in), make_tv(w), make_tv(bias), args,
                  numel(out));
}

int tconv2d_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                   const mlel_tensor *bias, const mlel_tconv2d_attr *a) {
    const TconvArgs args{a->input_zp, a->weight_zp, a->out_pad[0], a->out_pad[2], a->stride[0], a->stride[1], a->acc_type};
    return launch("transpose_conv2d", tconv2d_kernel, numel(out), s, make_tv(out), make_tv(in), make_tv(w),
                  make_tv(bias), args, numel(out));
}

int argmax_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t nan_mode) {
    return launch("argmax", argmax_kernel, numel(out), s, make_tv(out), make_tv(in), axis, nan_mode, numel(out));
}

int arshift_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2, uint32_t round) {
    return launch("arithmetic_right_shift", arshift_kernel, numel(out), s, make_tv(out), make_tv(in1), make_tv(in2),
                  round, numel(out));
}

int gather_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *values, const mlel_tensor *indices) {
    return launch("gather", gather_kernel, numel(out), s, make_tv(out), make_tv(values), make_tv(indices), numel(out));
}

int scatter_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *values_in, const mlel_tensor *indices,
                   const mlel_tensor *input) {
    return launch("scatter", scatter_kernel, numel(out), s, make_tv(out), make_tv(values_in), make_tv(indices),
                  make_tv(input), numel(out));
}

int reverse_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis) {
    return launch("reverse", rearrange_kernel, numel(out), s, (int)kReverse, make_tv(out), make_tv(in), axis, numel(out));
}

int tile_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in) {
    return launch("tile", rearrange_kernel, numel(out), s, (int)kTile, make_tv(out), make_tv(in), 0u, numel(out));
}

int select_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *cond, const mlel_tensor *a,
                  const mlel_tensor *b) {
    return launch("select", select_kernel, numel(out), s, make_tv(out), make_tv(cond), make_tv(a), make_tv(b), numel(out));
}

int resize_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_resize_attr *a) {
    const ResizeArgs args{a->scale[0], a->scale[1], a->scale[2], a->scale[3], a->offset[0], a->offset[1], a->mode};
    return launch("resize", resize_kernel, numel(out), s, make_tv(out), make_tv(in), args, numel(out));
}

int fft2d_launch(hipStream_t s, const mlel_tensor *out_r, const mlel_tensor *out_i, const mlel_tensor *in_r,
                 const mlel_tensor *in_i, bool inverse) {
    return launch("fft2d", fft2d_kernel, numel(out_r), s, make_tv(out_r), make_tv(out_i), make_tv(in_r), make_tv(in_i),
                  inverse ? -1.0f : 1.0f, numel(out_r));
}

int rfft2d_launch(hipStream_t s, const mlel_tensor *out_r, const mlel_tensor *out_i, const mlel_tensor *in) {
    return launch("rfft2d", rfft2d_kernel, numel(out_r), s, make_tv(out_r), make_tv(out_i), make_tv(in), numel(out_r));
}

}  // namespace mlel
