// extern "C" operator entry points of include/mlel_hip.h: argument validation (the host-side checks that keep
// every kernel's indexing assumptions true), then dispatch to a specialised gfx950 kernel or the generic path.
#include <vector>

#include "common.hpp"
#include "dispatch.hpp"

using namespace mlel;

namespace {

int require_ctx(mlel_ctx *ctx, const char *what) {
    MLEL_REQUIRE(ctx != nullptr, MLEL_ERR_INVALID, "%s: null context", what);
    hipError_t e = hipSetDevice(ctx->device);
    if (e != hipSuccess) return set_error(MLEL_ERR_DEVICE, "%s: hipSetDevice: %s", what, hipGetErrorString(e));
    return 0;
}

bool is_arith_dtype(int dt) { return dt_is_int(dt) || dt_is_float(dt); }

int check_supported(const mlel_tensor *t, const char *what) {
    MLEL_TRY(check_tensor(t, what));
    MLEL_REQUIRE(is_arith_dtype(t->dtype), MLEL_ERR_UNSUPPORTED,
                 "%s: element type %d (bf16/fp8 storage) has no kernel yet", what, t->dtype);
    return 0;
}

int check_conv(const char *name, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
               const mlel_tensor *bias, const mlel_conv2d_attr *a) {
    MLEL_REQUIRE(a != nullptr, MLEL_ERR_INVALID, "%s: null attributes", name);
    MLEL_TRY(check_supported(out, name));
    MLEL_TRY(check_supported(in, name));
    MLEL_TRY(check_supported(w, name));
    MLEL_TRY(check_supported(bias, name));
    MLEL_REQUIRE(out->rank == 4 && in->rank == 4 && w->rank == 4 && bias->rank == 1, MLEL_ERR_INVALID,
                 "%s: ranks must be 4,4,4,1", name);
    MLEL_REQUIRE(a->acc_type >= 1 && a->acc_type <= 4, MLEL_ERR_INVALID, "Unsupported acc type %u", a->acc_type);
    const bool facc = a->acc_type == MLEL_ACC_F16 || a->acc_type == MLEL_ACC_F32;
    // a floating-point accumulator needs floating-point tensors; an integer accumulator over floating-point storage
    // truncates the operands toward zero like the shaders' ACC_TYPE(v) conversion (common.comp:636-660)
    MLEL_REQUIRE(!facc || (dt_is_float(in->dtype) && dt_is_float(out->dtype)), MLEL_ERR_INVALID,
                 "%s: accumulator type %u does not match the tensor types", name, a->acc_type);
    MLEL_REQUIRE(dt_is_float(in->dtype) == dt_is_float(out->dtype), MLEL_ERR_INVALID,
                 "%s: input and output must both be integer or both floating point", name);
    MLEL_REQUIRE(bias->dtype == out->dtype, MLEL_ERR_INVALID, "%s: bias must have the output type", name);
    return 0;
}

int make_epilogue(const mlel_epilogue *epi, int in_dtype, const mlel_tensor *out, int64_t channels,
                  FusedEpilogue *fe) {
    MLEL_REQUIRE(epi != nullptr && epi->multiplier != nullptr && epi->shift != nullptr, MLEL_ERR_INVALID,
                 "fused epilogue: null argument");
    MLEL_TRY(check_scale_tensors(epi->multiplier, epi->shift, &epi->rescale, channels));
    MLEL_REQUIRE(is_packed(epi->multiplier) && is_packed(epi->shift), MLEL_ERR_INVALID,
                 "fused epilogue: multiplier/shift must be contiguous");
    MLEL_REQUIRE(dt_is_int(out->dtype) && dt_size(out->dtype) <= 4 && out->dtype != MLEL_BOOL, MLEL_ERR_INVALID,
                 "fused epilogue: output must be an 8/16/32-bit integer tensor");
    MLEL_TRY(make_rescale_params(&epi->rescale, in_dtype, out->dtype, epi->has_clamp ? &epi->clamp : nullptr, &fe->p));
    fe->mult = epi->multiplier;
    fe->shift = epi->shift;
    fe->scale32 = epi->rescale.scale32 != 0;
    fe->in_dt = dt_unsigned_twin(in_dtype, epi->rescale.input_unsigned != 0);
    return 0;
}

// scratch int32 tensor for a fused request that no specialised kernel takes: the unfused sequence is run instead
struct Scratch {
    void *ptr = nullptr;
    ~Scratch() {
        if (ptr) (void)hipFree(ptr);
    }
};

// Temporary of a fused entry point's operator-by-operator route.  That route allocates, and synchronises the stream
// before the temporary is freed on return; a stream that is being captured can do neither, so the call is refused there.
int alloc_fallback(Scratch &t, size_t bytes, void *stream, const char *what) {
    MLEL_REQUIRE(!stream_is_capturing((hipStream_t)stream), MLEL_ERR_UNSUPPORTED,
                 "%s: no one-pass kernel takes these operands, and the operator-by-operator route allocates a temporary "
                 "and synchronises, which is not possible on a stream that is being captured",
                 what);
    MLEL_HIP_CHECK(hipMalloc(&t.ptr, bytes));
    return 0;
}

int run_unfused_tail(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *acc,
                     const mlel_epilogue *epi) {
    // RESCALE into `out`, then CLAMP in place: exactly the operator sequence the fused kernels replace
    MLEL_TRY(mlel_hip_rescale(ctx, s, out, acc, epi->multiplier, epi->shift, &epi->rescale));
    if (epi->has_clamp) MLEL_TRY(mlel_hip_clamp(ctx, s, out, out, &epi->clamp));
    return 0;
}

mlel_tensor packed_like(const mlel_tensor *t, int dtype, void *ptr) {
    mlel_tensor r = *t;
    r.dtype = dtype;
    r.ptr = ptr;
    int64_t s = dt_size(dtype);
    for (int i = r.rank - 1; i >= 0; i--) {
        r.strides[i] = s;
        s *= r.dims[i];
    }
    return r;
}

// CONV3D over int8 operands with an int32 result as ONE CONV2D on the matrix cores: the depth taps become channels
// (launch_conv3d_regroup), which costs KD copies of the input in a temporary.  A kernel one slice deep without depth
// padding needs no copy at all: its operands are CONV2D's already.  Returns 1 when done, 0 to decline.
int try_conv3d_as_conv2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                         const mlel_tensor *bias, const mlel_conv3d_attr *a) {
    if (in->dtype != MLEL_I8 || w->dtype != MLEL_I8 || out->dtype != MLEL_I32 || bias->dtype != MLEL_I32 ||
        a->acc_type != MLEL_ACC_I32)
        return 0;
    if (!is_packed(in) || !is_packed(w) || !is_packed(out)) return 0;
    const int64_t N = out->dims[0], OD = out->dims[1], OH = out->dims[2], OW = out->dims[3], OC = out->dims[4];
    const int64_t D = in->dims[1], H = in->dims[2], W = in->dims[3], IC = in->dims[4];
    const int64_t KD = w->dims[1], KH = w->dims[2], KW = w->dims[3];
    if (in->dims[0] != N || w->dims[0] != OC || w->dims[4] != IC || N <= 0 || OD <= 0 || OH <= 0 || OW <= 0 || OC <= 0 ||
        IC <= 0 || KD <= 0 || KH <= 0 || KW <= 0 || D <= 0)
        return 0;
    if (a->stride[0] <= 0 || a->dilation[0] <= 0 || a->pad[0] < 0 || a->pad[1] < 0) return 0;
    mlel_conv2d_attr a2{};
    a2.input_zp = a->input_zp, a2.weight_zp = a->weight_zp, a2.acc_type = a->acc_type;
    for (int i = 0; i < 4; i++) a2.pad[i] = a->pad[2 + i];
    a2.stride[0] = a->stride[1], a2.stride[1] = a->stride[2];
    a2.dilation[0] = a->dilation[1], a2.dilation[1] = a->dilation[2];
    mlel_tensor o2{};
    o2.dtype = MLEL_I32, o2.rank = 4, o2.ptr = out->ptr;
    o2.dims[0] = N * OD, o2.dims[1] = OH, o2.dims[2] = OW, o2.dims[3] = OC;
    mlel_tensor x2 = o2, w2 = o2;
    x2.dtype = w2.dtype = MLEL_I8;
    x2.dims[1] = H, x2.dims[2] = W, x2.dims[3] = KD * IC;
    w2.dims[0] = OC, w2.dims[1] = KH, w2.dims[2] = KW, w2.dims[3] = KD * IC;
    const auto pack = [](mlel_tensor &t) {
        int64_t st = dt_size(t.dtype);
        for (int i = t.rank - 1; i >= 0; i--) t.strides[i] = st, st *= t.dims[i];
        return st;
    };
    pack(o2);
    const int64_t x_bytes = pack(x2), w_bytes = pack(w2);
    if (KD == 1 && a->pad[0] == 0 && a->pad[1] == 0 && a->stride[0] == 1 && OD == D) {
        x2.ptr = in->ptr, w2.ptr = w->ptr;  // [N * D][H][W][IC] and [OC][KH][KW][IC] as they lie
        MLEL_TRY(mlel_hip_conv2d(ctx, stream, &o2, &x2, &w2, bias, &a2));
        return 1;
    }
    // the copies pay from a few million multiply-adds on; they go to the stream's staging memory (no allocation and no
    // wait once it is large enough; when it is not and cannot grow -- a capturing stream -- the generic kernel runs)
    const int64_t macs = N * OD * OH * OW * OC * KD * KH * KW * IC;
    if (macs < (int64_t(1) << 22) || x_bytes >= (int64_t(1) << 31) || w_bytes >= (int64_t(1) << 31)) return 0;
    const size_t x_room = ((size_t)x_bytes + 255) & ~size_t(255);
    char *stage = stage_workspace(ctx, (hipStream_t)stream, x_room + (size_t)w_bytes + 256);
    if (stage == nullptr) return 0;
    x2.ptr = stage, w2.ptr = stage + x_room;
    MLEL_TRY(launch_conv3d_regroup((hipStream_t)stream, x2.ptr, w2.ptr, in, w, OD, a));
    MLEL_TRY(mlel_hip_conv2d(ctx, stream, &o2, &x2, &w2, bias, &a2));
    return 1;
}

}  // namespace

extern "C" {

int mlel_hip_conv2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                    const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv2d_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "conv2d"));
    MLEL_TRY(check_conv("conv2d", out, in, weights, bias, attr));
    int rc = try_conv2d_i8_direct(ctx, (hipStream_t)stream, out, in, weights, bias, attr, nullptr);
    if (rc == 0) rc = try_conv2d_i8_mfma(ctx, (hipStream_t)stream, out, in, weights, bias, attr, nullptr);
    if (rc != 0) return rc < 0 ? rc : 0;
    return conv2d_generic_launch((hipStream_t)stream, out, in, weights, bias, attr);
}

int mlel_hip_depthwise_conv2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                              const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv2d_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "depthwise_conv2d"));
    MLEL_TRY(check_conv("depthwise_conv2d", out, in, weights, bias, attr));
    MLEL_REQUIRE(weights->dims[3] > 0, MLEL_ERR_INVALID, "depthwise_conv2d: channel multiplier must be > 0");
    const int rc = try_dwconv_i8_fast(ctx, (hipStream_t)stream, out, in, weights, bias, attr, nullptr);
    if (rc != 0) return rc < 0 ? rc : 0;
    return dwconv_generic_launch((hipStream_t)stream, out, in, weights, bias, attr);
}

int mlel_hip_matmul(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a, const mlel_tensor *b,
                    const mlel_matmul_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "matmul"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "matmul: null attributes");
    MLEL_TRY(check_supported(out, "matmul out"));
    MLEL_TRY(check_supported(a, "matmul a"));
    MLEL_TRY(check_supported(b, "matmul b"));
    MLEL_REQUIRE(out->rank == 3 && a->rank == 3 && b->rank == 3, MLEL_ERR_INVALID, "matmul: rank must be 3");
    MLEL_REQUIRE(a->dtype == b->dtype, MLEL_ERR_INVALID, "matmul: operand types differ");
    MLEL_REQUIRE(dt_is_float(a->dtype) == dt_is_float(out->dtype), MLEL_ERR_INVALID,
                 "matmul: integer/float mismatch between operands and output");
    int rc = try_matmul_i8_mfma(ctx, (hipStream_t)stream, out, a, b, attr, nullptr);
    if (rc == 0) rc = try_matmul_f16_mfma(ctx, (hipStream_t)stream, out, a, b, attr);
    if (rc != 0) return rc < 0 ? rc : 0;
    return matmul_generic_launch((hipStream_t)stream, out, a, b, attr);
}

int mlel_hip_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                     const mlel_tensor *multiplier, const mlel_tensor *shift, const mlel_rescale_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "rescale"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "rescale: null attributes");
    MLEL_TRY(check_tensor(out, "rescale out"));
    MLEL_TRY(check_tensor(in, "rescale in"));
    MLEL_REQUIRE(in->rank == out->rank, MLEL_ERR_INVALID, "rescale: ranks differ");
    MLEL_TRY(check_scale_tensors(multiplier, shift, attr, out->dims[out->rank - 1]));
    RescaleParams p;
    MLEL_TRY(make_rescale_params(attr, in->dtype, out->dtype, nullptr, &p));
    const int rc = try_rescale_fast(ctx, (hipStream_t)stream, out, in, multiplier, shift, attr, p);
    if (rc != 0) return rc < 0 ? rc : 0;
    return rescale_generic_launch((hipStream_t)stream, out, in, multiplier, shift, attr, p);
}

int mlel_hip_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                   const mlel_clamp_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "clamp"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "clamp: null attributes");
    MLEL_TRY(check_supported(out, "clamp out"));
    MLEL_TRY(check_supported(in, "clamp in"));
    MLEL_REQUIRE(in->dtype == out->dtype && in->rank == out->rank, MLEL_ERR_INVALID, "clamp: type/rank mismatch");
    const int rc = try_clamp_fast(ctx, (hipStream_t)stream, out, in, attr);
    if (rc != 0) return rc < 0 ? rc : 0;
    return clamp_generic_launch((hipStream_t)stream, out, in, attr);
}

int mlel_hip_elementwise_binary(mlel_ctx *ctx, void *stream, int32_t op, const mlel_tensor *out,
                                const mlel_tensor *in1, const mlel_tensor *in2, uint32_t nan_mode) {
    MLEL_TRY(require_ctx(ctx, "elementwise_binary"));
    MLEL_REQUIRE(op >= 0 && op < MLEL_BIN_COUNT, MLEL_ERR_INVALID, "elementwise_binary: unknown op %d", op);
    MLEL_TRY(check_supported(out, "binary out"));
    MLEL_TRY(check_supported(in1, "binary in1"));
    MLEL_TRY(check_supported(in2, "binary in2"));
    MLEL_REQUIRE(in1->dtype == in2->dtype, MLEL_ERR_INVALID, "elementwise_binary: input types differ");
    MLEL_REQUIRE(in1->rank == out->rank && in2->rank == out->rank, MLEL_ERR_INVALID,
                 "elementwise_binary: ranks differ");
    int rc = try_binary_fast(ctx, (hipStream_t)stream, op, out, in1, in2);
    if (rc == 0) rc = try_binary_float_fast(ctx, (hipStream_t)stream, op, out, in1, in2);
    if (rc != 0) return rc < 0 ? rc : 0;
    return binary_generic_launch((hipStream_t)stream, op, out, in1, in2, nan_mode);
}

int mlel_hip_mul(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2,
                 uint32_t shift) {
    MLEL_TRY(require_ctx(ctx, "mul"));
    MLEL_TRY(check_supported(out, "mul out"));
    MLEL_TRY(check_supported(in1, "mul in1"));
    MLEL_TRY(check_supported(in2, "mul in2"));
    MLEL_REQUIRE(in1->dtype == in2->dtype, MLEL_ERR_INVALID, "mul: input types differ");
    MLEL_REQUIRE(in1->rank == out->rank && in2->rank == out->rank, MLEL_ERR_INVALID, "mul: ranks differ");
    MLEL_REQUIRE(shift <= 63, MLEL_ERR_INVALID, "mul: shift %u", shift);
    {
        const int rc = try_mul_float_fast(ctx, (hipStream_t)stream, out, in1, in2);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return mul_generic_launch((hipStream_t)stream, out, in1, in2, shift);
}

int mlel_hip_elementwise_unary(mlel_ctx *ctx, void *stream, int32_t op, const mlel_tensor *out,
                               const mlel_tensor *in) {
    MLEL_TRY(require_ctx(ctx, "elementwise_unary"));
    MLEL_REQUIRE(op >= 0 && op < MLEL_UN_COUNT, MLEL_ERR_INVALID, "elementwise_unary: unknown op %d", op);
    MLEL_TRY(check_supported(out, "unary out"));
    MLEL_TRY(check_supported(in, "unary in"));
    MLEL_REQUIRE(in->dtype == out->dtype && in->rank == out->rank, MLEL_ERR_INVALID, "unary: type/rank mismatch");
    {
        const int rc = try_unary_float_fast(ctx, (hipStream_t)stream, op, out, in);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return unary_generic_launch((hipStream_t)stream, op, out, in);
}

int mlel_hip_reduce(mlel_ctx *ctx, void *stream, int32_t op, const mlel_tensor *out, const mlel_tensor *in,
                    uint32_t axis, uint32_t nan_mode) {
    MLEL_TRY(require_ctx(ctx, "reduce"));
    MLEL_REQUIRE(op >= 0 && op < MLEL_RED_COUNT, MLEL_ERR_INVALID, "reduce: unknown op %d", op);
    MLEL_TRY(check_supported(out, "reduce out"));
    MLEL_TRY(check_supported(in, "reduce in"));
    MLEL_REQUIRE(in->dtype == out->dtype && in->rank == out->rank, MLEL_ERR_INVALID, "reduce: type/rank mismatch");
    MLEL_REQUIRE((int)axis < in->rank, MLEL_ERR_INVALID, "reduce: axis %u outside rank %d", axis, in->rank);
    if (!dt_is_float(in->dtype)) nan_mode = MLEL_NAN_PROPAGATE;  // reference: compute_graph_op.cpp:1674-1680
    {
        const int rc = try_reduce_float_fast(ctx, (hipStream_t)stream, op, out, in, axis, nan_mode);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return reduce_generic_launch((hipStream_t)stream, op, out, in, axis, nan_mode);
}

int mlel_hip_avg_pool2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                        const mlel_pool2d_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "avg_pool2d"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "avg_pool2d: null attributes");
    MLEL_TRY(check_supported(out, "avg_pool2d out"));
    MLEL_TRY(check_supported(in, "avg_pool2d in"));
    MLEL_REQUIRE(out->rank == 4 && in->rank == 4 && in->dtype == out->dtype, MLEL_ERR_INVALID,
                 "avg_pool2d: rank 4 tensors of one type");
    MLEL_REQUIRE(attr->acc_type >= 1 && attr->acc_type <= 4, MLEL_ERR_INVALID, "Unsupported AVG_POOL2D acc type %u",
                 attr->acc_type);
    const int rc = try_avgpool_fast(ctx, (hipStream_t)stream, out, in, attr);
    if (rc != 0) return rc < 0 ? rc : 0;
    return pool_generic_launch((hipStream_t)stream, true, out, in, attr);
}

int mlel_hip_max_pool2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                        const mlel_pool2d_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "max_pool2d"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "max_pool2d: null attributes");
    MLEL_TRY(check_supported(out, "max_pool2d out"));
    MLEL_TRY(check_supported(in, "max_pool2d in"));
    MLEL_REQUIRE(out->rank == 4 && in->rank == 4 && in->dtype == out->dtype, MLEL_ERR_INVALID,
                 "max_pool2d: rank 4 tensors of one type");
    const int rc = try_maxpool_fast(ctx, (hipStream_t)stream, out, in, attr);
    if (rc != 0) return rc < 0 ? rc : 0;
    return pool_generic_launch((hipStream_t)stream, false, out, in, attr);
}

int mlel_hip_table(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                   const mlel_tensor *table) {
    MLEL_TRY(require_ctx(ctx, "table"));
    MLEL_TRY(check_tensor(out, "table out"));
    MLEL_TRY(check_tensor(in, "table in"));
    MLEL_TRY(check_tensor(table, "table table"));
    MLEL_REQUIRE(in->dtype == MLEL_I8 || in->dtype == MLEL_I16, MLEL_ERR_UNSUPPORTED, "table: input must be i8 or i16");
    MLEL_REQUIRE(table->dtype == in->dtype && table->rank == 1, MLEL_ERR_INVALID,
                 "table: the table is a rank-1 tensor of the input type");
    MLEL_REQUIRE(out->dtype == (in->dtype == MLEL_I8 ? MLEL_I8 : MLEL_I32) && out->rank == in->rank, MLEL_ERR_INVALID,
                 "table: i8 -> i8 or i16 -> i32");
    const int rc = try_table_fast(ctx, (hipStream_t)stream, out, in, table);
    if (rc != 0) return rc < 0 ? rc : 0;
    return table_generic_launch((hipStream_t)stream, out, in, table);
}

int mlel_hip_cast(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in) {
    MLEL_TRY(require_ctx(ctx, "cast"));
    MLEL_TRY(check_supported(out, "cast out"));
    MLEL_TRY(check_supported(in, "cast in"));
    MLEL_REQUIRE(in->rank == out->rank, MLEL_ERR_INVALID, "cast: ranks differ");
    {
        const int rc = try_cast_float_fast(ctx, (hipStream_t)stream, out, in);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return cast_generic_launch((hipStream_t)stream, out, in);
}

int mlel_hip_negate(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, int32_t input_zp,
                    int32_t output_zp) {
    MLEL_TRY(require_ctx(ctx, "negate"));
    MLEL_TRY(check_supported(out, "negate out"));
    MLEL_TRY(check_supported(in, "negate in"));
    MLEL_REQUIRE(in->dtype == out->dtype && in->rank == out->rank, MLEL_ERR_INVALID, "negate: type/rank mismatch");
    return negate_generic_launch((hipStream_t)stream, out, in, input_zp, output_zp);
}

int mlel_hip_reshape(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in) {
    MLEL_TRY(require_ctx(ctx, "reshape"));
    MLEL_TRY(check_tensor(out, "reshape out"));
    MLEL_TRY(check_tensor(in, "reshape in"));
    MLEL_REQUIRE(dt_size(in->dtype) == dt_size(out->dtype), MLEL_ERR_INVALID, "reshape: element size differs");
    // two packed tensors of the same element count: RESHAPE (reshape.comp:16-27, a flat-index copy) is a plain copy
    if (is_packed(in) && is_packed(out) && numel(in) == numel(out) && ((uintptr_t)in->ptr % 16) == 0 &&
        ((uintptr_t)out->ptr % 16) == 0)
        return mlel_hip_copy_kernel(ctx, stream, out->ptr, in->ptr, (size_t)numel(out) * dt_size(out->dtype));
    return move_generic_launch((hipStream_t)stream, kReshape, out, in, nullptr, 0, 0);
}

int mlel_hip_transpose(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                       const uint32_t *perms) {
    MLEL_TRY(require_ctx(ctx, "transpose"));
    MLEL_TRY(check_tensor(out, "transpose out"));
    MLEL_TRY(check_tensor(in, "transpose in"));
    MLEL_REQUIRE(perms != nullptr && in->rank == out->rank && dt_size(in->dtype) == dt_size(out->dtype),
                 MLEL_ERR_INVALID, "transpose: bad arguments");
    for (int i = 0; i < out->rank; i++)
        MLEL_REQUIRE((int)perms[i] < out->rank, MLEL_ERR_INVALID, "transpose: perms[%d] = %u", i, perms[i]);
    {
        const int rc = try_transpose_fast(ctx, (hipStream_t)stream, out, in, perms);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return move_generic_launch((hipStream_t)stream, kTranspose, out, in, perms, 0, 0);
}

int mlel_hip_concat(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis,
                    uint32_t offset) {
    MLEL_TRY(require_ctx(ctx, "concat"));
    MLEL_TRY(check_tensor(out, "concat out"));
    MLEL_TRY(check_tensor(in, "concat in"));
    MLEL_REQUIRE(in->rank == out->rank && (int)axis < in->rank && dt_size(in->dtype) == dt_size(out->dtype),
                 MLEL_ERR_INVALID, "concat: bad arguments");
    {
        const int rc = try_concat_fast((hipStream_t)stream, out, in, axis, offset);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return move_generic_launch((hipStream_t)stream, kConcat, out, in, nullptr, axis, offset);
}

int mlel_hip_slice(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                   const uint32_t *start) {
    MLEL_TRY(require_ctx(ctx, "slice"));
    MLEL_TRY(check_tensor(out, "slice out"));
    MLEL_TRY(check_tensor(in, "slice in"));
    MLEL_REQUIRE(start != nullptr && in->rank == out->rank && dt_size(in->dtype) == dt_size(out->dtype),
                 MLEL_ERR_INVALID, "slice: bad arguments");
    {
        const int rc = try_slice_fast((hipStream_t)stream, out, in, start);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return move_generic_launch((hipStream_t)stream, kSlice, out, in, start, 0, 0);
}

int mlel_hip_pad(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                 const mlel_tensor *padding, double pad_const, int32_t pad_const_int) {
    MLEL_TRY(require_ctx(ctx, "pad"));
    MLEL_TRY(check_supported(out, "pad out"));
    MLEL_TRY(check_supported(in, "pad in"));
    MLEL_TRY(check_tensor(padding, "pad padding"));
    MLEL_REQUIRE(in->rank == out->rank && in->dtype == out->dtype, MLEL_ERR_INVALID, "pad: type/rank mismatch");
    MLEL_REQUIRE(padding->rank == 1 && padding->dtype == MLEL_I32 && padding->dims[0] >= 2 * in->rank,
                 MLEL_ERR_INVALID, "pad: padding must be int32[2*rank]");
    {
        const int rc = try_pad_fast((hipStream_t)stream, out, in, padding, pad_const, pad_const_int);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return pad_generic_launch((hipStream_t)stream, out, in, padding, pad_const, pad_const_int);
}

// ---- the TOSA operators outside the benchmark graphs (kernels: ops_extra.hip) ----

int mlel_hip_argmax(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis,
                    uint32_t nan_mode) {
    MLEL_TRY(require_ctx(ctx, "argmax"));
    MLEL_TRY(check_supported(out, "argmax out"));
    MLEL_TRY(check_supported(in, "argmax in"));
    MLEL_REQUIRE((int)axis < in->rank && out->rank == in->rank - 1 && out->dtype == MLEL_I32, MLEL_ERR_INVALID,
                 "argmax: the output is int32 with the axis removed");
    return argmax_launch((hipStream_t)stream, out, in, axis, nan_mode);
}

int mlel_hip_arithmetic_right_shift(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in1,
                                    const mlel_tensor *in2, uint32_t round) {
    MLEL_TRY(require_ctx(ctx, "arithmetic_right_shift"));
    MLEL_TRY(check_supported(out, "arithmetic_right_shift out"));
    MLEL_TRY(check_supported(in1, "arithmetic_right_shift in1"));
    MLEL_TRY(check_supported(in2, "arithmetic_right_shift in2"));
    MLEL_REQUIRE(dt_is_int(out->dtype) && in1->dtype == out->dtype && in2->dtype == out->dtype &&
                     in1->rank == out->rank && in2->rank == out->rank,
                 MLEL_ERR_INVALID, "arithmetic_right_shift: one integer type, equal ranks");
    return arshift_launch((hipStream_t)stream, out, in1, in2, round);
}

int mlel_hip_conv3d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                    const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv3d_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "conv3d"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "conv3d: null attribute");
    MLEL_TRY(check_supported(out, "conv3d out"));
    MLEL_TRY(check_supported(in, "conv3d in"));
    MLEL_TRY(check_supported(weights, "conv3d weights"));
    MLEL_TRY(check_supported(bias, "conv3d bias"));
    MLEL_REQUIRE(out->rank == 5 && in->rank == 5 && weights->rank == 5 && bias->rank == 1, MLEL_ERR_INVALID,
                 "conv3d: ranks must be 5,5,5,1");
    MLEL_REQUIRE(attr->acc_type >= MLEL_ACC_I32 && attr->acc_type <= MLEL_ACC_I64, MLEL_ERR_INVALID,
                 "Unsupported acc type %u", attr->acc_type);
    {
        const int r = try_conv3d_as_conv2d(ctx, stream, out, in, weights, bias, attr);
        if (r != 0) return r < 0 ? r : 0;
    }
    return conv3d_launch((hipStream_t)stream, out, in, weights, bias, attr);
}

int mlel_hip_transpose_conv2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                              const mlel_tensor *weights, const mlel_tensor *bias, const mlel_tconv2d_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "transpose_conv2d"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "transpose_conv2d: null attribute");
    MLEL_TRY(check_supported(out, "transpose_conv2d out"));
    MLEL_TRY(check_supported(in, "transpose_conv2d in"));
    MLEL_TRY(check_supported(weights, "transpose_conv2d weights"));
    MLEL_TRY(check_supported(bias, "transpose_conv2d bias"));
    MLEL_REQUIRE(out->rank == 4 && in->rank == 4 && weights->rank == 4 && bias->rank == 1, MLEL_ERR_INVALID,
                 "transpose_conv2d: ranks must be 4,4,4,1");
    MLEL_REQUIRE(attr->stride[0] > 0 && attr->stride[1] > 0, MLEL_ERR_INVALID, "transpose_conv2d: stride must be positive");
    MLEL_REQUIRE(attr->acc_type >= MLEL_ACC_I32 && attr->acc_type <= MLEL_ACC_I64, MLEL_ERR_INVALID,
                 "Unsupported acc type %u", attr->acc_type);
    return tconv2d_launch((hipStream_t)stream, out, in, weights, bias, attr);
}

int mlel_hip_fft2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out_real, const mlel_tensor *out_imag,
                   const mlel_tensor *in_real, const mlel_tensor *in_imag, int32_t inverse) {
    MLEL_TRY(require_ctx(ctx, "fft2d"));
    const mlel_tensor *all[4] = {out_real, out_imag, in_real, in_imag};
    for (const mlel_tensor *t : all) {
        MLEL_TRY(check_supported(t, "fft2d tensor"));
        MLEL_REQUIRE(t->rank == 3 && t->dtype == MLEL_F32, MLEL_ERR_INVALID, "fft2d: float32 tensors of rank 3");
    }
    return fft2d_launch((hipStream_t)stream, out_real, out_imag, in_real, in_imag, inverse != 0);
}

int mlel_hip_rfft2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out_real, const mlel_tensor *out_imag,
                    const mlel_tensor *in) {
    MLEL_TRY(require_ctx(ctx, "rfft2d"));
    const mlel_tensor *all[3] = {out_real, out_imag, in};
    for (const mlel_tensor *t : all) {
        MLEL_TRY(check_supported(t, "rfft2d tensor"));
        MLEL_REQUIRE(t->rank == 3 && t->dtype == MLEL_F32, MLEL_ERR_INVALID, "rfft2d: float32 tensors of rank 3");
    }
    return rfft2d_launch((hipStream_t)stream, out_real, out_imag, in);
}

int mlel_hip_gather(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *values,
                    const mlel_tensor *indices) {
    MLEL_TRY(require_ctx(ctx, "gather"));
    MLEL_TRY(check_tensor(out, "gather out"));
    MLEL_TRY(check_tensor(values, "gather values"));
    MLEL_TRY(check_supported(indices, "gather indices"));
    MLEL_REQUIRE(out->rank == 3 && values->rank == 3 && indices->rank == 2 && dt_is_int(indices->dtype) &&
                     dt_size(out->dtype) == dt_size(values->dtype),
                 MLEL_ERR_INVALID, "gather: [N,W,C] from [N,K,C] with integer indices [N,W]");
    {
        const int rc = try_gather_fast((hipStream_t)stream, out, values, indices);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return gather_launch((hipStream_t)stream, out, values, indices);
}

int mlel_hip_scatter(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *values_in,
                     const mlel_tensor *indices, const mlel_tensor *input) {
    MLEL_TRY(require_ctx(ctx, "scatter"));
    MLEL_TRY(check_tensor(out, "scatter out"));
    MLEL_TRY(check_tensor(values_in, "scatter values_in"));
    MLEL_TRY(check_supported(indices, "scatter indices"));
    MLEL_TRY(check_tensor(input, "scatter input"));
    MLEL_REQUIRE(out->rank == 3 && values_in->rank == 3 && input->rank == 3 && indices->rank == 2 &&
                     dt_is_int(indices->dtype) && dt_size(out->dtype) == dt_size(values_in->dtype) &&
                     dt_size(out->dtype) == dt_size(input->dtype),
                 MLEL_ERR_INVALID, "scatter: [N,K,C] from [N,K,C], integer indices [N,W] and [N,W,C]");
    return scatter_launch((hipStream_t)stream, out, values_in, indices, input);
}

int mlel_hip_resize(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                    const mlel_resize_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "resize"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "resize: null attribute");
    MLEL_TRY(check_supported(out, "resize out"));
    MLEL_TRY(check_supported(in, "resize in"));
    MLEL_REQUIRE(out->rank == 4 && in->rank == 4 && dt_is_float(out->dtype) == dt_is_float(in->dtype), MLEL_ERR_INVALID,
                 "resize: rank 4, integer to integer or float to float");
    MLEL_REQUIRE(attr->scale[0] > 0 && attr->scale[2] > 0, MLEL_ERR_INVALID, "resize: scale numerators must be positive");
    MLEL_REQUIRE(attr->mode == MLEL_RESIZE_NEAREST || attr->mode == MLEL_RESIZE_BILINEAR, MLEL_ERR_INVALID,
                 "resize: mode %u", attr->mode);
    return resize_launch((hipStream_t)stream, out, in, attr);
}

int mlel_hip_reverse(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis) {
    MLEL_TRY(require_ctx(ctx, "reverse"));
    MLEL_TRY(check_tensor(out, "reverse out"));
    MLEL_TRY(check_tensor(in, "reverse in"));
    MLEL_REQUIRE(in->rank == out->rank && (int)axis < out->rank && dt_size(in->dtype) == dt_size(out->dtype),
                 MLEL_ERR_INVALID, "reverse: bad arguments");
    {
        const int rc = try_reverse_fast((hipStream_t)stream, out, in, axis);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return reverse_launch((hipStream_t)stream, out, in, axis);
}

int mlel_hip_tile(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in) {
    MLEL_TRY(require_ctx(ctx, "tile"));
    MLEL_TRY(check_tensor(out, "tile out"));
    MLEL_TRY(check_tensor(in, "tile in"));
    MLEL_REQUIRE(in->rank == out->rank && dt_size(in->dtype) == dt_size(out->dtype), MLEL_ERR_INVALID,
                 "tile: bad arguments");
    {
        const int rc = try_tile_fast((hipStream_t)stream, out, in);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    return tile_launch((hipStream_t)stream, out, in);
}

int mlel_hip_select(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *condition,
                    const mlel_tensor *in_true, const mlel_tensor *in_false) {
    MLEL_TRY(require_ctx(ctx, "select"));
    MLEL_TRY(check_tensor(out, "select out"));
    MLEL_TRY(check_supported(condition, "select condition"));
    MLEL_TRY(check_tensor(in_true, "select in_true"));
    MLEL_TRY(check_tensor(in_false, "select in_false"));
    MLEL_REQUIRE(dt_size(condition->dtype) == 1 && condition->rank == out->rank && in_true->rank == out->rank &&
                     in_false->rank == out->rank && dt_size(in_true->dtype) == dt_size(out->dtype) &&
                     dt_size(in_false->dtype) == dt_size(out->dtype),
                 MLEL_ERR_INVALID, "select: one-byte condition, equal ranks and element sizes");
    return select_launch((hipStream_t)stream, out, condition, in_true, in_false);
}

// ---- fused entry points ----

int mlel_hip_conv2d_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                  const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv2d_attr *attr,
                                  const mlel_epilogue *epi) {
    MLEL_TRY(require_ctx(ctx, "conv2d_rescale_clamp"));
    MLEL_REQUIRE(out != nullptr && attr != nullptr, MLEL_ERR_INVALID, "conv2d_rescale_clamp: null argument");
    MLEL_TRY(check_tensor(out, "conv2d_rescale_clamp out"));
    mlel_tensor acc_view = packed_like(out, MLEL_I32, out->ptr);  // shape carrier for validation
    MLEL_TRY(check_conv("conv2d_rescale_clamp", &acc_view, in, weights, bias, attr));
    FusedEpilogue fe;
    MLEL_TRY(make_epilogue(epi, MLEL_I32, out, out->dims[3], &fe));
    int rc = try_conv2d_i8_direct(ctx, (hipStream_t)stream, out, in, weights, bias, attr, &fe);
    if (rc == 0) rc = try_conv2d_i8_mfma(ctx, (hipStream_t)stream, out, in, weights, bias, attr, &fe);
    if (rc != 0) return rc < 0 ? rc : 0;
    // no specialised kernel for this layout: run the unfused operator sequence through an int32 scratch tensor
    Scratch scratch;
    MLEL_TRY(alloc_fallback(scratch, (size_t)numel(out) * 4 + 16, stream, __func__));
    mlel_tensor acc = packed_like(out, MLEL_I32, scratch.ptr);
    MLEL_TRY(mlel_hip_conv2d(ctx, stream, &acc, in, weights, bias, attr));
    MLEL_TRY(run_unfused_tail(ctx, (hipStream_t)stream, out, &acc, epi));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_conv2d_rescale_clamp_static(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                         const mlel_tensor *weights, const mlel_tensor *bias,
                                         const mlel_conv2d_attr *attr, const mlel_epilogue *epi) {
    MLEL_TRY(require_ctx(ctx, "conv2d_rescale_clamp_static"));
    MLEL_REQUIRE(out != nullptr && attr != nullptr, MLEL_ERR_INVALID, "conv2d_rescale_clamp_static: null argument");
    MLEL_REQUIRE(ctx->static_scratch != nullptr, MLEL_ERR_DEVICE,
                 "conv2d_rescale_clamp_static: the static scratch has no address on device %d", ctx->device);
    MLEL_TRY(check_tensor(out, "conv2d_rescale_clamp_static out"));
    mlel_tensor acc_view = packed_like(out, MLEL_I32, out->ptr);  // shape carrier for validation
    MLEL_TRY(check_conv("conv2d_rescale_clamp_static", &acc_view, in, weights, bias, attr));
    FusedEpilogue fe;
    MLEL_TRY(make_epilogue(epi, MLEL_I32, out, out->dims[3], &fe));
    // the fused kernels; a split-K launch keeps its partial tiles and counters in the static array
    bool used_split = false;
    const GemmScratch gs{ctx->static_scratch,
                         reinterpret_cast<uint32_t *>(ctx->static_scratch + kStaticScratchPartialBytes),
                         kStaticScratchPartialBytes, &used_split};
    int rc = try_conv2d_i8_direct(ctx, (hipStream_t)stream, out, in, weights, bias, attr, &fe);
    if (rc == 0) rc = try_conv2d_i8_mfma(ctx, (hipStream_t)stream, out, in, weights, bias, attr, &fe, nullptr, &gs);
    ctx->static_last_use = used_split ? 1 : 0;
    if (rc != 0) return rc < 0 ? rc : 0;
    // no fused kernel for this layout: the operator sequence, its int32 accumulator staged in the static array
    const size_t need = (size_t)numel(out) * 4;
    MLEL_REQUIRE(need <= kStaticScratchPartialBytes, MLEL_ERR_LIMIT,
                 "conv2d_rescale_clamp_static: no one-pass kernel takes these operands and the int32 accumulator of "
                 "the operator sequence (%zu bytes) exceeds the static scratch (%zu bytes); use "
                 "mlel_hip_conv2d_rescale_clamp, which allocates",
                 need, kStaticScratchPartialBytes);
    mlel_tensor acc = packed_like(out, MLEL_I32, ctx->static_scratch);
    ctx->static_last_use = 2;
    const GemmScratch no_split{nullptr, nullptr, 0, nullptr};  // the array is taken: the contraction must not split K
    rc = try_conv2d_i8_direct(ctx, (hipStream_t)stream, &acc, in, weights, bias, attr, nullptr);
    if (rc == 0) rc = try_conv2d_i8_mfma(ctx, (hipStream_t)stream, &acc, in, weights, bias, attr, nullptr, nullptr, &no_split);
    if (rc < 0) return rc;
    if (rc == 0) MLEL_TRY(conv2d_generic_launch((hipStream_t)stream, &acc, in, weights, bias, attr));
    MLEL_TRY(run_unfused_tail(ctx, (hipStream_t)stream, out, &acc, epi));
    return 0;
}

int mlel_hip_static_scratch_last_use(mlel_ctx *ctx) {
    if (ctx == nullptr) return set_error(MLEL_ERR_INVALID, "static_scratch_last_use: null ctx");
    return ctx->static_last_use;
}

int mlel_hip_conv2d_rescale_add_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                        const mlel_tensor *weights, const mlel_tensor *bias,
                                        const mlel_conv2d_attr *attr, const mlel_epilogue *epi,
                                        const mlel_epilogue *scale_conv, const mlel_tensor *residual,
                                        const mlel_epilogue *scale_residual, const mlel_epilogue *scale_out,
                                        int residual_first) {
    MLEL_TRY(require_ctx(ctx, "conv2d_rescale_add_rescale"));
    MLEL_REQUIRE(out != nullptr && attr != nullptr && epi != nullptr, MLEL_ERR_INVALID,
                 "conv2d_rescale_add_rescale: null argument");
    MLEL_TRY(check_tensor(out, "conv2d_rescale_add_rescale out"));
    MLEL_TRY(check_tensor(residual, "conv2d_rescale_add_rescale residual"));
    MLEL_REQUIRE(same_shape(out, residual), MLEL_ERR_INVALID, "conv2d_rescale_add_rescale: residual shape differs");
    MLEL_REQUIRE(scale_conv && scale_residual && scale_out, MLEL_ERR_INVALID,
                 "conv2d_rescale_add_rescale: null scale");
    MLEL_REQUIRE(!scale_conv->has_clamp && !scale_residual->has_clamp, MLEL_ERR_INVALID,
                 "conv2d_rescale_add_rescale: only the output stage of the addition may carry a clamp");
    // the convolution's own result has the shape and the (8-bit) type of `out`
    MLEL_REQUIRE(dt_size(out->dtype) == 1 && out->dtype != MLEL_BOOL, MLEL_ERR_INVALID,
                 "conv2d_rescale_add_rescale: 8-bit output expected");
    const int conv_dt = out->dtype;
    mlel_tensor acc_view = packed_like(out, MLEL_I32, out->ptr);  // shape carrier for validation
    MLEL_TRY(check_conv("conv2d_rescale_add_rescale", &acc_view, in, weights, bias, attr));
    const int64_t ch = out->dims[3];
    const bool one_pass = out->dtype == MLEL_I8 && residual->dtype == MLEL_I8 && conv_dt == MLEL_I8 &&
                          is_packed(out) && is_packed(residual) && !scale_conv->rescale.per_channel &&
                          !scale_residual->rescale.per_channel && !scale_out->rescale.per_channel;
    if (one_pass) {
        mlel_tensor conv_view = packed_like(out, MLEL_I8, out->ptr);
        ConvResidual cr;
        cr.res = residual;
        FusedEpilogue fe;
        MLEL_TRY(make_epilogue(epi, MLEL_I32, &conv_view, ch, &fe));
        MLEL_TRY(make_epilogue(scale_residual, residual->dtype, &acc_view, ch, &cr.f_res));
        MLEL_TRY(make_epilogue(scale_conv, conv_dt, &acc_view, ch, &cr.f_conv));
        MLEL_TRY(make_epilogue(scale_out, MLEL_I32, out, ch, &cr.f_out));
        // the kernels requantise the sum as an accumulator, which assumes the output stage's input_zp is 0
        if (cr.f_res.in_dt == MLEL_I8 && cr.f_conv.in_dt == MLEL_I8 && cr.f_out.p.in_zp == 0) {
            const int rc = try_conv2d_i8_mfma(ctx, (hipStream_t)stream, out, in, weights, bias, attr, &fe, &cr);
            if (rc != 0) return rc < 0 ? rc : 0;
        }
    }
    // otherwise the two fused halves in sequence through an 8-bit temporary
    Scratch scratch;
    MLEL_TRY(alloc_fallback(scratch, (size_t)numel(out) + 16, stream, __func__));
    mlel_tensor conv_out = packed_like(out, conv_dt, scratch.ptr);
    MLEL_TRY(mlel_hip_conv2d_rescale_clamp(ctx, stream, &conv_out, in, weights, bias, attr, epi));
    if (residual_first)
        MLEL_TRY(mlel_hip_rescale_add_rescale(ctx, stream, out, residual, scale_residual, &conv_out, scale_conv, scale_out));
    else
        MLEL_TRY(mlel_hip_rescale_add_rescale(ctx, stream, out, &conv_out, scale_conv, residual, scale_residual, scale_out));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_matmul_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                            const mlel_tensor *b, const mlel_matmul_attr *attr, const mlel_epilogue *epi) {
    MLEL_TRY(require_ctx(ctx, "matmul_rescale"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "matmul_rescale: null attributes");
    MLEL_TRY(check_tensor(out, "matmul_rescale out"));
    MLEL_TRY(check_supported(a, "matmul_rescale a"));
    MLEL_TRY(check_supported(b, "matmul_rescale b"));
    MLEL_REQUIRE(out->rank == 3 && a->rank == 3 && b->rank == 3, MLEL_ERR_INVALID, "matmul_rescale: rank must be 3");
    MLEL_REQUIRE(a->dtype == b->dtype && dt_is_int(a->dtype), MLEL_ERR_INVALID, "matmul_rescale: integer operands");
    FusedEpilogue fe;
    MLEL_TRY(make_epilogue(epi, MLEL_I32, out, out->dims[2], &fe));
    const int rc = try_matmul_i8_mfma(ctx, (hipStream_t)stream, out, a, b, attr, &fe);
    if (rc != 0) return rc < 0 ? rc : 0;
    Scratch scratch;
    MLEL_TRY(alloc_fallback(scratch, (size_t)numel(out) * 4 + 16, stream, __func__));
    mlel_tensor acc = packed_like(out, MLEL_I32, scratch.ptr);
    MLEL_TRY(mlel_hip_matmul(ctx, stream, &acc, a, b, attr));
    MLEL_TRY(run_unfused_tail(ctx, (hipStream_t)stream, out, &acc, epi));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_elementwise_chain(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_chain *chain) {
    MLEL_TRY(require_ctx(ctx, "elementwise_chain"));
    MLEL_REQUIRE(chain != nullptr, MLEL_ERR_INVALID, "elementwise_chain: null chain");
    MLEL_REQUIRE(chain->n_inputs >= 1 && chain->n_inputs <= MLEL_CHAIN_MAX_INPUTS && chain->n_steps >= 1 &&
                     chain->n_steps <= MLEL_CHAIN_MAX_STEPS,
                 MLEL_ERR_INVALID, "elementwise_chain: %d inputs, %d steps", chain->n_inputs, chain->n_steps);
    MLEL_TRY(check_supported(out, "elementwise_chain out"));
    for (int i = 0; i < chain->n_inputs; i++) MLEL_TRY(check_supported(chain->inputs[i], "elementwise_chain input"));
    bool reduces = false;
    for (int i = 0; i < chain->n_steps; i++) reduces = reduces || chain->steps[i].kind == MLEL_CHAIN_REDUCE;
    const int rc = reduces ? row_chain_launch((hipStream_t)stream, out, chain)
                           : elementwise_chain_launch((hipStream_t)stream, out, chain);
    if (rc != MLEL_ERR_UNSUPPORTED) return rc;
    // the one-pass kernel declined (strides, alignment, too many live values): the operators one after another,
    // every intermediate in a temporary of its own with the broadcast shape of its operands
    std::vector<Scratch> temps(static_cast<size_t>(chain->n_steps));
    std::vector<mlel_tensor> values;
    for (int i = 0; i < chain->n_inputs; i++) values.push_back(*chain->inputs[i]);
    for (int i = 0; i < chain->n_steps; i++) {
        const mlel_chain_step &st = chain->steps[i];
        const int n = static_cast<int>(values.size());
        const bool two = st.kind == MLEL_CHAIN_BINARY || st.kind == MLEL_CHAIN_MUL;
        MLEL_REQUIRE(st.a >= 0 && st.a < n && (!two || (st.b >= 0 && st.b < n)), MLEL_ERR_INVALID,
                     "elementwise_chain: step %d reads a value that does not exist yet", i);
        const mlel_tensor *a = &values[static_cast<size_t>(st.a)], *b = two ? &values[static_cast<size_t>(st.b)] : nullptr;
        mlel_tensor result;
        if (i == chain->n_steps - 1) {
            result = *out;
        } else {
            mlel_tensor shape = *a;
            if (two) {
                MLEL_REQUIRE(a->rank == b->rank, MLEL_ERR_INVALID, "elementwise_chain: step %d: operand ranks differ", i);
                for (int d = 0; d < a->rank; d++) shape.dims[d] = std::max(a->dims[d], b->dims[d]);
            }
            if (st.kind == MLEL_CHAIN_REDUCE) shape.dims[shape.rank - 1] = 1;
            MLEL_TRY(alloc_fallback(temps[static_cast<size_t>(i)], (size_t)numel(&shape) * 4 + 16, stream, __func__));
            result = packed_like(&shape, st.dtype, temps[static_cast<size_t>(i)].ptr);
        }
        switch (st.kind) {
        case MLEL_CHAIN_BINARY:
            MLEL_TRY(mlel_hip_elementwise_binary(ctx, stream, st.selector, &result, a, b, MLEL_NAN_PROPAGATE));
            break;
        case MLEL_CHAIN_MUL: MLEL_TRY(mlel_hip_mul(ctx, stream, &result, a, b, 0)); break;
        case MLEL_CHAIN_UNARY: MLEL_TRY(mlel_hip_elementwise_unary(ctx, stream, st.selector, &result, a)); break;
        case MLEL_CHAIN_CAST: MLEL_TRY(mlel_hip_cast(ctx, stream, &result, a)); break;
        case MLEL_CHAIN_REDUCE:
            MLEL_REQUIRE(a->rank >= 1, MLEL_ERR_INVALID, "elementwise_chain: step %d reduces a rank-0 value", i);
            MLEL_TRY(mlel_hip_reduce(ctx, stream, st.selector, &result, a, (uint32_t)(a->rank - 1), MLEL_NAN_PROPAGATE));
            break;
        default: MLEL_REQUIRE(false, MLEL_ERR_INVALID, "elementwise_chain: step kind %d", st.kind);
        }
        values.push_back(result);
    }
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_softmax_rows(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in) {
    MLEL_TRY(require_ctx(ctx, "softmax_rows"));
    MLEL_TRY(check_supported(out, "softmax_rows out"));
    MLEL_TRY(check_supported(in, "softmax_rows in"));
    MLEL_REQUIRE(in->rank >= 1 && same_shape(out, in) && in->dtype == out->dtype && dt_is_float(in->dtype), MLEL_ERR_INVALID,
                 "softmax_rows: input and output must be floating-point tensors of one shape and type");
    // the six operators as one chain: value 0 is the input, steps produce values 1 .. 6
    mlel_chain c{};
    c.n_inputs = 1;
    c.n_steps = 6;
    c.inputs[0] = in;
    const int dt = in->dtype;
    c.steps[0] = mlel_chain_step{MLEL_CHAIN_REDUCE, MLEL_RED_MAX, 0, 0, dt};
    c.steps[1] = mlel_chain_step{MLEL_CHAIN_BINARY, MLEL_BIN_SUB, 0, 1, dt};
    c.steps[2] = mlel_chain_step{MLEL_CHAIN_UNARY, MLEL_UN_EXP, 2, 0, dt};
    c.steps[3] = mlel_chain_step{MLEL_CHAIN_REDUCE, MLEL_RED_SUM, 3, 0, dt};
    c.steps[4] = mlel_chain_step{MLEL_CHAIN_UNARY, MLEL_UN_RECIPROCAL, 4, 0, dt};
    c.steps[5] = mlel_chain_step{MLEL_CHAIN_MUL, 0, 3, 5, dt};
    return mlel_hip_elementwise_chain(ctx, stream, out, &c);
}

int mlel_hip_matmul_bias_cast(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                              const mlel_tensor *b, const mlel_tensor *bias, const mlel_matmul_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "matmul_bias_cast"));
    MLEL_REQUIRE(attr != nullptr, MLEL_ERR_INVALID, "matmul_bias_cast: null attributes");
    MLEL_TRY(check_supported(out, "matmul_bias_cast out"));
    MLEL_TRY(check_supported(a, "matmul_bias_cast a"));
    MLEL_TRY(check_supported(b, "matmul_bias_cast b"));
    if (bias) MLEL_TRY(check_supported(bias, "matmul_bias_cast bias"));
    MLEL_REQUIRE((out->rank == 3 || out->rank == 6) && a->rank == 3 && b->rank == 3, MLEL_ERR_INVALID,
                 "matmul_bias_cast: operands of rank 3, output of rank 3 or a six-dimensional view");
    MLEL_REQUIRE(a->dtype == MLEL_F16 && b->dtype == MLEL_F16 && out->dtype == MLEL_F16 &&
                     (bias == nullptr || (bias->dtype == MLEL_F32 && bias->rank == 3)),
                 MLEL_ERR_INVALID, "matmul_bias_cast: fp16 operands and output, fp32 bias of rank 3");
    const int rc = try_matmul_f16_mfma(ctx, (hipStream_t)stream, out, a, b, attr, true, bias);
    if (rc != 0) return rc < 0 ? rc : 0;
    if (out->rank == 6) {
        // the view without the fused kernel: the product into a dense temporary, then a strided copy
        Scratch dense_mem;
        MLEL_TRY(alloc_fallback(dense_mem, (size_t)numel(out) * 2 + 16, stream, __func__));
        mlel_tensor dense3 = *out;
        dense3.rank = 3;
        dense3.dims[0] = out->dims[0] * out->dims[1];
        dense3.dims[1] = out->dims[2] * out->dims[3];
        dense3.dims[2] = out->dims[4] * out->dims[5];
        dense3 = packed_like(&dense3, MLEL_F16, dense_mem.ptr);
        MLEL_TRY(mlel_hip_matmul_bias_cast(ctx, stream, &dense3, a, b, bias, attr));
        const mlel_tensor dense6 = packed_like(out, MLEL_F16, dense_mem.ptr);
        MLEL_TRY(mlel_hip_cast(ctx, stream, out, &dense6));
        MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
        return 0;
    }
    // no fused kernel for these strides / alignments: the three operators one after another through temporaries
    Scratch acc_mem, sum_mem;
    MLEL_TRY(alloc_fallback(acc_mem, (size_t)numel(out) * 4 + 16, stream, __func__));
    mlel_tensor acc = packed_like(out, MLEL_F32, acc_mem.ptr);
    MLEL_TRY(mlel_hip_matmul(ctx, stream, &acc, a, b, attr));
    const mlel_tensor *cast_in = &acc;
    mlel_tensor sum{};
    if (bias) {
        MLEL_TRY(alloc_fallback(sum_mem, (size_t)numel(out) * 4 + 16, stream, __func__));
        sum = packed_like(out, MLEL_F32, sum_mem.ptr);
        MLEL_TRY(mlel_hip_elementwise_binary(ctx, stream, MLEL_BIN_ADD, &sum, &acc, bias, MLEL_NAN_PROPAGATE));
        cast_in = &sum;
    }
    MLEL_TRY(mlel_hip_cast(ctx, stream, out, cast_in));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_matmul_bias_cast_chain(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                                    const mlel_tensor *b, const mlel_tensor *bias, const mlel_matmul_attr *attr,
                                    const mlel_chain *chain) {
    MLEL_TRY(require_ctx(ctx, "matmul_bias_cast_chain"));
    MLEL_REQUIRE(attr != nullptr && chain != nullptr && out != nullptr, MLEL_ERR_INVALID, "matmul_bias_cast_chain: null argument");
    MLEL_REQUIRE(chain->n_inputs >= 1 && chain->n_inputs <= MLEL_CHAIN_MAX_INPUTS && chain->n_steps >= 1 &&
                     chain->n_steps <= MLEL_CHAIN_MAX_STEPS,
                 MLEL_ERR_INVALID, "matmul_bias_cast_chain: %d inputs, %d steps", chain->n_inputs, chain->n_steps);
    MLEL_TRY(check_supported(out, "matmul_bias_cast_chain out"));
    MLEL_TRY(check_supported(a, "matmul_bias_cast_chain a"));
    MLEL_TRY(check_supported(b, "matmul_bias_cast_chain b"));
    if (bias) MLEL_TRY(check_supported(bias, "matmul_bias_cast_chain bias"));
    for (int i = 1; i < chain->n_inputs; i++)  // input 0 is the product itself
        MLEL_TRY(check_supported(chain->inputs[i], "matmul_bias_cast_chain chain input"));
    if (out->rank == 3 && out->dtype == MLEL_F16 && a->rank == 3 && b->rank == 3 &&
        a->dtype == MLEL_F16 && b->dtype == MLEL_F16 && (bias == nullptr || (bias->dtype == MLEL_F32 && bias->rank == 3)) &&
        chain_is_gelu_tanh(chain)) {
        const int rc = try_matmul_f16_mfma(ctx, (hipStream_t)stream, out, a, b, attr, true, bias, nullptr, &chain->inputs[1]);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    // the product into a temporary, then the chain over it
    Scratch product_mem;
    MLEL_TRY(alloc_fallback(product_mem, (size_t)numel(out) * 2 + 16, stream, __func__));
    const mlel_tensor product = packed_like(out, MLEL_F16, product_mem.ptr);
    MLEL_TRY(mlel_hip_matmul_bias_cast(ctx, stream, &product, a, b, bias, attr));
    mlel_chain over = *chain;
    over.inputs[0] = &product;
    MLEL_TRY(mlel_hip_elementwise_chain(ctx, stream, out, &over));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_attention_f16(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *q,
                           const mlel_tensor *kt, const mlel_tensor *v, const mlel_chain *softmax) {
    MLEL_TRY(require_ctx(ctx, "attention_f16"));
    MLEL_REQUIRE(softmax != nullptr, MLEL_ERR_INVALID, "attention_f16: null chain");
    MLEL_REQUIRE(softmax->n_inputs >= 1 && softmax->n_inputs <= MLEL_CHAIN_MAX_INPUTS && softmax->n_steps >= 1 &&
                     softmax->n_steps <= MLEL_CHAIN_MAX_STEPS,
                 MLEL_ERR_INVALID, "attention_f16: %d inputs, %d steps", softmax->n_inputs, softmax->n_steps);
    MLEL_TRY(check_supported(out, "attention_f16 out"));
    MLEL_TRY(check_supported(q, "attention_f16 q"));
    MLEL_TRY(check_supported(kt, "attention_f16 kt"));
    MLEL_TRY(check_supported(v, "attention_f16 v"));
    for (int i = 1; i < softmax->n_inputs; i++)  // input 0 is the first product
        MLEL_TRY(check_supported(softmax->inputs[i], "attention_f16 chain input"));
    const int rc = try_attention_f16(ctx, (hipStream_t)stream, out, q, kt, v, softmax);
    if (rc != 0) return rc < 0 ? rc : 0;
    return set_error(MLEL_ERR_UNSUPPORTED,
                     "attention_f16: fp16 heads of 64, M a multiple of 64, 64 <= S <= 512 in multiples of 64, dense "
                     "16-byte aligned rows and the softmax chain only; run the three operators instead");
}

int mlel_hip_attention_f16_in_kernel(const mlel_tensor *out, const mlel_tensor *q, const mlel_tensor *kt,
                                     const mlel_tensor *v, const mlel_chain *softmax) {
    if (out == nullptr || q == nullptr || kt == nullptr || v == nullptr || softmax == nullptr) return 0;
    if (softmax->n_inputs < 1 || softmax->n_inputs > MLEL_CHAIN_MAX_INPUTS || softmax->n_steps < 1 ||
        softmax->n_steps > MLEL_CHAIN_MAX_STEPS)
        return 0;
    for (int i = 1; i < softmax->n_inputs; i++)
        if (softmax->inputs[i] == nullptr) return 0;
    return attention_f16_supported(out, q, kt, v, softmax) ? 1 : 0;
}

int mlel_hip_matmul_chain_in_kernel(const mlel_chain *chain) {
    return chain != nullptr && chain->n_inputs >= 1 && chain->n_inputs <= MLEL_CHAIN_MAX_INPUTS && chain->n_steps >= 1 &&
                   chain->n_steps <= MLEL_CHAIN_MAX_STEPS && chain_is_gelu_tanh(chain)
               ? 1
               : 0;
}

int mlel_hip_matmul_bias_cast_group(mlel_ctx *ctx, void *stream, const mlel_matmul_product *products, int n_products,
                                    const mlel_tensor *a, const mlel_matmul_attr *attr) {
    MLEL_TRY(require_ctx(ctx, "matmul_bias_cast_group"));
    MLEL_REQUIRE(products != nullptr && n_products >= 1 && n_products <= MLEL_MATMUL_GROUP_MAX && attr != nullptr,
                 MLEL_ERR_INVALID, "matmul_bias_cast_group: 1 to %d products", MLEL_MATMUL_GROUP_MAX);
    const mlel_tensor *outs[MLEL_MATMUL_GROUP_MAX], *bs[MLEL_MATMUL_GROUP_MAX], *biases[MLEL_MATMUL_GROUP_MAX];
    MLEL_TRY(check_supported(a, "matmul_bias_cast_group a"));
    bool fusable = a->rank == 3 && a->dtype == MLEL_F16;
    for (int i = 0; i < n_products; i++) {
        outs[i] = products[i].out, bs[i] = products[i].b, biases[i] = products[i].bias;
        MLEL_TRY(check_supported(outs[i], "matmul_bias_cast_group out"));
        MLEL_TRY(check_supported(bs[i], "matmul_bias_cast_group b"));
        if (biases[i]) MLEL_TRY(check_supported(biases[i], "matmul_bias_cast_group bias"));
        fusable = fusable && bs[i]->rank == 3 && bs[i]->dtype == MLEL_F16 && outs[i]->dtype == MLEL_F16 &&
                  (outs[i]->rank == 3 || outs[i]->rank == 6) &&
                  (biases[i] == nullptr || (biases[i]->dtype == MLEL_F32 && biases[i]->rank == 3));
    }
    if (fusable && n_products > 1) {
        const int rc = try_matmul_f16_group(ctx, (hipStream_t)stream, n_products, outs, a, bs, biases, attr);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    for (int i = 0; i < n_products; i++) MLEL_TRY(mlel_hip_matmul_bias_cast(ctx, stream, outs[i], a, bs[i], biases[i], attr));
    return 0;
}

int mlel_hip_matmul_bias_cast_add(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                                  const mlel_tensor *b, const mlel_tensor *bias, const mlel_matmul_attr *attr,
                                  const mlel_tensor *residual) {
    MLEL_TRY(require_ctx(ctx, "matmul_bias_cast_add"));
    MLEL_REQUIRE(attr != nullptr && residual != nullptr, MLEL_ERR_INVALID, "matmul_bias_cast_add: null argument");
    MLEL_TRY(check_supported(out, "matmul_bias_cast_add out"));
    MLEL_TRY(check_supported(residual, "matmul_bias_cast_add residual"));
    MLEL_TRY(check_supported(a, "matmul_bias_cast_add a"));
    MLEL_TRY(check_supported(b, "matmul_bias_cast_add b"));
    if (bias) MLEL_TRY(check_supported(bias, "matmul_bias_cast_add bias"));
    MLEL_REQUIRE(out->rank == 3 && residual->dtype == MLEL_F16 && out->dtype == MLEL_F16 && same_shape(out, residual),
                 MLEL_ERR_INVALID, "matmul_bias_cast_add: the residual is an fp16 tensor of the output's shape");
    if (a->dtype == MLEL_F16 && b->dtype == MLEL_F16 && a->rank == 3 && b->rank == 3 &&
        (bias == nullptr || (bias->dtype == MLEL_F32 && bias->rank == 3))) {
        const int rc = try_matmul_f16_mfma(ctx, (hipStream_t)stream, out, a, b, attr, true, bias, residual);
        if (rc != 0) return rc < 0 ? rc : 0;
    }
    // no fused kernel for these strides / alignments: the projection into a temporary, then the addition
    Scratch proj_mem;
    MLEL_TRY(alloc_fallback(proj_mem, (size_t)numel(out) * 2 + 16, stream, __func__));
    const mlel_tensor proj = packed_like(out, MLEL_F16, proj_mem.ptr);
    MLEL_TRY(mlel_hip_matmul_bias_cast(ctx, stream, &proj, a, b, bias, attr));
    MLEL_TRY(mlel_hip_elementwise_binary(ctx, stream, MLEL_BIN_ADD, out, &proj, residual, MLEL_NAN_PROPAGATE));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_dwconv_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                  const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv2d_attr *attr,
                                  const mlel_epilogue *epi) {
    MLEL_TRY(require_ctx(ctx, "dwconv_rescale_clamp"));
    MLEL_REQUIRE(out != nullptr && attr != nullptr, MLEL_ERR_INVALID, "dwconv_rescale_clamp: null argument");
    MLEL_TRY(check_tensor(out, "dwconv_rescale_clamp out"));
    mlel_tensor acc_view = packed_like(out, MLEL_I32, out->ptr);
    MLEL_TRY(check_conv("dwconv_rescale_clamp", &acc_view, in, weights, bias, attr));
    MLEL_REQUIRE(weights->dims[3] > 0, MLEL_ERR_INVALID, "dwconv_rescale_clamp: channel multiplier must be > 0");
    FusedEpilogue fe;
    MLEL_TRY(make_epilogue(epi, MLEL_I32, out, out->dims[3], &fe));
    const int rc = try_dwconv_i8_fast(ctx, (hipStream_t)stream, out, in, weights, bias, attr, &fe);
    if (rc != 0) return rc < 0 ? rc : 0;
    Scratch scratch;
    MLEL_TRY(alloc_fallback(scratch, (size_t)numel(out) * 4 + 16, stream, __func__));
    mlel_tensor acc = packed_like(out, MLEL_I32, scratch.ptr);
    MLEL_TRY(mlel_hip_depthwise_conv2d(ctx, stream, &acc, in, weights, bias, attr));
    MLEL_TRY(run_unfused_tail(ctx, (hipStream_t)stream, out, &acc, epi));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

namespace {
// the intermediate tensor [N, H, W, C] of the fused pair, as the first operator would have written it (no memory)
int conv_dw_prepare(const char *name, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w1,
                    const mlel_tensor *b1, const mlel_conv2d_attr *a1, const mlel_epilogue *e1, const mlel_tensor *w2,
                    const mlel_tensor *b2, const mlel_conv2d_attr *a2, const mlel_epilogue *e2, FusedEpilogue *f1,
                    FusedEpilogue *f2) {
    MLEL_REQUIRE(out != nullptr && in != nullptr && w1 != nullptr && b1 != nullptr && a1 != nullptr && e1 != nullptr &&
                     w2 != nullptr && b2 != nullptr && a2 != nullptr && e2 != nullptr,
                 MLEL_ERR_INVALID, "%s: null argument", name);
    MLEL_TRY(check_tensor(out, name));
    MLEL_TRY(check_tensor(in, name));
    MLEL_TRY(check_tensor(w1, name));
    MLEL_REQUIRE(in->rank == 4 && w1->rank == 4 && out->rank == 4, MLEL_ERR_INVALID, "%s: rank-4 tensors expected", name);
    mlel_tensor mid{};
    mid.dtype = MLEL_I8;
    mid.rank = 4;
    mid.dims[0] = in->dims[0], mid.dims[1] = in->dims[1], mid.dims[2] = in->dims[2], mid.dims[3] = w1->dims[0];
    mid.strides[3] = 1;
    for (int i = 2; i >= 0; i--) mid.strides[i] = mid.strides[i + 1] * mid.dims[i + 1];
    mid.ptr = out->ptr;  // shape carrier for validation only
    mlel_tensor acc1 = packed_like(&mid, MLEL_I32, out->ptr);
    MLEL_TRY(check_conv(name, &acc1, in, w1, b1, a1));
    mlel_tensor acc2 = packed_like(out, MLEL_I32, out->ptr);
    MLEL_TRY(check_conv(name, &acc2, &mid, w2, b2, a2));
    MLEL_TRY(make_epilogue(e1, MLEL_I32, &mid, mid.dims[3], f1));
    MLEL_TRY(make_epilogue(e2, MLEL_I32, out, out->dims[3], f2));
    return 0;
}
}  // namespace

int mlel_hip_conv2d_dwconv_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                         const mlel_tensor *w1, const mlel_tensor *b1, const mlel_conv2d_attr *a1,
                                         const mlel_epilogue *e1, const mlel_tensor *w2, const mlel_tensor *b2,
                                         const mlel_conv2d_attr *a2, const mlel_epilogue *e2) {
    MLEL_TRY(require_ctx(ctx, "conv2d_dwconv_rescale_clamp"));
    FusedEpilogue f1, f2;
    MLEL_TRY(conv_dw_prepare("conv2d_dwconv_rescale_clamp", out, in, w1, b1, a1, e1, w2, b2, a2, e2, &f1, &f2));
    const int rc = try_conv2d_dwconv_i8(ctx, (hipStream_t)stream, out, in, w1, b1, a1, &f1, w2, b2, a2, &f2, true);
    if (rc != 0) return rc < 0 ? rc : 0;
    return set_error(MLEL_ERR_UNSUPPORTED,
                     "conv2d_dwconv_rescale_clamp: int8, 1x1 unit-stride convolution of 32..160 input channels (a "
                     "multiple of 32) to a multiple of 32 channels, 3x3 depthwise of stride 1 or 2, images of at most "
                     "32 x 32 positions, zero weight zero points, dense 16-byte aligned operands only; run the two "
                     "operators instead");
}

int mlel_hip_conv2d_dwconv_in_kernel(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w1,
                                     const mlel_tensor *b1, const mlel_conv2d_attr *a1, const mlel_tensor *w2,
                                     const mlel_tensor *b2, const mlel_conv2d_attr *a2) {
    if (out == nullptr || in == nullptr || w1 == nullptr || b1 == nullptr || a1 == nullptr || w2 == nullptr ||
        b2 == nullptr || a2 == nullptr)
        return 0;
    const FusedEpilogue unused{};  // the requantisation constants do not decide whether the kernel takes the case
    return try_conv2d_dwconv_i8(nullptr, nullptr, out, in, w1, b1, a1, &unused, w2, b2, a2, &unused, false) == 1 ? 1 : 0;
}

int mlel_hip_conv2d_conv2d_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *mid,
                                         const mlel_tensor *in, const mlel_tensor *w1, const mlel_tensor *b1,
                                         const mlel_conv2d_attr *a1, const mlel_epilogue *e1, const mlel_tensor *w2,
                                         const mlel_tensor *b2, const mlel_conv2d_attr *a2, const mlel_epilogue *e2) {
    MLEL_TRY(require_ctx(ctx, "conv2d_conv2d_rescale_clamp"));
    FusedEpilogue f1, f2;
    MLEL_TRY(conv_dw_prepare("conv2d_conv2d_rescale_clamp", out, in, w1, b1, a1, e1, w2, b2, a2, e2, &f1, &f2));
    if (mid != nullptr) {
        MLEL_TRY(check_tensor(mid, "conv2d_conv2d_rescale_clamp mid"));
        MLEL_REQUIRE(mid->rank == 4 && mid->dims[0] == in->dims[0] && mid->dims[1] == in->dims[1] &&
                         mid->dims[2] == in->dims[2] && mid->dims[3] == w1->dims[0] && dt_size(mid->dtype) == 1,
                     MLEL_ERR_INVALID, "conv2d_conv2d_rescale_clamp: the intermediate tensor is 8-bit [N, H, W, OC1]");
    }
    const int mid_dt = mid != nullptr ? mid->dtype : MLEL_I8;
    const int rc = try_conv2d_pair_rows(ctx, (hipStream_t)stream, out, mid, in, w1, b1, a1, &f1, mid_dt, w2, b2, a2, &f2, false);
    if (rc != 0) return rc < 0 ? rc : 0;
    // no one-pass kernel for these operands: the two fused operators one after the other, through the caller's
    // intermediate tensor or a temporary
    if (mid != nullptr) {
        MLEL_TRY(mlel_hip_conv2d_rescale_clamp(ctx, stream, mid, in, w1, b1, a1, e1));
        return mlel_hip_conv2d_rescale_clamp(ctx, stream, out, mid, w2, b2, a2, e2);
    }
    Scratch scratch;
    const size_t bytes = (size_t)(in->dims[0] * in->dims[1] * in->dims[2] * w1->dims[0]);
    MLEL_TRY(alloc_fallback(scratch, bytes + 16, stream, __func__));
    mlel_tensor tmp{};
    tmp.dtype = MLEL_I8;
    tmp.rank = 4;
    tmp.dims[0] = in->dims[0], tmp.dims[1] = in->dims[1], tmp.dims[2] = in->dims[2], tmp.dims[3] = w1->dims[0];
    tmp.strides[3] = 1;
    for (int i = 2; i >= 0; i--) tmp.strides[i] = tmp.strides[i + 1] * tmp.dims[i + 1];
    tmp.ptr = scratch.ptr;
    MLEL_TRY(mlel_hip_conv2d_rescale_clamp(ctx, stream, &tmp, in, w1, b1, a1, e1));
    MLEL_TRY(mlel_hip_conv2d_rescale_clamp(ctx, stream, out, &tmp, w2, b2, a2, e2));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_conv2d_conv2d_in_kernel(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w1,
                                     const mlel_tensor *b1, const mlel_conv2d_attr *a1, const mlel_tensor *w2,
                                     const mlel_tensor *b2, const mlel_conv2d_attr *a2) {
    if (out == nullptr || in == nullptr || w1 == nullptr || b1 == nullptr || a1 == nullptr || w2 == nullptr ||
        b2 == nullptr || a2 == nullptr)
        return 0;
    const FusedEpilogue unused{};  // the requantisation constants do not decide whether the kernel takes the case
    return try_conv2d_pair_rows(nullptr, nullptr, out, nullptr, in, w1, b1, a1, &unused, MLEL_I8, w2, b2, a2, &unused, true) == 1 ? 1 : 0;
}

namespace {
// the convolution's result as a dense tensor of `dtype` at `ptr`: [N, OH, OW, OC] from the operands and attributes
bool conv_result_like(mlel_tensor *t, const mlel_tensor *in, const mlel_tensor *w, const mlel_conv2d_attr *a, int dtype,
                      void *ptr) {
    if (in == nullptr || w == nullptr || a == nullptr || in->rank != 4 || w->rank != 4) return false;
    if (a->stride[0] <= 0 || a->stride[1] <= 0 || a->dilation[0] <= 0 || a->dilation[1] <= 0) return false;
    const int64_t eh = (w->dims[1] - 1) * a->dilation[0] + 1, ew = (w->dims[2] - 1) * a->dilation[1] + 1;
    const int64_t ih = in->dims[1] + a->pad[0] + a->pad[1], iw = in->dims[2] + a->pad[2] + a->pad[3];
    if (ih < eh || iw < ew) return false;
    *t = mlel_tensor{};
    t->dtype = dtype, t->rank = 4, t->ptr = ptr;
    t->dims[0] = in->dims[0], t->dims[1] = (ih - eh) / a->stride[0] + 1, t->dims[2] = (iw - ew) / a->stride[1] + 1;
    t->dims[3] = w->dims[0];
    int64_t st = dt_size(dtype);
    for (int i = 3; i >= 0; i--) t->strides[i] = st, st *= t->dims[i];
    return true;
}
}  // namespace

int mlel_hip_conv2d_rescale_clamp_avgpool(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                          const mlel_tensor *weights, const mlel_tensor *bias,
                                          const mlel_conv2d_attr *attr, const mlel_epilogue *epi, int32_t conv_dtype,
                                          const mlel_pool2d_attr *pool) {
    MLEL_TRY(require_ctx(ctx, "conv2d_rescale_clamp_avgpool"));
    MLEL_REQUIRE(out != nullptr && attr != nullptr && pool != nullptr && epi != nullptr, MLEL_ERR_INVALID,
                 "conv2d_rescale_clamp_avgpool: null argument");
    MLEL_TRY(check_tensor(out, "conv2d_rescale_clamp_avgpool out"));
    mlel_tensor mid;
    // (the pooled tensor's pointer stands in where validation wants one: the convolution's result has no memory here)
    MLEL_REQUIRE(conv_result_like(&mid, in, weights, attr, conv_dtype, out->ptr), MLEL_ERR_INVALID,
                 "conv2d_rescale_clamp_avgpool: operands do not describe a convolution");
    MLEL_REQUIRE(dt_is_int(conv_dtype) && dt_size(conv_dtype) <= 4 && conv_dtype == out->dtype, MLEL_ERR_INVALID,
                 "conv2d_rescale_clamp_avgpool: the convolution's result and the pooled tensor have one integer type");
    mlel_tensor acc_view = packed_like(&mid, MLEL_I32, out->ptr);  // shape carrier for validation
    MLEL_TRY(check_conv("conv2d_rescale_clamp_avgpool", &acc_view, in, weights, bias, attr));
    FusedEpilogue fe;
    MLEL_TRY(make_epilogue(epi, MLEL_I32, &mid, mid.dims[3], &fe));
    const int rc = try_conv2d_avgpool_cols((hipStream_t)stream, out, &mid, in, weights, bias, attr, &fe, pool, false);
    if (rc != 0) return rc < 0 ? rc : 0;
    // no one-pass kernel for these operands: the fused convolution into a temporary, then the pooling
    Scratch scratch;
    MLEL_TRY(alloc_fallback(scratch, (size_t)numel(&mid) * dt_size(conv_dtype) + 16, stream, __func__));
    mid.ptr = scratch.ptr;
    MLEL_TRY(mlel_hip_conv2d_rescale_clamp(ctx, stream, &mid, in, weights, bias, attr, epi));
    MLEL_TRY(mlel_hip_avg_pool2d(ctx, stream, out, &mid, pool));
    MLEL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int mlel_hip_conv2d_avgpool_in_kernel(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *weights,
                                      const mlel_tensor *bias, const mlel_conv2d_attr *attr, int32_t conv_dtype,
                                      const mlel_pool2d_attr *pool) {
    if (out == nullptr || in == nullptr || weights == nullptr || bias == nullptr || attr == nullptr || pool == nullptr) return 0;
    mlel_tensor mid;
    if (!conv_result_like(&mid, in, weights, attr, conv_dtype, nullptr)) return 0;
    const FusedEpilogue unused{};  // the requantisation constants do not decide whether the kernel takes the case
    return try_conv2d_avgpool_cols(nullptr, out, &mid, in, weights, bias, attr, &unused, pool, true) == 1 ? 1 : 0;
}

int mlel_hip_rescale_add_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in1,
                                 const mlel_epilogue *scale1, const mlel_tensor *in2, const mlel_epilogue *scale2,
                                 const mlel_epilogue *scale_out) {
    MLEL_TRY(require_ctx(ctx, "rescale_add_rescale"));
    MLEL_TRY(check_tensor(out, "rescale_add_rescale out"));
    MLEL_TRY(check_tensor(in1, "rescale_add_rescale in1"));
    MLEL_TRY(check_tensor(in2, "rescale_add_rescale in2"));
    MLEL_REQUIRE(same_shape(out, in1) && same_shape(out, in2), MLEL_ERR_INVALID,
                 "rescale_add_rescale: shapes differ (no broadcast in the fused form)");
    MLEL_REQUIRE(scale1 && scale2 && scale_out, MLEL_ERR_INVALID, "rescale_add_rescale: null scale");
    MLEL_REQUIRE(!scale1->has_clamp && !scale2->has_clamp, MLEL_ERR_INVALID,
                 "rescale_add_rescale: only the output stage may carry a clamp");
    const int64_t ch = out->dims[out->rank - 1];
    // the two input stages produce int32; build their parameters against a virtual int32 tensor
    mlel_tensor mid = packed_like(out, MLEL_I32, out->ptr);
    FusedEpilogue f1, f2, fo;
    MLEL_TRY(make_epilogue(scale1, in1->dtype, &mid, ch, &f1));
    MLEL_TRY(make_epilogue(scale2, in2->dtype, &mid, ch, &f2));
    MLEL_TRY(make_epilogue(scale_out, MLEL_I32, out, ch, &fo));
    return rescale_add_rescale_launch(ctx, (hipStream_t)stream, out, in1, f1, in2, f2, fo);
}

}  // extern "C"
