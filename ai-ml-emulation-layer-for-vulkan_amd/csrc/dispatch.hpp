// Internal launch functions behind the C ABI: the generic one-thread-per-element path and the specialised
// gfx950 kernels.  The `try_*` functions return 1 when they took the case, 0 when the caller must fall through to
// the generic path, and a negative mlel_status on error.
#pragma once

#include "common.hpp"

namespace mlel {

enum MoveKind { kReshape = 0, kTranspose = 1, kConcat = 2, kSlice = 3 };

// ---- generic path (ops_generic.hip) ----
int conv2d_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                          const mlel_tensor *bias, const mlel_conv2d_attr *a);
int dwconv_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                          const mlel_tensor *bias, const mlel_conv2d_attr *a);
int matmul_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *a, const mlel_tensor *b,
                          const mlel_matmul_attr *attr);
int rescale_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *mult,
                           const mlel_tensor *shift, const mlel_rescale_attr *attr, const RescaleParams &p);
int clamp_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_clamp_attr *a);
int binary_generic_launch(hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in1,
                          const mlel_tensor *in2, uint32_t nan_mode);
int mul_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2,
                       uint32_t shift);
int unary_generic_launch(hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in);
int reduce_generic_launch(hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis,
                          uint32_t nan_mode);
int pool_generic_launch(hipStream_t s, bool avg, const mlel_tensor *out, const mlel_tensor *in,
                        const mlel_pool2d_attr *a);
int table_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *table);
int cast_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in);
int negate_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, int32_t zi, int32_t zo);
int move_generic_launch(hipStream_t s, int kind, const mlel_tensor *out, const mlel_tensor *in, const uint32_t *v,
                        uint32_t axis, uint32_t offset);
int pad_generic_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *padding,
                       double pad_const, int32_t pad_const_int);

int elementwise_chain_launch(hipStream_t s, const mlel_tensor *out, const mlel_chain *chain);
// the same for a chain with reductions over the last axis in it (fp16)
int row_chain_launch(hipStream_t s, const mlel_tensor *out, const mlel_chain *chain);

// ops_extra.hip: the TOSA operators outside the benchmark graphs
int conv3d_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                  const mlel_tensor *bias, const mlel_conv3d_attr *a);
int tconv2d_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                   const mlel_tensor *bias, const mlel_tconv2d_attr *a);
int argmax_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t nan_mode);
int arshift_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2, uint32_t round);
int gather_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *values, const mlel_tensor *indices);
int scatter_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *values_in, const mlel_tensor *indices,
                   const mlel_tensor *input);
int reverse_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis);
int tile_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in);
int select_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *cond, const mlel_tensor *a,
                  const mlel_tensor *b);
int resize_launch(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_resize_attr *a);
int fft2d_launch(hipStream_t s, const mlel_tensor *out_r, const mlel_tensor *out_i, const mlel_tensor *in_r,
                 const mlel_tensor *in_i, bool inverse);
int rfft2d_launch(hipStream_t s, const mlel_tensor *out_r, const mlel_tensor *out_i, const mlel_tensor *in);

// ---- int8 MFMA contractions (gemm_i8.hip) ----
// Optional fused epilogue: when `epi` is non-null the int32 accumulator is requantised (RESCALE [+CLAMP]) and
// stored as int8/int16/int32 `out`; otherwise the int32 accumulator (plus bias) is stored.
struct FusedEpilogue {
    const mlel_tensor *mult;
    const mlel_tensor *shift;
    RescaleParams p;
    bool scale32;
    int in_dt;  // input storage type viewed through input_unsigned
};
// The same, as a kernel argument: raw pointers to the multiplier (int32 or int16) and shift (int8) arrays.
struct ScaleRef {
    const char *mult;
    const int8_t *shift;
    int32_t mult16;
    RescaleParams p;
};
inline ScaleRef make_ref(const FusedEpilogue &f) {
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

// residual stage fused behind an int8 convolution: out = rescale_out(rescale_res(res) + rescale_conv(conv result))
struct ConvResidual {
    const mlel_tensor *res;
    FusedEpilogue f_res, f_conv, f_out;
};
// `static_scratch`: where a split-K launch keeps its partial tiles and counters instead of the context's per-stream
// workspace (the counters must be zero); `used_split` reports whether the launch split K
struct GemmScratch {
    char *partials;
    uint32_t *counters;
    size_t partial_bytes;
    bool *used_split;
};
int try_conv2d_i8_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                       const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                       const FusedEpilogue *epi, const ConvResidual *residual = nullptr,
                       const GemmScratch *static_scratch = nullptr);
// ---- direct (dot4) convolution for very small input channel counts (conv_direct.hip) ----
int try_conv2d_i8_direct(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                         const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                         const FusedEpilogue *epi);
int try_matmul_i8_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *a,
                       const mlel_tensor *b, const mlel_matmul_attr *attr, const FusedEpilogue *epi);

// ---- fp16 MFMA MATMUL with fp32 result (gemm_f16.hip) ----
// `residual`: an fp16 tensor of the output's shape added to the fused form's fp16 result (a second, fp16 ADD)
int try_matmul_f16_mfma(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *a,
                        const mlel_tensor *b, const mlel_matmul_attr *attr, bool bias_cast = false,
                        const mlel_tensor *bias = nullptr, const mlel_tensor *residual = nullptr,
                        const mlel_tensor *const *gelu_inputs = nullptr);
// `gelu_inputs`: the four single-element fp16 inputs of the tanh form of GELU (see chain_is_gelu_tanh), applied to
// the fused form's rounded result
// The chain is the tanh form of GELU over its value 0, as the graph's region builder emits it: inputs 1 .. 4 are
// single fp16 elements, nine steps (ops_float.hip).
bool chain_is_gelu_tanh(const mlel_chain *chain);

// two or three fused products (fp16 out = CAST(MATMUL + bias)) of one A in a single launch
int try_matmul_f16_group(mlel_ctx *ctx, hipStream_t s, int n, const mlel_tensor *const *outs, const mlel_tensor *a,
                         const mlel_tensor *const *bs, const mlel_tensor *const *biases, const mlel_matmul_attr *attr);

// ---- 1x1 CONV2D + RESCALE (+CLAMP) and 3x3 DEPTHWISE_CONV2D + RESCALE (+CLAMP) in one launch (conv_dw_i8.hip) ----
// 1 when taken (with `launch` false: when the extents, types and strides are covered; pointers are not looked at)
int try_conv2d_dwconv_i8(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                         const mlel_tensor *w1, const mlel_tensor *b1, const mlel_conv2d_attr *a1,
                         const FusedEpilogue *e1, const mlel_tensor *w2, const mlel_tensor *b2,
                         const mlel_conv2d_attr *a2, const FusedEpilogue *e2, bool launch);

// ---- scores, softmax and the product with V of fp16 attention heads in one launch (attention_f16.hip) ----
bool attention_f16_supported(const mlel_tensor *out, const mlel_tensor *q, const mlel_tensor *kt, const mlel_tensor *v,
                             const mlel_chain *chain);
int try_attention_f16(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *q, const mlel_tensor *kt,
                      const mlel_tensor *v, const mlel_chain *chain);

// ---- floating-point elementwise / reduce specialisations (ops_float.hip) ----
int try_binary_float_fast(mlel_ctx *ctx, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in1,
                          const mlel_tensor *in2);
int try_mul_float_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1,
                       const mlel_tensor *in2);
int try_unary_float_fast(mlel_ctx *ctx, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in);
int try_cast_float_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in);
int try_reduce_float_fast(mlel_ctx *ctx, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in,
                          uint32_t axis, uint32_t nan_mode);

// ---- bandwidth-bound specialisations (ops_fast.hip) ----
int try_dwconv_i8_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                       const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                       const FusedEpilogue *epi);
int try_rescale_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                     const mlel_tensor *mult, const mlel_tensor *shift, const mlel_rescale_attr *attr,
                     const RescaleParams &p);
int try_clamp_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                   const mlel_clamp_attr *a);
int try_binary_fast(mlel_ctx *ctx, hipStream_t s, int op, const mlel_tensor *out, const mlel_tensor *in1,
                    const mlel_tensor *in2);
int try_avgpool_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                     const mlel_pool2d_attr *a);
// ops_vec.hip: packed integer tensors, 128 bits per thread
int try_maxpool_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                     const mlel_pool2d_attr *a);
int try_table_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                   const mlel_tensor *table);
int try_transpose_fast(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in,
                       const uint32_t *perms);
int rescale_add_rescale_launch(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *in1,
                               const FusedEpilogue &s1, const mlel_tensor *in2, const FusedEpilogue &s2,
                               const FusedEpilogue &so);

// ---- two 1x1 CONV2D + RESCALE (+CLAMP) in a row, one launch (conv_direct.hip); `probe`: judge only ----
int try_conv2d_pair_rows(mlel_ctx *ctx, hipStream_t s, const mlel_tensor *out, const mlel_tensor *mid,
                         const mlel_tensor *in, const mlel_tensor *w1, const mlel_tensor *b1, const mlel_conv2d_attr *a1,
                         const FusedEpilogue *e1, int mid_dtype, const mlel_tensor *w2, const mlel_tensor *b2,
                         const mlel_conv2d_attr *a2, const FusedEpilogue *e2, bool probe);
// 1x1 CONV2D + RESCALE (+CLAMP) + global AVG_POOL2D in one launch (gemm_i8.hip / gemm_i8_cols.hip); `conv_out` is a
// shape and type carrier
int try_conv2d_avgpool_cols(hipStream_t s, const mlel_tensor *pool_out, const mlel_tensor *conv_out, const mlel_tensor *in,
                            const mlel_tensor *w, const mlel_tensor *bias, const mlel_conv2d_attr *a,
                            const FusedEpilogue *epi, const mlel_pool2d_attr *pool, bool probe);
// ---- data movement in whole pieces on packed tensors (ops_move.hip); each returns 1 when launched, 0 to decline ----
int try_slice_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const uint32_t *start);
int try_concat_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t offset);
int try_pad_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *padding,
                 double pad_const, int32_t pad_const_int);
int try_tile_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in);
int try_reverse_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis);
int try_gather_fast(hipStream_t s, const mlel_tensor *out, const mlel_tensor *values, const mlel_tensor *indices);
// CONV3D as CONV2D (ops_move.hip): the depth taps side by side along the channels of x2, the weights regrouped to match
int launch_conv3d_regroup(hipStream_t s, void *x2, void *w2, const mlel_tensor *in, const mlel_tensor *w, int64_t OD,
                          const mlel_conv3d_attr *a);

}  // namespace mlel
