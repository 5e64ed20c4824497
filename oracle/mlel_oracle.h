/*
 * mlel_oracle.h -- CPU restatement of the reference's TOSA operator shaders.  TEST INFRASTRUCTURE ONLY.
 *
 * Only the tests, the smoke check and the benchmark's CPU-baseline leg may link or call this library; it is
 * never part of the product path (the HIP backend fails loudly instead of falling back to it).
 *
 * Every function takes the same tensor views and attribute structs as the HIP C ABI (include/mlel_hip.h), with
 * host pointers, and follows the arithmetic of one reference shader:
 *
 *   mlel_cpu_conv2d            graph/shaders/graph_op/tosa/conv2d.comp:40-116
 *   mlel_cpu_depthwise_conv2d  .../depthwise_conv2d.comp:31-78
 *   mlel_cpu_matmul            .../matmul.comp:30-73
 *   mlel_cpu_rescale           .../rescale.comp:27-72
 *   mlel_cpu_clamp             .../clamp.comp:24-53
 *   mlel_cpu_elementwise_binary.../elementwise_binary.comp:146-173 (+ operation strings,
 *                              graph/compute_graph_op.cpp:2527-2946)
 *   mlel_cpu_mul               .../mul.comp:24-59
 *   mlel_cpu_elementwise_unary .../elementwise_unary.comp:136-205
 *   mlel_cpu_reduce            .../reduce.comp:24-70 (+ init strings graph/compute_graph_op.cpp:2819-2859)
 *   mlel_cpu_avg_pool2d        .../avgpool2d.comp:27-75
 *   mlel_cpu_max_pool2d        .../maxpool2d.comp:23-72
 *   mlel_cpu_table             .../table.comp:17-52
 *   mlel_cpu_cast              .../cast.comp:22-103
 *   mlel_cpu_negate            .../negate.comp:29-47
 *   mlel_cpu_reshape/transpose/concat/slice/pad   the shaders of the same names
 *   index helpers              graph/shaders/graph_op/common.comp:64-182, tensor/shaders/tensor.glsl:26-86
 *
 * Parity status.  Integer paths are closed-form and pinned by the reference's known-answer tests (CONV2D,
 * MAX_POOL2D, RESCALE+ADD, CAST, CONCAT, SLICE, MAXIMUM, RESHAPE) plus brute-force / library cross-checks in
 * tests/ (MATMUL, DEPTHWISE_CONV2D, AVG_POOL2D, TABLE, CLAMP, MUL, SUB, REDUCE, TRANSPOSE, PAD: no reference test
 * exists; they are pinned against numpy int64 restatements of the TOSA formulae and hand-computed cases).
 * The floating-point unary operators (EXP, LOG, COS, SIGMOID, RECIPROCAL, RSQRT, CEIL, FLOOR, ERF, TANH with its
 * three branches, SIN), the remaining binary operators (BITWISE_*, LOGICAL_*, shifts, comparisons, MINIMUM, INTDIV,
 * POW) and REDUCE PRODUCT / MIN / MAX are pinned by tests/test_oracle_pins.py against the C library in double
 * precision rounded once, Python integers and the shader's polynomial coefficients in exact rationals.
 * What stays PARITY UNPINNED is what only a run of the reference on its Vulkan driver could fix: the last-ulp
 * behaviour of the driver's builtins (exp, log, inversesqrt, tanh, sin, cos, pow; this restatement returns the
 * correctly rounded value) and the payload / sign of NaN results.
 */
#ifndef MLEL_ORACLE_H
#define MLEL_ORACLE_H

#include "../include/mlel_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

const char *mlel_cpu_last_error(void);
int mlel_cpu_num_threads(void);

int mlel_cpu_conv2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *weights,
                    const mlel_tensor *bias, const mlel_conv2d_attr *attr);
int mlel_cpu_depthwise_conv2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *weights,
                              const mlel_tensor *bias, const mlel_conv2d_attr *attr);
int mlel_cpu_matmul(const mlel_tensor *out, const mlel_tensor *a, const mlel_tensor *b,
                    const mlel_matmul_attr *attr);
int mlel_cpu_rescale(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *multiplier,
                     const mlel_tensor *shift, const mlel_rescale_attr *attr);
int mlel_cpu_clamp(const mlel_tensor *out, const mlel_tensor *in, const mlel_clamp_attr *attr);
int mlel_cpu_elementwise_binary(int32_t op, const mlel_tensor *out, const mlel_tensor *in1,
                                const mlel_tensor *in2, uint32_t nan_mode);
int mlel_cpu_mul(const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2, uint32_t shift);
int mlel_cpu_elementwise_unary(int32_t op, const mlel_tensor *out, const mlel_tensor *in);
int mlel_cpu_reduce(int32_t op, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t nan_mode);
int mlel_cpu_avg_pool2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_pool2d_attr *attr);
int mlel_cpu_max_pool2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_pool2d_attr *attr);
int mlel_cpu_table(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *table);
int mlel_cpu_cast(const mlel_tensor *out, const mlel_tensor *in);
int mlel_cpu_negate(const mlel_tensor *out, const mlel_tensor *in, int32_t input_zp, int32_t output_zp);
int mlel_cpu_reshape(const mlel_tensor *out, const mlel_tensor *in);
int mlel_cpu_transpose(const mlel_tensor *out, const mlel_tensor *in, const uint32_t *perms);
int mlel_cpu_concat(const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t offset);
int mlel_cpu_slice(const mlel_tensor *out, const mlel_tensor *in, const uint32_t *start);
int mlel_cpu_pad(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *padding, double pad_const,
                 int32_t pad_const_int);
int mlel_cpu_argmax(const mlel_tensor *out, const mlel_tensor *in, uint32_t axis, uint32_t nan_mode);
int mlel_cpu_arithmetic_right_shift(const mlel_tensor *out, const mlel_tensor *in1, const mlel_tensor *in2,
                                    uint32_t round);
int mlel_cpu_conv3d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w, const mlel_tensor *bias,
                    const mlel_conv3d_attr *attr);
int mlel_cpu_transpose_conv2d(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w,
                              const mlel_tensor *bias, const mlel_tconv2d_attr *attr);
int mlel_cpu_fft2d(const mlel_tensor *out_real, const mlel_tensor *out_imag, const mlel_tensor *in_real,
                   const mlel_tensor *in_imag, int32_t inverse);
int mlel_cpu_rfft2d(const mlel_tensor *out_real, const mlel_tensor *out_imag, const mlel_tensor *in);
int mlel_cpu_gather(const mlel_tensor *out, const mlel_tensor *values, const mlel_tensor *indices);
int mlel_cpu_scatter(const mlel_tensor *out, const mlel_tensor *values_in, const mlel_tensor *indices,
                     const mlel_tensor *input);
int mlel_cpu_resize(const mlel_tensor *out, const mlel_tensor *in, const mlel_resize_attr *attr);
int mlel_cpu_reverse(const mlel_tensor *out, const mlel_tensor *in, uint32_t axis);
int mlel_cpu_tile(const mlel_tensor *out, const mlel_tensor *in);
int mlel_cpu_select(const mlel_tensor *out, const mlel_tensor *condition, const mlel_tensor *in_true,
                    const mlel_tensor *in_false);

/* IEEE binary16 <-> binary32 helpers (round to nearest even), exported for the tests. */
uint16_t mlel_cpu_f32_to_f16(float f);
float mlel_cpu_f16_to_f32(uint16_t h);
/* bf16 / fp8 storage codecs as the shaders define them (graph/shaders/graph_op/common.comp:184-232, 300-418);
 * `dtype` is MLEL_F8E4M3 or MLEL_F8E5M2 */
uint16_t mlel_cpu_f32_to_bf16(float x, int nearest_even);
uint8_t mlel_cpu_f32_to_f8(float x, int dtype);
float mlel_cpu_f8_to_f32(uint8_t x, int dtype);

#ifdef __cplusplus
}
#endif
#endif
