/*
 * mlel_hip.h -- C ABI of the MI355X (gfx950) execution backend for TOSA 1.0 data-graph operators.
 *
 * This is the boundary the host-side operator surface (GraphPipeline::make<Op>, the mirror of the
 * reference's graph/compute_graph_op.hpp:1204-1549) calls instead of building a VkPipeline and recording
 * vkCmdDispatch (reference: graph/compute_graph_op.cpp:526-590).  One entry point per TOSA operator class
 * of the reference; each takes tensor views (device pointer, dims, byte strides) and an attribute struct that
 * is field-for-field the reference's push-constant + specialisation-constant set for that operator.
 *
 * Conventions
 *   - plain C, no exceptions; every function returns 0 on success or a negative mlel_status and leaves a
 *     human readable message retrievable with mlel_hip_last_error() (thread local);
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); launches are asynchronous;
 *   - tensor pointers are device pointers; strides are in BYTES (reference: tensor/tensor_arm.cpp:67-93),
 *     rank <= 6 (reference: graph/shaders/graph_op/common.comp:11);
 *   - reads outside a tensor's dims yield 0 and writes outside are dropped
 *     (reference: tensor/shaders/tensor.glsl:26-81);
 *   - nothing here falls back to a CPU implementation: without a GPU every launch returns MLEL_ERR_DEVICE.
 */
#ifndef MLEL_HIP_H
#define MLEL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLEL_MAX_RANK 6

/* Status codes. */
typedef enum mlel_status {
    MLEL_OK = 0,
    MLEL_ERR_INVALID = -1,     /* bad argument: shape / dtype / attribute combination not accepted */
    MLEL_ERR_UNSUPPORTED = -2, /* valid TOSA, but no kernel for this dtype combination              */
    MLEL_ERR_DEVICE = -3,      /* HIP runtime error (no device, launch failure, out of memory)       */
    MLEL_ERR_LIMIT = -4        /* size beyond a documented limit                                     */
} mlel_status;

/* Element types.  Mirrors the VkFormat -> shader type table of the reference (common/utils.cpp:119-228). */
typedef enum mlel_dtype {
    MLEL_BOOL = 0, /* VK_FORMAT_R8_BOOL_ARM, one byte, 0/1 */
    MLEL_I8 = 1,
    MLEL_U8 = 2,
    MLEL_I16 = 3,
    MLEL_U16 = 4,
    MLEL_I32 = 5,
    MLEL_U32 = 6,
    MLEL_I64 = 7,
    MLEL_U64 = 8,
    MLEL_F16 = 9,
    MLEL_BF16 = 10,   /* upper half of an fp32; arithmetic in fp32 (graph/shaders/graph_op/common.comp:184-189) */
    MLEL_F32 = 11,
    MLEL_F64 = 12,
    MLEL_F8E4M3 = 13, /* bias 7, no infinities, NaN = 0x7f; arithmetic in fp16 (common.comp:197-215) */
    MLEL_F8E5M2 = 14, /* upper byte of an fp16; arithmetic in fp16 (common.comp:191-195) */
    MLEL_DTYPE_COUNT = 15
} mlel_dtype;

/* Accumulator type codes as decoded from the SPIR-V operand (reference: graph/compute_graph_op.cpp:39-67). */
enum { MLEL_ACC_I32 = 1, MLEL_ACC_F16 = 2, MLEL_ACC_F32 = 3, MLEL_ACC_I64 = 4 };
/* NaN propagation modes (reference: graph/compute_graph_op.hpp:32-35). */
enum { MLEL_NAN_PROPAGATE = 1, MLEL_NAN_IGNORE = 2 };
/* RESCALE rounding modes (reference: graph/graph_tosa_1_0_ext_inst.cpp:29-33). */
enum { MLEL_ROUND_SINGLE = 1, MLEL_ROUND_INEXACT = 2, MLEL_ROUND_DOUBLE = 3 };

/* Tensor view.  Replaces the reference's tensor descriptor {address, dims[6], strides[6]}
 * (reference: tensor/tensor_descriptor.cpp:56-80). */
typedef struct mlel_tensor {
    void *ptr;
    int32_t dtype; /* mlel_dtype */
    int32_t rank;  /* 1..6 */
    int64_t dims[MLEL_MAX_RANK];
    int64_t strides[MLEL_MAX_RANK]; /* bytes */
} mlel_tensor;

/* ---- attribute structs (same fields as the reference push constants) ---- */

/* CONV2D / DEPTHWISE_CONV2D (reference: graph/compute_graph_op.hpp:418-425, 509-515).
 * pad = {top, bottom, left, right}; stride = {y, x}; dilation = {y, x}. */
typedef struct mlel_conv2d_attr {
    int32_t input_zp;
    int32_t weight_zp;
    int32_t pad[4];
    int32_t stride[2];
    int32_t dilation[2];
    uint32_t acc_type; /* MLEL_ACC_* */
} mlel_conv2d_attr;

/* MATMUL (reference: graph/compute_graph_op.hpp:655-658). */
typedef struct mlel_matmul_attr {
    int32_t a_zp;
    int32_t b_zp;
} mlel_matmul_attr;

/* RESCALE (reference: push constants graph/compute_graph_op.hpp:846-849, specialisation constants
 * {rank, scale32, doubleRound, perChannel} graph/compute_graph_op.cpp:1729, unsigned twins :1761-1762). */
typedef struct mlel_rescale_attr {
    int32_t input_zp;
    int32_t output_zp;
    uint32_t scale32;
    uint32_t double_round;
    uint32_t per_channel;
    uint32_t input_unsigned;
    uint32_t output_unsigned;
} mlel_rescale_attr;

/* CLAMP (reference: graph/compute_graph_op.hpp:352-356); min/max travel as double. */
typedef struct mlel_clamp_attr {
    double min_val;
    double max_val;
    uint32_t nan_mode;
} mlel_clamp_attr;

/* AVG_POOL2D / MAX_POOL2D (reference: graph/compute_graph_op.hpp:296-302, 688-693).
 * kernel = {y, x}; stride = {y, x}; pad = {top, bottom, left, right}. */
typedef struct mlel_pool2d_attr {
    int32_t kernel[2];
    int32_t stride[2];
    int32_t pad[4];
    int32_t input_zp;  /* AVG only */
    int32_t output_zp; /* AVG only */
    uint32_t acc_type; /* AVG only */
    uint32_t nan_mode; /* MAX only */
} mlel_pool2d_attr;

/* CONV3D (reference: conv3d.comp:29-35 push constants).  pad = {front, back, top, bottom, left, right};
 * stride = {d, y, x}; dilation = {d, y, x}. */
typedef struct mlel_conv3d_attr {
    int32_t input_zp;
    int32_t weight_zp;
    int32_t pad[6];
    int32_t stride[3];
    int32_t dilation[3];
    uint32_t acc_type; /* MLEL_ACC_* */
} mlel_conv3d_attr;

/* TRANSPOSE_CONV2D (reference: transpose_conv2d.comp:25-30).  out_pad = {top, bottom, left, right}; stride = {y, x}. */
typedef struct mlel_tconv2d_attr {
    int32_t input_zp;
    int32_t weight_zp;
    int32_t out_pad[4];
    int32_t stride[2];
    uint32_t acc_type; /* MLEL_ACC_* */
} mlel_tconv2d_attr;

/* RESIZE (reference: resize.comp:21-44).  scale = {y_n, y_d, x_n, x_d}; offset = {y, x}; border = {y, x}. */
enum { MLEL_RESIZE_NEAREST = 1, MLEL_RESIZE_BILINEAR = 2 };
typedef struct mlel_resize_attr {
    int32_t scale[4];
    int32_t offset[2];
    int32_t border[2];
    uint32_t mode; /* MLEL_RESIZE_* */
} mlel_resize_attr;

/* Elementwise binary operator selector.  One value per `%operation%` string the reference substitutes into
 * elementwise_binary.comp (reference: graph/compute_graph_op.cpp:2527-2946). */
typedef enum mlel_binary_op {
    MLEL_BIN_ADD = 0,
    MLEL_BIN_SUB,
    MLEL_BIN_BITWISE_AND,
    MLEL_BIN_BITWISE_OR,
    MLEL_BIN_BITWISE_XOR,
    MLEL_BIN_INTDIV,
    MLEL_BIN_LOGICAL_AND,
    MLEL_BIN_LOGICAL_OR,
    MLEL_BIN_LOGICAL_XOR,
    MLEL_BIN_LOGICAL_LEFT_SHIFT,
    MLEL_BIN_LOGICAL_RIGHT_SHIFT,
    MLEL_BIN_MAXIMUM,
    MLEL_BIN_MINIMUM,
    MLEL_BIN_POW,
    MLEL_BIN_EQUAL,
    MLEL_BIN_GREATER,
    MLEL_BIN_GREATER_EQUAL,
    MLEL_BIN_COUNT
} mlel_binary_op;

/* Elementwise unary operator selector (reference: elementwise_unary.comp `%operation%` strings,
 * graph/compute_graph_op.cpp:2527-2946). */
typedef enum mlel_unary_op {
    MLEL_UN_ABS = 0,
    MLEL_UN_BITWISE_NOT,
    MLEL_UN_CEIL,
    MLEL_UN_CLZ,
    MLEL_UN_COS,
    MLEL_UN_ERF,
    MLEL_UN_EXP,
    MLEL_UN_FLOOR,
    MLEL_UN_LOG,
    MLEL_UN_LOGICAL_NOT,
    MLEL_UN_RECIPROCAL,
    MLEL_UN_RSQRT,
    MLEL_UN_SIGMOID,
    MLEL_UN_SIN,
    MLEL_UN_TANH,
    MLEL_UN_COUNT
} mlel_unary_op;

/* Reduction selector (reference: reduce.comp init/operation strings, graph/compute_graph_op.cpp:2819-2859). */
typedef enum mlel_reduce_op {
    MLEL_RED_ALL = 0,
    MLEL_RED_ANY,
    MLEL_RED_MAX,
    MLEL_RED_MIN,
    MLEL_RED_PRODUCT,
    MLEL_RED_SUM,
    MLEL_RED_COUNT
} mlel_reduce_op;

/* Fused epilogue of a contraction: RESCALE (always) then optional CLAMP, applied to the int32 accumulator
 * before it is narrowed and stored.  Bit-identical to running the three operators one after another. */
typedef struct mlel_epilogue {
    const mlel_tensor *multiplier; /* i32[C] (scale32) or i16[C]; C == 1 unless per_channel */
    const mlel_tensor *shift;      /* i8[C] */
    mlel_rescale_attr rescale;
    int32_t has_clamp;
    mlel_clamp_attr clamp;
} mlel_epilogue;

/* ---- context, memory, streams, events ---- */

typedef struct mlel_ctx mlel_ctx;

/* Thread-local description of the last failure on the calling thread. */
const char *mlel_hip_last_error(void);

/* Library / device queries.  mlel_hip_device_count() never fails: it returns 0 when no GPU is visible. */
int mlel_hip_device_count(void);
int mlel_hip_init(int device, mlel_ctx **out_ctx);
void mlel_hip_destroy(mlel_ctx *ctx);
/* Fills compute units, engine clock (kHz), memory clock (kHz), bus width (bits), name (<=255 chars). */
int mlel_hip_device_info(mlel_ctx *ctx, int32_t *cu_count, int32_t *clock_khz, int32_t *mem_clock_khz,
                         int32_t *bus_width_bits, char *name, size_t name_len);

/* Device arena (hipMalloc'd HBM).  Replaces VkDeviceMemory allocation of the reference
 * (graph/tensor.cpp:95-114 for constants, utilities/tensor.cpp:100-108 for test tensors, zero-filled). */
int mlel_hip_arena_alloc(mlel_ctx *ctx, size_t bytes, void **dptr);
int mlel_hip_arena_free(mlel_ctx *ctx, void *dptr);
/* Import of a Vulkan allocation exported as an opaque fd (VK_KHR_external_memory_fd) into the HIP address
 * space; the returned pointer aliases the VkDeviceMemory. */
int mlel_hip_arena_import_fd(mlel_ctx *ctx, int fd, size_t bytes, void **dptr, void **out_handle);
int mlel_hip_arena_release_import(mlel_ctx *ctx, void *handle);
int mlel_hip_memcpy_h2d(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream);
int mlel_hip_memcpy_d2h(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream);
int mlel_hip_memcpy_d2d(mlel_ctx *ctx, void *dst, const void *src, size_t bytes, void *stream);
/* Asynchronous byte fill on `stream`.  On a stream that is being captured into a graph the fill is recorded as a
 * kernel, not as a memset node. */
int mlel_hip_memset(mlel_ctx *ctx, void *dst, int value, size_t bytes, void *stream);

int mlel_hip_stream_create(mlel_ctx *ctx, void **out_stream);
/* Waits for the stream, frees the split-K workspace the context kept for it (if it ever split), destroys it. */
int mlel_hip_stream_destroy(mlel_ctx *ctx, void *stream);
/* Number of per-stream split-K workspaces (16 MiB + 16 KiB each, at most 16) the context holds right now. */
int mlel_hip_split_workspaces(mlel_ctx *ctx);
int mlel_hip_sync(mlel_ctx *ctx, void *stream); /* NULL = whole device */

/* Per-operator timing.  Replaces the reference's timestamp queries around each dispatch
 * (graph/graph_profiler.cpp:157-191). */
int mlel_hip_event_create(mlel_ctx *ctx, void **out_event);
int mlel_hip_event_destroy(mlel_ctx *ctx, void *event);
int mlel_hip_event_record(mlel_ctx *ctx, void *event, void *stream);
/* Work issued to `stream` after this call starts when the work recorded in `event` (its latest record) is done:
 * the fork and the join of a dispatch that runs on two streams.  Legal on a stream that is being captured (the
 * other stream joins the capture).  Reference counterpart: a pipeline barrier between two queues' submissions. */
int mlel_hip_stream_wait_event(mlel_ctx *ctx, void *stream, void *event);
int mlel_hip_event_elapsed_ms(mlel_ctx *ctx, void *start, void *stop, float *ms); /* synchronises on stop */

/* HIP-graph capture of a sequence of launches on `stream`, used to replay a whole TOSA graph with one
 * submission.  Replaces command-buffer recording + vkQueueSubmit (reference: graph/graph_layer.cpp:1844-1980). */
int mlel_hip_capture_begin(mlel_ctx *ctx, void *stream);
int mlel_hip_capture_end(mlel_ctx *ctx, void *stream, void **out_graph_exec);
int mlel_hip_graph_launch(mlel_ctx *ctx, void *graph_exec, void *stream);
int mlel_hip_graph_destroy(mlel_ctx *ctx, void *graph_exec);

/* ---- operators ---- */

/* CONV2D.  in [N,H,W,IC], w [OC,KH,KW,IC], bias [OC] or [1] typed as the output, out [N,OH,OW,OC].
 * Replaces class Conv2D (reference: graph/compute_graph_op.cpp:914-1023) running conv2d.comp:40-116. */
int mlel_hip_conv2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                    const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv2d_attr *attr);

/* DEPTHWISE_CONV2D.  w [KH,KW,C,M], out channel = c*M+m.
 * Replaces class DepthwiseConv2D (reference: graph/compute_graph_op.cpp:1116-1199), depthwise_conv2d.comp:31-78. */
int mlel_hip_depthwise_conv2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                              const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv2d_attr *attr);

/* MATMUL.  a [N,H,C], b [N,C,W], out [N,H,W].
 * Replaces class Matmul (reference: graph/compute_graph_op.cpp:1387-1436), matmul.comp:30-73. */
int mlel_hip_matmul(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                    const mlel_tensor *b, const mlel_matmul_attr *attr);

/* RESCALE.  Replaces class Rescale (reference: graph/compute_graph_op.cpp:1719-1779), rescale.comp:27-72. */
int mlel_hip_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                     const mlel_tensor *multiplier, const mlel_tensor *shift, const mlel_rescale_attr *attr);

/* CLAMP.  Replaces class Clamp (reference: graph/compute_graph_op.cpp:811-853), clamp.comp:24-53. */
int mlel_hip_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                   const mlel_clamp_attr *attr);

/* ADD, SUB, MAXIMUM, ... with size-1 broadcast.  Replaces class ElementwiseBinary
 * (reference: graph/compute_graph_op.cpp:1205-1255), elementwise_binary.comp:146-173. */
int mlel_hip_elementwise_binary(mlel_ctx *ctx, void *stream, int32_t op, const mlel_tensor *out,
                                const mlel_tensor *in1, const mlel_tensor *in2, uint32_t nan_mode);

/* MUL.  Replaces class Mul (reference: graph/compute_graph_op.cpp:1508-1557), mul.comp:24-59. */
int mlel_hip_mul(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in1,
                 const mlel_tensor *in2, uint32_t shift);

/* ABS ... TANH.  Replaces class ElementwiseUnary (reference: graph/compute_graph_op.cpp:1261-1297),
 * elementwise_unary.comp:188-205. */
int mlel_hip_elementwise_unary(mlel_ctx *ctx, void *stream, int32_t op, const mlel_tensor *out,
                               const mlel_tensor *in);

/* REDUCE_*.  Output keeps the reduced axis with extent 1.  Replaces class Reduce
 * (reference: graph/compute_graph_op.cpp:1665-1713), reduce.comp:24-70. */
int mlel_hip_reduce(mlel_ctx *ctx, void *stream, int32_t op, const mlel_tensor *out, const mlel_tensor *in,
                    uint32_t axis, uint32_t nan_mode);

/* AVG_POOL2D / MAX_POOL2D.  Replace classes AvgPool2D / MaxPool2D
 * (reference: graph/compute_graph_op.cpp:694-760, 1442-1502), avgpool2d.comp:27-75, maxpool2d.comp:23-72. */
int mlel_hip_avg_pool2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                        const mlel_pool2d_attr *attr);
int mlel_hip_max_pool2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                        const mlel_pool2d_attr *attr);

/* TABLE.  Replaces class Table (reference: graph/compute_graph_op.cpp:2090-2126), table.comp:17-52. */
int mlel_hip_table(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                   const mlel_tensor *table);

/* CAST.  Replaces class Cast (reference: graph/compute_graph_op.cpp:766-805), cast.comp:22-103. */
int mlel_hip_cast(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in);

/* NEGATE.  Replaces class Negate (reference: negate.comp:29-47). */
int mlel_hip_negate(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                    int32_t input_zp, int32_t output_zp);

/* Data movement.  Replace classes Reshape, Transpose, Concat (one call per input, running `offset` along
 * `axis`, reference: graph/compute_graph_op.cpp:2607-2615), Slice, Pad and the shaders of the same names. */
int mlel_hip_reshape(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in);
int mlel_hip_transpose(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                       const uint32_t *perms);
int mlel_hip_concat(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis,
                    uint32_t offset);
int mlel_hip_slice(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                   const uint32_t *start);
int mlel_hip_pad(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                 const mlel_tensor *padding, double pad_const, int32_t pad_const_int);

/* ---- the remaining TOSA operators: one thread per output element, any strides ---- */

/* ARGMAX: output int32 with the axis removed; first maximum wins.  Replaces class ArgMax, argmax.comp:26-66. */
int mlel_hip_argmax(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis,
                    uint32_t nan_mode);
/* ARITHMETIC_RIGHT_SHIFT with size-1 broadcast.  Replaces class ArithmeticRightShift,
 * arithmetic_right_shift.comp:22-48. */
int mlel_hip_arithmetic_right_shift(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in1,
                                    const mlel_tensor *in2, uint32_t round);
/* CONV3D: NDHWC x ODHWI.  Replaces class Conv3D (reference: graph/compute_graph_op.cpp:1029-1110), conv3d.comp:37-104.
 * Dense int8 operands with an int32 result and at least four million multiply-adds run as ONE CONV2D on the matrix
 * cores: the KD depth taps of an output slice are laid side by side along the channels of a copy of the input in the
 * stream's staging memory (KD times the input; grown on demand outside a capture, released by
 * mlel_hip_stream_destroy / mlel_hip_destroy), the weights regrouped to match.  A kernel one slice deep without depth
 * padding or stride needs no copy.  Everything else, and a capturing stream whose staging memory is too small, takes
 * the one-thread-per-output kernel.  The bits are the same. */
int mlel_hip_conv3d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                    const mlel_tensor *weights, const mlel_tensor *bias, const mlel_conv3d_attr *attr);
/* TRANSPOSE_CONV2D: NHWC x OHWI.  Replaces class TransposeConv2D (reference: graph/compute_graph_op.cpp:2211-2290),
 * transpose_conv2d.comp:31-70. */
int mlel_hip_transpose_conv2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                              const mlel_tensor *weights, const mlel_tensor *bias, const mlel_tconv2d_attr *attr);
/* FFT2D / RFFT2D on float32 [N, H, W]: direct evaluation of the transform sums.  Replace classes Fft2D / Rfft2D
 * (reference: graph/compute_graph_op.cpp:1303-1381, 1931-1990), fft2d.comp:17-52, rfft2d.comp:13-71. */
int mlel_hip_fft2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out_real, const mlel_tensor *out_imag,
                   const mlel_tensor *in_real, const mlel_tensor *in_imag, int32_t inverse);
int mlel_hip_rfft2d(mlel_ctx *ctx, void *stream, const mlel_tensor *out_real, const mlel_tensor *out_imag,
                    const mlel_tensor *in);
/* GATHER: out[n,w,c] = values[n, indices[n,w], c].  SCATTER: out = values_in with rows named by indices replaced
 * by the rows of input.  Replace classes Gather / Scatter, gather.comp:13-25, scatter.comp:14-34. */
int mlel_hip_gather(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *values,
                    const mlel_tensor *indices);
int mlel_hip_scatter(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *values_in,
                     const mlel_tensor *indices, const mlel_tensor *input);
/* RESIZE (nearest / bilinear, integer or float).  Replaces class Resize (reference:
 * graph/compute_graph_op.cpp:1820-1925), resize.comp:57-134. */
int mlel_hip_resize(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                    const mlel_resize_attr *attr);
/* REVERSE, TILE, SELECT.  Replace the classes and shaders of the same names (reverse.comp:14-30, tile.comp:12-30,
 * select.comp:15-41). */
int mlel_hip_reverse(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in, uint32_t axis);
int mlel_hip_tile(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in);
int mlel_hip_select(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *condition,
                    const mlel_tensor *in_true, const mlel_tensor *in_false);

/* ---- fused entry points (chosen only by the host-side fusion pass; no counterpart in the reference, which
 * runs one dispatch per TOSA instruction: graph/compute_graph_op.cpp:2500-2509).  Each equals, bit for bit,
 * the unfused sequence <contraction> -> RESCALE -> [CLAMP] with an int32 intermediate.
 * When no one-pass kernel takes the operands (strided views, unusual types) these entry points run that operator
 * sequence themselves: they then hipMalloc temporaries, and synchronise the stream before freeing them on return.
 * On a stream that is being captured into a graph that route returns MLEL_ERR_UNSUPPORTED instead (nothing is
 * launched).  The int8 contractions may split K over several blocks when a layer has fewer tiles than the GPU has
 * compute units; the partial tiles live in a per-stream workspace owned by the context (16 MiB, created the first
 * time a stream needs it outside a capture; MLEL_SPLIT_K=0 in the environment at mlel_hip_init switches the mode
 * off).  Integer addition wraps, so a split result is bit-identical. ---- */
int mlel_hip_conv2d_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                  const mlel_tensor *weights, const mlel_tensor *bias,
                                  const mlel_conv2d_attr *attr, const mlel_epilogue *epi);
/* mlel_hip_conv2d_rescale_clamp for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and the
 * same bits in `out`; it calls no hipMalloc / hipFree or allocating library routine.  Whatever scratch its kernels
 * need -- the partial tiles and arrival counters of a split-K contraction, or the int32 accumulator when no one-pass
 * kernel takes the operands and the operator sequence runs instead -- lives in one statically allocated device array
 * of 8 MiB + 16 KiB that each GPU the library runs on holds until the process ends.  A call whose accumulator would
 * not fit (more than 2 097 152 output elements on the operator-sequence route) returns MLEL_ERR_LIMIT.  All calls on
 * one GPU share the array: calls that overlap on one GPU (two streams, two threads) race; order them. */
int mlel_hip_conv2d_rescale_clamp_static(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                         const mlel_tensor *weights, const mlel_tensor *bias,
                                         const mlel_conv2d_attr *attr, const mlel_epilogue *epi);
/* What the last mlel_hip_conv2d_rescale_clamp_static call on this context kept in the static array: 0 nothing (a
 * one-pass kernel without scratch), 1 the partial tiles and counters of a split-K contraction, 2 the int32
 * accumulator of the operator sequence.  No counterpart in the reference; for tests and for callers that want to
 * know which route a shape takes. */
int mlel_hip_static_scratch_last_use(mlel_ctx *ctx);
/* out = RESCALE_out( RESCALE_conv( CONV2D -> RESCALE -> [CLAMP] (epi) ) + RESCALE_residual(residual) ): the
 * residual connection behind a projecting convolution, bit for bit mlel_hip_conv2d_rescale_clamp into an 8-bit
 * temporary of `out`'s type followed by mlel_hip_rescale_add_rescale.  The integer addition wraps, so the operand order
 * (`residual_first`) only matters to the unfused fallback's argument order. */
int mlel_hip_conv2d_rescale_add_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                        const mlel_tensor *weights, const mlel_tensor *bias,
                                        const mlel_conv2d_attr *attr, const mlel_epilogue *epi,
                                        const mlel_epilogue *scale_conv, const mlel_tensor *residual,
                                        const mlel_epilogue *scale_residual, const mlel_epilogue *scale_out,
                                        int residual_first);
int mlel_hip_matmul_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                            const mlel_tensor *b, const mlel_matmul_attr *attr, const mlel_epilogue *epi);
/* The softmax operator sequence over the last axis in one pass:
 *   m = REDUCE_MAX(in); d = SUB(in, m); e = EXP(d); s = REDUCE_SUM(e); r = RECIPROCAL(s); out = MUL(e, r)
 * (NaN propagating reductions), every intermediate rounded to the tensors' type as the stand-alone operators round
 * it: a shorthand for the six-step mlel_chain below (same kernel, same guarantees). */
int mlel_hip_softmax_rows(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in);
/* out(fp16) = CAST( MATMUL(a, b) + bias ): fp16 operands, fp32 accumulation, the fp32 bias [1,1,N] or [1,1,1] (or
 * NULL) added in fp32, one rounding to fp16 -- bit for bit the unfused MATMUL -> ADD -> CAST (or MATMUL -> CAST).
 * `out` has rank 3, or is a six-dimensional view [NB1, NB2, M1, M2, N1, N2] with byte strides of its own (the last
 * one 2, N2 a multiple of 8; or, for a view that transposes, the stride of M2 2 and M2 a multiple of 8) through which
 * element (nb1 * NB2 + nb2, m1 * M2 + m2, n1 * N2 + n2) of the product is written: the RESHAPE -> TRANSPOSE that splits
 * or merges attention heads behind a projection costs no pass.
 * `b` is the operator's [NB, K, N] tensor; its byte strides may describe a matrix that is stored row-wise ([N][K]:
 * strides[1] == 2, strides[2] the pitch of a row of K) -- with K a multiple of 32 such a B takes the faster
 * direct-to-LDS loop, with the same bits.  A caller whose B is a constant lays it down that way once (the graph layer
 * does at pipeline creation); the same holds for the _add, _group and _chain forms below. */
int mlel_hip_matmul_bias_cast(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                              const mlel_tensor *b, const mlel_tensor *bias, const mlel_matmul_attr *attr);
/* Several such products of one `a` (the query, key and value projections of an attention block) in one launch:
 * products[k].out = CAST( MATMUL(a, products[k].b) + products[k].bias ), every product with the same extents; an
 * output may be a six-dimensional view as above.  Equals the products computed one after another bit for bit (which
 * is also what happens when the grouped kernel does not apply). */
#define MLEL_MATMUL_GROUP_MAX 3
typedef struct mlel_matmul_product {
    const mlel_tensor *out;
    const mlel_tensor *b;
    const mlel_tensor *bias; /* may be NULL */
} mlel_matmul_product;
int mlel_hip_matmul_bias_cast_group(mlel_ctx *ctx, void *stream, const mlel_matmul_product *products, int n_products,
                                    const mlel_tensor *a, const mlel_matmul_attr *attr);
/* The same followed by the ADD of a residual connection: out(fp16) = ADD( CAST( MATMUL(a, b) + bias ), residual ),
 * `residual` an fp16 tensor of the output's shape; the second addition is an fp16 ADD (one rounding of the exact sum
 * of two halfs), as the stand-alone operator computes it. */
int mlel_hip_matmul_bias_cast_add(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                                  const mlel_tensor *b, const mlel_tensor *bias, const mlel_matmul_attr *attr,
                                  const mlel_tensor *residual);
int mlel_hip_dwconv_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                  const mlel_tensor *weights, const mlel_tensor *bias,
                                  const mlel_conv2d_attr *attr, const mlel_epilogue *epi);
/* out = RESCALE_o( RESCALE_a(in1) + RESCALE_b(in2) ): the residual-add pattern with both operands brought to
 * a common int32 scale, added with wraparound, and requantised. */
int mlel_hip_rescale_add_rescale(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in1,
                                 const mlel_epilogue *scale1, const mlel_tensor *in2, const mlel_epilogue *scale2,
                                 const mlel_epilogue *scale_out);

/* A chain of floating-point elementwise operators executed in one pass: ADD, SUB, MUL (shift 0), EXP, RECIPROCAL,
 * RSQRT, TANH and CAST between fp16 and fp32.  Value v < n_inputs is inputs[v]; step i produces value n_inputs + i
 * from values a (and b) and rounds it into `dtype` exactly as the stand-alone operator would; the last step's value
 * is written to `out`.  Every step has the shape of `out`; an input has that shape, or is broadcast along the rows
 * (all leading extents 1), along the last axis (last extent 1), or both.  Equals the operators run one after
 * another bit for bit (no counterpart in the reference, which runs one dispatch per operator).
 *
 * A chain may also hold REDUCE_SUM / REDUCE_MAX steps over the last axis (LayerNorm's moments, softmax).  Values then
 * have the full shape, the full shape with a last extent of 1 (what a reduction yields), or are broadcast inputs as
 * above; a step's shape is the broadcast of its operands' shapes, a reduction takes a full value, and `out` has the
 * last step's shape.  Non-NaN results equal the operators run one after another bit for bit; where those yield a NaN
 * so does the chain, but not necessarily one of the same sign and payload. */
#define MLEL_CHAIN_MAX_STEPS 24
#define MLEL_CHAIN_MAX_INPUTS 8
enum { MLEL_CHAIN_BINARY = 0, MLEL_CHAIN_MUL = 1, MLEL_CHAIN_UNARY = 2, MLEL_CHAIN_CAST = 3, MLEL_CHAIN_REDUCE = 4 };
typedef struct mlel_chain_step {
    int32_t kind;     /* MLEL_CHAIN_* */
    int32_t selector; /* mlel_binary_op (ADD, SUB), mlel_unary_op (EXP, RECIPROCAL, RSQRT, TANH) or, for
                         MLEL_CHAIN_REDUCE, mlel_reduce_op (SUM, MAX) over the last axis, NaN propagated */
    int32_t a, b;     /* operand values; b is ignored by unary steps and casts */
    int32_t dtype;    /* MLEL_F16 or MLEL_F32: the type of the step's result */
} mlel_chain_step;
typedef struct mlel_chain {
    int32_t n_inputs;
    int32_t n_steps;
    const mlel_tensor *inputs[MLEL_CHAIN_MAX_INPUTS];
    mlel_chain_step steps[MLEL_CHAIN_MAX_STEPS];
} mlel_chain;
int mlel_hip_elementwise_chain(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_chain *chain);
/* out(fp16) = chain( CAST( MATMUL(a, b) + bias ) ): the fused product above followed by an elementwise chain whose
 * value 0 is the product (chain->inputs[0] is ignored and may be NULL; the other inputs are the chain's own).  The
 * activation of a feed-forward layer costs no pass when the chain is one the product's kernel knows (the tanh form
 * of GELU); otherwise the product goes through a temporary and the chain runs over it.  Bit for bit the product
 * followed by mlel_hip_elementwise_chain. */
int mlel_hip_matmul_bias_cast_chain(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *a,
                                    const mlel_tensor *b, const mlel_tensor *bias, const mlel_matmul_attr *attr,
                                    const mlel_chain *chain);
/* 1 when mlel_hip_matmul_bias_cast_chain applies this chain inside the product's kernel, 0 when it would run the
 * chain as a pass of its own over a temporary (then a caller gains nothing by handing the chain over).  Reads only
 * the steps and the extents and types of inputs 1 and up; touches no device.  No counterpart in the reference, which
 * has no fused operators. */
int mlel_hip_matmul_chain_in_kernel(const mlel_chain *chain);

/* out(fp16) = CAST( MATMUL( softmax( CAST( MATMUL(q, kt) ) ), v ) ) for fp16 attention heads of 64: q [NB, M, 64],
 * kt [NB, 64, S], v [NB, S, 64], out [NB, M, 64] or a rank-6 view of it as in mlel_hip_matmul_bias_cast.  `softmax` is
 * the chain between the two products as a TOSA graph spells it (REDUCE_MAX, SUB, EXP, REDUCE_SUM, RECIPROCAL, MUL over
 * the last axis, optionally a MUL by a single-element scale in front; its input 0 is the first product and may be
 * NULL).  One launch that keeps the scores on the chip; bit for bit mlel_hip_matmul_bias_cast, mlel_hip_elementwise_chain
 * and mlel_hip_matmul_bias_cast one after another wherever the result is a number (rows that meet a NaN or an infinity
 * are NaN in both).  M a multiple of 64, S a multiple of 64 up to 512, dense 16-byte aligned rows; anything else is
 * MLEL_ERR_UNSUPPORTED (nothing is allocated and nothing falls back).  Replaces three of the reference's dispatches
 * (matmul.comp, the elementwise / reduce shaders of the softmax, matmul.comp); it has no single counterpart there. */
int mlel_hip_attention_f16(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *q,
                           const mlel_tensor *kt, const mlel_tensor *v, const mlel_chain *softmax);
/* 1 when mlel_hip_attention_f16 takes these operands, judged by types, extents, strides and the chain's steps only
 * (data pointers are not looked at; no device is touched), else 0. */
int mlel_hip_attention_f16_in_kernel(const mlel_tensor *out, const mlel_tensor *q, const mlel_tensor *kt,
                                     const mlel_tensor *v, const mlel_chain *softmax);

/* out(int8) = CLAMP?(RESCALE(DEPTHWISE_CONV2D( CLAMP?(RESCALE(CONV2D(in, w1, b1))), w2, b2 ))): the expansion (1x1,
 * unit stride, no padding) and the 3x3 depthwise stage (stride 1 or 2) of an inverted-residual block in one launch.  A
 * thread block keeps 32 expanded channels of a whole image in shared memory, so the expanded tensor never reaches
 * memory.  Byte for byte mlel_hip_conv2d_rescale_clamp followed by mlel_hip_dwconv_rescale_clamp.  in [N, H, W, IC]
 * with IC a multiple of 32 up to 160 and H, W <= 32; w1 [C, 1, 1, IC] with C a multiple of 32; w2 [3, 3, C, 1];
 * out [N, OH, OW, C]; zero weight zero points; dense operands, `in` and `w1` 16-byte aligned.  Anything else is
 * MLEL_ERR_UNSUPPORTED (nothing is allocated and nothing falls back).  Replaces two pairs of the reference's
 * dispatches (conv2d.comp + rescale.comp, depthwise_conv2d.comp + rescale.comp, each with clamp.comp when present);
 * it has no single counterpart there. */
int mlel_hip_conv2d_dwconv_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                         const mlel_tensor *w1, const mlel_tensor *b1, const mlel_conv2d_attr *a1,
                                         const mlel_epilogue *e1, const mlel_tensor *w2, const mlel_tensor *b2,
                                         const mlel_conv2d_attr *a2, const mlel_epilogue *e2);
/* out(int8) = CLAMP?(RESCALE(CONV2D( CLAMP?(RESCALE(CONV2D(in, w1, b1))), w2, b2 ))): two 1x1 convolutions in a row
 * (unit stride, no padding), the projection of one inverted-residual block and the expansion of the next, in one
 * launch: a wavefront requantises 32 positions of the first operator into shared memory and reads them back as the
 * second product's row operand.  `mid` (may be NULL): the intermediate tensor [N, H, W, OC1] when another operator
 * reads it too -- it is then stored as well; with NULL it never reaches memory.  Byte for byte
 * mlel_hip_conv2d_rescale_clamp twice.  One pass for int8, IC a multiple of 16, OC1 a multiple of 8 up to 32, OC2 a
 * multiple of 16 up to 192, zero weight zero points, dense operands (the shapes of
 * mlel_hip_conv2d_conv2d_in_kernel); anything else runs the two fused operators one after the other, through `mid`
 * or, with NULL, through a temporary (which allocates and synchronises: MLEL_ERR_UNSUPPORTED on a capturing stream).
 * Replaces two pairs of the reference's dispatches (conv2d.comp + rescale.comp [+ clamp.comp], twice). */
int mlel_hip_conv2d_conv2d_rescale_clamp(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *mid,
                                         const mlel_tensor *in, const mlel_tensor *w1, const mlel_tensor *b1,
                                         const mlel_conv2d_attr *a1, const mlel_epilogue *e1, const mlel_tensor *w2,
                                         const mlel_tensor *b2, const mlel_conv2d_attr *a2, const mlel_epilogue *e2);
/* 1 when mlel_hip_conv2d_conv2d_rescale_clamp runs these operands in one pass, judged by types, extents, strides and
 * attributes only (data pointers are not looked at; no device is touched), else 0. */
int mlel_hip_conv2d_conv2d_in_kernel(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w1,
                                     const mlel_tensor *b1, const mlel_conv2d_attr *a1, const mlel_tensor *w2,
                                     const mlel_tensor *b2, const mlel_conv2d_attr *a2);

/* 1x1 CONV2D + RESCALE (+CLAMP) whose int8 result is read only by an AVG_POOL2D over all positions of an image (the
 * head of a classification network), as one launch: the convolution's result stays in registers.  `out` is the pooled
 * tensor [N, 1, 1, OC]; `conv_dtype` is the type the convolution's result would have had.  Composition of
 * conv2d.comp:40-116, rescale.comp:28-63, clamp.comp:18-31 and avgpool2d.comp:27-75: the bytes are those of
 * mlel_hip_conv2d_rescale_clamp followed by mlel_hip_avg_pool2d, which is also what runs (through a temporary: the call
 * then allocates and waits, and is refused on a capturing stream) when the one-launch kernel declines the operands:
 * int8, zero weight zero point, RESCALE input zero point 0, at most 64 positions per image, input channels in 16-byte
 * units, no padding, dense operands.  mlel_hip_conv2d_avgpool_in_kernel answers that beforehand without touching the
 * device (1: one launch). */
int mlel_hip_conv2d_rescale_clamp_avgpool(mlel_ctx *ctx, void *stream, const mlel_tensor *out, const mlel_tensor *in,
                                          const mlel_tensor *weights, const mlel_tensor *bias,
                                          const mlel_conv2d_attr *attr, const mlel_epilogue *epi, int32_t conv_dtype,
                                          const mlel_pool2d_attr *pool);
int mlel_hip_conv2d_avgpool_in_kernel(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *weights,
                                      const mlel_tensor *bias, const mlel_conv2d_attr *attr, int32_t conv_dtype,
                                      const mlel_pool2d_attr *pool);
/* 1 when mlel_hip_conv2d_dwconv_rescale_clamp takes these operands, judged by types, extents, strides and attributes
 * only (data pointers are not looked at; no device is touched), else 0. */
int mlel_hip_conv2d_dwconv_in_kernel(const mlel_tensor *out, const mlel_tensor *in, const mlel_tensor *w1,
                                     const mlel_tensor *b1, const mlel_conv2d_attr *a1, const mlel_tensor *w2,
                                     const mlel_tensor *b2, const mlel_conv2d_attr *a2);

/* Plain device-to-device copy kernel of `bytes` bytes with 128-bit accesses; the calibration kernel for
 * memory-traffic counters and the measured HBM ceiling. */
int mlel_hip_copy_kernel(mlel_ctx *ctx, void *stream, void *dst, const void *src, size_t bytes);
/* The same kernel with its launch geometry as arguments, for measuring what this part's memory system delivers:
 * `blocks` of 256 threads (<= 0: as many as give every thread one pass), 1 / 2 / 4 / 8 16-byte pieces in flight per
 * thread, temporal or non-temporal accesses; mode 0 copies, 1 only reads `src`, 2 only writes `dst`.  `bytes` in whole
 * 16-byte pieces.  No counterpart in the reference; a measurement aid. */
int mlel_hip_copy_kernel_variant(mlel_ctx *ctx, void *stream, void *dst, const void *src, size_t bytes, int blocks,
                                 int pieces_in_flight, int non_temporal, int mode);
/* The matrix cores without operand delivery: `blocks` blocks of four wavefronts, each wavefront `iters` rounds of
 * eight independent v_mfma_i32_32x32x32_i8 on operands held in registers, which it reads once from `operands`
 * (64 KiB: zeros or random bytes -- the sustained rate depends on the data); `out` receives blocks x 256 int32.
 * 2 x 32 x 32 x 32 x 8 x iters operations per wavefront.  No counterpart in the reference; a measurement aid: the
 * rate a contraction kernel on this part is to be read against beside the published peak. */
int mlel_hip_mfma_rate_probe(mlel_ctx *ctx, void *stream, const void *operands, void *out, int blocks, int iters);
/* What a wavefront that is alone on its SIMD issues while its matrix instructions run: one block of four wavefronts
 * per compute unit, `iters` rounds of the instruction mix `mode` each (0 four v_mfma_i32_32x32x32_i8; 1 sixteen
 * v_dot4, 2 behind the four matrix instructions, 3 dealt out between them; 4 / 5 / 6 the same with v_add_u32, 7 with
 * v_sad_u8 dealt out; 8 / 9 / 10 six 128-bit shared-memory reads; 11 / 12 / 13 four loads into shared memory; 14 four
 * v_mfma_i32_16x16x64_i8 dealt out).  `operands`: 64 KiB; `out`: (2 + 256 x compute units) dwords, of which the first two
 * receive the clocks the first wavefront took for all rounds.  No counterpart in the reference; a measurement aid:
 * the order of the instructions in the contraction kernels' loops follows from these figures. */
int mlel_hip_issue_probe(mlel_ctx *ctx, void *stream, const void *operands, void *out, int mode, int iters);

#ifdef __cplusplus
}
#endif

#endif /* MLEL_HIP_H */
