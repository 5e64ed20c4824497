/*
 * mlel_graph.h -- C view of the host-side operator surface (class mlel::graph::GraphPipeline).
 *
 * The C++ class is the drop-in for the reference's GraphPipeline (graph/compute_graph_op.hpp:1204-1549); this C
 * wrapper exists so that harnesses without a C++ toolchain (ctypes, cgo, JNI ...) can build and run a data graph.
 * Tensors are referred to by non-negative integer handles; every function returns 0 / a handle on success or a
 * negative mlel_status, with the message in mlel_graph_last_error().  C++ exceptions (the reference's inner layer
 * throws std::runtime_error: graph/compute_graph_op.cpp:50,363,477) are caught at this boundary.
 */
#ifndef MLEL_GRAPH_H
#define MLEL_GRAPH_H

#include "mlel_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mlel_graph mlel_graph;

const char *mlel_graph_last_error(void);

/* Reference: GraphPipeline constructor (compute_graph_op.cpp:2379-2390). */
int mlel_graph_create(mlel_ctx *ctx, mlel_graph **out);
void mlel_graph_destroy(mlel_graph *g);

/* Reference: makeConstTensor / getConstTensor / makeConstCompositeTensor (compute_graph_op.cpp:2398-2420).
 * strides may be NULL (packed).  The data is copied. */
int mlel_graph_make_const_tensor(mlel_graph *g, uint32_t id, int32_t dtype, int32_t rank, const int64_t *dims,
                                 const int64_t *strides, const void *data);
int mlel_graph_get_const_tensor(mlel_graph *g, uint32_t id);
int mlel_graph_make_const_composite_tensor(mlel_graph *g, int32_t dtype, int32_t rank, const int64_t *dims,
                                           const void *data);
/* Reference: makeDescriptorSetBinding / getTensor (compute_graph_op.cpp:2441-2455). */
int mlel_graph_make_descriptor_set_binding(mlel_graph *g, uint32_t set, uint32_t binding, uint32_t array_index,
                                           int32_t dtype, int32_t rank, const int64_t *dims, const int64_t *strides);
int mlel_graph_get_tensor(mlel_graph *g, uint32_t set, uint32_t binding, uint32_t array_index);
/* Reference: makeTensor (compute_graph_op.cpp:2457-2469). */
int mlel_graph_make_tensor(mlel_graph *g, int32_t dtype, int32_t rank, const int64_t *dims, const int64_t *strides);
int mlel_graph_make_input(mlel_graph *g, int tensor);
int mlel_graph_make_output(mlel_graph *g, int tensor);

/* One TOSA operator, named as in the TOSA.001000.1 extended instruction set ("CONV2D", "RESCALE", "ADD", ...).
 * `inputs` / `outputs` are tensor handles in the order of the corresponding GraphPipeline::make<Op> signature
 * (tensor arguments only); `iattr` carries the integer attributes and `fattr` the real-valued ones in signature
 * order (vectors flattened).  See the table in the implementation (graph/c_api.cpp) for each operator. */
int mlel_graph_make_op(mlel_graph *g, const char *tosa_name, const int *inputs, int n_inputs, const int *outputs,
                       int n_outputs, const int64_t *iattr, int n_iattr, const double *fattr, int n_fattr,
                       const char *debug_name);

/* Front-end: a data graph written as SPIR-V assembly text (SPV_ARM_graph + SPV_ARM_tensors, "TOSA.001000.1"
 * extended instructions) is decoded into make<Op> calls on `g` (reference: the layer's SPIR-V pass and
 * GraphTosa10ExtInst::handleOp, graph/graph_tosa_1_0_ext_inst.cpp:37-1032; constants and tensor shapes that the
 * reference takes from VkDataGraphPipelineConstantARM / VkTensorDescriptionARM, graph_layer.cpp:343-420, are the
 * `constants` / `bindings` arguments).  `bindings` give the shape of every interface tensor whose SPIR-V type is
 * unshaped; `constants` the payload of every OpGraphConstantARM; `specializations` the values of specialization
 * constants that differ from their defaults (reference: graph_layer.cpp:71-107).  On return io[0..3*n_in) holds {set, binding,
 * array element} of the graph inputs in index order, followed by the same for the outputs.  Returns the number of
 * TOSA instructions decoded. */
typedef struct mlel_graph_spv_binding {
    uint32_t set, binding, array_index;
    int32_t rank;
    const int64_t *dims;
} mlel_graph_spv_binding;
typedef struct mlel_graph_spv_constant {
    uint32_t id;
    int32_t rank;         /* 0 when the SPIR-V type is shaped */
    const int64_t *dims;
    const void *data;
} mlel_graph_spv_constant;
typedef struct mlel_graph_spv_specialization {
    uint32_t spec_id; /* the SpecId decoration */
    uint64_t bits;    /* value as the bit pattern of the constant's type; booleans 0 / 1 */
} mlel_graph_spv_specialization;
int mlel_graph_load_spvasm(mlel_graph *g, const char *text, size_t length, const mlel_graph_spv_binding *bindings,
                           int n_bindings, const mlel_graph_spv_constant *constants, int n_constants,
                           const mlel_graph_spv_specialization *specializations, int n_specializations, uint32_t *io,
                           int io_capacity, int *n_inputs, int *n_outputs);
/* The same for a binary module: `words` is the word stream a Vulkan application passes to vkCreateShaderModule
 * (VkShaderModuleCreateInfo::pCode, codeSize / 4 words; either byte order), which the reference hands to
 * SPIRV-Tools in GraphLayer::vkCreateShaderModule (graph/graph_layer.cpp:2015-2046). */
int mlel_graph_load_spirv(mlel_graph *g, const uint32_t *words, size_t n_words, const mlel_graph_spv_binding *bindings,
                          int n_bindings, const mlel_graph_spv_constant *constants, int n_constants,
                          const mlel_graph_spv_specialization *specializations, int n_specializations, uint32_t *io,
                          int io_capacity, int *n_inputs, int *n_outputs);
/* dtype, rank and dimensions of a tensor handle (dims: room for MLEL_MAX_RANK entries); returns the rank. */
int mlel_graph_tensor_info(mlel_graph *g, int tensor, int32_t *dtype, int64_t *dims);

/* Session-memory planner, chosen before mlel_graph_finalize: 0 interval (default), 1 linear, 2 best fit.  A new graph
 * takes its default from the environment variable VMEL_MEMORY_PLANNER = "Linear" | "BestFit", as the reference does
 * when a session is created (graph_layer.cpp:282-297; planners: graph/memory_planner.cpp:52-382,
 * graph/interval_memory_planner.cpp). */
int mlel_graph_set_memory_planner(mlel_graph *g, int planner);
int mlel_graph_get_memory_planner(mlel_graph *g);

/* Batch split, opt-in, before mlel_graph_finalize.  The reference records a graph as one chain of dispatches
 * (cmdBindAndDispatch, graph/compute_graph_op.cpp:2379-2521); with the split, the leading run of operators that
 * treat the images of a batch independently is issued as two launches each -- the first and the second half of the
 * batch -- on two streams that fork where the dispatch starts and join behind the run, so that one chain's launch
 * latencies are covered by the other's work.  Same bytes in every output as the unsplit dispatch.  The session needs
 * the memory mlel_graph_session_memory_requirements reports after finalize (the tensors inside the run are stored as
 * two halves).  Interval and linear planners; a graph the split cannot serve is left unsplit.
 * mlel_graph_get_batch_split: after finalize, the number of launches that are issued per half (0: not split). */
int mlel_graph_set_batch_split(mlel_graph *g, int enabled);
int mlel_graph_get_batch_split(mlel_graph *g);
/* Fusion + session memory planning; then the session requirements
 * (reference: vkGetDataGraphPipelineSessionMemoryRequirementsARM, graph_layer.cpp:1382-1389). */
int mlel_graph_finalize(mlel_graph *g, int enable_fusion);
int mlel_graph_session_memory_requirements(mlel_graph *g, uint64_t *size, uint64_t *alignment);
/* Reference: vkBindDataGraphPipelineSessionMemoryARM (graph_layer.cpp:1391-1420). */
int mlel_graph_bind_session_memory(mlel_graph *g, void *device_base);
int mlel_graph_bind_external(mlel_graph *g, uint32_t set, uint32_t binding, uint32_t array_index, void *device_ptr);
/* Reference: vkCmdDispatchDataGraphARM -> cmdBindAndDispatch (graph_layer.cpp:1844-1980). */
int mlel_graph_dispatch(mlel_graph *g, void *stream);

/* ---- sessions: one pipeline, several sets of bound memory in flight at once ----
 * Reference: vkCreateDataGraphPipelineSessionARM (graph/graph_layer.cpp:1297-1330),
 * vkGetDataGraphPipelineSessionBindPointRequirementsARM (:1332-1380), vkGetDataGraphPipelineSessionMemoryRequirementsARM
 * (:1382-1389), vkBindDataGraphPipelineSessionMemoryARM (:1391-1420), vkCmdDispatchDataGraphARM (:1844-1980).
 * A session holds its own transient (session) memory and its own external tensor bindings; the functions above that
 * take the graph itself (mlel_graph_bind_session_memory, mlel_graph_bind_external, mlel_graph_dispatch) work on a
 * session the graph creates for itself.  External tensors may be re-bound between dispatches (update-after-bind);
 * the pointers are resolved when a dispatch is issued, so dispatches of two sessions issued one after the other on
 * two streams overlap on the GPU.  A session is used from the thread that uses its graph (neither is locked, as in
 * the reference) and destroyed before its graph. */
typedef struct mlel_graph_session mlel_graph_session;
#define MLEL_GRAPH_INCOMPLETE 5 /* positive, like VK_INCOMPLETE: the array was too short, *count entries exist */
enum { MLEL_GRAPH_BIND_POINT_TRANSIENT = 0 };   /* VK_DATA_GRAPH_PIPELINE_SESSION_BIND_POINT_TRANSIENT_ARM */
enum { MLEL_GRAPH_BIND_POINT_TYPE_MEMORY = 0 }; /* VK_DATA_GRAPH_PIPELINE_SESSION_BIND_POINT_TYPE_MEMORY_ARM */
typedef struct mlel_graph_bind_point_requirement {
    uint32_t bind_point, bind_point_type, num_objects;
} mlel_graph_bind_point_requirement;
int mlel_graph_session_create(mlel_graph *g, mlel_graph_session **out); /* after mlel_graph_finalize */
void mlel_graph_session_destroy(mlel_graph_session *s);
/* Two-call pattern: requirements == NULL writes the number of bind points to *count (0 for a graph without
 * intermediate tensors, else 1); otherwise at most *count entries are written, *count becomes the number that exist
 * and the result is MLEL_GRAPH_INCOMPLETE when the array was shorter than that. */
int mlel_graph_session_bind_point_requirements(mlel_graph_session *s, uint32_t *count,
                                               mlel_graph_bind_point_requirement *requirements);
int mlel_graph_session_get_memory_requirements(mlel_graph_session *s, uint32_t bind_point, uint64_t *size,
                                               uint64_t *alignment);
int mlel_graph_session_bind_memory(mlel_graph_session *s, uint32_t bind_point, void *device_base);
int mlel_graph_session_bind_external(mlel_graph_session *s, uint32_t set, uint32_t binding, uint32_t array_index,
                                     void *device_ptr);
int mlel_graph_session_dispatch(mlel_graph_session *s, void *stream);
/* The same dispatch with its launches recorded into a HIP graph the first time (and again after a bind on this session,
 * or on another stream) and replayed with one submission afterwards: the host's share of a dispatch drops from one
 * launch call per operator (about 4 us each) to one, which is what bounds several sessions in flight.  Same results.
 * The recording holds the addresses bound at that moment; `stream` must not be capturing already.  Reference
 * counterpart: a command buffer with vkCmdDispatchDataGraphARM recorded once and submitted many times
 * (graph/graph_layer.cpp:1844-1980).  With profiling enabled the dispatch runs eagerly (per-operator events). */
int mlel_graph_session_dispatch_replayed(mlel_graph_session *s, void *stream);
/* The operators `first` .. `first + count - 1` of the executed list only (profiling single layers). */
int mlel_graph_session_dispatch_range(mlel_graph_session *s, void *stream, int first, int count);

/* Dispatch with a pair of events around every operator; per-operator milliseconds are written to `ms`
 * (reference: the profiler's timestamp pairs, graph/graph_profiler.cpp:157-191).  Returns the operator count. */
int mlel_graph_dispatch_profiled(mlel_graph *g, void *stream, float *ms, int capacity);
/* Per-operator profiling of every mlel_graph_dispatch (reference: GraphProfiler, enabled by the environment variable
 * VMEL_GRAPH_PROFILING, graph/graph_profiler.cpp:107; a new graph takes its default from the same variable).  A
 * profiled dispatch waits for its own events.  mlel_graph_profiling_json writes the report of
 * graph/graph_profiler.cpp:563-625 ("samples", "by_operator"; no cycle counts: times come from event pairs) into
 * `buf` (truncated to `capacity`) and returns the number of bytes the whole text needs, or a negative status. */
int mlel_graph_set_profiling(mlel_graph *g, int enabled);
int mlel_graph_get_profiling(mlel_graph *g);
int64_t mlel_graph_profiling_json(mlel_graph *g, char *buf, size_t capacity);

/* The graph layer's log (reference: graphLog, graph/graph_log.cpp:19, common/log.cpp:29-87).  The environment variable
 * VMEL_GRAPH_SEVERITY = Error | Warning | Info | Debug (case-insensitive, default Error) is read when the first message
 * is considered; lines go to standard output as "<date> <time>,<ms> [Graph][<severity>] <text>".  Info: one line per
 * decoded TOSA instruction (graph_tosa_1_0_ext_inst.cpp:453-457), the memory planner in use (graph_layer.cpp:286-295),
 * a summary per created pipeline; Error: every failure a mlel_graph_* call reports; Debug: tensor creation
 * (graph/tensor.cpp:90).  mlel_graph_log_level returns 0 .. 3 for Error .. Debug; mlel_graph_log_reload reads the
 * variable again and returns the new level. */
int mlel_graph_log_level(void);
int mlel_graph_log_reload(void);

/* Introspection (tests, profiler). */
int mlel_graph_op_count(mlel_graph *g);        /* operators executed after fusion */
int mlel_graph_op_name(mlel_graph *g, int index, char *buf, size_t len); /* "CONV2D+RESCALE+CLAMP", ... */
int mlel_graph_session_tensor_count(mlel_graph *g);
/* offset == UINT64_MAX: the tensor was folded into a fused kernel and has no storage */
int mlel_graph_session_tensor_info(mlel_graph *g, int index, int *tensor, uint64_t *offset, uint64_t *size,
                                   uint32_t *first_use, uint32_t *last_use);

/* The interval allocator on its own (reference: details::allocateIntervals, interval_memory_planner.cpp:170-215).
 * intervals: n x {id, first, last, size, order}; unseen: m x {id, size}; out_offsets: (n + m) x {id, offset}. */
int mlel_graph_allocate_intervals(const uint64_t *intervals, int n, const uint64_t *unseen, int m,
                                  uint64_t alignment, uint64_t *out_offsets, uint64_t *out_memory_size);

/* VkFormat number -> mlel_dtype (reference: getFormatInfo, common/utils.cpp:119-228); negative when unsupported. */
int mlel_graph_dtype_from_vk_format(int32_t vk_format);

#ifdef __cplusplus
}
#endif
#endif /* MLEL_GRAPH_H */
