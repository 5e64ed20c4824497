// Host-side operator surface of the TOSA data-graph backend.
//
// class GraphPipeline mirrors the reference's class of the same name (graph/compute_graph_op.hpp:1204-1549): the
// SPIR-V graph decoder (graph/graph_tosa_1_0_ext_inst.cpp) calls make<Op>() once per TOSA instruction, the layer
// registers constants / external tensors / session tensors through makeConstTensor, makeDescriptorSetBinding and
// makeTensor, and finally dispatches.  Where the reference builds one VkPipeline per operator and records
// vkCmdDispatch (compute_graph_op.cpp:526-590, 2500-2509), this class records an operator node and, at dispatch,
// calls the C ABI of include/mlel_hip.h, which launches hand-written gfx950 kernels.
//
// Differences that follow from running on HIP instead of Vulkan:
//   * tensors are (device pointer, dims, byte strides); the element type is mlel_dtype (the VkFormat -> type table
//     of common/utils.cpp:119-228 is provided by dtypeFromVkFormat());
//   * finalize() runs a fusion pass (CONV2D/DEPTHWISE_CONV2D/MATMUL + RESCALE [+ CLAMP] into one launch,
//     RESCALE + RESCALE + ADD + RESCALE into one launch; the fused kernels are bit-identical to the sequence) and
//     the interval memory planner over the fused operator list;
//   * dispatch(stream) replaces cmdBindAndDispatch(commandBuffer, ...): operators run in creation order on one HIP
//     stream, which gives the same ordering the reference enforces with a barrier on every input tensor.
#pragma once

#include <array>
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/mlel_hip.h"
#include "session_planner.hpp"

namespace mlel::graph {

using real_t = double;  // reference: common/include/mlel/float.hpp (double unless VMEL_USE_FLOAT_AS_DOUBLE)

// VkFormat values of the tensor formats the reference accepts (Vulkan-Headers; only the numbers are used here).
enum VkFormatValue : int32_t {
    VK_FORMAT_R8_UINT = 13,
    VK_FORMAT_R8_SINT = 14,
    VK_FORMAT_R16_UINT = 74,
    VK_FORMAT_R16_SINT = 75,
    VK_FORMAT_R16_SFLOAT = 76,
    VK_FORMAT_R32_UINT = 98,
    VK_FORMAT_R32_SINT = 99,
    VK_FORMAT_R32_SFLOAT = 100,
    VK_FORMAT_R64_UINT = 110,
    VK_FORMAT_R64_SINT = 111,
    VK_FORMAT_R64_SFLOAT = 112,
    VK_FORMAT_S8_UINT = 127,
    VK_FORMAT_R8_BOOL_ARM = 1000460000,
};
// Throws std::runtime_error("Unsupported tensor buffer format: <n>") like getFormatInfo (common/utils.cpp:185).
mlel_dtype dtypeFromVkFormat(int32_t vkFormat);
size_t dtypeSize(int32_t dtype);

enum class TensorKind { Session, Constant, External };

class OpNode;

// Reference counterpart: class TensorDescriptor (graph/tensor.hpp, graph/tensor.cpp:70-114,185-255).
class TensorDescriptor {
  public:
    TensorDescriptor(int32_t dtype, std::vector<int64_t> dimensions, std::vector<int64_t> strides, TensorKind kind);

    int32_t getFormat() const { return dtype; }
    const std::vector<int64_t> &getDimensions() const { return dimensions; }
    const std::vector<int64_t> &getStrides() const { return strides; }
    uint32_t getRank() const { return static_cast<uint32_t>(dimensions.size()); }
    size_t getShapeSize() const;
    size_t getSize() const;  // dims[0] * strides[0]: the extent in bytes (reference: tensor.cpp:197-203)
    TensorKind getKind() const { return kind; }
    bool isPacked() const;

    OpNode *getProducer() const { return producer; }
    void setProducer(OpNode *op) { producer = op; }

    void *devicePointer() const { return ptr; }
    void bind(void *devicePtr) { ptr = devicePtr; }
    mlel_tensor view() const;

    int id = -1;  // handle used by the C API
    bool isGraphInput = false, isGraphOutput = false;

  private:
    int32_t dtype;
    std::vector<int64_t> dimensions;
    std::vector<int64_t> strides;
    TensorKind kind;
    OpNode *producer = nullptr;
    void *ptr = nullptr;
};
using TensorPtr = std::shared_ptr<TensorDescriptor>;

enum class OpKind {
    Conv2D, DepthwiseConv2D, Matmul, Rescale, Clamp, Binary, Mul, Unary, Reduce, AvgPool2D, MaxPool2D, Table, Cast,
    Negate, Reshape, Transpose, Concat, Slice, Pad,
    Argmax, ArithmeticRightShift, Conv3D, TransposeConv2D, Fft2D, Rfft2D, Gather, Scatter, Resize, Reverse, Tile, Select,
    // produced by the fusion pass only
    FusedConv2D, FusedDepthwiseConv2D, FusedMatmul, FusedRescaleAddRescale, FusedMatmulBiasCast, FusedElementwise,
    FusedConv2DResidual, FusedAttention, FusedConv2DDepthwise, FusedConv2DConv2D, FusedConv2DAvgPool,
};

struct RescaleSpec {
    TensorPtr multiplier, shift;
    mlel_rescale_attr attr{};
};

// One recorded operator.  Reference counterpart: the ComputePipeline subclasses (compute_graph_op.hpp:226-1198).
class OpNode {
  public:
    OpKind kind{};
    std::string tosaName;   // "CONV2D", "RESCALE", ... as in graph_tosa_1_0_ext_inst.cpp:41-108
    std::string debugName;
    std::vector<TensorPtr> inputs;   // data inputs first, then parameter tensors (weights, bias, multiplier ...)
    std::vector<TensorPtr> outputs;
    std::vector<const TensorDescriptor *> originalTensors;  // operands as recorded, before any fusion
    // attributes (a plain union-of-fields record; only the fields of `kind` are meaningful)
    mlel_conv2d_attr conv{};
    mlel_matmul_attr matmul{};
    mlel_rescale_attr rescale{};
    mlel_clamp_attr clamp{};
    mlel_pool2d_attr pool{};
    mlel_conv3d_attr conv3d{};
    mlel_tconv2d_attr tconv{};
    mlel_resize_attr resize{};
    bool flag = false;  // ARITHMETIC_RIGHT_SHIFT: round; FFT2D: inverse
    std::vector<mlel_chain_step> chain;  // FusedElementwise: the program over `inputs` (see mlel_chain)
    int32_t selector = 0;  // mlel_binary_op / mlel_unary_op / mlel_reduce_op
    uint32_t nanMode = MLEL_NAN_PROPAGATE, axis = 0, shift = 0, offset = 0;
    int32_t inputZeroPoint = 0, outputZeroPoint = 0, padConstInt = 0;
    real_t padConst = 0;
    std::array<uint32_t, MLEL_MAX_RANK> vec{};  // perms / start
    // fusion results
    bool fusedAway = false;          // folded into another node; not executed
    RescaleSpec epilogue;            // Fused*: RESCALE applied to the accumulator
    bool hasClamp = false;           // Fused*: CLAMP after the RESCALE
    bool hasBias = false;            // FusedMatmulBiasCast: inputs[2] is the fp32 bias; `flag`: the last input is an
                                     // fp16 residual added to the rounded result
    // FusedMatmulBiasCast whose result is written through a view [NB1, NB2, M1, M2, N1, N2] of the output tensor's
    // storage (a RESHAPE -> TRANSPOSE behind the product folded into its stores); extents 0: no view
    std::array<int64_t, 6> viewDims{}, viewStrides{};
    // FusedMatmulBiasCast that computes several products of inputs[0] in one launch: product k > 0 reads the inputs
    // appended for it (its B, then its bias when hasBias), writes outputs[k], through the view k - 1 of this list
    // when that view's extents are non-zero
    std::vector<std::pair<std::array<int64_t, 6>, std::array<int64_t, 6>>> extraProductViews;
    // FusedAttention: inputs = {q, kt, v, the softmax chain's inputs from 1 on}; `chain` is the softmax region between
    // the two products (its value 0 is the first product); viewDims / viewStrides as for FusedMatmulBiasCast
    RescaleSpec scaleA, scaleB;      // FusedRescaleAddRescale: the two input stages (epilogue = output stage)
    // FusedConv2DResidual: epilogue (+ clamp) belongs to the convolution; scaleA rescales its 8-bit result, scaleB the
    // residual (inputs[3]), scaleOut their sum; `flag` is set when the residual was the addition's first operand
    RescaleSpec scaleOut;
    // FusedConv2DDepthwise: inputs = {x, the 1x1 convolution's weights and bias, the depthwise weights and bias};
    // conv / epilogue / hasClamp / clamp belong to the depthwise stage, convFirst / scaleA / hasClampFirst /
    // clampFirst to the 1x1 convolution in front of it
    // FusedConv2DConv2D: two 1x1 convolutions in a row; inputs = {x, the first convolution's weights and bias, the
    // second's}; conv / epilogue / hasClamp / clamp belong to the second, convFirst / scaleA / hasClampFirst / clampFirst
    // to the first; outputs[1], when present, is the first convolution's result, which a later operator reads too
    // FusedConv2DAvgPool: a 1x1 convolution (+RESCALE, +CLAMP) and the AVG_POOL2D over all positions behind it; inputs =
    // {x, weights, bias}; conv / epilogue / hasClamp / clamp belong to the convolution, pool to the pooling, selector
    // is the type the convolution's result had
    mlel_conv2d_attr convFirst{};
    mlel_clamp_attr clampFirst{};
    bool hasClampFirst = false;
};

class GraphPipeline {
  public:
    explicit GraphPipeline(mlel_ctx *ctx);
    ~GraphPipeline();
    GraphPipeline(const GraphPipeline &) = delete;
    GraphPipeline &operator=(const GraphPipeline &) = delete;

    // ---- constant tensors owned by the pipeline; the data is copied (reference: compute_graph_op.cpp:2398-2420)
    void makeConstTensor(uint32_t id, int32_t dtype, const std::vector<int64_t> &dimensions,
                         const std::vector<int64_t> &strides, const void *data);
    TensorPtr getConstTensor(uint32_t id) const;  // throws std::out_of_range like the reference's map::at
    TensorPtr makeConstCompositeTensor(int32_t dtype, std::vector<int64_t> dimensions, const void *data);

    // ---- external tensors owned by the application (reference: compute_graph_op.cpp:2441-2455)
    void makeDescriptorSetBinding(uint32_t set, uint32_t binding, uint32_t arrayIndex, int32_t dtype,
                                  const std::vector<int64_t> &dimensions, const std::vector<int64_t> &strides);
    TensorPtr getTensor(uint32_t set, uint32_t binding, uint32_t arrayIndex = 0) const;

    // ---- tensors allocated in session RAM (reference: compute_graph_op.cpp:2457-2471)
    TensorPtr makeTensor(int32_t dtype, std::vector<int64_t> dimensions = {}, std::vector<int64_t> strides = {});
    const std::vector<TensorPtr> &getTensors() const { return tensors; }

    void makeInput(const TensorPtr &tensor);
    void makeOutput(const TensorPtr &tensor);
    const std::vector<TensorPtr> &getInputs() const { return inputs; }
    const std::vector<TensorPtr> &getOutputs() const { return outputs; }
    const std::vector<std::shared_ptr<OpNode>> &getPipelines() const { return ops; }

    // ---- TOSA operators: names, argument order and meaning as in compute_graph_op.hpp:1249-1483
    void makeAbs(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeAdd(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output, const std::string &debugName);
    void makeArgmax(const TensorPtr &input, const TensorPtr &output, uint32_t axis, uint32_t nanMode,
                    const std::string &debugName);
    void makeArithmeticRightShift(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output, bool round,
                                  const std::string &debugName);
    void makeAvgPool2D(const TensorPtr &input, const TensorPtr &output, const std::vector<int32_t> &kernel,
                       const std::vector<int32_t> &stride, const std::vector<int32_t> &pad, uint32_t accType,
                       int8_t inputZeroPoint, int8_t outputZeroPoint, const std::string &debugName);
    void makeBitwiseAnd(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                        const std::string &debugName);
    void makeBitwiseNot(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeBitwiseOr(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                       const std::string &debugName);
    void makeBitwiseXor(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                        const std::string &debugName);
    void makeCast(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeCeil(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeClamp(const TensorPtr &input, const TensorPtr &output, real_t min, real_t max, uint32_t nanMode,
                   const std::string &debugName);
    void makeClz(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeConcat(const std::vector<TensorPtr> &inputs, const TensorPtr &output, uint32_t axis,
                    const std::string &debugName);
    void makeConv2D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights, const TensorPtr &biases,
                    const std::vector<int32_t> &pad, const std::vector<int32_t> &stride,
                    const std::vector<int32_t> &dilation, int8_t inputZeroPoint, int8_t weightZeroPoint,
                    uint32_t accType, const std::string &debugName);
    void makeConv3D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights, const TensorPtr &biases,
                    const std::vector<int32_t> &pad, const std::vector<int32_t> &stride,
                    const std::vector<int32_t> &dilation, int8_t inputZeroPoint, int8_t weightZeroPoint,
                    uint32_t accType, const std::string &debugName);
    void makeCos(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeDepthwiseConv2D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights,
                             const TensorPtr &biases, const std::vector<int32_t> &pad,
                             const std::vector<int32_t> &stride, const std::vector<int32_t> &dilation,
                             int8_t inputZeroPoint, int8_t weightZeroPoint, uint32_t accType,
                             const std::string &debugName);
    void makeEqual(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                   const std::string &debugName);
    void makeErf(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeExp(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeFft2D(const TensorPtr &inputReal, const TensorPtr &inputImag, const TensorPtr &outputReal,
                   const TensorPtr &outputImag, bool inverse, const std::string &debugName);
    void makeFloor(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeGather(const TensorPtr &values, const TensorPtr &indices, const TensorPtr &output,
                    const std::string &debugName);
    void makeGreater(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                     const std::string &debugName);
    void makeGreaterEqual(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                          const std::string &debugName);
    void makeIntdiv(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                    const std::string &debugName);
    void makeLog(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeLogicalAnd(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                        const std::string &debugName);
    void makeLogicalLeftShift(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                              const std::string &debugName);
    void makeLogicalNot(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeLogicalRightShift(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                               const std::string &debugName);
    void makeLogicalOr(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                       const std::string &debugName);
    void makeLogicalXor(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                        const std::string &debugName);
    void makeMaximum(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output, uint32_t nanMode,
                     const std::string &debugName);
    void makeMinimum(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output, uint32_t nanMode,
                     const std::string &debugName);
    void makeMatmul(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output, int32_t inputZeroPoint1,
                    int32_t inputZeroPoint2, const std::string &debugName);
    void makeMaxPool2D(const TensorPtr &input, const TensorPtr &output, const std::vector<int32_t> &kernel,
                       const std::vector<int32_t> &stride, const std::vector<int32_t> &pad, uint32_t nanMode,
                       const std::string &debugName);
    void makeMul(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output, uint32_t shift,
                 const std::string &debugName);
    void makeNegate(const TensorPtr &input, const TensorPtr &output, int32_t inputZeroPoint, int32_t outputZeroPoint,
                    const std::string &debugName);
    void makePad(const TensorPtr &input, const TensorPtr &output, const TensorPtr &padding, real_t padConst,
                 int32_t padConstInt, const std::string &debugName);
    void makePow(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                 const std::string &debugName);
    void makeReciprocal(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeReduceAll(const TensorPtr &input, const TensorPtr &output, uint32_t axis, const std::string &debugName);
    void makeReduceAny(const TensorPtr &input, const TensorPtr &output, uint32_t axis, const std::string &debugName);
    void makeReduceMax(const TensorPtr &input, const TensorPtr &output, uint32_t axis, uint32_t nanMode,
                       const std::string &debugName);
    void makeReduceMin(const TensorPtr &input, const TensorPtr &output, uint32_t axis, uint32_t nanMode,
                       const std::string &debugName);
    void makeReduceProduct(const TensorPtr &input, const TensorPtr &output, uint32_t axis,
                           const std::string &debugName);
    void makeReduceSum(const TensorPtr &input, const TensorPtr &output, uint32_t axis, const std::string &debugName);
    void makeRescale(const TensorPtr &input, const TensorPtr &output, int32_t inputZeroPoint, int32_t outputZeroPoint,
                     const TensorPtr &multiplier, const TensorPtr &shift, bool scale32, bool doubleRound,
                     bool perChannel, bool inputUnsigned, bool outputUnsigned, const std::string &debugName);
    void makeReshape(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeResize(const TensorPtr &input, const TensorPtr &output, const std::vector<int32_t> &scale,
                    const std::vector<int32_t> &offset, const std::vector<int32_t> &border, uint32_t mode,
                    const std::string &debugName);
    void makeReverse(const TensorPtr &input, const TensorPtr &output, uint32_t axis, const std::string &debugName);
    void makeRfft2D(const TensorPtr &input, const TensorPtr &outputReal, const TensorPtr &outputImag,
                    const std::string &debugName);
    void makeRsqrt(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeScatter(const TensorPtr &input, const TensorPtr &values, const TensorPtr &indices,
                     const TensorPtr &output, const std::string &debugName);
    void makeSelect(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &input3, const TensorPtr &output,
                    const std::string &debugName);
    void makeSigmoid(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeSin(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeSlice(const TensorPtr &input, const TensorPtr &output, const std::vector<uint32_t> &start,
                   const std::string &debugName);
    void makeSub(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                 const std::string &debugName);
    void makeTable(const TensorPtr &input, const TensorPtr &output, const TensorPtr &table,
                   const std::string &debugName);
    void makeTanh(const TensorPtr &input1, const TensorPtr &output, const std::string &debugName);
    void makeTile(const TensorPtr &input, const TensorPtr &output, const std::string &debugName);
    void makeTranspose(const TensorPtr &input, const TensorPtr &output, const std::vector<uint32_t> &perms,
                       const std::string &debugName);
    void makeTransposeConv2D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights,
                             const TensorPtr &biases, const std::vector<int32_t> &pad,
                             const std::vector<int32_t> &stride, int8_t inputZeroPoint, int8_t weightZeroPoint,
                             uint32_t accType, const std::string &debugName);

    // ---- HIP side ------------------------------------------------------------------------------------------
    // Runs the fusion pass (unless disabled) and plans session memory.  Called once, after the last make<Op>().
    // Session-memory planner (reference: GraphPipelineSession::createMemoryPlanner, graph_layer.cpp:282-297).  The
    // default is read from VMEL_MEMORY_PLANNER ("Linear", "BestFit", anything else: the interval planner) when the
    // pipeline is created; set before finalize().
    enum class MemoryPlanner { Interval, Linear, BestFit };
    void setMemoryPlanner(MemoryPlanner p);
    MemoryPlanner memoryPlanner() const { return planner; }
    void finalize(bool enableFusion = true);
    bool isFinalized() const { return finalized; }
    // Batch split (opt-in, set before finalize()).  The reference records a graph as one chain of dispatches
    // (cmdBindAndDispatch, compute_graph_op.cpp:2379-2521); on a GPU of 256 compute units a chain of short dependent
    // launches leaves most of the machine idle.  With the split the leading run of operators that treat the images of
    // a batch independently (convolutions, depthwise convolutions, pooling, RESCALE / CLAMP / TABLE, the residual
    // additions; activations [N, ...] with N even) is issued as two launches each, over the first and the second half
    // of the batch, on two streams that fork at the start of the dispatch and join behind the run; the operators
    // after it run on whole tensors as before.  Every launch computes the bytes it computes unsplit.  Session
    // tensors that only the run touches live in two regions, one per half, planned like a graph of half the batch, so
    // the two streams never share a byte while they are out of step; everything else keeps one contiguous
    // allocation.  Interval and linear planners only (the best-fit planner's sharing rules assume one chain).
    void setBatchSplit(bool enabled);
    bool batchSplitRequested() const { return splitRequested; }
    uint32_t batchSplitLaunches() const { return splitPrefix - splitFirst; }  // executed operators issued per half (0: not split)
    uint32_t batchSplitFirst() const { return splitFirst; }
    struct SplitLane {  // the second stream of a split dispatch and its fork / join events (owned by the session)
        void *stream = nullptr, *fork = nullptr, *join = nullptr;
    };
    // Session memory requirements (reference: vkGetDataGraphPipelineSessionMemoryRequirementsARM,
    // graph_layer.cpp:1382-1389): size and alignment of the one allocation all intermediates live in.
    size_t sessionMemorySize() const { return sessionSize; }
    size_t sessionMemoryAlignment() const { return kSessionAlignment; }
    // Reference: vkBindDataGraphPipelineSessionMemoryARM -> bindGraphPipelineSessionMemory
    // (interval_memory_planner.cpp:251-272): every planned tensor is bound at base + its offset.
    void bindSessionMemory(void *deviceBase);
    // External tensors may be re-bound between dispatches (update-after-bind in the reference).
    void bindExternal(uint32_t set, uint32_t binding, uint32_t arrayIndex, void *devicePtr);
    // Reference: cmdBindAndDispatch (compute_graph_op.cpp:2500-2509).  The decorator, when set, brackets every
    // executed operator (the reference's ComputePipelineDispatchDecorator, used by its profiler).
    using DispatchDecorator = std::function<void(const OpNode &, uint32_t index, bool before)>;
    // `first` / `count` select a run of the executed operators (positions in executionList()); profiling tools time
    // single operators with it.
    // `lane`: with a batch split, the half-batch launches of the second half go to the lane's stream (a whole
    // dispatch without decorator only; otherwise, and without a lane, both halves are issued to `stream` in turn).
    void dispatch(void *stream, const DispatchDecorator &decorator = {}, uint32_t first = 0, uint32_t count = UINT32_MAX,
                  const SplitLane *lane = nullptr);

    // introspection used by tests and the profiler
    std::vector<const OpNode *> executionList() const;
    const std::map<const TensorDescriptor *, size_t> &sessionOffsets() const { return offsets; }
    std::vector<std::array<uint32_t, 2>> liveRanges() const;  // per getTensors() entry: {first, last} or {~0,~0}

    static constexpr size_t kSessionAlignment = 256;

  private:
    std::shared_ptr<OpNode> addOp(OpKind kind, const char *tosaName, const std::string &debugName,
                                  std::vector<TensorPtr> ins, std::vector<TensorPtr> outs);
    void makeBinary(int32_t op, const char *name, const TensorPtr &a, const TensorPtr &b, const TensorPtr &out,
                    uint32_t nanMode, const std::string &debugName);
    void makeUnary(int32_t op, const char *name, const TensorPtr &in, const TensorPtr &out,
                   const std::string &debugName);
    void makeReduce(int32_t op, const char *name, const TensorPtr &in, const TensorPtr &out, uint32_t axis,
                    uint32_t nanMode, const std::string &debugName);
    TensorPtr registerTensor(TensorPtr t);
    void *uploadConstant(const TensorDescriptor &t, const void *data);
    void fuse();
    void prepackConstants();
    void plan();
    std::vector<details::BestFitTensor> bestFitTensors(const std::vector<details::LiveInterval> &planned,
                                                       const std::vector<details::UnseenAllocation> &unseen);
    void run(const OpNode &op, void *stream, int half = -1);  // half 0 / 1: that half of the batch (split run only)
    void analyzeBatchSplit();
    void validateSplitPlan() const;
    [[noreturn]] void unsupported(const char *tosaName) const;

    mlel_ctx *ctx;
    std::vector<std::shared_ptr<OpNode>> ops;
    std::vector<TensorPtr> tensors;             // session tensors in creation order
    std::set<TensorPtr> tensorSet;
    std::vector<TensorPtr> allTensors;          // every tensor this pipeline knows (handles)
    std::map<uint32_t, TensorPtr> constTensorMap;
    std::vector<TensorPtr> compositeTensors;
    std::map<uint32_t, std::map<uint32_t, std::vector<TensorPtr>>> tensorMap;  // set -> binding -> array
    std::vector<void *> constantsDeviceMemory;
    std::vector<TensorPtr> inputs, outputs;
    std::map<const TensorDescriptor *, size_t> offsets;
    std::map<const TensorDescriptor *, std::array<uint32_t, 2>> ranges;
    std::map<const TensorDescriptor *, const TensorDescriptor *> aliasOf;  // elided RESHAPE: output -> input
    size_t sessionSize = 0;
    bool splitRequested = false;
    uint32_t splitFirst = 0;      // executed operators [splitFirst, splitPrefix) are issued as two half-batch launches
    uint32_t splitPrefix = 0;
    int64_t splitBatch = 0;       // N of the activations of that run
    size_t splitFullRegion = 0;   // session memory: [whole tensors | first halves | second halves]
    size_t splitHalfRegion = 0;
    std::set<const TensorDescriptor *> splitInterior;  // session tensors stored as two halves, one per region
    MemoryPlanner planner = MemoryPlanner::Interval;
    bool finalized = false;

    friend class CApi;
    friend class GraphSession;
    const class GraphSession *appliedSession = nullptr;  // whose bindings the tensor descriptors hold right now
    uint64_t appliedVersion = 0;
  public:
    const std::vector<TensorPtr> &handles() const { return allTensors; }
};

// One session of a pipeline: its own transient (session) memory and its own external tensor bindings, so that several
// sessions of one pipeline can be in flight at the same time, each on its own stream.  Reference counterpart:
// DataGraphPipelineSessionARM (graph/graph_layer.cpp:215-330; entry points :1297-1425).  A session is used from the
// thread that uses its pipeline (neither is locked, as in the reference); pointers are resolved on the host when a
// dispatch is issued, so dispatches of different sessions issued one after the other overlap on the GPU.
class GraphSession {
  public:
    explicit GraphSession(GraphPipeline &pipeline);  // the pipeline must be finalized and outlive the session
    ~GraphSession();
    GraphSession(const GraphSession &) = delete;
    GraphSession &operator=(const GraphSession &) = delete;

    // reference: needsTransientRequirements (graph_layer.cpp:239-241): a graph without intermediates needs none
    bool needsTransientMemory() const { return pipeline.sessionMemorySize() != 0; }
    size_t memorySize() const { return pipeline.sessionMemorySize(); }
    size_t memoryAlignment() const { return pipeline.sessionMemoryAlignment(); }
    // reference: bindTransientMemory (graph_layer.cpp:260-271)
    void bindTransientMemory(void *deviceBase);
    // external tensors of this session; may be re-bound between dispatches (update-after-bind)
    void bindExternal(uint32_t set, uint32_t binding, uint32_t arrayIndex, void *devicePtr);
    // reference: vkCmdDispatchDataGraphARM with this session (graph_layer.cpp:1844-1980)
    void dispatch(void *stream, const GraphPipeline::DispatchDecorator &decorator = {}, uint32_t first = 0,
                  uint32_t count = UINT32_MAX);
    // The same launches, recorded into a HIP graph the first time (and again after a bind or on another stream) and
    // replayed with one submission afterwards: the host side of a dispatch shrinks from one launch call per operator
    // to one.  Reference counterpart: a command buffer with vkCmdDispatchDataGraphARM recorded once and submitted
    // many times (graph_layer.cpp:1844-1980).
    void dispatchReplayed(void *stream);

  private:
    void apply();
    void dropRecording();
    void *recording = nullptr;       // the instantiated HIP graph of this session's dispatch
    void *recordingStream = nullptr;
    uint64_t recordingVersion = 0;
    const GraphPipeline::SplitLane *lane();  // created on first use when the pipeline splits the batch
    GraphPipeline::SplitLane splitLane;
    uint64_t eagerVersion = UINT64_MAX;  // bindings under which recording failed: replayed dispatches run eagerly
    void *eagerStream = nullptr;
    GraphPipeline &pipeline;
    void *base = nullptr;
    bool transientMemoryBound = false;
    std::map<TensorDescriptor *, void *> externals;
    uint64_t version = 1;  // bumped by every bind: the pipeline re-applies the bindings only when they changed
};

}  // namespace mlel::graph
