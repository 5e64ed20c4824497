#include "graph_pipeline.hpp"

#include "graph_log.hpp"

#include <cstdlib>

#include <algorithm>
#include <cstring>
#include <map>
#include <unordered_map>

#include "session_planner.hpp"

namespace mlel::graph {

namespace {

[[noreturn]] void fail(const std::string &what) { throw std::runtime_error(what); }

void check(int rc, const char *what) {
    if (rc != 0) fail(std::string(what) + ": " + mlel_hip_last_error());
}

std::vector<int64_t> packedStrides(int32_t dtype, const std::vector<int64_t> &dims) {
    // reference: tensor/tensor_arm.cpp:82-92
    std::vector<int64_t> s(dims.size());
    int64_t v = static_cast<int64_t>(dtypeSize(dtype));
    for (size_t i = dims.size(); i-- > 0;) {
        s[i] = v;
        v *= dims[i];
    }
    return s;
}

}  // namespace

mlel_dtype dtypeFromVkFormat(const int32_t f) {
    switch (f) {
    case VK_FORMAT_R8_SINT: return MLEL_I8;
    case VK_FORMAT_R8_UINT:
    case VK_FORMAT_S8_UINT: return MLEL_U8;
    case VK_FORMAT_R8_BOOL_ARM: return MLEL_BOOL;
    case VK_FORMAT_R16_SINT: return MLEL_I16;
    case VK_FORMAT_R16_UINT: return MLEL_U16;
    case VK_FORMAT_R16_SFLOAT: return MLEL_F16;
    case VK_FORMAT_R32_SINT: return MLEL_I32;
    case VK_FORMAT_R32_UINT: return MLEL_U32;
    case VK_FORMAT_R32_SFLOAT: return MLEL_F32;
    case VK_FORMAT_R64_SINT: return MLEL_I64;
    case VK_FORMAT_R64_UINT: return MLEL_U64;
    case VK_FORMAT_R64_SFLOAT: return MLEL_F64;
    default: fail("Unsupported tensor buffer format: " + std::to_string(f));
    }
}

size_t dtypeSize(const int32_t dtype) {
    switch (dtype) {
    case MLEL_BOOL: case MLEL_I8: case MLEL_U8: case MLEL_F8E4M3: case MLEL_F8E5M2: return 1;
    case MLEL_I16: case MLEL_U16: case MLEL_F16: case MLEL_BF16: return 2;
    case MLEL_I32: case MLEL_U32: case MLEL_F32: return 4;
    case MLEL_I64: case MLEL_U64: case MLEL_F64: return 8;
    default: fail("Unsupported tensor element type: " + std::to_string(dtype));
    }
}

/*******************************************************************************
 * TensorDescriptor
 *******************************************************************************/

TensorDescriptor::TensorDescriptor(const int32_t _dtype, std::vector<int64_t> _dimensions,
                                   std::vector<int64_t> _strides, const TensorKind _kind)
    : dtype{_dtype}, dimensions{std::move(_dimensions)}, strides{std::move(_strides)}, kind{_kind} {
    (void)dtypeSize(dtype);
    if (dimensions.empty() || dimensions.size() > MLEL_MAX_RANK)
        fail("Tensor rank must be between 1 and " + std::to_string(MLEL_MAX_RANK));
    if (strides.empty()) strides = packedStrides(dtype, dimensions);
    if (strides.size() != dimensions.size()) fail("Tensor strides and dimensions differ in length");
    if (strides[0] < 0) fail("Strides must be greater than zero.");
}

size_t TensorDescriptor::getShapeSize() const {
    size_t n = 1;
    for (const auto d : dimensions) n *= static_cast<size_t>(d);
    return n;
}

size_t TensorDescriptor::getSize() const { return static_cast<size_t>(dimensions[0] * strides[0]); }

bool TensorDescriptor::isPacked() const { return strides == packedStrides(dtype, dimensions); }

mlel_tensor TensorDescriptor::view() const {
    mlel_tensor t{};
    t.ptr = ptr;
    t.dtype = dtype;
    t.rank = static_cast<int32_t>(dimensions.size());
    for (size_t i = 0; i < dimensions.size(); i++) {
        t.dims[i] = dimensions[i];
        t.strides[i] = strides[i];
    }
    return t;
}

/*******************************************************************************
 * GraphPipeline: tensors
 *******************************************************************************/

// A null context is accepted for building and planning a graph (host-side logic needs no device); constants are
// then not uploaded and dispatch() refuses to run.
GraphPipeline::GraphPipeline(mlel_ctx *_ctx) : ctx{_ctx} {
    if (const char *env = std::getenv("VMEL_MEMORY_PLANNER")) {
        if (std::string(env) == "Linear") planner = MemoryPlanner::Linear;
        if (std::string(env) == "BestFit") planner = MemoryPlanner::BestFit;
    }
}

GraphPipeline::~GraphPipeline() {
    if (ctx != nullptr)
        for (void *p : constantsDeviceMemory) (void)mlel_hip_arena_free(ctx, p);
}

TensorPtr GraphPipeline::registerTensor(TensorPtr t) {
    t->id = static_cast<int>(allTensors.size());
    allTensors.push_back(t);
    MLEL_GRAPH_LOG(Debug, "Create tensor. tensor=" << t->id << " dtype=" << t->getFormat() << " rank=" << t->getRank()
                                                   << " bytes=" << t->getSize());
    return t;
}

void *GraphPipeline::uploadConstant(const TensorDescriptor &t, const void *data) {
    if (data == nullptr || ctx == nullptr) return nullptr;  // reference: null data -> VK_NULL_HANDLE
    void *dptr = nullptr;
    check(mlel_hip_arena_alloc(ctx, t.getSize(), &dptr), "allocating constant tensor");
    constantsDeviceMemory.push_back(dptr);
    check(mlel_hip_memcpy_h2d(ctx, dptr, data, t.getSize(), nullptr), "uploading constant tensor");
    return dptr;
}

void GraphPipeline::makeConstTensor(const uint32_t id, const int32_t dtype, const std::vector<int64_t> &dimensions,
                                    const std::vector<int64_t> &strides, const void *data) {
    auto t = std::make_shared<TensorDescriptor>(dtype, dimensions, strides, TensorKind::Constant);
    t->bind(uploadConstant(*t, data));
    constTensorMap[id] = registerTensor(std::move(t));
}

TensorPtr GraphPipeline::getConstTensor(const uint32_t id) const { return constTensorMap.at(id); }

TensorPtr GraphPipeline::makeConstCompositeTensor(const int32_t dtype, std::vector<int64_t> dimensions,
                                                  const void *data) {
    auto t = std::make_shared<TensorDescriptor>(dtype, std::move(dimensions), std::vector<int64_t>{},
                                                TensorKind::Constant);
    t->bind(uploadConstant(*t, data));
    compositeTensors.push_back(registerTensor(t));
    return t;
}

void GraphPipeline::makeDescriptorSetBinding(const uint32_t set, const uint32_t binding, const uint32_t arrayIndex,
                                             const int32_t dtype, const std::vector<int64_t> &dimensions,
                                             const std::vector<int64_t> &strides) {
    auto t = std::make_shared<TensorDescriptor>(dtype, dimensions, strides, TensorKind::External);
    auto &vec = tensorMap[set][binding];
    vec.resize(std::max(vec.size(), static_cast<size_t>(arrayIndex) + 1));
    vec[arrayIndex] = registerTensor(std::move(t));
}

TensorPtr GraphPipeline::getTensor(const uint32_t set, const uint32_t binding, const uint32_t arrayIndex) const {
    return tensorMap.at(set).at(binding).at(arrayIndex);
}

TensorPtr GraphPipeline::makeTensor(const int32_t dtype, std::vector<int64_t> dimensions,
                                    std::vector<int64_t> strides) {
    auto t = std::make_shared<TensorDescriptor>(dtype, std::move(dimensions), std::move(strides), TensorKind::Session);
    if (tensorSet.insert(t).second) tensors.push_back(t);
    return registerTensor(t);
}

void GraphPipeline::makeInput(const TensorPtr &tensor) {
    tensor->isGraphInput = true;
    inputs.push_back(tensor);
}

void GraphPipeline::makeOutput(const TensorPtr &tensor) {
    tensor->isGraphOutput = true;
    outputs.push_back(tensor);
}

/*******************************************************************************
 * GraphPipeline: operators
 *******************************************************************************/

std::shared_ptr<OpNode> GraphPipeline::addOp(const OpKind kind, const char *tosaName, const std::string &debugName,
                                             std::vector<TensorPtr> ins, std::vector<TensorPtr> outs) {
    if (finalized) fail("GraphPipeline is finalized; no more operators can be added");
    for (const auto &t : ins)
        if (!t) fail(std::string(tosaName) + ": null input tensor");
    for (const auto &t : outs)
        if (!t) fail(std::string(tosaName) + ": null output tensor");
    auto op = std::make_shared<OpNode>();
    op->kind = kind;
    op->tosaName = tosaName;
    op->debugName = debugName;
    op->inputs = std::move(ins);
    op->outputs = std::move(outs);
    for (const auto &t : op->outputs) t->setProducer(op.get());
    for (const auto &t : op->inputs) op->originalTensors.push_back(t.get());
    for (const auto &t : op->outputs) op->originalTensors.push_back(t.get());
    ops.push_back(op);
    return op;
}

void GraphPipeline::unsupported(const char *tosaName) const {
    fail(std::string("TOSA operator ") + tosaName + " has no kernel on the HIP backend yet");
}

namespace {

mlel_conv2d_attr convAttr(const std::vector<int32_t> &pad, const std::vector<int32_t> &stride,
                          const std::vector<int32_t> &dilation, const int8_t zi, const int8_t zw,
                          const uint32_t accType) {
    if (pad.size() < 4 || stride.size() < 2 || dilation.size() < 2)
        fail("convolution: pad/stride/dilation need 4/2/2 values");
    if (accType < 1 || accType > 4) fail("Unsupported acc type " + std::to_string(accType));
    mlel_conv2d_attr a{};
    a.input_zp = zi;
    a.weight_zp = zw;
    for (int i = 0; i < 4; i++) a.pad[i] = pad[static_cast<size_t>(i)];
    for (int i = 0; i < 2; i++) {
        a.stride[i] = stride[static_cast<size_t>(i)];
        a.dilation[i] = dilation[static_cast<size_t>(i)];
    }
    a.acc_type = accType;
    return a;
}

mlel_pool2d_attr poolAttr(const std::vector<int32_t> &kernel, const std::vector<int32_t> &stride,
                          const std::vector<int32_t> &pad) {
    if (kernel.size() < 2 || stride.size() < 2 || pad.size() < 4) fail("pooling: kernel/stride/pad need 2/2/4 values");
    mlel_pool2d_attr a{};
    for (int i = 0; i < 2; i++) {
        a.kernel[i] = kernel[static_cast<size_t>(i)];
        a.stride[i] = stride[static_cast<size_t>(i)];
    }
    for (int i = 0; i < 4; i++) a.pad[i] = pad[static_cast<size_t>(i)];
    a.acc_type = MLEL_ACC_I32;
    a.nan_mode = MLEL_NAN_PROPAGATE;
    return a;
}

}  // namespace

void GraphPipeline::makeBinary(const int32_t op, const char *name, const TensorPtr &a, const TensorPtr &b,
                               const TensorPtr &out, const uint32_t nanMode, const std::string &debugName) {
    auto n = addOp(OpKind::Binary, name, debugName, {a, b}, {out});
    n->selector = op;
    n->nanMode = nanMode;
}

void GraphPipeline::makeUnary(const int32_t op, const char *name, const TensorPtr &in, const TensorPtr &out,
                              const std::string &debugName) {
    addOp(OpKind::Unary, name, debugName, {in}, {out})->selector = op;
}

void GraphPipeline::makeReduce(const int32_t op, const char *name, const TensorPtr &in, const TensorPtr &out,
                               const uint32_t axis, const uint32_t nanMode, const std::string &debugName) {
    auto n = addOp(OpKind::Reduce, name, debugName, {in}, {out});
    n->selector = op;
    n->axis = axis;
    n->nanMode = nanMode;
}

#define MLEL_UNARY(Method, Enum, Name)                                                                                 \
    void GraphPipeline::Method(const TensorPtr &i, const TensorPtr &o, const std::string &d) {                        \
        makeUnary(Enum, Name, i, o, d);                                                                                \
    }
MLEL_UNARY(makeAbs, MLEL_UN_ABS, "ABS")
MLEL_UNARY(makeBitwiseNot, MLEL_UN_BITWISE_NOT, "BITWISE_NOT")
MLEL_UNARY(makeCeil, MLEL_UN_CEIL, "CEIL")
MLEL_UNARY(makeClz, MLEL_UN_CLZ, "CLZ")
MLEL_UNARY(makeCos, MLEL_UN_COS, "COS")
MLEL_UNARY(makeErf, MLEL_UN_ERF, "ERF")
MLEL_UNARY(makeExp, MLEL_UN_EXP, "EXP")
MLEL_UNARY(makeFloor, MLEL_UN_FLOOR, "FLOOR")
MLEL_UNARY(makeLog, MLEL_UN_LOG, "LOG")
MLEL_UNARY(makeLogicalNot, MLEL_UN_LOGICAL_NOT, "LOGICAL_NOT")
MLEL_UNARY(makeReciprocal, MLEL_UN_RECIPROCAL, "RECIPROCAL")
MLEL_UNARY(makeRsqrt, MLEL_UN_RSQRT, "RSQRT")
MLEL_UNARY(makeSigmoid, MLEL_UN_SIGMOID, "SIGMOID")
MLEL_UNARY(makeSin, MLEL_UN_SIN, "SIN")
MLEL_UNARY(makeTanh, MLEL_UN_TANH, "TANH")
#undef MLEL_UNARY

#define MLEL_BINARY(Method, Enum, Name)                                                                                \
    void GraphPipeline::Method(const TensorPtr &a, const TensorPtr &b, const TensorPtr &o, const std::string &d) {    \
        makeBinary(Enum, Name, a, b, o, MLEL_NAN_PROPAGATE, d);                                                        \
    }
MLEL_BINARY(makeAdd, MLEL_BIN_ADD, "ADD")
MLEL_BINARY(makeSub, MLEL_BIN_SUB, "SUB")
MLEL_BINARY(makeBitwiseAnd, MLEL_BIN_BITWISE_AND, "BITWISE_AND")
MLEL_BINARY(makeBitwiseOr, MLEL_BIN_BITWISE_OR, "BITWISE_OR")
MLEL_BINARY(makeBitwiseXor, MLEL_BIN_BITWISE_XOR, "BITWISE_XOR")
MLEL_BINARY(makeIntdiv, MLEL_BIN_INTDIV, "INTDIV")
MLEL_BINARY(makeLogicalAnd, MLEL_BIN_LOGICAL_AND, "LOGICAL_AND")
MLEL_BINARY(makeLogicalOr, MLEL_BIN_LOGICAL_OR, "LOGICAL_OR")
MLEL_BINARY(makeLogicalXor, MLEL_BIN_LOGICAL_XOR, "LOGICAL_XOR")
MLEL_BINARY(makeLogicalLeftShift, MLEL_BIN_LOGICAL_LEFT_SHIFT, "LOGICAL_LEFT_SHIFT")
MLEL_BINARY(makeLogicalRightShift, MLEL_BIN_LOGICAL_RIGHT_SHIFT, "LOGICAL_RIGHT_SHIFT")
MLEL_BINARY(makePow, MLEL_BIN_POW, "POW")
MLEL_BINARY(makeEqual, MLEL_BIN_EQUAL, "EQUAL")
MLEL_BINARY(makeGreater, MLEL_BIN_GREATER, "GREATER")
MLEL_BINARY(makeGreaterEqual, MLEL_BIN_GREATER_EQUAL, "GREATER_EQUAL")
#undef MLEL_BINARY

void GraphPipeline::makeMaximum(const TensorPtr &a, const TensorPtr &b, const TensorPtr &o, const uint32_t nanMode,
                                const std::string &d) {
    makeBinary(MLEL_BIN_MAXIMUM, "MAXIMUM", a, b, o, nanMode, d);
}
void GraphPipeline::makeMinimum(const TensorPtr &a, const TensorPtr &b, const TensorPtr &o, const uint32_t nanMode,
                                const std::string &d) {
    makeBinary(MLEL_BIN_MINIMUM, "MINIMUM", a, b, o, nanMode, d);
}

void GraphPipeline::makeReduceAll(const TensorPtr &i, const TensorPtr &o, const uint32_t axis, const std::string &d) {
    makeReduce(MLEL_RED_ALL, "REDUCE_ALL", i, o, axis, MLEL_NAN_PROPAGATE, d);
}
void GraphPipeline::makeReduceAny(const TensorPtr &i, const TensorPtr &o, const uint32_t axis, const std::string &d) {
    makeReduce(MLEL_RED_ANY, "REDUCE_ANY", i, o, axis, MLEL_NAN_PROPAGATE, d);
}
void GraphPipeline::makeReduceMax(const TensorPtr &i, const TensorPtr &o, const uint32_t axis, const uint32_t nanMode,
                                  const std::string &d) {
    makeReduce(MLEL_RED_MAX, "REDUCE_MAX", i, o, axis, nanMode, d);
}
void GraphPipeline::makeReduceMin(const TensorPtr &i, const TensorPtr &o, const uint32_t axis, const uint32_t nanMode,
                                  const std::string &d) {
    makeReduce(MLEL_RED_MIN, "REDUCE_MIN", i, o, axis, nanMode, d);
}
void GraphPipeline::makeReduceProduct(const TensorPtr &i, const TensorPtr &o, const uint32_t axis,
                                      const std::string &d) {
    makeReduce(MLEL_RED_PRODUCT, "REDUCE_PRODUCT", i, o, axis, MLEL_NAN_PROPAGATE, d);
}
void GraphPipeline::makeReduceSum(const TensorPtr &i, const TensorPtr &o, const uint32_t axis, const std::string &d) {
    makeReduce(MLEL_RED_SUM, "REDUCE_SUM", i, o, axis, MLEL_NAN_PROPAGATE, d);
}

void GraphPipeline::makeAvgPool2D(const TensorPtr &input, const TensorPtr &output, const std::vector<int32_t> &kernel,
                                  const std::vector<int32_t> &stride, const std::vector<int32_t> &pad,
                                  const uint32_t accType, const int8_t inputZeroPoint, const int8_t outputZeroPoint,
                                  const std::string &debugName) {
    if (accType < 1 || accType > 4) fail("Unsupported AVG_POOL2D acc type " + std::to_string(accType));
    auto n = addOp(OpKind::AvgPool2D, "AVG_POOL2D", debugName, {input}, {output});
    n->pool = poolAttr(kernel, stride, pad);
    n->pool.acc_type = accType;
    n->pool.input_zp = inputZeroPoint;
    n->pool.output_zp = outputZeroPoint;
}

void GraphPipeline::makeMaxPool2D(const TensorPtr &input, const TensorPtr &output, const std::vector<int32_t> &kernel,
                                  const std::vector<int32_t> &stride, const std::vector<int32_t> &pad,
                                  const uint32_t nanMode, const std::string &debugName) {
    auto n = addOp(OpKind::MaxPool2D, "MAX_POOL2D", debugName, {input}, {output});
    n->pool = poolAttr(kernel, stride, pad);
    n->pool.nan_mode = nanMode;
}

void GraphPipeline::makeCast(const TensorPtr &input, const TensorPtr &output, const std::string &debugName) {
    addOp(OpKind::Cast, "CAST", debugName, {input}, {output});
}

void GraphPipeline::makeClamp(const TensorPtr &input, const TensorPtr &output, const real_t min, const real_t max,
                              const uint32_t nanMode, const std::string &debugName) {
    auto n = addOp(OpKind::Clamp, "CLAMP", debugName, {input}, {output});
    n->clamp = mlel_clamp_attr{min, max, nanMode};
}

void GraphPipeline::makeConcat(const std::vector<TensorPtr> &_inputs, const TensorPtr &output, const uint32_t axis,
                               const std::string &debugName) {
    // one operator per input with a running offset along `axis` (reference: compute_graph_op.cpp:2607-2615)
    uint32_t offset = 0;
    for (const auto &input : _inputs) {
        auto n = addOp(OpKind::Concat, "CONCAT", debugName, {input}, {output});
        n->axis = axis;
        n->offset = offset;
        if (axis >= input->getRank()) fail("CONCAT: axis outside the input rank");
        offset += static_cast<uint32_t>(input->getDimensions()[axis]);
    }
}

void GraphPipeline::makeConv2D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights,
                               const TensorPtr &biases, const std::vector<int32_t> &pad,
                               const std::vector<int32_t> &stride, const std::vector<int32_t> &dilation,
                               const int8_t inputZeroPoint, const int8_t weightZeroPoint, const uint32_t accType,
                               const std::string &debugName) {
    const auto attr = convAttr(pad, stride, dilation, inputZeroPoint, weightZeroPoint, accType);
    addOp(OpKind::Conv2D, "CONV2D", debugName, {input, weights, biases}, {output})->conv = attr;
}

void GraphPipeline::makeDepthwiseConv2D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights,
                                        const TensorPtr &biases, const std::vector<int32_t> &pad,
                                        const std::vector<int32_t> &stride, const std::vector<int32_t> &dilation,
                                        const int8_t inputZeroPoint, const int8_t weightZeroPoint,
                                        const uint32_t accType, const std::string &debugName) {
    const auto attr = convAttr(pad, stride, dilation, inputZeroPoint, weightZeroPoint, accType);
    addOp(OpKind::DepthwiseConv2D, "DEPTHWISE_CONV2D", debugName, {input, weights, biases}, {output})->conv = attr;
}

void GraphPipeline::makeMatmul(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                               const int32_t inputZeroPoint1, const int32_t inputZeroPoint2,
                               const std::string &debugName) {
    addOp(OpKind::Matmul, "MATMUL", debugName, {input1, input2}, {output})->matmul =
        mlel_matmul_attr{inputZeroPoint1, inputZeroPoint2};
}

void GraphPipeline::makeMul(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                            const uint32_t shift, const std::string &debugName) {
    addOp(OpKind::Mul, "MUL", debugName, {input1, input2}, {output})->shift = shift;
}

void GraphPipeline::makeNegate(const TensorPtr &input, const TensorPtr &output, const int32_t inputZeroPoint,
                               const int32_t outputZeroPoint, const std::string &debugName) {
    auto n = addOp(OpKind::Negate, "NEGATE", debugName, {input}, {output});
    n->inputZeroPoint = inputZeroPoint;
    n->outputZeroPoint = outputZeroPoint;
}

void GraphPipeline::makePad(const TensorPtr &input, const TensorPtr &output, const TensorPtr &padding,
                            const real_t padConst, const int32_t padConstInt, const std::string &debugName) {
    auto n = addOp(OpKind::Pad, "PAD", debugName, {input, padding}, {output});
    n->padConst = padConst;
    n->padConstInt = padConstInt;
}

void GraphPipeline::makeRescale(const TensorPtr &input, const TensorPtr &output, const int32_t inputZeroPoint,
                                const int32_t outputZeroPoint, const TensorPtr &multiplier, const TensorPtr &shift,
                                const bool scale32, const bool doubleRound, const bool perChannel,
                                const bool inputUnsigned, const bool outputUnsigned, const std::string &debugName) {
    auto n = addOp(OpKind::Rescale, "RESCALE", debugName, {input, multiplier, shift}, {output});
    n->rescale = mlel_rescale_attr{inputZeroPoint, outputZeroPoint, scale32, doubleRound, perChannel,
                                   inputUnsigned,  outputUnsigned};
}

void GraphPipeline::makeReshape(const TensorPtr &input, const TensorPtr &output, const std::string &debugName) {
    addOp(OpKind::Reshape, "RESHAPE", debugName, {input}, {output});
}

void GraphPipeline::makeSlice(const TensorPtr &input, const TensorPtr &output, const std::vector<uint32_t> &start,
                              const std::string &debugName) {
    auto n = addOp(OpKind::Slice, "SLICE", debugName, {input}, {output});
    if (start.size() < input->getRank()) fail("SLICE: start has fewer values than the tensor rank");
    for (uint32_t i = 0; i < input->getRank(); i++) n->vec[i] = start[i];
}

void GraphPipeline::makeTable(const TensorPtr &input, const TensorPtr &output, const TensorPtr &table,
                              const std::string &debugName) {
    addOp(OpKind::Table, "TABLE", debugName, {input, table}, {output});
}

void GraphPipeline::makeTranspose(const TensorPtr &input, const TensorPtr &output, const std::vector<uint32_t> &perms,
                                  const std::string &debugName) {
    auto n = addOp(OpKind::Transpose, "TRANSPOSE", debugName, {input}, {output});
    if (perms.size() < input->getRank()) fail("TRANSPOSE: perms has fewer values than the tensor rank");
    for (uint32_t i = 0; i < input->getRank(); i++) n->vec[i] = perms[i];
}

void GraphPipeline::makeArgmax(const TensorPtr &input, const TensorPtr &output, const uint32_t axis,
                               const uint32_t nanMode, const std::string &debugName) {
    auto n = addOp(OpKind::Argmax, "ARGMAX", debugName, {input}, {output});
    n->axis = axis;
    n->nanMode = nanMode;
}

void GraphPipeline::makeArithmeticRightShift(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &output,
                                             const bool round, const std::string &debugName) {
    addOp(OpKind::ArithmeticRightShift, "ARITHMETIC_RIGHT_SHIFT", debugName, {input1, input2}, {output})->flag = round;
}

void GraphPipeline::makeConv3D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights,
                               const TensorPtr &biases, const std::vector<int32_t> &pad,
                               const std::vector<int32_t> &stride, const std::vector<int32_t> &dilation,
                               const int8_t inputZeroPoint, const int8_t weightZeroPoint, const uint32_t accType,
                               const std::string &debugName) {
    if (pad.size() < 6 || stride.size() < 3 || dilation.size() < 3) fail("CONV3D: pad/stride/dilation need 6/3/3 values");
    auto n = addOp(OpKind::Conv3D, "CONV3D", debugName, {input, weights, biases}, {output});
    n->conv3d.input_zp = inputZeroPoint;
    n->conv3d.weight_zp = weightZeroPoint;
    for (int i = 0; i < 6; i++) n->conv3d.pad[i] = pad[static_cast<size_t>(i)];
    for (int i = 0; i < 3; i++) {
        n->conv3d.stride[i] = stride[static_cast<size_t>(i)];
        n->conv3d.dilation[i] = dilation[static_cast<size_t>(i)];
    }
    n->conv3d.acc_type = accType;
}

void GraphPipeline::makeTransposeConv2D(const TensorPtr &input, const TensorPtr &output, const TensorPtr &weights,
                                        const TensorPtr &biases, const std::vector<int32_t> &pad,
                                        const std::vector<int32_t> &stride, const int8_t inputZeroPoint,
                                        const int8_t weightZeroPoint, const uint32_t accType,
                                        const std::string &debugName) {
    if (pad.size() < 4 || stride.size() < 2) fail("TRANSPOSE_CONV2D: outPad/stride need 4/2 values");
    auto n = addOp(OpKind::TransposeConv2D, "TRANSPOSE_CONV2D", debugName, {input, weights, biases}, {output});
    n->tconv.input_zp = inputZeroPoint;
    n->tconv.weight_zp = weightZeroPoint;
    for (int i = 0; i < 4; i++) n->tconv.out_pad[i] = pad[static_cast<size_t>(i)];
    for (int i = 0; i < 2; i++) n->tconv.stride[i] = stride[static_cast<size_t>(i)];
    n->tconv.acc_type = accType;
}

void GraphPipeline::makeFft2D(const TensorPtr &inputReal, const TensorPtr &inputImag, const TensorPtr &outputReal,
                              const TensorPtr &outputImag, const bool inverse, const std::string &debugName) {
    addOp(OpKind::Fft2D, "FFT2D", debugName, {inputReal, inputImag}, {outputReal, outputImag})->flag = inverse;
}

void GraphPipeline::makeRfft2D(const TensorPtr &input, const TensorPtr &outputReal, const TensorPtr &outputImag,
                               const std::string &debugName) {
    addOp(OpKind::Rfft2D, "RFFT2D", debugName, {input}, {outputReal, outputImag});
}

void GraphPipeline::makeGather(const TensorPtr &values, const TensorPtr &indices, const TensorPtr &output,
                               const std::string &debugName) {
    addOp(OpKind::Gather, "GATHER", debugName, {values, indices}, {output});
}

// `input` is the [N, W, C] tensor whose rows are written into `values` [N, K, C] at the rows named by `indices`
void GraphPipeline::makeScatter(const TensorPtr &input, const TensorPtr &values, const TensorPtr &indices,
                                const TensorPtr &output, const std::string &debugName) {
    addOp(OpKind::Scatter, "SCATTER", debugName, {values, indices, input}, {output});
}

void GraphPipeline::makeResize(const TensorPtr &input, const TensorPtr &output, const std::vector<int32_t> &scale,
                               const std::vector<int32_t> &offset, const std::vector<int32_t> &border,
                               const uint32_t mode, const std::string &debugName) {
    if (scale.size() < 4 || offset.size() < 2 || border.size() < 2) fail("RESIZE: scale/offset/border need 4/2/2 values");
    auto n = addOp(OpKind::Resize, "RESIZE", debugName, {input}, {output});
    for (int i = 0; i < 4; i++) n->resize.scale[i] = scale[static_cast<size_t>(i)];
    for (int i = 0; i < 2; i++) {
        n->resize.offset[i] = offset[static_cast<size_t>(i)];
        n->resize.border[i] = border[static_cast<size_t>(i)];
    }
    n->resize.mode = mode;
}

void GraphPipeline::makeReverse(const TensorPtr &input, const TensorPtr &output, const uint32_t axis,
                                const std::string &debugName) {
    addOp(OpKind::Reverse, "REVERSE", debugName, {input}, {output})->axis = axis;
}

void GraphPipeline::makeSelect(const TensorPtr &input1, const TensorPtr &input2, const TensorPtr &input3,
                               const TensorPtr &output, const std::string &debugName) {
    addOp(OpKind::Select, "SELECT", debugName, {input1, input2, input3}, {output});
}

void GraphPipeline::makeTile(const TensorPtr &input, const TensorPtr &output, const std::string &debugName) {
    addOp(OpKind::Tile, "TILE", debugName, {input}, {output});
}

/*******************************************************************************
 * GraphPipeline: fusion
 *******************************************************************************/

namespace {

// operators (not folded away) that read `t`
std::vector<OpNode *> consumersOf(const std::vector<std::shared_ptr<OpNode>> &ops, const TensorDescriptor *t) {
    std::vector<OpNode *> r;
    for (const auto &op : ops) {
        if (op->fusedAway) continue;
        for (const auto &in : op->inputs)
            if (in.get() == t) {
                r.push_back(op.get());
                break;
            }
    }
    return r;
}

bool sameShape(const TensorDescriptor &a, const TensorDescriptor &b) { return a.getDimensions() == b.getDimensions(); }

// an intermediate may disappear only if nothing outside the fused group can observe it
bool isPrivateIntermediate(const TensorDescriptor &t) {
    return t.getKind() == TensorKind::Session && !t.isGraphOutput && !t.isGraphInput && t.isPacked();
}

bool scaleTensorsOk(const OpNode &rescale) {
    const auto &m = rescale.inputs[1], &s = rescale.inputs[2];
    // read at the fused node's (earlier) position: they must not be produced inside the graph
    if (m->getKind() == TensorKind::Session || s->getKind() == TensorKind::Session) return false;
    return m->getRank() == 1 && s->getRank() == 1 && m->isPacked() && s->isPacked() &&
           m->getFormat() == (rescale.rescale.scale32 ? MLEL_I32 : MLEL_I16) && s->getFormat() == MLEL_I8;
}

bool isSmallInt(int32_t dt) { return dt == MLEL_I8 || dt == MLEL_I16 || dt == MLEL_I32; }

}  // namespace

void GraphPipeline::fuse() {
    // Pattern 1: CONV2D | DEPTHWISE_CONV2D | MATMUL (int8 x int8 -> int32)  ->  RESCALE  [-> CLAMP]
    // Legal when the int32 accumulator tensor (and, for the CLAMP, the RESCALE result) is a private intermediate
    // with exactly one consumer.  The fused kernels compute exactly RESCALE(CLAMP) of the int32 accumulator, so the
    // result is bit-identical to the three operators run one after another.
    for (const auto &opPtr : ops) {
        OpNode &op = *opPtr;
        if (op.fusedAway) continue;
        const bool isConv = op.kind == OpKind::Conv2D, isDw = op.kind == OpKind::DepthwiseConv2D,
                   isMm = op.kind == OpKind::Matmul;
        if (!isConv && !isDw && !isMm) continue;
        const auto &acc = op.outputs[0];
        if (acc->getFormat() != MLEL_I32 || op.inputs[0]->getFormat() != MLEL_I8 ||
            op.inputs[1]->getFormat() != MLEL_I8 || !isPrivateIntermediate(*acc))
            continue;
        if (!isMm && op.conv.acc_type != MLEL_ACC_I32) continue;
        const auto users = consumersOf(ops, acc.get());
        if (users.size() != 1 || users[0]->kind != OpKind::Rescale || users[0]->inputs[0].get() != acc.get()) continue;
        OpNode &rs = *users[0];
        const auto &rsOut = rs.outputs[0];
        if (!isSmallInt(rsOut->getFormat()) || !sameShape(*acc, *rsOut) || !rsOut->isPacked() || !scaleTensorsOk(rs) ||
            rs.rescale.input_unsigned)
            continue;
        // optional CLAMP
        OpNode *clamp = nullptr;
        if (isPrivateIntermediate(*rsOut) && !rs.rescale.output_unsigned) {
            const auto rsUsers = consumersOf(ops, rsOut.get());
            if (rsUsers.size() == 1 && rsUsers[0]->kind == OpKind::Clamp &&
                rsUsers[0]->outputs[0]->getFormat() == rsOut->getFormat() && sameShape(*rsOut, *rsUsers[0]->outputs[0]) &&
                rsUsers[0]->outputs[0]->isPacked() && rsUsers[0]->clamp.min_val <= rsUsers[0]->clamp.max_val)
                clamp = rsUsers[0];
        }
        op.kind = isConv ? OpKind::FusedConv2D : (isDw ? OpKind::FusedDepthwiseConv2D : OpKind::FusedMatmul);
        op.epilogue = RescaleSpec{rs.inputs[1], rs.inputs[2], rs.rescale};
        rs.fusedAway = true;
        TensorPtr finalOut = rsOut;
        if (clamp) {
            op.hasClamp = true;
            op.clamp = clamp->clamp;
            clamp->fusedAway = true;
            finalOut = clamp->outputs[0];
        }
        op.outputs[0] = finalOut;
        finalOut->setProducer(&op);
    }

    // Pattern 2 (residual add): RESCALE(a -> i32), RESCALE(b -> i32), ADD(i32), RESCALE(-> i8/i16/i32)
    for (const auto &opPtr : ops) {
        OpNode &add = *opPtr;
        if (add.fusedAway || add.kind != OpKind::Binary || add.selector != MLEL_BIN_ADD) continue;
        const auto &sum = add.outputs[0];
        if (sum->getFormat() != MLEL_I32 || !isPrivateIntermediate(*sum)) continue;
        OpNode *ra = add.inputs[0]->getProducer(), *rb = add.inputs[1]->getProducer();
        if (!ra || !rb || ra == rb || ra->fusedAway || rb->fusedAway || ra->kind != OpKind::Rescale ||
            rb->kind != OpKind::Rescale)
            continue;
        const auto &ta = add.inputs[0], &tb = add.inputs[1];
        if (!isPrivateIntermediate(*ta) || !isPrivateIntermediate(*tb) || ta->getFormat() != MLEL_I32 ||
            tb->getFormat() != MLEL_I32 || !sameShape(*ta, *sum) || !sameShape(*tb, *sum))
            continue;
        if (consumersOf(ops, ta.get()).size() != 1 || consumersOf(ops, tb.get()).size() != 1) continue;
        const auto users = consumersOf(ops, sum.get());
        if (users.size() != 1 || users[0]->kind != OpKind::Rescale || users[0]->inputs[0].get() != sum.get()) continue;
        OpNode &ro = *users[0];
        if (!isSmallInt(ro.outputs[0]->getFormat()) || !sameShape(*sum, *ro.outputs[0]) || !scaleTensorsOk(*ra) ||
            !scaleTensorsOk(*rb) || !scaleTensorsOk(ro) || ro.rescale.input_unsigned ||
            !sameShape(*ra->inputs[0], *sum) || !sameShape(*rb->inputs[0], *sum) ||
            !isSmallInt(ra->inputs[0]->getFormat()) || !isSmallInt(rb->inputs[0]->getFormat()))
            continue;
        // the fused node takes the place of the ADD (all three producers precede it in creation order)
        add.kind = OpKind::FusedRescaleAddRescale;
        add.scaleA = RescaleSpec{ra->inputs[1], ra->inputs[2], ra->rescale};
        add.scaleB = RescaleSpec{rb->inputs[1], rb->inputs[2], rb->rescale};
        add.epilogue = RescaleSpec{ro.inputs[1], ro.inputs[2], ro.rescale};
        add.inputs = {ra->inputs[0], rb->inputs[0]};
        add.outputs[0] = ro.outputs[0];
        ro.outputs[0]->setProducer(&add);
        ra->fusedAway = rb->fusedAway = ro.fusedAway = true;
    }

    // Pattern 3 (residual connection behind a projection): a fused addition one of whose operands is the 8-bit result
    // of a fused 1x1 convolution read nowhere else moves into that convolution's epilogue, which then reads the
    // other operand at the position it is about to write.  Legal when the other operand exists before the
    // convolution runs and all three RESCALE stages of the addition are per tensor; the epilogue applies the same
    // three stages to the same two 8-bit values, so the result is bit-identical.  Restricted to the layouts the
    // one-pass kernel takes (dense 1x1, stride 1, unpadded, channel counts in whole 16-byte / 4-byte units), since
    // the fallback behind the entry point allocates.
    {
        std::unordered_map<const OpNode *, size_t> position;
        for (size_t i = 0; i < ops.size(); i++) position[ops[i].get()] = i;
        for (const auto &opPtr : ops) {
            OpNode &add = *opPtr;
            if (add.fusedAway || add.kind != OpKind::FusedRescaleAddRescale) continue;
            if (add.outputs[0]->getFormat() != MLEL_I8 || !add.outputs[0]->isPacked()) continue;
            if (add.scaleA.attr.per_channel || add.scaleB.attr.per_channel || add.epilogue.attr.per_channel ||
                add.scaleA.attr.input_unsigned || add.scaleB.attr.input_unsigned)
                continue;
            for (int side = 0; side < 2; side++) {
                const TensorPtr &convOut = add.inputs[side], &residual = add.inputs[1 - side];
                OpNode *conv = convOut->getProducer();
                if (!conv || conv->fusedAway || conv->kind != OpKind::FusedConv2D || conv->outputs[0].get() != convOut.get())
                    continue;
                if (convOut->getFormat() != MLEL_I8 || residual->getFormat() != MLEL_I8 || convOut.get() == residual.get() ||
                    !isPrivateIntermediate(*convOut) || consumersOf(ops, convOut.get()).size() != 1 || !residual->isPacked())
                    continue;
                const OpNode *resProducer = residual->getProducer();
                if (resProducer != nullptr && position.at(resProducer) >= position.at(conv)) continue;
                if (residual->getKind() == TensorKind::Session && resProducer == nullptr && !residual->isGraphInput) continue;
                const auto &x = conv->inputs[0], &w = conv->inputs[1];
                const auto &wd = w->getDimensions();
                const mlel_conv2d_attr &a = conv->conv;
                const bool pointwise = wd[1] == 1 && wd[2] == 1 && a.stride[0] == 1 && a.stride[1] == 1 && a.pad[0] == 0 &&
                                       a.pad[1] == 0 && a.pad[2] == 0 && a.pad[3] == 0;
                if (!pointwise || !x->isPacked() || !w->isPacked() || wd[3] % 16 != 0 || wd[0] % 4 != 0 ||
                    conv->epilogue.attr.output_unsigned)
                    continue;
                conv->kind = OpKind::FusedConv2DResidual;
                conv->scaleA = side == 0 ? add.scaleA : add.scaleB;
                conv->scaleB = side == 0 ? add.scaleB : add.scaleA;
                conv->scaleOut = add.epilogue;
                conv->flag = side == 1;
                conv->inputs.push_back(residual);
                conv->outputs[0] = add.outputs[0];
                add.outputs[0]->setProducer(conv);
                add.fusedAway = true;
                break;
            }
        }
    }

    // Pattern 4 (fp16 projections): MATMUL (fp16 x fp16 -> fp32)  [-> ADD of an fp32 constant of one or N values]
    // -> CAST to fp16.  The fused kernel adds in fp32 and rounds once to fp16, exactly like the operators it replaces.
    for (const auto &opPtr : ops) {
        OpNode &mm = *opPtr;
        if (mm.fusedAway || mm.kind != OpKind::Matmul) continue;
        const auto &acc = mm.outputs[0];
        if (acc->getFormat() != MLEL_F32 || mm.inputs[0]->getFormat() != MLEL_F16 || mm.inputs[1]->getFormat() != MLEL_F16 ||
            mm.matmul.a_zp != 0 || mm.matmul.b_zp != 0 || !isPrivateIntermediate(*acc) || acc->getRank() != 3)
            continue;
        const int64_t K = mm.inputs[0]->getDimensions()[2], N = acc->getDimensions()[2];
        if (K % 8 != 0 || N % 8 != 0 || !mm.inputs[0]->isPacked() || !mm.inputs[1]->isPacked()) continue;
        auto users = consumersOf(ops, acc.get());
        if (users.size() != 1) continue;
        OpNode *add = nullptr;
        TensorPtr bias;
        TensorPtr value = acc;
        if (users[0]->kind == OpKind::Binary && users[0]->selector == MLEL_BIN_ADD) {
            OpNode *cand = users[0];
            const bool accFirst = cand->inputs[0].get() == acc.get();
            const TensorPtr other = cand->inputs[accFirst ? 1 : 0];
            const auto &od = other->getDimensions();
            const int64_t n = static_cast<int64_t>(other->getShapeSize());
            const bool vectorOnLastAxis = other->getRank() == 3 && od[2] == n && (n == 1 || n == N);
            if (other->getKind() != TensorKind::Constant || other->getFormat() != MLEL_F32 || !vectorOnLastAxis ||
                !other->isPacked() || cand->outputs[0]->getFormat() != MLEL_F32 || !sameShape(*acc, *cand->outputs[0]) ||
                !isPrivateIntermediate(*cand->outputs[0]))
                continue;
            add = cand;
            bias = other;
            value = cand->outputs[0];
            users = consumersOf(ops, value.get());
            if (users.size() != 1) continue;
        }
        OpNode *cast = users[0];
        if (cast->kind != OpKind::Cast || cast->inputs[0].get() != value.get() ||
            cast->outputs[0]->getFormat() != MLEL_F16 || !sameShape(*acc, *cast->outputs[0]) ||
            !cast->outputs[0]->isPacked())
            continue;
        mm.kind = OpKind::FusedMatmulBiasCast;
        if (bias) mm.inputs.push_back(bias);
        mm.hasBias = bias != nullptr;
        mm.outputs[0] = cast->outputs[0];
        cast->outputs[0]->setProducer(&mm);
        cast->fusedAway = true;
        if (add) add->fusedAway = true;
    }

    // Pattern 4e (head split / merge behind an fp16 product): the fp16 result [NB, M, N], private, read only by a
    // RESHAPE that splits each of NB, M, N into at most two extents, itself read only by a TRANSPOSE that keeps the
    // innermost extent innermost or makes the inner row extent the innermost one (K transposed for the scores).
    // The product then writes the transposed tensor directly, through a strided view
    // (mlel_hip_matmul_bias_cast with a six-dimensional output); the two data-movement operators disappear.
    for (const auto &opPtr : ops) {
        OpNode &mm = *opPtr;
        if (mm.fusedAway || mm.kind != OpKind::FusedMatmulBiasCast || mm.flag) continue;
        const TensorPtr h = mm.outputs[0];
        if (!isPrivateIntermediate(*h) || h->getRank() != 3) continue;
        auto users = consumersOf(ops, h.get());
        if (users.size() != 1 || users[0]->kind != OpKind::Reshape) continue;
        OpNode *reshape = users[0];
        const TensorPtr split = reshape->outputs[0];
        if (!isPrivateIntermediate(*split) || split->getFormat() != MLEL_F16) continue;
        users = consumersOf(ops, split.get());
        if (users.size() != 1 || users[0]->kind != OpKind::Transpose) continue;
        OpNode *transpose = users[0];
        const TensorPtr moved = transpose->outputs[0];
        if (moved->getFormat() != MLEL_F16 || !moved->isPacked() || moved->getRank() != split->getRank()) continue;
        // the split extents, in order, grouped by the product extent they come from (extents of 1 address nothing)
        const auto &sd = split->getDimensions();
        const auto &hd = h->getDimensions();
        std::array<std::vector<size_t>, 3> groups;
        size_t at = 0;
        bool ok = true;
        for (int part = 0; part < 3 && ok; part++) {
            int64_t product = 1;
            while (product < hd[static_cast<size_t>(part)] && at < sd.size()) {
                if (sd[at] != 1) groups[static_cast<size_t>(part)].push_back(at);
                product *= sd[at++];
            }
            ok = product == hd[static_cast<size_t>(part)] && groups[static_cast<size_t>(part)].size() <= 2;
        }
        for (; at < sd.size() && ok; at++) ok = sd[at] == 1;
        if (!ok || groups[2].empty()) continue;
        // byte strides of the split extents inside the (packed) transposed tensor
        const size_t rank = sd.size();
        std::vector<int64_t> movedStride(rank), splitStride(rank);
        int64_t stride = 2;
        for (size_t k = rank; k-- > 0;) {
            movedStride[k] = stride;
            stride *= moved->getDimensions()[k];
        }
        for (size_t k = 0; k < rank; k++) splitStride[transpose->vec[k]] = movedStride[k];
        std::array<int64_t, 6> vd{}, vs{};
        for (size_t part = 0; part < 3; part++) {
            const auto &gr = groups[part];
            // one extent: (extent, 1); two: (outer, inner); none (the product extent is 1): (1, 1)
            vd[2 * part] = gr.empty() ? 1 : sd[gr[0]];
            vs[2 * part] = gr.empty() ? 0 : splitStride[gr[0]];
            vd[2 * part + 1] = gr.size() == 2 ? sd[gr[1]] : 1;
            vs[2 * part + 1] = gr.size() == 2 ? splitStride[gr[1]] : 0;
        }
        if (groups[2].size() == 1) {  // the columns were not split: they are the inner extent
            vd[5] = vd[4], vs[5] = vs[4];
            vd[4] = 1, vs[4] = 0;
        }
        // eight contiguous elements along the innermost column extent or, for a transposing view, along the
        // innermost row extent
        const size_t inner = vs[5] == 2 ? 5 : 3;
        bool aligned = vs[inner] == 2 && vd[inner] % 8 == 0;
        for (size_t k = 0; k < 6; k++) aligned = aligned && (k == inner || vs[k] % 16 == 0);
        if (!aligned) continue;
        mm.viewDims = vd;
        mm.viewStrides = vs;
        mm.outputs[0] = moved;
        moved->setProducer(&mm);
        reshape->fusedAway = transpose->fusedAway = true;
    }

    // Pattern 4d (residual connection behind an fp16 projection): the fp16 result of the pattern above, private and
    // read only by an fp16 ADD whose other operand has the same shape and exists before the projection runs, takes
    // that addition into the projection's epilogue (mlel_hip_matmul_bias_cast_add).
    for (size_t at = 0; at < ops.size(); at++) {
        OpNode &mm = *ops[at];
        if (mm.fusedAway || mm.kind != OpKind::FusedMatmulBiasCast || mm.flag || mm.viewDims[5] != 0) continue;
        TensorPtr h = mm.outputs[0];
        if (!isPrivateIntermediate(*h)) continue;
        auto users = consumersOf(ops, h.get());
        // a RESHAPE in between only renames the extents of the same packed bytes ([1, rows, N] -> [batch, seq, N])
        OpNode *reshape = nullptr;
        if (users.size() == 1 && users[0]->kind == OpKind::Reshape && isPrivateIntermediate(*users[0]->outputs[0]) &&
            users[0]->outputs[0]->getFormat() == MLEL_F16 && users[0]->outputs[0]->getSize() == h->getSize()) {
            reshape = users[0];
            h = reshape->outputs[0];
            users = consumersOf(ops, h.get());
        }
        if (users.size() != 1 || users[0]->kind != OpKind::Binary || users[0]->selector != MLEL_BIN_ADD) continue;
        OpNode *add = users[0];
        const TensorPtr other = add->inputs[add->inputs[0].get() == h.get() ? 1 : 0];
        if (other.get() == h.get() || other->getFormat() != MLEL_F16 || !sameShape(*other, *h) || !other->isPacked() ||
            add->outputs[0]->getFormat() != MLEL_F16 || !sameShape(*add->outputs[0], *h) || !add->outputs[0]->isPacked())
            continue;
        bool early = other->getProducer() == nullptr;
        for (size_t k = 0; k < at && !early; k++) early = ops[k].get() == other->getProducer();
        if (!early) continue;
        mm.inputs.push_back(other);
        mm.flag = true;
        mm.outputs[0] = add->outputs[0];
        add->outputs[0]->setProducer(&mm);
        add->fusedAway = true;
        if (reshape) reshape->fusedAway = true;
    }

    // Pattern 4f (projections of one tensor): fused fp16 products (pattern 4, possibly with the view of pattern 4e,
    // without a residual) that read the same A and whose B and bias are not produced by the graph, of equal extents,
    // become one launch of up to three products (mlel_hip_matmul_bias_cast_group): the query, key and value
    // projections of an attention block.  The later ones run at the first one's place.
    for (const auto &opPtr : ops) {
        OpNode &first = *opPtr;
        if (first.fusedAway || first.kind != OpKind::FusedMatmulBiasCast || first.flag || !first.extraProductViews.empty()) continue;
        const auto constantOperands = [](const OpNode &op) {
            for (size_t i = 1; i < op.inputs.size(); i++)
                if (op.inputs[i]->getProducer() != nullptr) return false;
            return true;
        };
        if (!constantOperands(first)) continue;
        bool after = false;
        for (const auto &otherPtr : ops) {
            OpNode &other = *otherPtr;
            if (&other == &first) {
                after = true;
                continue;
            }
            if (!after || first.outputs.size() >= 3) continue;
            if (other.fusedAway || other.kind != OpKind::FusedMatmulBiasCast || other.flag || !other.extraProductViews.empty() ||
                other.outputs.size() != 1 || other.inputs[0].get() != first.inputs[0].get() || other.hasBias != first.hasBias ||
                !constantOperands(other) || !sameShape(*other.inputs[1], *first.inputs[1]) ||
                (first.hasBias && !sameShape(*other.inputs[2], *first.inputs[2])) ||
                other.matmul.a_zp != first.matmul.a_zp || other.matmul.b_zp != first.matmul.b_zp)
                continue;
            for (size_t i = 1; i < other.inputs.size(); i++) first.inputs.push_back(other.inputs[i]);
            first.outputs.push_back(other.outputs[0]);
            other.outputs[0]->setProducer(&first);
            first.extraProductViews.emplace_back(other.viewDims, other.viewStrides);
            other.fusedAway = true;
        }
    }

    // Pattern 5: regions of floating-point elementwise operators (ADD, SUB, MUL, EXP, RECIPROCAL, RSQRT, TANH, CAST
    // between fp16 and fp32) collapse into one pass.  A region grows backwards from an operator whose result is needed
    // elsewhere: a producer is absorbed when it is elementwise too, has the region's shape, and its result is a
    // private intermediate read only here; everything else the region reads becomes an input and must have the
    // region's shape or be broadcast along rows and / or the last axis.  The one-pass kernel rounds after every step
    // like the stand-alone operators, so the result is bit-identical.
    const auto chainStepOf = [](const OpNode &op, mlel_chain_step *st) {
        const auto &out = op.outputs[0];
        const int dt = out->getFormat();
        if (op.fusedAway || (dt != MLEL_F16 && dt != MLEL_F32) || op.outputs.size() != 1) return false;
        const auto sameType = [&](size_t n) {
            for (size_t i = 0; i < n; i++)
                if (op.inputs[i]->getFormat() != dt) return false;
            return true;
        };
        *st = mlel_chain_step{0, 0, -1, -1, dt};
        switch (op.kind) {
        case OpKind::Binary:
            st->kind = MLEL_CHAIN_BINARY;
            st->selector = op.selector;
            return (op.selector == MLEL_BIN_ADD || op.selector == MLEL_BIN_SUB) && sameType(2);
        case OpKind::Mul: st->kind = MLEL_CHAIN_MUL; return op.shift == 0 && sameType(2);
        case OpKind::Unary:
            st->kind = MLEL_CHAIN_UNARY;
            st->selector = op.selector;
            return (op.selector == MLEL_UN_EXP || op.selector == MLEL_UN_RECIPROCAL || op.selector == MLEL_UN_RSQRT ||
                    op.selector == MLEL_UN_TANH) && sameType(1);
        case OpKind::Cast:
            st->kind = MLEL_CHAIN_CAST;
            return op.inputs[0]->getFormat() == MLEL_F16 || op.inputs[0]->getFormat() == MLEL_F32;
        default: return false;
        }
    };
    // Pattern 4c: regions of fp16 operators that hold reductions over the last axis (REDUCE_SUM / REDUCE_MAX with the
    // elementwise operators around them: LayerNorm, softmax with its scale) become one pass over the rows.  A region
    // starts at an operator, takes the later operators that read its values while everything they read is either in
    // the region or exists before it, and ends at the longest prefix from which exactly one value escapes: the last
    // one, with the full shape.  All values have the full shape [.., cols], its per-row shape [.., 1], or are inputs
    // broadcast along rows and / or the last axis.
    {
        const auto rowStepOf = [&](const OpNode &op, mlel_chain_step *st) {
            if (op.fusedAway || op.outputs.size() != 1 || op.outputs[0]->getFormat() != MLEL_F16) return false;
            if (op.kind == OpKind::Reduce) {
                const auto &in = op.inputs[0];
                *st = mlel_chain_step{MLEL_CHAIN_REDUCE, op.selector, -1, -1, MLEL_F16};
                return (op.selector == MLEL_RED_SUM || op.selector == MLEL_RED_MAX) && op.nanMode == MLEL_NAN_PROPAGATE &&
                       in->getFormat() == MLEL_F16 && in->getRank() >= 1 && op.axis + 1 == in->getRank();
            }
            return op.kind != OpKind::Cast && chainStepOf(op, st);
        };
        for (size_t first = 0; first < ops.size(); first++) {
            mlel_chain_step firstStep{};
            if (!rowStepOf(*ops[first], &firstStep)) continue;
            // the full shape: the largest operand or result of the first operator
            const TensorDescriptor *full = ops[first]->outputs[0].get();
            for (const auto &in : ops[first]->inputs)
                if (in->getShapeSize() > full->getShapeSize()) full = in.get();
            const auto &dims = full->getDimensions();
            if (dims.empty() || dims.back() % 8 != 0 || dims.back() < 8) continue;
            enum { kNone, kFull, kRow, kBroadcast };
            const auto shapeClass = [&](const TensorDescriptor &t) {
                const auto &d = t.getDimensions();
                if (d.size() != dims.size() || !t.isPacked() || t.getFormat() != MLEL_F16) return int(kNone);
                bool same = true, ones = true;
                for (size_t i = 0; i + 1 < d.size(); i++) {
                    same = same && d[i] == dims[i];
                    ones = ones && d[i] == 1;
                }
                if (d.back() != dims.back() && d.back() != 1) return int(kNone);
                if (same) return d.back() == dims.back() ? int(kFull) : int(kRow);
                return ones ? int(kBroadcast) : int(kNone);
            };
            std::vector<OpNode *> region;
            std::vector<mlel_chain_step> regionSteps;
            const auto inRegion = [&](const OpNode *p) { return std::find(region.begin(), region.end(), p) != region.end(); };
            for (size_t i = first; i < ops.size() && region.size() < MLEL_CHAIN_MAX_STEPS; i++) {
                OpNode &op = *ops[i];
                mlel_chain_step st{};
                if (!rowStepOf(op, &st)) continue;
                const int outClass = shapeClass(*op.outputs[0]);
                if (outClass != kFull && outClass != kRow) continue;
                bool connected = region.empty(), readable = true;
                for (const auto &in : op.inputs) {
                    OpNode *p = in->getProducer();
                    if (p && inRegion(p)) {
                        connected = true;
                    } else {
                        // produced before the region starts (or not by the graph at all) and of a usable shape
                        bool early = p == nullptr;
                        for (size_t k = 0; k < first && !early; k++) early = ops[k].get() == p;
                        readable = readable && early && shapeClass(*in) != kNone;
                    }
                }
                if (!connected || !readable) continue;
                region.push_back(&op);
                regionSteps.push_back(st);
            }
            // the longest prefix with one escaping value, the last, full-shaped, and at least one reduction inside
            size_t best = 0;
            for (size_t n = region.size(); n >= 3 && best == 0; n--) {
                bool ok = shapeClass(*region[n - 1]->outputs[0]) == kFull, reduces = false;
                for (size_t k = 0; k < n && ok; k++) {
                    reduces = reduces || region[k]->kind == OpKind::Reduce;
                    if (k + 1 == n) break;
                    const auto &t = region[k]->outputs[0];
                    ok = isPrivateIntermediate(*t);
                    for (OpNode *user : consumersOf(ops, t.get())) {
                        bool inside = false;
                        for (size_t m = 0; m < n; m++) inside = inside || region[m] == user;
                        ok = ok && inside;
                    }
                }
                if (ok && reduces) best = n;
            }
            if (best == 0) continue;
            // values: region inputs first, then one per step
            std::vector<TensorPtr> regionInputs;
            std::vector<mlel_chain_step> steps;
            bool fits = true;
            const auto valueOf = [&](const TensorPtr &t) {
                for (size_t k = 0; k < best; k++)
                    if (region[k]->outputs[0].get() == t.get() && k < steps.size()) return -static_cast<int>(k) - 1;
                for (size_t k = 0; k < regionInputs.size(); k++)
                    if (regionInputs[k].get() == t.get()) return static_cast<int>(k);
                if (regionInputs.size() >= MLEL_CHAIN_MAX_INPUTS) {
                    fits = false;
                    return 0;
                }
                regionInputs.push_back(t);
                return static_cast<int>(regionInputs.size()) - 1;
            };
            for (size_t k = 0; k < best; k++) {
                mlel_chain_step st = regionSteps[k];
                const bool two = st.kind == MLEL_CHAIN_BINARY || st.kind == MLEL_CHAIN_MUL;
                st.a = valueOf(region[k]->inputs[0]);
                st.b = two ? valueOf(region[k]->inputs[1]) : 0;
                steps.push_back(st);
            }
            bool anyFull = false;
            for (const auto &t : regionInputs) anyFull = anyFull || shapeClass(*t) == kFull;
            if (!fits || !anyFull) continue;
            const int nIn = static_cast<int>(regionInputs.size());
            for (auto &st : steps) {
                if (st.a < 0) st.a = nIn + (-st.a - 1);
                if (st.b < 0) st.b = nIn + (-st.b - 1);
            }
            OpNode &root = *region[best - 1];
            for (size_t k = 0; k + 1 < best; k++) region[k]->fusedAway = true;
            root.kind = OpKind::FusedElementwise;
            root.inputs = regionInputs;
            root.chain = steps;
        }
    }

    for (auto it = ops.rbegin(); it != ops.rend(); ++it) {
        OpNode &root = **it;
        mlel_chain_step rootStep{};
        if (!chainStepOf(root, &rootStep)) continue;
        const TensorDescriptor &shape = *root.outputs[0];
        const auto &dims = shape.getDimensions();
        const bool flat = !dims.empty() && dims.back() % 8 != 0;  // short rows: walked as one long row
        if (!shape.isPacked() || dims.empty() || (flat && shape.getShapeSize() % 8 != 0)) continue;
        const auto broadcastable = [&](const TensorDescriptor &t) {
            const auto &d = t.getDimensions();
            if (d.size() != dims.size() || !t.isPacked()) return false;
            if (flat) return t.getShapeSize() == 1 || sameShape(t, shape);
            bool same = true, ones = true;
            for (size_t i = 0; i + 1 < d.size(); i++) {
                same = same && d[i] == dims[i];
                ones = ones && d[i] == 1;
            }
            return (same || ones) && (d.back() == dims.back() || d.back() == 1);
        };
        std::vector<TensorPtr> regionInputs;
        std::vector<mlel_chain_step> steps;   // operands: value >= 0 input index, value < 0 -(step index + 1)
        std::vector<OpNode *> absorbed;
        std::map<const TensorDescriptor *, int> emitted;  // an absorbed intermediate read twice (MUL(t, t)) is one step
        bool ok = true;
        std::function<int(const TensorPtr &)> valueOf;
        const auto emit = [&](OpNode &op, mlel_chain_step st) {
            const bool two = st.kind == MLEL_CHAIN_BINARY || st.kind == MLEL_CHAIN_MUL;
            st.a = valueOf(op.inputs[0]);
            st.b = two ? valueOf(op.inputs[1]) : 0;
            steps.push_back(st);
            return -static_cast<int>(steps.size());
        };
        valueOf = [&](const TensorPtr &t) -> int {
            OpNode *p = t->getProducer();
            mlel_chain_step st{};
            const auto seen = emitted.find(t.get());
            if (seen != emitted.end()) return seen->second;
            if (p && p != &root && isPrivateIntermediate(*t) && sameShape(*t, shape) && chainStepOf(*p, &st) &&
                consumersOf(ops, t.get()).size() == 1 && steps.size() + absorbed.size() < MLEL_CHAIN_MAX_STEPS - 1) {
                absorbed.push_back(p);
                const int value = emit(*p, st);
                emitted[t.get()] = value;
                return value;
            }
            for (size_t i = 0; i < regionInputs.size(); i++)
                if (regionInputs[i].get() == t.get()) return static_cast<int>(i);
            if (!broadcastable(*t) || regionInputs.size() >= MLEL_CHAIN_MAX_INPUTS) {
                ok = false;
                return 0;
            }
            regionInputs.push_back(t);
            return static_cast<int>(regionInputs.size()) - 1;
        };
        emit(root, rootStep);
        if (!ok || steps.size() < 2 || steps.size() > MLEL_CHAIN_MAX_STEPS) continue;
        const int nIn = static_cast<int>(regionInputs.size());
        for (auto &st : steps) {
            if (st.a < 0) st.a = nIn + (-st.a - 1);
            if (st.b < 0) st.b = nIn + (-st.b - 1);
        }
        for (OpNode *p : absorbed) p->fusedAway = true;
        root.kind = OpKind::FusedElementwise;
        root.inputs = regionInputs;
        root.chain = steps;
    }

    // Pattern 6 (activation behind an fp16 product): a fused product (pattern 4; no view, residual or group) whose
    // private result is read only by a fused elementwise region as its first input, the region's other inputs not
    // produced by the graph, and the chain one that the product's kernel applies to the tile on its way out (the tanh
    // form of GELU; mlel_hip_matmul_chain_in_kernel): the region moves into the product's call
    // (mlel_hip_matmul_bias_cast_chain).
    for (const auto &opPtr : ops) {
        OpNode &mm = *opPtr;
        if (mm.fusedAway || mm.kind != OpKind::FusedMatmulBiasCast || mm.flag || mm.viewDims[5] != 0 ||
            !mm.extraProductViews.empty() || !mm.chain.empty())
            continue;
        const TensorPtr h = mm.outputs[0];
        if (!isPrivateIntermediate(*h)) continue;
        const auto users = consumersOf(ops, h.get());
        if (users.size() != 1 || users[0]->kind != OpKind::FusedElementwise) continue;
        OpNode *ew = users[0];
        if (ew->inputs.empty() || ew->inputs[0].get() != h.get() || !sameShape(*ew->outputs[0], *h) ||
            ew->outputs[0]->getFormat() != MLEL_F16 || !ew->outputs[0]->isPacked() ||
            mm.inputs.size() + ew->inputs.size() - 1 > 8)
            continue;
        bool ok = true;
        for (size_t i = 1; i < ew->inputs.size(); i++)
            ok = ok && ew->inputs[i].get() != h.get() && ew->inputs[i]->getProducer() == nullptr;
        for (const auto &st : ew->chain) ok = ok && st.kind != MLEL_CHAIN_REDUCE;
        if (!ok || ew->inputs.size() > MLEL_CHAIN_MAX_INPUTS || ew->chain.size() > MLEL_CHAIN_MAX_STEPS) continue;
        // only a chain the product's kernel applies itself: any other would run as a pass of its own over a temporary
        // that the call has to allocate, which the stand-alone region does without
        std::array<mlel_tensor, MLEL_CHAIN_MAX_INPUTS> described{};
        mlel_chain query{};
        query.n_inputs = static_cast<int32_t>(ew->inputs.size());
        query.n_steps = static_cast<int32_t>(ew->chain.size());
        for (size_t i = 1; i < ew->inputs.size(); i++) {
            described[i] = ew->inputs[i]->view();
            query.inputs[i] = &described[i];
        }
        for (size_t i = 0; i < ew->chain.size(); i++) query.steps[i] = ew->chain[i];
        if (mlel_hip_matmul_chain_in_kernel(&query) == 0) continue;
        mm.chain = ew->chain;
        for (size_t i = 1; i < ew->inputs.size(); i++) mm.inputs.push_back(ew->inputs[i]);
        mm.outputs[0] = ew->outputs[0];
        ew->outputs[0]->setProducer(&mm);
        ew->fusedAway = true;
    }

    // Pattern 7 (attention): a fused fp16 product (no bias, view, residual, group or chain) whose private result is
    // read only by a fused region as its value 0, the region being the softmax chain over the last axis
    // (mlel_hip_attention_f16_in_kernel decides), and the region's private result read only as the first operand of
    // another such product (which may carry the view of a head merge): the three become one launch that keeps the
    // scores on the chip (mlel_hip_attention_f16), bit for bit the three launches.
    for (const auto &opPtr : ops) {
        OpNode &sm = *opPtr;
        if (sm.fusedAway || sm.kind != OpKind::FusedElementwise || sm.inputs.empty() || sm.inputs.size() > 4) continue;
        const TensorPtr scores = sm.inputs[0];
        OpNode *first = scores->getProducer();
        const auto plainProduct = [](const OpNode *mm) {
            return mm != nullptr && !mm->fusedAway && mm->kind == OpKind::FusedMatmulBiasCast && !mm->hasBias && !mm->flag &&
                   mm->extraProductViews.empty() && mm->chain.empty();
        };
        if (!plainProduct(first) || first->viewDims[5] != 0 || !isPrivateIntermediate(*scores)) continue;
        const auto scoreUsers = consumersOf(ops, scores.get());
        if (scoreUsers.size() != 1 || scoreUsers[0] != &sm) continue;
        const TensorPtr prob = sm.outputs[0];
        if (!isPrivateIntermediate(*prob) || !sameShape(*prob, *scores)) continue;
        const auto probUsers = consumersOf(ops, prob.get());
        if (probUsers.size() != 1 || !plainProduct(probUsers[0])) continue;
        OpNode *second = probUsers[0];
        if (second->inputs[0].get() != prob.get() || second->inputs[1].get() == prob.get()) continue;
        bool ok = true;
        for (size_t i = 1; i < sm.inputs.size(); i++)
            ok = ok && sm.inputs[i].get() != scores.get() && sm.inputs[i]->getProducer() == nullptr;
        if (!ok || sm.chain.size() > MLEL_CHAIN_MAX_STEPS) continue;
        std::array<mlel_tensor, MLEL_CHAIN_MAX_INPUTS> described{};
        mlel_chain query{};
        query.n_inputs = static_cast<int32_t>(sm.inputs.size());
        query.n_steps = static_cast<int32_t>(sm.chain.size());
        for (size_t i = 1; i < sm.inputs.size(); i++) {
            described[i] = sm.inputs[i]->view();
            query.inputs[i] = &described[i];
        }
        for (size_t i = 0; i < sm.chain.size(); i++) query.steps[i] = sm.chain[i];
        const mlel_tensor q = first->inputs[0]->view(), kt = first->inputs[1]->view(), v = second->inputs[1]->view();
        mlel_tensor out = second->outputs[0]->view();
        if (second->viewDims[5] != 0) {
            out.rank = 6;
            for (size_t k = 0; k < 6; k++) {
                out.dims[k] = second->viewDims[k];
                out.strides[k] = second->viewStrides[k];
            }
        }
        if (mlel_hip_attention_f16_in_kernel(&out, &q, &kt, &v, &query) == 0) continue;
        const TensorPtr qT = first->inputs[0], ktT = first->inputs[1], vT = second->inputs[1];
        second->kind = OpKind::FusedAttention;
        second->inputs = {qT, ktT, vT};
        for (size_t i = 1; i < sm.inputs.size(); i++) second->inputs.push_back(sm.inputs[i]);
        second->chain = sm.chain;
        first->fusedAway = true;
        sm.fusedAway = true;
    }

    // Pattern 8 (expansion + depthwise): a fused 1x1 CONV2D (+RESCALE, +CLAMP) whose private int8 result is read only
    // by a fused 3x3 DEPTHWISE_CONV2D (+RESCALE, +CLAMP) as its image, on shapes the one-launch kernel takes
    // (mlel_hip_conv2d_dwconv_in_kernel decides: small images, channel counts in multiples of 32).  The expanded
    // tensor then lives in shared memory only; byte for byte the two launches.
    for (const auto &opPtr : ops) {
        OpNode &dw = *opPtr;
        if (dw.fusedAway || dw.kind != OpKind::FusedDepthwiseConv2D) continue;
        const TensorPtr mid = dw.inputs[0];
        OpNode *conv = mid->getProducer();
        if (!conv || conv->fusedAway || conv->kind != OpKind::FusedConv2D || conv->outputs[0].get() != mid.get() ||
            !isPrivateIntermediate(*mid) || consumersOf(ops, mid.get()).size() != 1)
            continue;
        // the one-launch kernel requantises int32 accumulators, whose RESCALE has input_zp 0 in TOSA; it has no
        // general route of its own for a graph that names another
        if (conv->epilogue.attr.input_zp != 0 || dw.epilogue.attr.input_zp != 0) continue;
        const mlel_tensor out = dw.outputs[0]->view(), x = conv->inputs[0]->view(), w1 = conv->inputs[1]->view(),
                          b1 = conv->inputs[2]->view(), w2 = dw.inputs[1]->view(), b2 = dw.inputs[2]->view();
        if (mlel_hip_conv2d_dwconv_in_kernel(&out, &x, &w1, &b1, &conv->conv, &w2, &b2, &dw.conv) == 0) continue;
        const TensorPtr w2T = dw.inputs[1], b2T = dw.inputs[2];
        dw.kind = OpKind::FusedConv2DDepthwise;
        dw.inputs = {conv->inputs[0], conv->inputs[1], conv->inputs[2], w2T, b2T};
        dw.convFirst = conv->conv;
        dw.scaleA = conv->epilogue;
        dw.hasClampFirst = conv->hasClamp;
        dw.clampFirst = conv->clamp;
        conv->fusedAway = true;
    }

    // Pattern 9 (projection + expansion): a fused 1x1 CONV2D whose int8 result is the image of another fused 1x1
    // CONV2D, on shapes the one-launch kernel takes (mlel_hip_conv2d_conv2d_in_kernel decides).  Positions are
    // independent in both operators, so a wavefront hands its 32 positions from one product to the next through
    // shared memory.  When the second convolution is the only reader the intermediate tensor disappears; when later
    // operators read it too (a residual connection) it is still written, by the same launch.  Byte for byte the two
    // launches.
    for (size_t bi = 0; bi < ops.size(); bi++) {
        OpNode &second = *ops[bi];
        if (second.fusedAway || second.kind != OpKind::FusedConv2D) continue;
        const TensorPtr mid = second.inputs[0];
        OpNode *first = mid->getProducer();
        if (!first || first->fusedAway || first->kind != OpKind::FusedConv2D || first->outputs[0].get() != mid.get() ||
            !isPrivateIntermediate(*mid))
            continue;
        if (first->epilogue.attr.input_zp != 0 || second.epilogue.attr.input_zp != 0) continue;
        // every other reader of the intermediate tensor runs after the second convolution
        bool later = true, others = false;
        for (size_t k = 0; k < ops.size(); k++) {
            if (ops[k]->fusedAway || ops[k].get() == &second) continue;
            bool reads = false;
            for (const auto &t : ops[k]->inputs) reads = reads || t.get() == mid.get();
            if (reads) {
                others = true;
                later = later && k > bi;
            }
        }
        if (!later) continue;
        const mlel_tensor out = second.outputs[0]->view(), x = first->inputs[0]->view(), w1 = first->inputs[1]->view(),
                          b1 = first->inputs[2]->view(), w2 = second.inputs[1]->view(), b2 = second.inputs[2]->view();
        if (mlel_hip_conv2d_conv2d_in_kernel(&out, &x, &w1, &b1, &first->conv, &w2, &b2, &second.conv) == 0) continue;
        const TensorPtr w2T = second.inputs[1], b2T = second.inputs[2];
        second.kind = OpKind::FusedConv2DConv2D;
        second.inputs = {first->inputs[0], first->inputs[1], first->inputs[2], w2T, b2T};
        second.convFirst = first->conv;
        second.scaleA = first->epilogue;
        second.hasClampFirst = first->hasClamp;
        second.clampFirst = first->clamp;
        if (others) {
            second.outputs.push_back(mid);
            mid->setProducer(&second);
        }
        first->fusedAway = true;
    }

    // Pattern 10 (head of a classifier): a fused 1x1 CONV2D whose private int8 result is read only by an AVG_POOL2D
    // over all positions of an image, on shapes the one-launch kernel takes (mlel_hip_conv2d_avgpool_in_kernel
    // decides).  The convolution's result then stays in registers; byte for byte the two launches.
    for (const auto &opPtr : ops) {
        OpNode &pool = *opPtr;
        if (pool.fusedAway || pool.kind != OpKind::AvgPool2D) continue;
        const TensorPtr mid = pool.inputs[0];
        OpNode *conv = mid->getProducer();
        if (!conv || conv->fusedAway || conv->kind != OpKind::FusedConv2D || conv->outputs[0].get() != mid.get() ||
            !isPrivateIntermediate(*mid) || consumersOf(ops, mid.get()).size() != 1)
            continue;
        if (conv->epilogue.attr.input_zp != 0) continue;
        const mlel_tensor out = pool.outputs[0]->view(), x = conv->inputs[0]->view(), w = conv->inputs[1]->view(),
                          b = conv->inputs[2]->view();
        const int32_t midType = mid->view().dtype;
        if (mlel_hip_conv2d_avgpool_in_kernel(&out, &x, &w, &b, &conv->conv, midType, &pool.pool) == 0) continue;
        pool.kind = OpKind::FusedConv2DAvgPool;
        pool.inputs = {conv->inputs[0], conv->inputs[1], conv->inputs[2]};
        pool.conv = conv->conv;
        pool.epilogue = conv->epilogue;
        pool.hasClamp = conv->hasClamp;
        pool.clamp = conv->clamp;
        pool.selector = midType;
        conv->fusedAway = true;
    }

    // Pattern 3: RESHAPE between two packed session tensors of the same byte size moves no data (the reference's
    // reshape.comp:16-27 copies by flat index): the output becomes a second view of the input's storage and the
    // operator is not executed.  plan() gives both tensors one allocation that lives as long as either is used.
    for (const auto &opPtr : ops) {
        OpNode &op = *opPtr;
        if (op.fusedAway || op.kind != OpKind::Reshape) continue;
        const auto &in = op.inputs[0];
        const auto &out = op.outputs[0];
        if (!isPrivateIntermediate(*in) || !isPrivateIntermediate(*out) || in->getSize() != out->getSize() ||
            in->getShapeSize() != out->getShapeSize() || dtypeSize(in->getFormat()) != dtypeSize(out->getFormat()))
            continue;
        aliasOf[out.get()] = in.get();
        op.fusedAway = true;
    }
}

/*******************************************************************************
 * GraphPipeline: planning, binding, dispatch
 *******************************************************************************/

std::vector<const OpNode *> GraphPipeline::executionList() const {
    std::vector<const OpNode *> r;
    for (const auto &op : ops)
        if (!op->fusedAway) r.push_back(op.get());
    return r;
}

void GraphPipeline::plan() {
    // Live ranges as the reference builds them (interval_memory_planner.cpp:53-115): execution index 0 belongs to the
    // graph inputs, operator i (in execution order) to index i + 1, the graph outputs to the index after the last
    // operator; every session tensor an operator reads or writes has its range stretched over that index.
    std::map<const TensorDescriptor *, size_t> order;
    for (size_t i = 0; i < tensors.size(); i++) order[tensors[i].get()] = i;
    ranges.clear();
    const auto root = [&](const TensorDescriptor *t) {
        for (auto it = aliasOf.find(t); it != aliasOf.end(); it = aliasOf.find(t)) t = it->second;
        return t;
    };
    const auto touch = [&](const TensorPtr &t, uint32_t idx) {
        if (!t || order.find(t.get()) == order.end()) return;
        auto [it, inserted] = ranges.emplace(root(t.get()), std::array<uint32_t, 2>{idx, idx});
        if (!inserted) {
            it->second[0] = std::min(it->second[0], idx);
            it->second[1] = std::max(it->second[1], idx);
        }
    };
    uint32_t idx = 0;
    for (const auto &t : inputs) touch(t, idx);
    idx++;
    for (const auto &op : ops) {
        if (op->fusedAway) continue;
        for (const auto &t : op->inputs) touch(t, idx);
        for (const auto &t : op->outputs) touch(t, idx);
        for (const auto *spec : {&op->epilogue, &op->scaleA, &op->scaleB, &op->scaleOut}) {
            touch(spec->multiplier, idx);
            touch(spec->shift, idx);
        }
        idx++;
    }
    for (const auto &t : outputs) touch(t, idx);

    const auto aligned = [](size_t v) { return (v + kSessionAlignment - 1) / kSessionAlignment * kSessionAlignment; };
    std::vector<details::LiveInterval> intervals;
    std::vector<details::UnseenAllocation> unseen;
    // a tensor some operator of the graph used, but no executed operator uses any more, was folded into a fused
    // kernel: it no longer exists at run time and gets no storage (a tensor no operator ever used keeps storage of
    // its own, as in the reference)
    std::set<const TensorDescriptor *> eliminated;
    for (const auto &op : ops) {
        for (const auto &t : op->originalTensors)
            if (ranges.find(t) == ranges.end()) eliminated.insert(t);
    }
    for (size_t i = 0; i < tensors.size(); i++) {
        const auto *t = tensors[i].get();
        const auto it = ranges.find(t);
        if (it != ranges.end())
            intervals.push_back({i, it->second[0], it->second[1], aligned(t->getSize()), i});
        else if (eliminated.find(t) == eliminated.end() || t->isGraphOutput)
            unseen.push_back({i, aligned(t->getSize())});
    }
    // Batch split: session tensors that only the split run touches are stored as two halves, each planned at half
    // its size in a region of its own (see setBatchSplit); a tensor with a view (an elided RESHAPE) stays whole.
    splitInterior.clear();
    std::vector<details::LiveInterval> halfIntervals;
    if (splitPrefix > 0 && planner == MemoryPlanner::Interval) {
        std::set<const TensorDescriptor *> viewed;
        for (const auto &[view, target] : aliasOf) {
            viewed.insert(view);
            viewed.insert(target);
        }
        std::vector<details::LiveInterval> whole;
        for (const auto &iv : intervals) {
            const auto *t = tensors[iv.id].get();
            const bool interior = iv.first >= splitFirst + 1 && iv.last <= splitPrefix && !t->isGraphInput && !t->isGraphOutput &&
                                  viewed.find(t) == viewed.end() && t->getRank() == 4 &&
                                  t->getDimensions()[0] == splitBatch && t->isPacked();
            if (interior) {
                splitInterior.insert(t);
                halfIntervals.push_back({iv.id, iv.first, iv.last, aligned(t->getSize() / 2), iv.order});
            } else {
                // a whole tensor the split run touches is written or read by two chains that are out of step: it
                // shares no byte with any other such tensor, which the planner sees as a range over the whole run
                auto w = iv;
                if (w.first <= splitPrefix && w.last >= splitFirst + 1) {
                    w.first = std::min<uint32_t>(w.first, splitFirst + 1);
                    w.last = std::max<uint32_t>(w.last, splitPrefix);
                }
                whole.push_back(w);
            }
        }
        intervals = std::move(whole);
    }
    details::AllocationPlan planResult;
    // the reference reports its choice at this severity when a session is created (graph_layer.cpp:286-295)
    MLEL_GRAPH_LOG(Info, (planner == MemoryPlanner::Interval ? "Using interval memory planner"
                          : planner == MemoryPlanner::Linear ? "Using linear memory planner"
                                                             : "Using best-fit memory planner"));
    if (planner == MemoryPlanner::Interval) {
        planResult = details::allocateIntervals(std::move(intervals), unseen, kSessionAlignment);
    } else if (planner == MemoryPlanner::Linear) {
        std::vector<details::UnseenAllocation> all;  // creation order, one slot each
        for (size_t i = 0; i < tensors.size(); i++) {
            const auto *t = tensors[i].get();
            if (ranges.find(t) != ranges.end() || eliminated.find(t) == eliminated.end() || t->isGraphOutput)
                all.push_back({i, aligned(t->getSize())});
        }
        planResult = details::allocateLinear(all, kSessionAlignment);
    } else {
        planResult = details::allocateBestFit(bestFitTensors(intervals, unseen), kSessionAlignment);
    }
    offsets.clear();
    for (const auto &[id, off] : planResult.offsets) offsets[tensors[id].get()] = static_cast<size_t>(off);
    splitFullRegion = static_cast<size_t>(planResult.memorySize);
    splitHalfRegion = 0;
    if (!halfIntervals.empty()) {
        const auto halfPlan = details::allocateIntervals(std::move(halfIntervals), {}, kSessionAlignment);
        splitHalfRegion = aligned(static_cast<size_t>(halfPlan.memorySize));
        splitFullRegion = aligned(splitFullRegion);
        for (const auto &[id, off] : halfPlan.offsets)
            offsets[tensors[id].get()] = splitFullRegion + static_cast<size_t>(off);  // the first half's place
    }
    for (const auto &[view, target] : aliasOf) {  // views share the storage of the tensor they alias
        (void)target;
        const auto it = offsets.find(root(view));
        if (it != offsets.end()) offsets[view] = it->second;
    }
    sessionSize = splitHalfRegion != 0 ? splitFullRegion + 2 * splitHalfRegion : static_cast<size_t>(planResult.memorySize);
}

// Safe-to-reuse sets of the best-fit planner (reference: BestFitMemoryPlanner::liveTensorAnalysis,
// memory_planner.cpp:139-226): a tensor T may share memory with the outputs of operator P once every operator that
// reads T is a strict ancestor of P in the operator graph, i.e. T is dead before P can run in ANY topological order.
// Tensors nobody reads, and tensors no executed operator writes, are never shared.
std::vector<details::BestFitTensor> GraphPipeline::bestFitTensors(const std::vector<details::LiveInterval> &planned,
                                                                  const std::vector<details::UnseenAllocation> &unseen) {
    std::map<const TensorDescriptor *, size_t> index;
    for (size_t i = 0; i < tensors.size(); i++) index[tensors[i].get()] = i;
    const auto root = [&](const TensorDescriptor *t) {
        for (auto it = aliasOf.find(t); it != aliasOf.end(); it = aliasOf.find(t)) t = it->second;
        return t;
    };
    std::vector<const OpNode *> executed;
    for (const auto &op : ops)
        if (!op->fusedAway) executed.push_back(op.get());
    const size_t n = executed.size(), words = (n + 63) / 64;
    std::map<size_t, size_t> producer;               // tensor index -> operator position
    std::map<size_t, std::vector<size_t>> consumers;
    for (size_t p = 0; p < n; p++) {
        const OpNode &op = *executed[p];
        const auto reads = [&](const TensorPtr &t) {
            if (!t) return;
            const auto it = index.find(root(t.get()));
            if (it != index.end()) consumers[it->second].push_back(p);
        };
        for (const auto &t : op.inputs) reads(t);
        for (const auto *spec : {&op.epilogue, &op.scaleA, &op.scaleB, &op.scaleOut}) {
            reads(spec->multiplier);
            reads(spec->shift);
        }
        for (const auto &t : op.outputs) {
            const auto it = index.find(root(t.get()));
            if (it != index.end() && producer.find(it->second) == producer.end()) producer[it->second] = p;
        }
    }
    // strict ancestors of every operator (operators are stored in a topological order: creation order)
    std::vector<std::vector<uint64_t>> ancestors(n, std::vector<uint64_t>(words, 0));
    for (size_t p = 0; p < n; p++) {
        const auto inherit = [&](const TensorPtr &t) {
            if (!t) return;
            const auto it = index.find(root(t.get()));
            if (it == index.end()) return;
            const auto pr = producer.find(it->second);
            if (pr == producer.end() || pr->second >= p) return;
            for (size_t w = 0; w < words; w++) ancestors[p][w] |= ancestors[pr->second][w];
            ancestors[p][pr->second / 64] |= uint64_t(1) << (pr->second % 64);
        };
        for (const auto &t : executed[p]->inputs) inherit(t);
    }
    std::map<size_t, std::set<size_t>> safe;
    for (const auto &[t, readers] : consumers) {
        if (producer.find(t) == producer.end() || tensors[t]->isGraphOutput || tensors[t]->isGraphInput) continue;
        for (const auto &[u, p] : producer) {
            if (u == t || tensors[u]->isGraphOutput || tensors[u]->isGraphInput) continue;
            const bool dead = std::all_of(readers.begin(), readers.end(), [&](size_t r) {
                return (ancestors[p][r / 64] >> (r % 64)) & 1;
            });
            if (dead) {
                safe[t].insert(u);
                safe[u].insert(t);
            }
        }
    }
    std::vector<details::BestFitTensor> out;
    std::map<size_t, uint64_t> sizes;
    for (const auto &iv : planned) sizes[iv.id] = iv.size;
    for (const auto &u : unseen) sizes[u.id] = u.size;
    for (const auto &[id, size] : sizes) {  // creation order
        details::BestFitTensor t{id, size, {}};
        const auto it = safe.find(id);
        if (it != safe.end())
            for (const size_t other : it->second)
                if (sizes.find(other) != sizes.end()) t.safe.push_back(other);
        out.push_back(std::move(t));
    }
    return out;
}

void GraphPipeline::setMemoryPlanner(const MemoryPlanner p) {
    if (finalized) fail("the memory planner is chosen before finalize()");
    planner = p;
}

std::vector<std::array<uint32_t, 2>> GraphPipeline::liveRanges() const {
    std::vector<std::array<uint32_t, 2>> r;
    for (const auto &t : tensors) {
        const auto it = ranges.find(t.get());
        r.push_back(it == ranges.end() ? std::array<uint32_t, 2>{~0u, ~0u} : it->second);
    }
    return r;
}

// Constant weight matrices of the fused products (fp16 MATMUL + bias + CAST, int8 MATMUL + RESCALE) are laid down
// row-wise once, [N][K] instead of the operator's [K][N] (one transposing launch per matrix while the pipeline is created), and handed to the kernel as the same [K][N]
// tensor with the two strides exchanged: both operands of the product are then rows of K, which the fp16 kernel
// fetches straight into shared memory (gemm_f16.hip) and the int8 kernels read like a convolution's weights.  The values and the operator are unchanged.  Pipeline creation is
// also where the reference spends its one-time work (shader specialisation, compute_graph_op.cpp:526-590).
void GraphPipeline::prepackConstants() {
    if (ctx == nullptr) return;
    std::map<const TensorDescriptor *, TensorPtr> rowWise;
    bool launched = false;
    for (const auto &opPtr : ops) {
        OpNode &op = *opPtr;
        if (op.fusedAway || (op.kind != OpKind::FusedMatmulBiasCast && op.kind != OpKind::FusedMatmul)) continue;
        const bool int8 = op.kind == OpKind::FusedMatmul;  // MATMUL + RESCALE: a fully connected layer
        const size_t perProduct = op.hasBias ? 2 : 1;
        const size_t products = int8 || op.extraProductViews.empty() ? 1 : op.outputs.size();
        for (size_t k = 0; k < products; k++) {
            const size_t idx = 1 + k * perProduct;
            if (idx >= op.inputs.size()) break;
            const TensorPtr b = op.inputs[idx];
            const auto &d = b->getDimensions();
            // what the row-wise form of the kernel takes: one fp16 matrix, K in whole 64-byte steps, N in 16-byte pieces
            // (fp16) or, for int8, K in 16-byte pieces and N in dwords
            const int32_t want = int8 ? MLEL_I8 : MLEL_F16;
            const int64_t es = int8 ? 1 : 2;
            if (b->getKind() != TensorKind::Constant || b->devicePointer() == nullptr || b->getFormat() != want ||
                d.size() != 3 || d[0] != 1 || !b->isPacked() || d[1] <= 1 || d[2] <= 1)
                continue;
            if (int8 ? (d[1] % 16 != 0 || d[2] % 4 != 0) : (d[1] % 32 != 0 || d[2] % 8 != 0)) continue;
            auto found = rowWise.find(b.get());
            if (found == rowWise.end()) {
                const int64_t K = d[1], N = d[2];
                auto t = std::make_shared<TensorDescriptor>(want, std::vector<int64_t>{1, K, N},
                                                            std::vector<int64_t>{K * N * es, es, K * es}, TensorKind::Constant);
                void *dptr = nullptr;
                check(mlel_hip_arena_alloc(ctx, static_cast<size_t>(K * N * es), &dptr), "allocating a row-wise weight matrix");
                constantsDeviceMemory.push_back(dptr);
                const mlel_tensor src = b->view();
                mlel_tensor dst{};
                dst.ptr = dptr;
                dst.dtype = want;
                dst.rank = 3;
                dst.dims[0] = 1, dst.dims[1] = N, dst.dims[2] = K;
                dst.strides[0] = K * N * es, dst.strides[1] = K * es, dst.strides[2] = es;
                const uint32_t perms[3] = {0, 2, 1};
                check(mlel_hip_transpose(ctx, nullptr, &dst, &src, perms), "laying a weight matrix down row-wise");
                launched = true;
                t->bind(dptr);
                found = rowWise.emplace(b.get(), registerTensor(std::move(t))).first;
            }
            op.inputs[idx] = found->second;
            MLEL_GRAPH_LOG(Debug, "Weight matrix row-wise. op=" << op.debugName << " input=" << idx << " tensor=" << found->second->id);
        }
    }
    if (!launched) return;
    check(mlel_hip_sync(ctx, nullptr), "laying weight matrices down row-wise");
    // the K-major copy of a matrix that no operator reads any more is given back (a weight then costs its size once)
    for (const auto &[kMajor, unused] : rowWise) {
        (void)unused;
        if (!consumersOf(ops, kMajor).empty()) continue;
        void *old = kMajor->devicePointer();
        const auto held = std::find(constantsDeviceMemory.begin(), constantsDeviceMemory.end(), old);
        if (held == constantsDeviceMemory.end()) continue;
        constantsDeviceMemory.erase(held);
        (void)mlel_hip_arena_free(ctx, old);
        const_cast<TensorDescriptor *>(kMajor)->bind(nullptr);
    }
}

void GraphPipeline::finalize(const bool enableFusion) {
    if (finalized) return;
    const size_t recorded = ops.size();
    if (enableFusion) fuse();
    if (enableFusion) prepackConstants();
    if (splitRequested) analyzeBatchSplit();
    plan();
    if (splitPrefix > 0) validateSplitPlan();
    finalized = true;
    size_t launches = 0;
    for (const auto &op : ops) launches += op->fusedAway ? 0 : 1;
    MLEL_GRAPH_LOG(Info, "Graph pipeline created: " << recorded << " operators recorded, " << launches
                                                    << " launches per dispatch, session memory " << sessionSize << " bytes");
    if (splitRequested)
        MLEL_GRAPH_LOG(Info, "Batch split: launches " << splitFirst << " to " << splitPrefix
                                                      << " (exclusive) issued per half batch of " << splitBatch / 2
                                                      << " on two streams");
}

void GraphPipeline::setBatchSplit(const bool enabled) {
    if (finalized) fail("setBatchSplit: the pipeline is already finalized");
    splitRequested = enabled;
}

namespace {

// The operands of `op` that carry the batch in their outermost extent (positions in op.inputs), for the operator kinds
// that treat the images of a batch independently; false for every other kind.
bool batchOperands(const OpNode &op, std::vector<size_t> &ins) {
    ins.clear();
    switch (op.kind) {
    case OpKind::Conv2D:
    case OpKind::DepthwiseConv2D:
    case OpKind::FusedConv2D:
    case OpKind::FusedDepthwiseConv2D:
    case OpKind::FusedConv2DDepthwise:
    case OpKind::FusedConv2DConv2D:
    case OpKind::FusedConv2DAvgPool:
    case OpKind::AvgPool2D:
    case OpKind::MaxPool2D:
    case OpKind::Rescale:
    case OpKind::Clamp:
    case OpKind::Table:
        ins = {0};
        return true;
    case OpKind::FusedConv2DResidual:
        ins = {0, 3};
        return true;
    case OpKind::FusedRescaleAddRescale:
        ins = {0, 1};
        return true;
    default:
        return false;
    }
}

}  // namespace

void GraphPipeline::analyzeBatchSplit() {
    splitFirst = 0;
    splitPrefix = 0;
    splitBatch = 0;
    if (planner == MemoryPlanner::BestFit || inputs.empty()) return;
    const auto &first = inputs.front();
    if (first->getRank() != 4) return;
    const int64_t n = first->getDimensions()[0];
    if (n < 2 || n % 2 != 0) return;
    const auto carriesBatch = [&](const TensorPtr &t) {
        return t && t->getKind() != TensorKind::Constant && t->getRank() == 4 && t->getDimensions()[0] == n &&
               t->isPacked();
    };
    uint32_t count = 0;
    std::vector<size_t> act;
    for (const auto &op : ops) {
        if (op->fusedAway) continue;
        if (!batchOperands(*op, act) || !carriesBatch(op->outputs[0])) break;
        // a second output only where the launch writes one (the stored intermediate of a convolution pair)
        if (op->outputs.size() != 1 &&
            !(op->kind == OpKind::FusedConv2DConv2D && op->outputs.size() == 2 && carriesBatch(op->outputs[1])))
            break;
        bool ok = true;
        for (size_t i = 0; i < op->inputs.size() && ok; i++) {
            const bool isAct = std::find(act.begin(), act.end(), i) != act.end();
            // everything but the activations is a constant of the pipeline (weights, bias, scales, tables)
            ok = isAct ? carriesBatch(op->inputs[i]) : (op->inputs[i] && op->inputs[i]->getKind() == TensorKind::Constant);
        }
        for (const auto *spec : {&op->epilogue, &op->scaleA, &op->scaleB, &op->scaleOut})
            for (const auto &t : {spec->multiplier, spec->shift}) ok = ok && (!t || t->getKind() == TensorKind::Constant);
        if (!ok) break;
        count++;
    }
    if (count < 2) return;
    // Where the two chains start: at the first launch.  Measured on the MobileNetV2-shaped graph at batch 32 (replayed
    // dispatch, 0.340 ms unsplit): 0.319 ms from launch 0, 0.314 from 4, 0.324 from 8, 0.329 from 12, 0.337 from 16,
    // 0.351 from 26 -- the large early launches lose nothing beside their other half and the short late ones gain
    // little, so the whole run is split.  MLEL_GRAPH_SPLIT_FROM in the environment names another position.
    uint32_t from = 0;
    if (const char *env = std::getenv("MLEL_GRAPH_SPLIT_FROM")) from = static_cast<uint32_t>(std::max(0, std::atoi(env)));
    if (from + 2 > count) return;
    splitFirst = from;
    splitPrefix = count;
    splitBatch = n;
}

// What the split dispatch relies on, checked on the host when the pipeline is finalized: inside either region no
// two tensors whose live ranges overlap share a byte (a region is used by one chain of launches), the half regions
// hold the halves they were planned for, and the three regions do not overlap.
void GraphPipeline::validateSplitPlan() const {
    struct Slot {
        const TensorDescriptor *t;
        size_t off, size;
        std::array<uint32_t, 2> range;
    };
    std::vector<Slot> whole, halves;
    for (const auto &[t, off] : offsets) {
        if (aliasOf.find(t) != aliasOf.end()) continue;  // a view of another tensor's storage
        const auto r = ranges.find(t);
        if (r == ranges.end()) continue;
        if (splitInterior.count(t))
            halves.push_back({t, off - splitFullRegion, t->getSize() / 2, r->second});
        else
            whole.push_back({t, off, t->getSize(), r->second});
    }
    const auto disjoint = [&](const std::vector<Slot> &v, size_t region, const char *what, bool wholeRegion) {
        for (size_t i = 0; i < v.size(); i++) {
            if (v[i].off + v[i].size > region) fail(std::string("batch split: a tensor leaves the ") + what + " region");
            for (size_t j = i + 1; j < v.size(); j++) {
                const bool bytes = v[i].off < v[j].off + v[j].size && v[j].off < v[i].off + v[i].size;
                // inside the split run two chains are out of step: every tensor it touches counts as live throughout
                const auto inRun = [&](const Slot &x) { return x.range[0] <= splitPrefix && x.range[1] >= splitFirst + 1; };
                const bool bothInRun = wholeRegion && inRun(v[i]) && inRun(v[j]);
                const bool time = bothInRun || (v[i].range[0] <= v[j].range[1] && v[j].range[0] <= v[i].range[1]);
                if (bytes && time) fail(std::string("batch split: two live tensors share bytes in the ") + what + " region");
            }
        }
    };
    disjoint(whole, splitHalfRegion != 0 ? splitFullRegion : sessionSize, "whole-tensor", true);
    disjoint(halves, splitHalfRegion, "half-batch", false);
    for (const auto &s : halves) {
        if (s.range[0] < splitFirst + 1 || s.range[1] > splitPrefix)
            fail("batch split: a half-stored tensor is used outside the split run");
        if (s.t->getDimensions().empty() || s.t->getDimensions()[0] != splitBatch || !s.t->isPacked())
            fail("batch split: a half-stored tensor does not carry the batch");
    }
    if (splitHalfRegion != 0 && sessionSize != splitFullRegion + 2 * splitHalfRegion)
        fail("batch split: session memory size does not match its regions");
}

void GraphPipeline::bindSessionMemory(void *deviceBase) {
    if (!finalized) fail("bindSessionMemory: finalize() has not run");
    if (sessionSize != 0 && deviceBase == nullptr) fail("bindSessionMemory: null session memory");
    if (reinterpret_cast<uintptr_t>(deviceBase) % kSessionAlignment != 0)
        fail("bindSessionMemory: session memory must be aligned to " + std::to_string(kSessionAlignment) + " bytes");
    for (const auto &[t, off] : offsets) const_cast<TensorDescriptor *>(t)->bind(static_cast<char *>(deviceBase) + off);
    appliedSession = nullptr;  // (a session that calls this records itself afterwards)
}

void GraphPipeline::bindExternal(const uint32_t set, const uint32_t binding, const uint32_t arrayIndex,
                                 void *devicePtr) {
    getTensor(set, binding, arrayIndex)->bind(devicePtr);
    appliedSession = nullptr;
}

// ---------------------------------------------------------------------------------------------------------------
// GraphSession
// ---------------------------------------------------------------------------------------------------------------
GraphSession::GraphSession(GraphPipeline &p) : pipeline(p) {
    if (!pipeline.isFinalized()) fail("session: the pipeline's finalize() has not run");
}

GraphSession::~GraphSession() {
    dropRecording();
    if (pipeline.ctx != nullptr) {
        if (splitLane.stream) {
            (void)mlel_hip_sync(pipeline.ctx, splitLane.stream);
            (void)mlel_hip_stream_destroy(pipeline.ctx, splitLane.stream);
        }
        if (splitLane.fork) (void)mlel_hip_event_destroy(pipeline.ctx, splitLane.fork);
        if (splitLane.join) (void)mlel_hip_event_destroy(pipeline.ctx, splitLane.join);
    }
    if (pipeline.appliedSession == this) pipeline.appliedSession = nullptr;
}

const GraphPipeline::SplitLane *GraphSession::lane() {
    if (pipeline.batchSplitLaunches() == 0) return nullptr;
    if (splitLane.stream == nullptr) {
        check(mlel_hip_stream_create(pipeline.ctx, &splitLane.stream), "creating the second stream of a split dispatch");
        check(mlel_hip_event_create(pipeline.ctx, &splitLane.fork), "creating the fork event");
        check(mlel_hip_event_create(pipeline.ctx, &splitLane.join), "creating the join event");
    }
    return &splitLane;
}

void GraphSession::dropRecording() {
    if (recording != nullptr && pipeline.ctx != nullptr) (void)mlel_hip_graph_destroy(pipeline.ctx, recording);
    recording = nullptr;
}

void GraphSession::bindTransientMemory(void *deviceBase) {
    if (needsTransientMemory() && deviceBase == nullptr) fail("bindTransientMemory: null session memory");
    if (reinterpret_cast<uintptr_t>(deviceBase) % GraphPipeline::kSessionAlignment != 0)
        fail("bindTransientMemory: session memory must be aligned to " +
             std::to_string(GraphPipeline::kSessionAlignment) + " bytes");
    base = deviceBase;
    transientMemoryBound = true;
    version++;
}

void GraphSession::bindExternal(const uint32_t set, const uint32_t binding, const uint32_t arrayIndex, void *devicePtr) {
    externals[pipeline.getTensor(set, binding, arrayIndex).get()] = devicePtr;
    version++;
}

void GraphSession::apply() {
    if (pipeline.appliedSession == this && pipeline.appliedVersion == version) return;
    if (needsTransientMemory()) pipeline.bindSessionMemory(base);
    // an external tensor this session has not bound must not keep another session's pointer
    for (const auto &[set, bindings] : pipeline.tensorMap)
        for (const auto &[binding, array] : bindings)
            for (const auto &t : array)
                if (t) t->bind(nullptr);
    for (const auto &[t, ptr] : externals) t->bind(ptr);
    pipeline.appliedSession = this;
    pipeline.appliedVersion = version;
}

void GraphSession::dispatch(void *stream, const GraphPipeline::DispatchDecorator &decorator, const uint32_t first,
                            const uint32_t count) {
    if (pipeline.ctx == nullptr)
        fail("dispatch: this GraphPipeline was built without a device context; there is no CPU path");
    // reference: "session transient memory is not bound" (graph_layer.cpp:1944-1947)
    if (needsTransientMemory() && !transientMemoryBound) fail("dispatch: session transient memory is not bound");
    apply();
    pipeline.dispatch(stream, decorator, first, count, lane());
}

void GraphSession::dispatchReplayed(void *stream) {
    if (pipeline.ctx == nullptr)
        fail("dispatch: this GraphPipeline was built without a device context; there is no CPU path");
    if (needsTransientMemory() && !transientMemoryBound) fail("dispatch: session transient memory is not bound");
    if (eagerVersion == version && eagerStream == stream) {
        // this session's dispatch could not be recorded with these bindings (below): it is issued launch by launch
        apply();
        pipeline.dispatch(stream, {}, 0, UINT32_MAX, lane());
        return;
    }
    if (recording == nullptr || recordingVersion != version || recordingStream != stream) {
        // the recording holds the addresses of this session's tensors as they are bound now
        dropRecording();
        apply();
        check(mlel_hip_capture_begin(pipeline.ctx, stream), "recording a dispatch");
        void *exec = nullptr;
        bool recorded = true;
        try {
            pipeline.dispatch(stream, {}, 0, UINT32_MAX, lane());
        } catch (...) {
            recorded = false;
        }
        // the stream must leave capture mode whatever happened
        const int endStatus = mlel_hip_capture_end(pipeline.ctx, stream, &exec);
        if (!recorded) {
            // An operator that needs a temporary (an operator-by-operator route of a fused call) refuses to run under
            // capture.  What was recorded is thrown away and the dispatch is issued eagerly, now and until the
            // bindings change; a failure that is not about the capture shows again there, with its own message.
            if (endStatus == 0 && exec != nullptr) (void)mlel_hip_graph_destroy(pipeline.ctx, exec);
            eagerVersion = version;
            eagerStream = stream;
            pipeline.dispatch(stream, {}, 0, UINT32_MAX, lane());
            return;
        }
        check(endStatus, "recording a dispatch");
        recording = exec;
        recordingVersion = version;
        recordingStream = stream;
    }
    check(mlel_hip_graph_launch(pipeline.ctx, recording, stream), "replaying a recorded dispatch");
}

namespace {

mlel_epilogue makeEpilogue(const RescaleSpec &spec, const mlel_tensor *mult, const mlel_tensor *shift, bool hasClamp,
                           const mlel_clamp_attr &clamp) {
    mlel_epilogue e{};
    e.multiplier = mult;
    e.shift = shift;
    e.rescale = spec.attr;
    e.has_clamp = hasClamp ? 1 : 0;
    e.clamp = clamp;
    return e;
}

}  // namespace

void GraphPipeline::run(const OpNode &op, void *stream, const int half) {
    std::array<mlel_tensor, 8> in{};
    // FusedElementwise describes its inputs itself (up to MLEL_CHAIN_MAX_INPUTS); every other kind reads `in`
    if (op.inputs.size() > in.size() && op.kind != OpKind::FusedElementwise)
        fail(op.tosaName + " (" + op.debugName + "): " + std::to_string(op.inputs.size()) +
             " inputs, more than an operator call carries");
    for (size_t i = 0; i < op.inputs.size() && i < in.size(); i++) {
        in[i] = op.inputs[i]->view();
        if (in[i].ptr == nullptr && op.inputs[i]->getShapeSize() != 0)
            fail(op.tosaName + " (" + op.debugName + "): input tensor " + std::to_string(i) + " has no memory bound");
    }
    mlel_tensor out = op.outputs[0]->view();
    if (out.ptr == nullptr && op.outputs[0]->getShapeSize() != 0)
        fail(op.tosaName + " (" + op.debugName + "): output tensor has no memory bound");
    // one half of the batch: half the outermost extent; the second half of a tensor stored as two halves lies one
    // region further, that of a whole tensor half its size further
    const auto halved = [&](mlel_tensor &v, const TensorDescriptor *t) {
        v.dims[0] = splitBatch / 2;
        const size_t step = splitInterior.count(t) ? splitHalfRegion : static_cast<size_t>(v.dims[0] * v.strides[0]);
        v.ptr = static_cast<char *>(v.ptr) + static_cast<size_t>(half) * step;
    };
    if (half >= 0) {
        std::vector<size_t> act;
        if (!batchOperands(op, act)) fail(op.tosaName + " (" + op.debugName + "): not an operator of the split run");
        for (const size_t i : act) halved(in[i], op.inputs[i].get());
        halved(out, op.outputs[0].get());
    }
    int rc = 0;
    switch (op.kind) {
    case OpKind::Conv2D: rc = mlel_hip_conv2d(ctx, stream, &out, &in[0], &in[1], &in[2], &op.conv); break;
    case OpKind::DepthwiseConv2D:
        rc = mlel_hip_depthwise_conv2d(ctx, stream, &out, &in[0], &in[1], &in[2], &op.conv);
        break;
    case OpKind::Matmul: rc = mlel_hip_matmul(ctx, stream, &out, &in[0], &in[1], &op.matmul); break;
    case OpKind::Rescale: rc = mlel_hip_rescale(ctx, stream, &out, &in[0], &in[1], &in[2], &op.rescale); break;
    case OpKind::Clamp: rc = mlel_hip_clamp(ctx, stream, &out, &in[0], &op.clamp); break;
    case OpKind::Binary:
        rc = mlel_hip_elementwise_binary(ctx, stream, op.selector, &out, &in[0], &in[1], op.nanMode);
        break;
    case OpKind::Mul: rc = mlel_hip_mul(ctx, stream, &out, &in[0], &in[1], op.shift); break;
    case OpKind::Unary: rc = mlel_hip_elementwise_unary(ctx, stream, op.selector, &out, &in[0]); break;
    case OpKind::Reduce: rc = mlel_hip_reduce(ctx, stream, op.selector, &out, &in[0], op.axis, op.nanMode); break;
    case OpKind::AvgPool2D: rc = mlel_hip_avg_pool2d(ctx, stream, &out, &in[0], &op.pool); break;
    case OpKind::MaxPool2D: rc = mlel_hip_max_pool2d(ctx, stream, &out, &in[0], &op.pool); break;
    case OpKind::Table: rc = mlel_hip_table(ctx, stream, &out, &in[0], &in[1]); break;
    case OpKind::Cast: rc = mlel_hip_cast(ctx, stream, &out, &in[0]); break;
    case OpKind::Negate:
        rc = mlel_hip_negate(ctx, stream, &out, &in[0], op.inputZeroPoint, op.outputZeroPoint);
        break;
    case OpKind::Reshape: rc = mlel_hip_reshape(ctx, stream, &out, &in[0]); break;
    case OpKind::Transpose: rc = mlel_hip_transpose(ctx, stream, &out, &in[0], op.vec.data()); break;
    case OpKind::Concat: rc = mlel_hip_concat(ctx, stream, &out, &in[0], op.axis, op.offset); break;
    case OpKind::Slice: rc = mlel_hip_slice(ctx, stream, &out, &in[0], op.vec.data()); break;
    case OpKind::Pad: rc = mlel_hip_pad(ctx, stream, &out, &in[0], &in[1], op.padConst, op.padConstInt); break;
    case OpKind::Argmax: rc = mlel_hip_argmax(ctx, stream, &out, &in[0], op.axis, op.nanMode); break;
    case OpKind::ArithmeticRightShift:
        rc = mlel_hip_arithmetic_right_shift(ctx, stream, &out, &in[0], &in[1], op.flag ? 1u : 0u);
        break;
    case OpKind::Conv3D: rc = mlel_hip_conv3d(ctx, stream, &out, &in[0], &in[1], &in[2], &op.conv3d); break;
    case OpKind::TransposeConv2D:
        rc = mlel_hip_transpose_conv2d(ctx, stream, &out, &in[0], &in[1], &in[2], &op.tconv);
        break;
    case OpKind::Fft2D:
    case OpKind::Rfft2D: {
        const mlel_tensor imag = op.outputs[1]->view();
        if (imag.ptr == nullptr && op.outputs[1]->getShapeSize() != 0)
            fail(op.tosaName + " (" + op.debugName + "): second output tensor has no memory bound");
        rc = op.kind == OpKind::Fft2D ? mlel_hip_fft2d(ctx, stream, &out, &imag, &in[0], &in[1], op.flag ? 1 : 0)
                                      : mlel_hip_rfft2d(ctx, stream, &out, &imag, &in[0]);
        break;
    }
    case OpKind::Gather: rc = mlel_hip_gather(ctx, stream, &out, &in[0], &in[1]); break;
    case OpKind::Scatter: rc = mlel_hip_scatter(ctx, stream, &out, &in[0], &in[1], &in[2]); break;
    case OpKind::Resize: rc = mlel_hip_resize(ctx, stream, &out, &in[0], &op.resize); break;
    case OpKind::Reverse: rc = mlel_hip_reverse(ctx, stream, &out, &in[0], op.axis); break;
    case OpKind::Tile: rc = mlel_hip_tile(ctx, stream, &out, &in[0]); break;
    case OpKind::Select: rc = mlel_hip_select(ctx, stream, &out, &in[0], &in[1], &in[2]); break;
    case OpKind::FusedConv2D:
    case OpKind::FusedDepthwiseConv2D:
    case OpKind::FusedMatmul: {
        const mlel_tensor mult = op.epilogue.multiplier->view(), shift = op.epilogue.shift->view();
        const mlel_epilogue e = makeEpilogue(op.epilogue, &mult, &shift, op.hasClamp, op.clamp);
        if (op.kind == OpKind::FusedConv2D)
            rc = mlel_hip_conv2d_rescale_clamp(ctx, stream, &out, &in[0], &in[1], &in[2], &op.conv, &e);
        else if (op.kind == OpKind::FusedDepthwiseConv2D)
            rc = mlel_hip_dwconv_rescale_clamp(ctx, stream, &out, &in[0], &in[1], &in[2], &op.conv, &e);
        else
            rc = mlel_hip_matmul_rescale(ctx, stream, &out, &in[0], &in[1], &op.matmul, &e);
        break;
    }
    case OpKind::FusedElementwise: {
        mlel_chain c{};
        std::vector<mlel_tensor> views;
        for (const auto &t : op.inputs) {
            views.push_back(t->view());
            if (views.back().ptr == nullptr && t->getShapeSize() != 0)
                fail(op.tosaName + " (" + op.debugName + "): an input of the fused region has no memory bound");
        }
        c.n_inputs = static_cast<int32_t>(views.size());
        for (size_t i = 0; i < views.size(); i++) c.inputs[i] = &views[i];
        c.n_steps = static_cast<int32_t>(op.chain.size());
        for (size_t i = 0; i < op.chain.size(); i++) c.steps[i] = op.chain[i];
        rc = mlel_hip_elementwise_chain(ctx, stream, &out, &c);
        break;
    }
    case OpKind::FusedMatmulBiasCast: {
        const auto viewed = [](mlel_tensor t, const std::array<int64_t, 6> &dims, const std::array<int64_t, 6> &strides) {
            t.rank = 6;  // the transposed tensor's storage, addressed with the product's split extents
            for (size_t k = 0; k < 6; k++) {
                t.dims[k] = dims[k];
                t.strides[k] = strides[k];
            }
            return t;
        };
        if (!op.extraProductViews.empty()) {
            const size_t perProduct = op.hasBias ? 2 : 1, count = op.outputs.size();
            std::vector<mlel_tensor> outs(count);
            std::vector<mlel_matmul_product> products(count);
            for (size_t k = 0; k < count; k++) {
                const auto &dims = k == 0 ? op.viewDims : op.extraProductViews[k - 1].first;
                const auto &strides = k == 0 ? op.viewStrides : op.extraProductViews[k - 1].second;
                outs[k] = op.outputs[k]->view();
                if (dims[5] != 0) outs[k] = viewed(outs[k], dims, strides);
                products[k] = mlel_matmul_product{&outs[k], &in[1 + k * perProduct], op.hasBias ? &in[2 + k * perProduct] : nullptr};
            }
            rc = mlel_hip_matmul_bias_cast_group(ctx, stream, products.data(), static_cast<int>(count), &in[0], &op.matmul);
            break;
        }
        const mlel_tensor *bias = op.hasBias ? &in[2] : nullptr;
        if (!op.chain.empty()) {  // the product, then the elementwise region over it
            mlel_chain c{};
            const size_t own = op.hasBias ? 3 : 2;  // a, b (, bias); the region's own inputs follow
            c.n_inputs = static_cast<int32_t>(op.inputs.size() - own + 1);
            c.n_steps = static_cast<int32_t>(op.chain.size());
            c.inputs[0] = nullptr;
            for (size_t i = own; i < op.inputs.size(); i++) c.inputs[i - own + 1] = &in[i];
            for (size_t i = 0; i < op.chain.size(); i++) c.steps[i] = op.chain[i];
            rc = mlel_hip_matmul_bias_cast_chain(ctx, stream, &out, &in[0], &in[1], bias, &op.matmul, &c);
            break;
        }
        if (op.flag) {
            // the addition may have been written with other extents over the same packed bytes: both tensors are
            // handed over with the product's extents [batches, rows, columns]
            const auto as_product = [&](mlel_tensor t) {
                t.rank = 3;
                t.dims[0] = in[0].dims[0], t.dims[1] = in[0].dims[1], t.dims[2] = in[1].dims[2];
                t.strides[2] = 2;
                t.strides[1] = t.dims[2] * 2;
                t.strides[0] = t.dims[1] * t.strides[1];
                return t;
            };
            const mlel_tensor out3 = as_product(out), res3 = as_product(in[op.inputs.size() - 1]);
            rc = mlel_hip_matmul_bias_cast_add(ctx, stream, &out3, &in[0], &in[1], bias, &op.matmul, &res3);
        } else if (op.viewDims[5] != 0) {
            mlel_tensor view = out;  // the transposed tensor's storage, addressed with the product's split extents
            view.rank = 6;
            for (size_t k = 0; k < 6; k++) {
                view.dims[k] = op.viewDims[k];
                view.strides[k] = op.viewStrides[k];
            }
            rc = mlel_hip_matmul_bias_cast(ctx, stream, &view, &in[0], &in[1], bias, &op.matmul);
        } else {
            rc = mlel_hip_matmul_bias_cast(ctx, stream, &out, &in[0], &in[1], bias, &op.matmul);
        }
        break;
    }
    case OpKind::FusedAttention: {
        mlel_chain c{};
        c.n_inputs = static_cast<int32_t>(op.inputs.size() - 3 + 1);  // q, kt, v, then the chain's inputs from 1 on
        c.n_steps = static_cast<int32_t>(op.chain.size());
        c.inputs[0] = nullptr;
        for (size_t i = 3; i < op.inputs.size(); i++) c.inputs[i - 3 + 1] = &in[i];
        for (size_t i = 0; i < op.chain.size(); i++) c.steps[i] = op.chain[i];
        mlel_tensor view = out;
        if (op.viewDims[5] != 0) {
            view.rank = 6;
            for (size_t k = 0; k < 6; k++) {
                view.dims[k] = op.viewDims[k];
                view.strides[k] = op.viewStrides[k];
            }
        }
        rc = mlel_hip_attention_f16(ctx, stream, &view, &in[0], &in[1], &in[2], &c);
        break;
    }
    case OpKind::FusedConv2DDepthwise: {
        const mlel_tensor m1 = op.scaleA.multiplier->view(), s1 = op.scaleA.shift->view();
        const mlel_tensor m2 = op.epilogue.multiplier->view(), s2 = op.epilogue.shift->view();
        const mlel_epilogue e1 = makeEpilogue(op.scaleA, &m1, &s1, op.hasClampFirst, op.clampFirst);
        const mlel_epilogue e2 = makeEpilogue(op.epilogue, &m2, &s2, op.hasClamp, op.clamp);
        rc = mlel_hip_conv2d_dwconv_rescale_clamp(ctx, stream, &out, &in[0], &in[1], &in[2], &op.convFirst, &e1, &in[3],
                                                  &in[4], &op.conv, &e2);
        break;
    }
    case OpKind::FusedConv2DAvgPool: {
        const mlel_tensor mult = op.epilogue.multiplier->view(), shift = op.epilogue.shift->view();
        const mlel_epilogue e = makeEpilogue(op.epilogue, &mult, &shift, op.hasClamp, op.clamp);
        rc = mlel_hip_conv2d_rescale_clamp_avgpool(ctx, stream, &out, &in[0], &in[1], &in[2], &op.conv, &e, op.selector,
                                                   &op.pool);
        break;
    }
    case OpKind::FusedConv2DConv2D: {
        const mlel_tensor m1 = op.scaleA.multiplier->view(), s1 = op.scaleA.shift->view();
        const mlel_tensor m2 = op.epilogue.multiplier->view(), s2 = op.epilogue.shift->view();
        const mlel_epilogue e1 = makeEpilogue(op.scaleA, &m1, &s1, op.hasClampFirst, op.clampFirst);
        const mlel_epilogue e2 = makeEpilogue(op.epilogue, &m2, &s2, op.hasClamp, op.clamp);
        mlel_tensor mid{};
        const bool keep = op.outputs.size() > 1;
        if (keep) {
            mid = op.outputs[1]->view();
            if (mid.ptr == nullptr && op.outputs[1]->getShapeSize() != 0)
                fail(op.tosaName + " (" + op.debugName + "): the intermediate tensor has no memory bound");
            if (half >= 0) halved(mid, op.outputs[1].get());
        }
        rc = mlel_hip_conv2d_conv2d_rescale_clamp(ctx, stream, &out, keep ? &mid : nullptr, &in[0], &in[1], &in[2],
                                                  &op.convFirst, &e1, &in[3], &in[4], &op.conv, &e2);
        break;
    }
    case OpKind::FusedConv2DResidual: {
        const mlel_tensor mult = op.epilogue.multiplier->view(), shift = op.epilogue.shift->view();
        const mlel_tensor ma = op.scaleA.multiplier->view(), sa = op.scaleA.shift->view();
        const mlel_tensor mb = op.scaleB.multiplier->view(), sb = op.scaleB.shift->view();
        const mlel_tensor mo = op.scaleOut.multiplier->view(), so = op.scaleOut.shift->view();
        const mlel_clamp_attr none{};
        const mlel_epilogue e = makeEpilogue(op.epilogue, &mult, &shift, op.hasClamp, op.clamp);
        const mlel_epilogue ea = makeEpilogue(op.scaleA, &ma, &sa, false, none);
        const mlel_epilogue eb = makeEpilogue(op.scaleB, &mb, &sb, false, none);
        const mlel_epilogue eo = makeEpilogue(op.scaleOut, &mo, &so, false, none);
        rc = mlel_hip_conv2d_rescale_add_rescale(ctx, stream, &out, &in[0], &in[1], &in[2], &op.conv, &e, &ea, &in[3], &eb,
                                                 &eo, op.flag ? 1 : 0);
        break;
    }
    case OpKind::FusedRescaleAddRescale: {
        const mlel_tensor ma = op.scaleA.multiplier->view(), sa = op.scaleA.shift->view();
        const mlel_tensor mb = op.scaleB.multiplier->view(), sb = op.scaleB.shift->view();
        const mlel_tensor mo = op.epilogue.multiplier->view(), so = op.epilogue.shift->view();
        const mlel_clamp_attr none{};
        const mlel_epilogue ea = makeEpilogue(op.scaleA, &ma, &sa, false, none);
        const mlel_epilogue eb = makeEpilogue(op.scaleB, &mb, &sb, false, none);
        const mlel_epilogue eo = makeEpilogue(op.epilogue, &mo, &so, false, none);
        rc = mlel_hip_rescale_add_rescale(ctx, stream, &out, &in[0], &ea, &in[1], &eb, &eo);
        break;
    }
    }
    if (rc != 0) fail(op.tosaName + " (" + op.debugName + "): " + mlel_hip_last_error());
}

void GraphPipeline::dispatch(void *stream, const DispatchDecorator &decorator, const uint32_t first,
                             const uint32_t count, const SplitLane *lane) {
    if (!finalized) fail("dispatch: finalize() has not run");
    if (ctx == nullptr) fail("dispatch: this GraphPipeline was built without a device context; there is no CPU path");
    // two streams only for a whole, undecorated dispatch; otherwise the two halves of a split launch follow each
    // other on `stream`
    const bool fork = splitPrefix > 0 && lane != nullptr && lane->stream != nullptr && !decorator && first == 0 &&
                      count == UINT32_MAX;
    const auto check = [&](int rc, const char *what) {
        if (rc != 0) fail(std::string("dispatch: ") + what + ": " + mlel_hip_last_error());
    };
    bool forked = false, joined = !fork;
    const auto forkNow = [&] {
        if (!fork || forked) return;
        check(mlel_hip_event_record(ctx, lane->fork, stream), "recording the fork");
        check(mlel_hip_stream_wait_event(ctx, lane->stream, lane->fork), "starting the second half");
        forked = true;
    };
    const auto join = [&] {
        if (joined || !forked) return;
        check(mlel_hip_event_record(ctx, lane->join, lane->stream), "recording the join");
        check(mlel_hip_stream_wait_event(ctx, stream, lane->join), "waiting for the second half");
        joined = true;
    };
    uint32_t index = 0;
    try {
        for (const auto &op : ops) {
            if (op->fusedAway) continue;
            if (index >= first && index - first < count) {
                if (decorator) decorator(*op, index, true);
                if (index >= splitFirst && index < splitPrefix) {
                    forkNow();
                    run(*op, stream, 0);
                    run(*op, fork ? lane->stream : stream, 1);
                } else {
                    join();
                    run(*op, stream);
                }
                if (decorator) decorator(*op, index, false);
            }
            index++;
        }
    } catch (...) {
        // the second stream must come back to `stream` whatever happened (a capture cannot end with it forked)
        if (forked && !joined) {
            (void)mlel_hip_event_record(ctx, lane->join, lane->stream);
            (void)mlel_hip_stream_wait_event(ctx, stream, lane->join);
        }
        throw;
    }
    join();
}

}  // namespace mlel::graph
