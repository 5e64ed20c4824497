// C wrapper over GraphPipeline (include/mlel_graph.h).  Exceptions stop here and become status codes.
//
// mlel_graph_make_op attribute layout per TOSA operator (tensor handles follow the make<Op> signature order):
//   CONV2D / DEPTHWISE_CONV2D  in: input, weights, biases   out: output
//        iattr: pad[4] stride[2] dilation[2] inputZp weightZp accType
//   MATMUL                     in: input1, input2           iattr: zp1 zp2
//   RESCALE                    in: input, multiplier, shift iattr: inZp outZp scale32 doubleRound perChannel
//                                                                  inputUnsigned outputUnsigned
//   CLAMP                      in: input                    fattr: min max      iattr: nanMode
//   AVG_POOL2D                 in: input                    iattr: kernel[2] stride[2] pad[4] accType inZp outZp
//   MAX_POOL2D                 in: input                    iattr: kernel[2] stride[2] pad[4] nanMode
//   MAXIMUM / MINIMUM          in: input1, input2           iattr: nanMode
//   MUL                        in: input1, input2           iattr: shift
//   REDUCE_MAX / REDUCE_MIN    in: input                    iattr: axis nanMode
//   REDUCE_ALL/ANY/PRODUCT/SUM in: input                    iattr: axis
//   TABLE                      in: input, table
//   NEGATE                     in: input                    iattr: inZp outZp
//   CONCAT                     in: input0, input1, ...      iattr: axis
//   SLICE                      in: input                    iattr: start[rank]
//   TRANSPOSE                  in: input                    iattr: perms[rank]
//   PAD                        in: input, padding           fattr: padConst     iattr: padConstInt
//   ARGMAX                     in: input                    iattr: axis nanMode
//   ARITHMETIC_RIGHT_SHIFT     in: input1, input2           iattr: round
//   CONV3D                     in: input, weights, biases   iattr: pad[6] stride[3] dilation[3] inputZp weightZp accType
//   TRANSPOSE_CONV2D           in: input, weights, biases   iattr: outPad[4] stride[2] inputZp weightZp accType
//   GATHER                     in: values, indices
//   SCATTER                    in: valuesIn, indices, input (the operand order of the TOSA instruction)
//   REVERSE                    in: input                    iattr: axis
//   TILE                       in: input
//   RESIZE                     in: input                    iattr: scale[4] offset[2] border[2] mode
//   SELECT                     in: condition, onTrue, onFalse
//   FFT2D                      in: real, imag               out: real, imag       iattr: inverse
//   RFFT2D                     in: input                    out: real, imag
//   binary (ADD SUB BITWISE_* LOGICAL_* INTDIV POW EQUAL GREATER GREATER_EQUAL): in: input1, input2
//   unary (ABS ... TANH), CAST, RESHAPE: in: input
#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <map>
#include <memory>
#include <sstream>
#include <string>

#include "../../../include/mlel_graph.h"
#include "graph_log.hpp"
#include "graph_pipeline.hpp"
#include "session_planner.hpp"
#include "spirv_graph_loader.hpp"

using namespace mlel::graph;

struct ProfileSample {
    uint64_t dispatch;  // which mlel_graph_dispatch call of this graph
    uint32_t index;     // position in the execution list
    std::string name;
    double ms;
};

struct mlel_graph {
    GraphPipeline pipeline;
    std::unique_ptr<GraphSession> defaultSession;  // behind mlel_graph_bind_* / mlel_graph_dispatch
    mlel_ctx *ctx;
    std::vector<void *> events;  // pairs of profiling events, created on demand
    bool profiling = false;      // mlel_graph_dispatch records a sample per operator (VMEL_GRAPH_PROFILING)
    uint64_t dispatches = 0;
    std::vector<ProfileSample> samples;
    explicit mlel_graph(mlel_ctx *c) : pipeline(c), ctx(c) {}
    GraphSession &session() {
        if (!defaultSession) defaultSession = std::make_unique<GraphSession>(pipeline);
        return *defaultSession;
    }
};

struct mlel_graph_session {
    mlel_graph *graph;
    GraphSession session;
    explicit mlel_graph_session(mlel_graph *g) : graph(g), session(g->pipeline) {}
};

namespace {

thread_local std::string g_error;

// VMEL_GRAPH_PROFILING: anything but empty, 0, false, off, no (graph/graph_profiler.cpp:29-38)
bool truthy(const char *value) {
    if (value == nullptr || value[0] == 0) return false;
    std::string v(value);
    for (auto &c : v) c = static_cast<char>(std::tolower(static_cast<unsigned char>(c)));
    return v != "0" && v != "false" && v != "off" && v != "no";
}

template <typename F>
int guarded(F &&f) {
    try {
        return f();
    } catch (const std::out_of_range &e) {
        g_error = std::string("not found: ") + e.what();
        MLEL_GRAPH_LOG(Error, g_error);
        return MLEL_ERR_INVALID;
    } catch (const std::exception &e) {
        g_error = e.what();
        MLEL_GRAPH_LOG(Error, g_error);
        const bool unsupported = g_error.find("has no kernel") != std::string::npos;
        return unsupported ? MLEL_ERR_UNSUPPORTED : MLEL_ERR_INVALID;
    }
}

std::vector<int64_t> vec64(const int64_t *p, int n) { return p ? std::vector<int64_t>(p, p + n) : std::vector<int64_t>{}; }

TensorPtr handle(mlel_graph *g, int h) {
    const auto &all = g->pipeline.handles();
    if (h < 0 || static_cast<size_t>(h) >= all.size()) throw std::runtime_error("bad tensor handle " + std::to_string(h));
    return all[static_cast<size_t>(h)];
}

struct Args {
    mlel_graph *g;
    std::vector<TensorPtr> in, out;
    const int64_t *ia;
    int nia;
    const double *fa;
    int nfa;
    std::string name;
    int64_t i(int k) const {
        if (k >= nia) throw std::runtime_error("too few integer attributes");
        return ia[k];
    }
    double f(int k) const {
        if (k >= nfa) throw std::runtime_error("too few real attributes");
        return fa[k];
    }
    std::vector<int32_t> iv(int from, int n) const {
        std::vector<int32_t> v;
        for (int k = 0; k < n; k++) v.push_back(static_cast<int32_t>(i(from + k)));
        return v;
    }
    std::vector<uint32_t> uv(int from, int n) const {
        std::vector<uint32_t> v;
        for (int k = 0; k < n; k++) v.push_back(static_cast<uint32_t>(i(from + k)));
        return v;
    }
    const TensorPtr &I(size_t k) const {
        if (k >= in.size()) throw std::runtime_error("too few input tensors");
        return in[k];
    }
    const TensorPtr &O(size_t k = 0) const {
        if (k >= out.size()) throw std::runtime_error("too few output tensors");
        return out[k];
    }
};

using Maker = void (*)(GraphPipeline &, const Args &);

#define BIN(NAME, METHOD)                                                                                              \
    { NAME, [](GraphPipeline &p, const Args &a) { p.METHOD(a.I(0), a.I(1), a.O(), a.name); } }
#define UN(NAME, METHOD)                                                                                               \
    { NAME, [](GraphPipeline &p, const Args &a) { p.METHOD(a.I(0), a.O(), a.name); } }

const std::map<std::string, Maker> &makers() {
    static const std::map<std::string, Maker> m = {
        {"CONV2D",
         [](GraphPipeline &p, const Args &a) {
             p.makeConv2D(a.I(0), a.O(), a.I(1), a.I(2), a.iv(0, 4), a.iv(4, 2), a.iv(6, 2),
                          static_cast<int8_t>(a.i(8)), static_cast<int8_t>(a.i(9)), static_cast<uint32_t>(a.i(10)),
                          a.name);
         }},
        {"DEPTHWISE_CONV2D",
         [](GraphPipeline &p, const Args &a) {
             p.makeDepthwiseConv2D(a.I(0), a.O(), a.I(1), a.I(2), a.iv(0, 4), a.iv(4, 2), a.iv(6, 2),
                                   static_cast<int8_t>(a.i(8)), static_cast<int8_t>(a.i(9)),
                                   static_cast<uint32_t>(a.i(10)), a.name);
         }},
        {"MATMUL",
         [](GraphPipeline &p, const Args &a) {
             p.makeMatmul(a.I(0), a.I(1), a.O(), static_cast<int32_t>(a.i(0)), static_cast<int32_t>(a.i(1)), a.name);
         }},
        {"RESCALE",
         [](GraphPipeline &p, const Args &a) {
             p.makeRescale(a.I(0), a.O(), static_cast<int32_t>(a.i(0)), static_cast<int32_t>(a.i(1)), a.I(1), a.I(2),
                           a.i(2) != 0, a.i(3) != 0, a.i(4) != 0, a.i(5) != 0, a.i(6) != 0, a.name);
         }},
        {"CLAMP",
         [](GraphPipeline &p, const Args &a) {
             p.makeClamp(a.I(0), a.O(), a.f(0), a.f(1), static_cast<uint32_t>(a.i(0)), a.name);
         }},
        {"AVG_POOL2D",
         [](GraphPipeline &p, const Args &a) {
             p.makeAvgPool2D(a.I(0), a.O(), a.iv(0, 2), a.iv(2, 2), a.iv(4, 4), static_cast<uint32_t>(a.i(8)),
                             static_cast<int8_t>(a.i(9)), static_cast<int8_t>(a.i(10)), a.name);
         }},
        {"MAX_POOL2D",
         [](GraphPipeline &p, const Args &a) {
             p.makeMaxPool2D(a.I(0), a.O(), a.iv(0, 2), a.iv(2, 2), a.iv(4, 4), static_cast<uint32_t>(a.i(8)), a.name);
         }},
        {"MAXIMUM",
         [](GraphPipeline &p, const Args &a) {
             p.makeMaximum(a.I(0), a.I(1), a.O(), static_cast<uint32_t>(a.i(0)), a.name);
         }},
        {"MINIMUM",
         [](GraphPipeline &p, const Args &a) {
             p.makeMinimum(a.I(0), a.I(1), a.O(), static_cast<uint32_t>(a.i(0)), a.name);
         }},
        {"MUL",
         [](GraphPipeline &p, const Args &a) {
             p.makeMul(a.I(0), a.I(1), a.O(), static_cast<uint32_t>(a.i(0)), a.name);
         }},
        {"REDUCE_MAX",
         [](GraphPipeline &p, const Args &a) {
             p.makeReduceMax(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), static_cast<uint32_t>(a.i(1)), a.name);
         }},
        {"REDUCE_MIN",
         [](GraphPipeline &p, const Args &a) {
             p.makeReduceMin(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), static_cast<uint32_t>(a.i(1)), a.name);
         }},
        {"REDUCE_ALL",
         [](GraphPipeline &p, const Args &a) { p.makeReduceAll(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), a.name); }},
        {"REDUCE_ANY",
         [](GraphPipeline &p, const Args &a) { p.makeReduceAny(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), a.name); }},
        {"REDUCE_PRODUCT",
         [](GraphPipeline &p, const Args &a) {
             p.makeReduceProduct(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), a.name);
         }},
        {"REDUCE_SUM",
         [](GraphPipeline &p, const Args &a) { p.makeReduceSum(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), a.name); }},
        {"TABLE", [](GraphPipeline &p, const Args &a) { p.makeTable(a.I(0), a.O(), a.I(1), a.name); }},
        {"NEGATE",
         [](GraphPipeline &p, const Args &a) {
             p.makeNegate(a.I(0), a.O(), static_cast<int32_t>(a.i(0)), static_cast<int32_t>(a.i(1)), a.name);
         }},
        {"CONCAT",
         [](GraphPipeline &p, const Args &a) { p.makeConcat(a.in, a.O(), static_cast<uint32_t>(a.i(0)), a.name); }},
        {"SLICE",
         [](GraphPipeline &p, const Args &a) {
             p.makeSlice(a.I(0), a.O(), a.uv(0, static_cast<int>(a.I(0)->getRank())), a.name);
         }},
        {"TRANSPOSE",
         [](GraphPipeline &p, const Args &a) {
             p.makeTranspose(a.I(0), a.O(), a.uv(0, static_cast<int>(a.I(0)->getRank())), a.name);
         }},
        {"PAD",
         [](GraphPipeline &p, const Args &a) {
             p.makePad(a.I(0), a.O(), a.I(1), a.f(0), static_cast<int32_t>(a.i(0)), a.name);
         }},
        BIN("ADD", makeAdd), BIN("SUB", makeSub), BIN("BITWISE_AND", makeBitwiseAnd), BIN("BITWISE_OR", makeBitwiseOr),
        BIN("BITWISE_XOR", makeBitwiseXor), BIN("INTDIV", makeIntdiv), BIN("LOGICAL_AND", makeLogicalAnd),
        BIN("LOGICAL_OR", makeLogicalOr), BIN("LOGICAL_XOR", makeLogicalXor),
        BIN("LOGICAL_LEFT_SHIFT", makeLogicalLeftShift), BIN("LOGICAL_RIGHT_SHIFT", makeLogicalRightShift),
        BIN("POW", makePow), BIN("EQUAL", makeEqual), BIN("GREATER", makeGreater),
        BIN("GREATER_EQUAL", makeGreaterEqual),
        UN("ABS", makeAbs), UN("BITWISE_NOT", makeBitwiseNot), UN("CEIL", makeCeil), UN("CLZ", makeClz),
        UN("COS", makeCos), UN("ERF", makeErf), UN("EXP", makeExp), UN("FLOOR", makeFloor), UN("LOG", makeLog),
        UN("LOGICAL_NOT", makeLogicalNot), UN("RECIPROCAL", makeReciprocal), UN("RSQRT", makeRsqrt),
        UN("SIGMOID", makeSigmoid), UN("SIN", makeSin), UN("TANH", makeTanh), UN("CAST", makeCast),
        UN("RESHAPE", makeReshape),
        {"ARGMAX",
         [](GraphPipeline &p, const Args &a) {
             p.makeArgmax(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), static_cast<uint32_t>(a.i(1)), a.name);
         }},
        {"ARITHMETIC_RIGHT_SHIFT",
         [](GraphPipeline &p, const Args &a) { p.makeArithmeticRightShift(a.I(0), a.I(1), a.O(), a.i(0) != 0, a.name); }},
        {"CONV3D",
         [](GraphPipeline &p, const Args &a) {
             p.makeConv3D(a.I(0), a.O(), a.I(1), a.I(2), a.iv(0, 6), a.iv(6, 3), a.iv(9, 3), static_cast<int8_t>(a.i(12)),
                          static_cast<int8_t>(a.i(13)), static_cast<uint32_t>(a.i(14)), a.name);
         }},
        {"TRANSPOSE_CONV2D",
         [](GraphPipeline &p, const Args &a) {
             p.makeTransposeConv2D(a.I(0), a.O(), a.I(1), a.I(2), a.iv(0, 4), a.iv(4, 2), static_cast<int8_t>(a.i(6)),
                                   static_cast<int8_t>(a.i(7)), static_cast<uint32_t>(a.i(8)), a.name);
         }},
        {"GATHER", [](GraphPipeline &p, const Args &a) { p.makeGather(a.I(0), a.I(1), a.O(), a.name); }},
        {"SCATTER", [](GraphPipeline &p, const Args &a) { p.makeScatter(a.I(2), a.I(0), a.I(1), a.O(), a.name); }},
        {"REVERSE",
         [](GraphPipeline &p, const Args &a) { p.makeReverse(a.I(0), a.O(), static_cast<uint32_t>(a.i(0)), a.name); }},
        {"TILE", [](GraphPipeline &p, const Args &a) { p.makeTile(a.I(0), a.O(), a.name); }},
        {"RESIZE",
         [](GraphPipeline &p, const Args &a) {
             p.makeResize(a.I(0), a.O(), a.iv(0, 4), a.iv(4, 2), a.iv(6, 2), static_cast<uint32_t>(a.i(8)), a.name);
         }},
        {"SELECT", [](GraphPipeline &p, const Args &a) { p.makeSelect(a.I(0), a.I(1), a.I(2), a.O(), a.name); }},
        {"FFT2D",
         [](GraphPipeline &p, const Args &a) { p.makeFft2D(a.I(0), a.I(1), a.O(0), a.O(1), a.i(0) != 0, a.name); }},
        {"RFFT2D", [](GraphPipeline &p, const Args &a) { p.makeRfft2D(a.I(0), a.O(0), a.O(1), a.name); }},
    };
    return m;
}

std::string opLabel(const OpNode &op) {
    switch (op.kind) {
    case OpKind::FusedConv2D: return std::string("CONV2D+RESCALE") + (op.hasClamp ? "+CLAMP" : "");
    case OpKind::FusedDepthwiseConv2D: return std::string("DEPTHWISE_CONV2D+RESCALE") + (op.hasClamp ? "+CLAMP" : "");
    case OpKind::FusedMatmul: return std::string("MATMUL+RESCALE") + (op.hasClamp ? "+CLAMP" : "");
    case OpKind::FusedRescaleAddRescale: return "RESCALE+RESCALE+ADD+RESCALE";
    case OpKind::FusedConv2DResidual:
        return std::string("CONV2D+RESCALE") + (op.hasClamp ? "+CLAMP" : "") + "+RESCALE+RESCALE+ADD+RESCALE";
    case OpKind::FusedElementwise: {
        bool reduces = false;
        for (const auto &st : op.chain) reduces = reduces || st.kind == MLEL_CHAIN_REDUCE;
        return (reduces ? "ELEMENTWISE+REDUCE x" : "ELEMENTWISE x") + std::to_string(op.chain.size());
    }
    case OpKind::FusedMatmulBiasCast:
    {
        std::string name = std::string(op.hasBias ? "MATMUL+ADD+CAST" : "MATMUL+CAST") + (op.flag ? "+ADD" : "") +
                           (op.viewDims[5] != 0 ? "+RESHAPE+TRANSPOSE" : "");
        if (!op.chain.empty()) name += "+ELEMENTWISE x" + std::to_string(op.chain.size());
        for (const auto &view : op.extraProductViews)
            name += std::string(" | ") + (op.hasBias ? "MATMUL+ADD+CAST" : "MATMUL+CAST") +
                    (view.first[5] != 0 ? "+RESHAPE+TRANSPOSE" : "");
        return name;
    }
    case OpKind::FusedConv2DDepthwise:
        return std::string("CONV2D+RESCALE") + (op.hasClampFirst ? "+CLAMP" : "") + "+DEPTHWISE_CONV2D+RESCALE" +
               (op.hasClamp ? "+CLAMP" : "");
    case OpKind::FusedConv2DConv2D:
        // "+KEEP": the first convolution's result is stored as well (a later operator reads it)
        return std::string("CONV2D+RESCALE") + (op.hasClampFirst ? "+CLAMP" : "") + (op.outputs.size() > 1 ? "+KEEP" : "") +
               "+CONV2D+RESCALE" + (op.hasClamp ? "+CLAMP" : "");
    case OpKind::FusedConv2DAvgPool:
        return std::string("CONV2D+RESCALE") + (op.hasClamp ? "+CLAMP" : "") + "+AVG_POOL2D";
    case OpKind::FusedAttention:
        return std::string("MATMUL+CAST+ELEMENTWISE+REDUCE x") + std::to_string(op.chain.size()) + "+MATMUL+CAST" +
               (op.viewDims[5] != 0 ? "+RESHAPE+TRANSPOSE" : "");
    default: return op.tosaName;
    }
}

}  // namespace

extern "C" {

const char *mlel_graph_last_error(void) { return g_error.c_str(); }

int mlel_graph_create(mlel_ctx *ctx, mlel_graph **out) {
    return guarded([&] {
        if (out == nullptr) throw std::runtime_error("null out pointer");
        *out = new mlel_graph(ctx);
        (*out)->profiling = truthy(std::getenv("VMEL_GRAPH_PROFILING"));
        return 0;
    });
}

void mlel_graph_destroy(mlel_graph *g) {
    if (!g) return;
    for (void *e : g->events) (void)mlel_hip_event_destroy(g->ctx, e);
    delete g;
}

int mlel_graph_make_const_tensor(mlel_graph *g, uint32_t id, int32_t dtype, int32_t rank, const int64_t *dims,
                                 const int64_t *strides, const void *data) {
    return guarded([&] {
        g->pipeline.makeConstTensor(id, dtype, vec64(dims, rank), vec64(strides, strides ? rank : 0), data);
        return g->pipeline.getConstTensor(id)->id;
    });
}

int mlel_graph_get_const_tensor(mlel_graph *g, uint32_t id) {
    return guarded([&] { return g->pipeline.getConstTensor(id)->id; });
}

int mlel_graph_make_const_composite_tensor(mlel_graph *g, int32_t dtype, int32_t rank, const int64_t *dims,
                                           const void *data) {
    return guarded([&] { return g->pipeline.makeConstCompositeTensor(dtype, vec64(dims, rank), data)->id; });
}

int mlel_graph_make_descriptor_set_binding(mlel_graph *g, uint32_t set, uint32_t binding, uint32_t array_index,
                                           int32_t dtype, int32_t rank, const int64_t *dims, const int64_t *strides) {
    return guarded([&] {
        g->pipeline.makeDescriptorSetBinding(set, binding, array_index, dtype, vec64(dims, rank),
                                             vec64(strides, strides ? rank : 0));
        return g->pipeline.getTensor(set, binding, array_index)->id;
    });
}

int mlel_graph_get_tensor(mlel_graph *g, uint32_t set, uint32_t binding, uint32_t array_index) {
    return guarded([&] {
        const auto t = g->pipeline.getTensor(set, binding, array_index);
        if (!t) throw std::out_of_range("tensor array element was never bound");
        return t->id;
    });
}

int mlel_graph_make_tensor(mlel_graph *g, int32_t dtype, int32_t rank, const int64_t *dims, const int64_t *strides) {
    return guarded(
        [&] { return g->pipeline.makeTensor(dtype, vec64(dims, rank), vec64(strides, strides ? rank : 0))->id; });
}

int mlel_graph_make_input(mlel_graph *g, int tensor) {
    return guarded([&] {
        g->pipeline.makeInput(handle(g, tensor));
        return 0;
    });
}

int mlel_graph_make_output(mlel_graph *g, int tensor) {
    return guarded([&] {
        g->pipeline.makeOutput(handle(g, tensor));
        return 0;
    });
}

int mlel_graph_make_op(mlel_graph *g, const char *tosa_name, const int *inputs, int n_inputs, const int *outputs,
                       int n_outputs, const int64_t *iattr, int n_iattr, const double *fattr, int n_fattr,
                       const char *debug_name) {
    return guarded([&] {
        const auto it = makers().find(tosa_name ? tosa_name : "");
        if (it == makers().end()) {
            g_error = std::string("Unsupported TOSA operator: ") + (tosa_name ? tosa_name : "(null)");
            return static_cast<int>(MLEL_ERR_UNSUPPORTED);
        }
        Args a{g, {}, {}, iattr, n_iattr, fattr, n_fattr, debug_name ? debug_name : ""};
        for (int i = 0; i < n_inputs; i++) a.in.push_back(handle(g, inputs[i]));
        for (int i = 0; i < n_outputs; i++) a.out.push_back(handle(g, outputs[i]));
        it->second(g->pipeline, a);
        return 0;
    });
}

}  // extern "C"

namespace {
// shared tail of the two SPIR-V entry points: converts the argument arrays, runs `load`, reports the interface
template <typename Load>
int load_spirv_module(const mlel_graph_spv_binding *bindings, int n_bindings, const mlel_graph_spv_constant *constants,
                      int n_constants, const mlel_graph_spv_specialization *specializations, int n_specializations,
                      uint32_t *io, int io_capacity, int *n_inputs, int *n_outputs, const Load &load) {
    std::vector<SpvBinding> b;
    for (int i = 0; i < n_bindings; i++)
        b.push_back({bindings[i].set, bindings[i].binding, bindings[i].array_index, vec64(bindings[i].dims, bindings[i].rank)});
    std::vector<SpvConstant> c;
    for (int i = 0; i < n_constants; i++)
        c.push_back({constants[i].id, constants[i].data, vec64(constants[i].dims, constants[i].rank)});
    std::vector<SpvSpecialization> sp;
    for (int i = 0; i < n_specializations; i++) sp.push_back({specializations[i].spec_id, specializations[i].bits});
    const SpvGraphInfo info = load(b, c, sp);
    const size_t total = info.inputs.size() + info.outputs.size();
    if (io && static_cast<size_t>(io_capacity) < 3 * total) throw std::runtime_error("io array too small");
    size_t k = 0;
    for (const auto *list : {&info.inputs, &info.outputs})
        for (const auto &key : *list)
            for (int j = 0; j < 3 && io; j++) io[k++] = key[static_cast<size_t>(j)];
    if (n_inputs) *n_inputs = static_cast<int>(info.inputs.size());
    if (n_outputs) *n_outputs = static_cast<int>(info.outputs.size());
    return static_cast<int>(info.instructions);
}
}  // namespace

extern "C" {

int mlel_graph_load_spvasm(mlel_graph *g, const char *text, size_t length, const mlel_graph_spv_binding *bindings,
                           int n_bindings, const mlel_graph_spv_constant *constants, int n_constants,
                           const mlel_graph_spv_specialization *specializations, int n_specializations, uint32_t *io,
                           int io_capacity, int *n_inputs, int *n_outputs) {
    return guarded([&] {
        if (!text) throw std::runtime_error("null SPIR-V text");
        return load_spirv_module(bindings, n_bindings, constants, n_constants, specializations, n_specializations, io,
                                 io_capacity, n_inputs, n_outputs, [&](const auto &b, const auto &c, const auto &sp) {
                                     return loadSpirvAssembly(g->pipeline, std::string(text, length), b, c, sp);
                                 });
    });
}

int mlel_graph_load_spirv(mlel_graph *g, const uint32_t *words, size_t n_words, const mlel_graph_spv_binding *bindings,
                          int n_bindings, const mlel_graph_spv_constant *constants, int n_constants,
                          const mlel_graph_spv_specialization *specializations, int n_specializations, uint32_t *io,
                          int io_capacity, int *n_inputs, int *n_outputs) {
    return guarded([&] {
        if (!words) throw std::runtime_error("null SPIR-V module");
        return load_spirv_module(bindings, n_bindings, constants, n_constants, specializations, n_specializations, io,
                                 io_capacity, n_inputs, n_outputs, [&](const auto &b, const auto &c, const auto &sp) {
                                     return loadSpirvBinary(g->pipeline, words, n_words, b, c, sp);
                                 });
    });
}

int mlel_graph_tensor_info(mlel_graph *g, int tensor, int32_t *dtype, int64_t *dims) {
    return guarded([&] {
        const TensorPtr t = handle(g, tensor);
        if (dtype) *dtype = t->getFormat();
        for (size_t i = 0; i < t->getDimensions().size() && dims; i++) dims[i] = t->getDimensions()[i];
        return static_cast<int>(t->getRank());
    });
}

int mlel_graph_set_memory_planner(mlel_graph *g, int planner) {
    return guarded([&] {
        if (planner < 0 || planner > 2) throw std::runtime_error("memory planner: 0 interval, 1 linear, 2 best fit");
        g->pipeline.setMemoryPlanner(static_cast<GraphPipeline::MemoryPlanner>(planner));
        return 0;
    });
}

int mlel_graph_get_memory_planner(mlel_graph *g) {
    return guarded([&] { return static_cast<int>(g->pipeline.memoryPlanner()); });
}

int mlel_graph_set_batch_split(mlel_graph *g, int enabled) {
    return guarded([&] {
        g->pipeline.setBatchSplit(enabled != 0);
        return 0;
    });
}

int mlel_graph_get_batch_split(mlel_graph *g) {
    return guarded([&] {
        return g->pipeline.isFinalized() ? static_cast<int>(g->pipeline.batchSplitLaunches())
                                         : (g->pipeline.batchSplitRequested() ? 1 : 0);
    });
}

int mlel_graph_finalize(mlel_graph *g, int enable_fusion) {
    return guarded([&] {
        g->pipeline.finalize(enable_fusion != 0);
        return 0;
    });
}

int mlel_graph_session_memory_requirements(mlel_graph *g, uint64_t *size, uint64_t *alignment) {
    return guarded([&] {
        if (!g->pipeline.isFinalized()) throw std::runtime_error("finalize() has not run");
        if (size) *size = g->pipeline.sessionMemorySize();
        if (alignment) *alignment = g->pipeline.sessionMemoryAlignment();
        return 0;
    });
}

int mlel_graph_bind_session_memory(mlel_graph *g, void *device_base) {
    return guarded([&] {
        g->session().bindTransientMemory(device_base);
        return 0;
    });
}

int mlel_graph_bind_external(mlel_graph *g, uint32_t set, uint32_t binding, uint32_t array_index, void *device_ptr) {
    return guarded([&] {
        g->session().bindExternal(set, binding, array_index, device_ptr);
        return 0;
    });
}

namespace {

// a pair of events around every operator; milliseconds per operator into `ms` (n entries)
void dispatchTimed(mlel_graph *g, GraphSession &session, void *stream, std::vector<float> &ms) {
    const size_t n = g->pipeline.executionList().size();
    while (g->events.size() < 2 * n) {
        void *e = nullptr;
        if (mlel_hip_event_create(g->ctx, &e) != 0) throw std::runtime_error(mlel_hip_last_error());
        g->events.push_back(e);
    }
    session.dispatch(stream, [&](const OpNode &, uint32_t index, bool before) {
        if (mlel_hip_event_record(g->ctx, g->events[2 * index + (before ? 0 : 1)], stream) != 0)
            throw std::runtime_error(mlel_hip_last_error());
    });
    ms.assign(n, 0.f);
    for (size_t i = 0; i < n; i++)
        if (mlel_hip_event_elapsed_ms(g->ctx, g->events[2 * i], g->events[2 * i + 1], &ms[i]) != 0)
            throw std::runtime_error(mlel_hip_last_error());
}

}  // namespace

namespace {

int dispatchSession(mlel_graph *g, GraphSession &session, void *stream) {
    if (!g->profiling) {
        session.dispatch(stream);
        return 0;
    }
    // profiling: this dispatch waits for its own events (the reference reads its timestamps back at the fence)
    std::vector<float> ms;
    dispatchTimed(g, session, stream, ms);
    const auto list = g->pipeline.executionList();
    for (size_t i = 0; i < list.size(); i++)
        g->samples.push_back(ProfileSample{g->dispatches, static_cast<uint32_t>(i), opLabel(*list[i]), ms[i]});
    g->dispatches++;
    return 0;
}

}  // namespace

int mlel_graph_dispatch(mlel_graph *g, void *stream) {
    return guarded([&] { return dispatchSession(g, g->session(), stream); });
}

// ---- sessions (reference: graph_layer.cpp:1297-1425) ----
int mlel_graph_session_create(mlel_graph *g, mlel_graph_session **out) {
    return guarded([&] {
        if (g == nullptr || out == nullptr) throw std::runtime_error("session_create: null argument");
        *out = new mlel_graph_session(g);
        return 0;
    });
}

void mlel_graph_session_destroy(mlel_graph_session *s) { delete s; }

int mlel_graph_session_bind_point_requirements(mlel_graph_session *s, uint32_t *count,
                                               mlel_graph_bind_point_requirement *requirements) {
    return guarded([&] {
        if (s == nullptr || count == nullptr) throw std::runtime_error("bind_point_requirements: null argument");
        const uint32_t required = s->session.needsTransientMemory() ? 1u : 0u;
        if (requirements == nullptr) {
            *count = required;
            return 0;
        }
        const uint32_t capacity = *count;
        uint32_t written = 0;
        if (required) {
            if (written < capacity)
                requirements[written] = mlel_graph_bind_point_requirement{MLEL_GRAPH_BIND_POINT_TRANSIENT,
                                                                          MLEL_GRAPH_BIND_POINT_TYPE_MEMORY, 1};
            ++written;
        }
        *count = written;
        return capacity < required ? MLEL_GRAPH_INCOMPLETE : 0;
    });
}

int mlel_graph_session_get_memory_requirements(mlel_graph_session *s, uint32_t bind_point, uint64_t *size,
                                               uint64_t *alignment) {
    return guarded([&] {
        if (s == nullptr) throw std::runtime_error("session memory requirements: null session");
        (void)bind_point;  // a graph pipeline answers with its planner's requirements whatever the bind point
        if (size) *size = s->session.memorySize();
        if (alignment) *alignment = s->session.memoryAlignment();
        return 0;
    });
}

int mlel_graph_session_bind_memory(mlel_graph_session *s, uint32_t bind_point, void *device_base) {
    return guarded([&] {
        if (s == nullptr) throw std::runtime_error("session bind memory: null session");
        if (bind_point != MLEL_GRAPH_BIND_POINT_TRANSIENT)
            throw std::runtime_error("Invalid bind point for pipeline type");
        s->session.bindTransientMemory(device_base);
        return 0;
    });
}

int mlel_graph_session_bind_external(mlel_graph_session *s, uint32_t set, uint32_t binding, uint32_t array_index,
                                     void *device_ptr) {
    return guarded([&] {
        if (s == nullptr) throw std::runtime_error("session bind external: null session");
        s->session.bindExternal(set, binding, array_index, device_ptr);
        return 0;
    });
}

int mlel_graph_session_dispatch(mlel_graph_session *s, void *stream) {
    return guarded([&] {
        if (s == nullptr) throw std::runtime_error("session dispatch: null session");
        return dispatchSession(s->graph, s->session, stream);
    });
}

int mlel_graph_session_dispatch_replayed(mlel_graph_session *s, void *stream) {
    return guarded([&] {
        if (s == nullptr) throw std::runtime_error("session dispatch: null session");
        if (s->graph->profiling) return dispatchSession(s->graph, s->session, stream);  // per-operator events: eagerly
        s->session.dispatchReplayed(stream);
        return 0;
    });
}

int mlel_graph_session_dispatch_range(mlel_graph_session *s, void *stream, int first, int count) {
    return guarded([&] {
        if (s == nullptr || first < 0 || count < 0) throw std::runtime_error("session dispatch range: bad argument");
        s->session.dispatch(stream, {}, static_cast<uint32_t>(first), static_cast<uint32_t>(count));
        return 0;
    });
}

int mlel_graph_dispatch_profiled(mlel_graph *g, void *stream, float *ms, int capacity) {
    return guarded([&] {
        std::vector<float> all;
        dispatchTimed(g, g->session(), stream, all);
        for (size_t i = 0; i < all.size() && static_cast<int>(i) < capacity; i++) ms[i] = all[i];
        return static_cast<int>(all.size());
    });
}

int mlel_graph_log_level(void) { return (int)mlel::graphlog::level(); }
int mlel_graph_log_reload(void) {
    mlel::graphlog::reload();
    return (int)mlel::graphlog::level();
}

int mlel_graph_set_profiling(mlel_graph *g, int enabled) {
    return guarded([&] {
        g->profiling = enabled != 0;
        return 0;
    });
}

int mlel_graph_get_profiling(mlel_graph *g) {
    return guarded([&] { return g->profiling ? 1 : 0; });
}

int64_t mlel_graph_profiling_json(mlel_graph *g, char *buf, size_t capacity) {
    int64_t needed = 0;
    const int rc = guarded([&] {
        // the report of the reference's profiler (graph/graph_profiler.cpp:563-625): every sample, then count / total /
        // average / min / max per operator name; times come from event pairs, so there are no cycle counts
        struct Agg {
            uint64_t count = 0;
            double total = 0, mn = 0, mx = 0;
        };
        std::map<std::string, Agg> by;
        std::ostringstream o;
        o.precision(9);
        o << "{\n  \"timestamp_period_ns\": null,\n  \"samples\": [";
        bool first = true;
        for (const auto &s : g->samples) {
            o << (first ? "\n" : ",\n") << "    {\"submission\": " << s.dispatch << ", \"graph_dispatch\": " << s.dispatch
              << ", \"pipeline_index\": " << s.index << ", \"pipeline_kind\": \"tosa\", \"operator_name\": \"" << s.name
              << "\", \"time_ms\": " << s.ms << "}";
            first = false;
            Agg &a = by[s.name];
            a.mn = a.count == 0 ? s.ms : std::min(a.mn, s.ms);
            a.mx = a.count == 0 ? s.ms : std::max(a.mx, s.ms);
            a.count++;
            a.total += s.ms;
        }
        o << (first ? "" : "\n  ") << "],\n  \"by_operator\": [";
        first = true;
        for (const auto &[name, a] : by) {
            o << (first ? "\n" : ",\n") << "    {\"pipeline_kind\": \"tosa\", \"operator_name\": \"" << name
              << "\", \"dispatch_count\": " << a.count << ", \"total_time_ms\": " << a.total
              << ", \"average_time_ms\": " << (a.count ? a.total / static_cast<double>(a.count) : 0.0)
              << ", \"min_time_ms\": " << a.mn << ", \"max_time_ms\": " << a.mx << "}";
            first = false;
        }
        o << (first ? "" : "\n  ") << "]\n}\n";
        const std::string text = o.str();
        needed = static_cast<int64_t>(text.size()) + 1;
        if (buf != nullptr && capacity > 0) {
            const size_t n = std::min(capacity - 1, text.size());
            std::memcpy(buf, text.data(), n);
            buf[n] = 0;
        }
        return 0;
    });
    return rc != 0 ? rc : needed;
}

int mlel_graph_op_count(mlel_graph *g) {
    return guarded([&] { return static_cast<int>(g->pipeline.executionList().size()); });
}

int mlel_graph_op_name(mlel_graph *g, int index, char *buf, size_t len) {
    return guarded([&] {
        const auto list = g->pipeline.executionList();
        if (index < 0 || static_cast<size_t>(index) >= list.size() || !buf || len == 0)
            throw std::runtime_error("bad operator index");
        const std::string label = opLabel(*list[static_cast<size_t>(index)]);
        std::strncpy(buf, label.c_str(), len - 1);
        buf[len - 1] = 0;
        return 0;
    });
}

int mlel_graph_session_tensor_count(mlel_graph *g) {
    return guarded([&] { return static_cast<int>(g->pipeline.getTensors().size()); });
}

int mlel_graph_session_tensor_info(mlel_graph *g, int index, int *tensor, uint64_t *offset, uint64_t *size,
                                   uint32_t *first_use, uint32_t *last_use) {
    return guarded([&] {
        const auto &ts = g->pipeline.getTensors();
        if (index < 0 || static_cast<size_t>(index) >= ts.size()) throw std::runtime_error("bad session tensor index");
        const auto &t = ts[static_cast<size_t>(index)];
        if (tensor) *tensor = t->id;
        if (size) *size = t->getSize();
        const auto &off = g->pipeline.sessionOffsets();
        const auto it = off.find(t.get());
        if (offset) *offset = it == off.end() ? std::numeric_limits<uint64_t>::max() : it->second;
        const auto ranges = g->pipeline.liveRanges();
        if (first_use) *first_use = ranges[static_cast<size_t>(index)][0];
        if (last_use) *last_use = ranges[static_cast<size_t>(index)][1];
        return 0;
    });
}

int mlel_graph_allocate_intervals(const uint64_t *intervals, int n, const uint64_t *unseen, int m, uint64_t alignment,
                                  uint64_t *out_offsets, uint64_t *out_memory_size) {
    return guarded([&] {
        std::vector<details::LiveInterval> iv;
        for (int i = 0; i < n; i++)
            iv.push_back({static_cast<size_t>(intervals[5 * i]), static_cast<uint32_t>(intervals[5 * i + 1]),
                          static_cast<uint32_t>(intervals[5 * i + 2]), intervals[5 * i + 3],
                          static_cast<size_t>(intervals[5 * i + 4])});
        std::vector<details::UnseenAllocation> un;
        for (int i = 0; i < m; i++) un.push_back({static_cast<size_t>(unseen[2 * i]), unseen[2 * i + 1]});
        const auto plan = details::allocateIntervals(std::move(iv), un, alignment);
        int k = 0;
        for (const auto &[id, off] : plan.offsets) {
            out_offsets[2 * k] = id;
            out_offsets[2 * k + 1] = off;
            k++;
        }
        if (out_memory_size) *out_memory_size = plan.memorySize;
        return k;
    });
}

int mlel_graph_dtype_from_vk_format(int32_t vk_format) {
    return guarded([&] { return static_cast<int>(dtypeFromVkFormat(vk_format)); });
}

}  // extern "C"
