// Front-end for data graphs as SPIR-V, assembly text or binary words (SPV_ARM_graph + SPV_ARM_tensors with the
// "TOSA.001000.1" extended instruction set): the module is read, its types, constants and interface variables are
// resolved, and every instruction of the graph body becomes one GraphPipeline::make<Op> call.
//
// Reference counterpart: the layer decodes the binary module with SPIRV-Tools passes and
// GraphTosa10ExtInst::handleOp (graph/graph_tosa_1_0_ext_inst.cpp:37-1032, graph/graph_ext_inst_context.cpp:77-353).
// The conventions kept from there: integer element types mean signed data whatever their declared signedness;
// zero points arrive as one-element tensors (read as int8 for CONV2D / MATMUL / AVG_POOL2D, int32 for RESCALE /
// NEGATE); a graph output whose value is produced by an operator IS that operator's result tensor, while a graph
// input or constant routed straight to an output is copied with a CAST; `OpGraphConstantARM` data and the shapes of
// unshaped tensor types come from the caller, as they come from VkDataGraphPipelineConstantARM /
// VkTensorDescriptionARM in the reference.
#pragma once

#include <array>
#include <cstdint>
#include <string>
#include <vector>

#include "graph_pipeline.hpp"

namespace mlel::graph {

// shape of an external tensor whose SPIR-V type carries no shape (array elements are listed one by one)
struct SpvBinding {
    uint32_t set, binding, arrayIndex;
    std::vector<int64_t> dims;
};

// payload of `OpGraphConstantARM <type> id`; dims only needed when the type carries no shape
struct SpvConstant {
    uint32_t id;
    const void *data;
    std::vector<int64_t> dims;
};

// value of the specialization constant decorated `SpecId specId` (the bit pattern of its type; booleans 0 / 1)
struct SpvSpecialization {
    uint32_t specId;
    uint64_t bits;
};

struct SpvGraphInfo {
    std::string entryPoint;
    std::vector<std::array<uint32_t, 3>> inputs;   // {set, binding, arrayIndex} per graph input, in index order
    std::vector<std::array<uint32_t, 3>> outputs;  // the same per graph output
    uint32_t instructions = 0;                     // TOSA instructions decoded
};

// Throws std::runtime_error with the offending line for malformed text, unknown instructions of the graph body,
// missing shapes or constants.
SpvGraphInfo loadSpirvAssembly(GraphPipeline &pipeline, const std::string &text, const std::vector<SpvBinding> &bindings,
                               const std::vector<SpvConstant> &constants,
                               const std::vector<SpvSpecialization> &specializations = {});

// The same for a binary module (the words handed to vkCreateShaderModule, either byte order).  Errors name the
// offset of the offending instruction's first word.  The opcode, enumerant and TOSA instruction numbers are the
// published ones; the reference takes them from the SPIRV-Headers package, which is not part of its source tree.
SpvGraphInfo loadSpirvBinary(GraphPipeline &pipeline, const uint32_t *words, size_t count,
                             const std::vector<SpvBinding> &bindings, const std::vector<SpvConstant> &constants,
                             const std::vector<SpvSpecialization> &specializations = {});

}  // namespace mlel::graph
