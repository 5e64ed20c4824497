// SPIR-V assembly text or binary words -> GraphPipeline (see spirv_graph_loader.hpp).
#include "spirv_graph_loader.hpp"

#include "graph_log.hpp"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>

namespace mlel::graph {
namespace {

struct Instruction {
    std::string result;                 // "%name" or empty
    std::string opcode;                 // "OpTypeInt", ...
    std::vector<std::string> operands;  // ids keep their '%'; string literals are stored without quotes
    int line = 0;                       // text: line number; binary: offset of the instruction's first word
    bool binary = false;
};

[[noreturn]] void fail(const Instruction &inst, const std::string &what) {
    throw std::runtime_error(std::string("SPIR-V graph, ") + (inst.binary ? "word " : "line ") + std::to_string(inst.line) +
                             " (" + inst.opcode + "): " + what);
}

// ---- lexer: one instruction per line, ';' starts a comment, "..." is one operand
std::vector<Instruction> tokenize(const std::string &text) {
    std::vector<Instruction> out;
    std::istringstream stream(text);
    std::string line;
    int number = 0;
    while (std::getline(stream, line)) {
        number++;
        std::vector<std::string> words;
        size_t i = 0;
        while (i < line.size()) {
            const char c = line[i];
            if (c == ';') break;
            if (c == ' ' || c == '\t' || c == '\r') {
                i++;
            } else if (c == '"') {
                size_t j = i + 1;
                std::string s;
                while (j < line.size() && line[j] != '"') {
                    if (line[j] == '\\' && j + 1 < line.size()) j++;
                    s.push_back(line[j++]);
                }
                words.push_back(s);
                i = j + 1;
            } else {
                size_t j = i;
                while (j < line.size() && line[j] != ' ' && line[j] != '\t' && line[j] != '\r' && line[j] != ';') j++;
                words.push_back(line.substr(i, j - i));
                i = j;
            }
        }
        if (words.empty()) continue;
        Instruction inst;
        inst.line = number;
        size_t first = 0;
        if (words.size() >= 3 && words[1] == "=") {
            inst.result = words[0];
            first = 2;
        }
        inst.opcode = words[first];
        inst.operands.assign(words.begin() + first + 1, words.end());
        out.push_back(std::move(inst));
    }
    return out;
}


// ---- binary modules: the word stream is turned into the same instruction records the lexer above produces (ids as
// "%<number>", enumerants the loader looks at by name, constants as raw words "!0x..."), so both forms share
// everything after this point.
//
// Operand layouts, one character per operand after the optional result type and result id:
//   i  one id                       I  ids up to the end of the instruction
//   l  one literal word             L  literal words up to the end
//   s  a nul-terminated string      c  the literal of OpConstant: one word, or two for 64-bit types (low word first)
//   d  Decoration                   f  FPEncoding (optional)          x  TOSA instruction number
struct OpcodeLayout {
    uint16_t code;
    const char *name;
    bool hasType, hasResult;
    const char *operands;
};

// Numbers as published in the SPIR-V specification and the SPV_ARM_tensors / SPV_ARM_graph /
// SPV_EXT_replicated_composites extension texts.
const OpcodeLayout kOpcodes[] = {
    {5, "OpName", false, false, "is"},
    {10, "OpExtension", false, false, "s"},
    {11, "OpExtInstImport", false, true, "s"},
    {12, "OpExtInst", true, true, "ixI"},
    {14, "OpMemoryModel", false, false, "ll"},
    {17, "OpCapability", false, false, "l"},
    {19, "OpTypeVoid", false, true, ""},
    {20, "OpTypeBool", false, true, ""},
    {21, "OpTypeInt", false, true, "ll"},
    {22, "OpTypeFloat", false, true, "lf"},
    {23, "OpTypeVector", false, true, "il"},
    {24, "OpTypeMatrix", false, true, "il"},
    {28, "OpTypeArray", false, true, "ii"},
    {29, "OpTypeRuntimeArray", false, true, "i"},
    {30, "OpTypeStruct", false, true, "I"},
    {32, "OpTypePointer", false, true, "li"},
    {33, "OpTypeFunction", false, true, "I"},
    {41, "OpConstantTrue", true, true, ""},
    {42, "OpConstantFalse", true, true, ""},
    {43, "OpConstant", true, true, "c"},
    {44, "OpConstantComposite", true, true, "I"},
    {46, "OpConstantNull", true, true, ""},
    {48, "OpSpecConstantTrue", true, true, ""},
    {49, "OpSpecConstantFalse", true, true, ""},
    {50, "OpSpecConstant", true, true, "c"},
    {51, "OpSpecConstantComposite", true, true, "I"},
    {59, "OpVariable", true, true, "lI"},
    {71, "OpDecorate", false, false, "idL"},
    {81, "OpCompositeExtract", true, true, "iL"},
    {4163, "OpTypeTensorARM", false, true, "I"},
    {4181, "OpGraphConstantARM", true, true, "l"},
    {4182, "OpGraphEntryPointARM", false, false, "isI"},
    {4183, "OpGraphARM", true, true, ""},
    {4184, "OpGraphInputARM", true, true, "I"},
    {4185, "OpGraphSetOutputARM", false, false, "I"},
    {4186, "OpGraphEndARM", false, false, ""},
    {4190, "OpTypeGraphARM", false, true, "lI"},
    {4461, "OpConstantCompositeReplicateEXT", true, true, "i"},
    {4462, "OpSpecConstantCompositeReplicateEXT", true, true, "i"},
};

// "TOSA.001000.1" instruction numbers: the operators in the order of the TOSA 1.0 specification's chapters
// (tensor operators, activations, elementwise binary, unary, ternary, comparison, reduction, data layout,
// scatter / gather, image, type conversion), numbered from 0.  The reference reads them as the TOSA* enumerators
// of the SPIRV-Headers package (graph/graph_tosa_1_0_ext_inst.cpp:43-110 maps those to the names below); that
// package is not part of the reference's tree, so these numbers are restated from the published grammar.
const char *const kTosaNames[] = {
    "ARGMAX", "AVG_POOL2D", "CONV2D", "CONV3D", "DEPTHWISE_CONV2D", "FFT2D", "MATMUL", "MAX_POOL2D", "RFFT2D",
    "TRANSPOSE_CONV2D", "CLAMP", "ERF", "SIGMOID", "TANH", "ADD", "ARITHMETIC_RIGHT_SHIFT", "BITWISE_AND",
    "BITWISE_OR", "BITWISE_XOR", "INTDIV", "LOGICAL_AND", "LOGICAL_LEFT_SHIFT", "LOGICAL_RIGHT_SHIFT", "LOGICAL_OR",
    "LOGICAL_XOR", "MAXIMUM", "MINIMUM", "MUL", "POW", "SUB", "TABLE", "ABS", "BITWISE_NOT", "CEIL", "CLZ", "COS",
    "EXP", "FLOOR", "LOG", "LOGICAL_NOT", "NEGATE", "RECIPROCAL", "RSQRT", "SIN", "SELECT", "EQUAL", "GREATER",
    "GREATER_EQUAL", "REDUCE_ALL", "REDUCE_ANY", "REDUCE_MAX", "REDUCE_MIN", "REDUCE_PRODUCT", "REDUCE_SUM", "CONCAT",
    "PAD", "RESHAPE", "REVERSE", "SLICE", "TILE", "TRANSPOSE", "GATHER", "SCATTER", "RESIZE", "CAST", "RESCALE"};

constexpr uint32_t kSpirvMagic = 0x07230203u;

std::vector<Instruction> decodeWords(const uint32_t *stream, const size_t count) {
    if (!stream || count < 5) throw std::runtime_error("SPIR-V graph: a binary module has at least a five-word header");
    std::vector<uint32_t> words(stream, stream + count);
    const auto swap = [](const uint32_t w) { return (w >> 24) | ((w >> 8) & 0xff00u) | ((w << 8) & 0xff0000u) | (w << 24); };
    if (words[0] == swap(kSpirvMagic))  // written on a machine of the other byte order
        for (auto &w : words) w = swap(w);
    if (words[0] != kSpirvMagic) throw std::runtime_error("SPIR-V graph: the first word is not the SPIR-V magic number");
    std::map<uint32_t, const OpcodeLayout *> layouts;
    for (const auto &l : kOpcodes) layouts[l.code] = &l;
    std::map<uint32_t, int> scalarWidth;  // result id of OpTypeInt / OpTypeFloat -> width in bits
    uint32_t tosaSet = 0;
    const auto hex = [](const uint64_t v) {
        char buf[24];
        std::snprintf(buf, sizeof buf, "!0x%llx", static_cast<unsigned long long>(v));
        return std::string(buf);
    };
    std::vector<Instruction> out;
    size_t at = 5;
    while (at < words.size()) {
        const uint32_t length = words[at] >> 16, code = words[at] & 0xffffu;
        Instruction inst;
        inst.binary = true;
        inst.line = static_cast<int>(at);
        const auto known = layouts.find(code);
        inst.opcode = known != layouts.end() ? known->second->name : "Op#" + std::to_string(code);
        if (length == 0) fail(inst, "instruction of zero words");
        if (at + length > words.size()) fail(inst, "instruction runs past the end of the module");
        const uint32_t *w = &words[at];
        size_t k = 1;
        const auto more = [&] { return k < length; };
        const auto next = [&] {
            if (!more()) fail(inst, "too few words");
            return w[k++];
        };
        const auto id = [&] { return "%" + std::to_string(next()); };
        at += length;
        if (known == layouts.end()) {  // nothing the loader reads: kept as raw words so that error messages can show it
            while (more()) inst.operands.push_back(std::to_string(next()));
            out.push_back(std::move(inst));
            continue;
        }
        const OpcodeLayout &layout = *known->second;
        uint32_t typeId = 0, resultId = 0;
        if (layout.hasType) {
            typeId = next();
            inst.operands.push_back("%" + std::to_string(typeId));
        }
        if (layout.hasResult) {
            resultId = next();
            inst.result = "%" + std::to_string(resultId);
        }
        uint32_t firstId = 0;
        for (const char *kind = layout.operands; *kind; kind++) {
            switch (*kind) {
            case 'i': {
                const uint32_t v = next();
                if (firstId == 0) firstId = v;
                inst.operands.push_back("%" + std::to_string(v));
                break;
            }
            case 'I':
                while (more()) inst.operands.push_back(id());
                break;
            case 'l': inst.operands.push_back(std::to_string(next())); break;
            case 'L':
                while (more()) inst.operands.push_back(std::to_string(next()));
                break;
            case 's': {
                std::string text;
                bool ended = false;
                while (!ended) {
                    const uint32_t v = next();
                    for (int b = 0; b < 4 && !ended; b++) {
                        const char c = static_cast<char>((v >> (8 * b)) & 0xffu);
                        if (c == 0)
                            ended = true;
                        else
                            text.push_back(c);
                    }
                }
                inst.operands.push_back(text);
                break;
            }
            case 'c': {
                const auto width = scalarWidth.find(typeId);
                if (width == scalarWidth.end()) fail(inst, "constant of a type that is not a scalar number");
                uint64_t bits = next();
                if (width->second > 32) bits |= static_cast<uint64_t>(next()) << 32;
                inst.operands.push_back(hex(bits));
                break;
            }
            case 'd': {
                const uint32_t v = next();
                inst.operands.push_back(v == 1 ? "SpecId" : v == 33 ? "Binding" : v == 34 ? "DescriptorSet" : std::to_string(v));
                break;
            }
            case 'f':
                if (more()) {
                    const uint32_t v = next();
                    inst.operands.push_back(v == 0 ? "BFloat16KHR"
                                            : v == 4214 ? "Float8E4M3EXT"
                                            : v == 4215 ? "Float8E5M2EXT"
                                                        : "FPEncoding#" + std::to_string(v));
                }
                break;
            case 'x': {
                const uint32_t v = next();
                if (firstId == tosaSet && tosaSet != 0 && v < sizeof kTosaNames / sizeof kTosaNames[0])
                    inst.operands.push_back(kTosaNames[v]);
                else
                    inst.operands.push_back("instruction#" + std::to_string(v));
                break;
            }
            default: break;
            }
        }
        if (more()) fail(inst, "more words than the instruction takes");
        if (code == 21 || code == 22) scalarWidth[resultId] = std::atoi(inst.operands[0].c_str());
        if (code == 11 && inst.operands[0] == "TOSA.001000.1") tosaSet = resultId;
        out.push_back(std::move(inst));
    }
    return out;
}

// ---- module objects
enum class TypeKind { Int, Float, Bool, Array, Tensor, Pointer, Graph, Struct, Other };

struct Type {
    TypeKind kind = TypeKind::Other;
    int width = 0;              // Int / Float
    bool bfloat = false;        // Float 16 with the BFloat16KHR encoding
    int fp8 = 0;                // Float 8: 1 = Float8E4M3EXT, 2 = Float8E5M2EXT
    std::string element;        // Array / Tensor / Pointer: element (pointee) type id
    int64_t length = 0;         // Array
    int rank = 0;               // Tensor
    bool shaped = false;        // Tensor
    std::vector<int64_t> dims;  // Tensor, when shaped
    int numInputs = 0;          // Graph
    std::vector<std::string> interfaceTypes;  // Graph; Struct: member types
};

enum class ConstKind { Scalar, Composite, Null, Replicate, GraphConstant };

struct Constant {
    ConstKind kind = ConstKind::Scalar;
    std::string type;
    uint64_t bits = 0;  // Scalar: the value in the storage encoding of its type (two's complement / IEEE bits)
    std::vector<std::string> members;  // Composite: member ids; Replicate: the one replicated id
    uint32_t graphConstantId = 0;
};

struct Variable {
    std::string pointerType;
    bool hasSet = false, hasBinding = false;
    uint32_t set = 0, binding = 0;
};

uint16_t floatToHalfBits(const float f) {  // round to nearest even
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const int32_t exponent = static_cast<int32_t>((x >> 23) & 0xff) - 127 + 15;
    uint32_t mantissa = x & 0x7fffffu;
    if (((x >> 23) & 0xff) == 0xff) return static_cast<uint16_t>(sign | 0x7c00u | (mantissa ? 0x200u : 0u));
    if (exponent >= 31) return static_cast<uint16_t>(sign | 0x7c00u);
    if (exponent <= 0) {
        if (exponent < -10) return static_cast<uint16_t>(sign);
        mantissa |= 0x800000u;
        const int shift = 14 - exponent;
        uint32_t half = mantissa >> shift;
        const uint32_t rest = mantissa & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rest > halfway || (rest == halfway && (half & 1))) half++;
        return static_cast<uint16_t>(sign | half);
    }
    uint32_t half = (static_cast<uint32_t>(exponent) << 10) | (mantissa >> 13);
    const uint32_t rest = mantissa & 0x1fffu;
    if (rest > 0x1000u || (rest == 0x1000u && (half & 1))) half++;
    return static_cast<uint16_t>(sign | half);
}

// fp8 literals, nearest even like the other widths (values of the formats: graph/shaders/graph_op/common.comp:191-215)
uint8_t floatToE5M2Bits(const float f) {
    const uint16_t h = floatToHalfBits(f);
    if ((h & 0x7c00u) == 0x7c00u) return static_cast<uint8_t>((h >> 8) | ((h & 0x3ffu) ? 0x02u : 0u));  // inf / NaN
    return static_cast<uint8_t>((h + 0x7fu + ((h >> 8) & 1u)) >> 8);
}
uint8_t floatToE4M3Bits(const float f) {
    const uint8_t sign = std::signbit(f) ? 0x80u : 0u;
    const float ax = std::fabs(f);
    if (std::isnan(f) || ax > 464.0f) return sign | 0x7fu;  // no infinities: the NaN code
    if (ax < 0.015625f) return sign | static_cast<uint8_t>(std::nearbyint(ax * 512.0f));  // multiples of 2^-9 (8 -> 0x08)
    int e;
    const float m = std::frexp(ax, &e);  // ax = m * 2^e, m in [0.5, 1)
    int mant = static_cast<int>(std::nearbyint((m * 2.0f - 1.0f) * 8.0f)), expo = e - 1;
    if (mant == 8) mant = 0, expo++;
    const int field = expo + 7;
    if (field > 15 || (field == 15 && mant == 7)) return sign | 0x7eu;  // rounds to the largest finite value, 448
    return sign | static_cast<uint8_t>((field << 3) | mant);
}
float e4m3BitsToFloat(const uint8_t x) {
    const int e = (x >> 3) & 0xf, m = x & 7;
    if (e == 15 && m == 7) return std::nanf("");
    const float v = e == 0 ? static_cast<float>(m) / 512.0f : std::ldexp(1.0f + static_cast<float>(m) / 8.0f, e - 7);
    return (x & 0x80u) ? -v : v;
}

class Module {
  public:
    Module(GraphPipeline &p, const std::vector<SpvBinding> &b, const std::vector<SpvConstant> &c,
           const std::vector<SpvSpecialization> &sp)
        : pipeline(p), bindings(b), constantData(c), specializations(sp) {}

    SpvGraphInfo build(const std::vector<Instruction> &program);

  private:
    // ---- declarations
    void declare(const Instruction &inst);
    const Type &typeOf(const Instruction &at, const std::string &id) const {
        const auto it = types.find(id);
        if (it == types.end()) fail(at, "unknown type " + id);
        return it->second;
    }
    const Constant &constantOf(const Instruction &at, const std::string &id) const {
        const auto it = consts.find(id);
        if (it == consts.end()) fail(at, id + " is not a constant");
        return it->second;
    }
    int32_t dtypeOfScalarType(const Instruction &at, const Type &t) const;
    uint64_t parseLiteral(const Instruction &at, const Type &t, const std::string &word) const;

    // ---- attribute readers (reference: getConstScalar / getConstVector)
    int64_t scalarValue(const Instruction &at, const std::string &id) const;            // sign-interpreted
    double scalarReal(const Instruction &at, const std::string &id) const;
    double realFromBits(const Type &t, uint64_t bits) const;
    std::vector<double> vectorReal(const Instruction &at, const std::string &id) const;
    std::vector<int64_t> vectorValue(const Instruction &at, const std::string &id) const;  // small integer tensor
    void flatten(const Instruction &at, const std::string &id, size_t elemSize, std::vector<uint8_t> &out) const;

    // ---- tensors
    TensorPtr tensorOperand(const Instruction &at, const std::string &id);
    void registerVariables(const Instruction &at);
    std::vector<int64_t> bindingDims(uint32_t set, uint32_t binding, uint32_t index) const;
    TensorPtr resultTensor(const Instruction &inst, int member = -1);
    std::map<std::pair<std::string, int>, std::string> extracts;  // (multi-result id, member) -> OpCompositeExtract id
    void decodeTosa(const Instruction &inst);

    GraphPipeline &pipeline;
    const std::vector<SpvBinding> &bindings;
    const std::vector<SpvConstant> &constantData;
    const std::vector<SpvSpecialization> &specializations;
    std::map<std::string, uint32_t> specIds;  // decorated ids -> SpecId
    // a specialization constant keeps its default unless the caller supplies a value for its SpecId
    // (reference: graph_layer.cpp:71-107 freezes them before the graph is decoded)
    bool specialized(const std::string &id, uint64_t *bits) const {
        const auto it = specIds.find(id);
        if (it == specIds.end()) return false;
        for (const auto &sp : specializations)
            if (sp.specId == it->second) {
                *bits = sp.bits;
                return true;
            }
        return false;
    }
    std::map<std::string, Type> types;
    std::map<std::string, Constant> consts;
    std::map<std::string, Variable> variables;
    std::vector<std::string> variableOrder;
    std::string tosaImport;
    std::map<std::string, TensorPtr> values;          // graph inputs, instruction results, materialised constants
    std::map<std::string, std::vector<TensorPtr>> members;  // results of multi-result instructions
    std::map<std::string, std::vector<TensorPtr>> outputTargets;  // value id -> output tensors it is routed to
    bool variablesRegistered = false;
};

int32_t Module::dtypeOfScalarType(const Instruction &at, const Type &t) const {
    switch (t.kind) {
    case TypeKind::Bool: return MLEL_BOOL;
    case TypeKind::Int:  // declared signedness is ignored: integer tensors hold signed data
        switch (t.width) {
        case 8: return MLEL_I8;
        case 16: return MLEL_I16;
        case 32: return MLEL_I32;
        case 64: return MLEL_I64;
        default: break;
        }
        break;
    case TypeKind::Float:
        if (t.width == 8 && t.fp8 != 0) return t.fp8 == 1 ? MLEL_F8E4M3 : MLEL_F8E5M2;
        if (t.width == 16) return t.bfloat ? MLEL_BF16 : MLEL_F16;
        if (t.width == 32) return MLEL_F32;
        if (t.width == 64) return MLEL_F64;
        break;
    default: break;
    }
    fail(at, "unsupported tensor element type");
}

uint64_t Module::parseLiteral(const Instruction &at, const Type &t, const std::string &word) const {
    if (word.empty()) fail(at, "missing literal");
    if (word[0] == '!') return std::strtoull(word.c_str() + 1, nullptr, 0);  // raw word
    if (t.kind == TypeKind::Int) {
        const uint64_t mask = t.width >= 64 ? ~uint64_t(0) : ((uint64_t(1) << t.width) - 1);
        if (word[0] == '-') return static_cast<uint64_t>(std::strtoll(word.c_str(), nullptr, 0)) & mask;
        return std::strtoull(word.c_str(), nullptr, 0) & mask;
    }
    if (t.kind == TypeKind::Float) {
        char *end = nullptr;
        const double v = std::strtod(word.c_str(), &end);  // decimal and hexadecimal floating literals
        if (end == word.c_str()) fail(at, "bad floating literal " + word);
        if (t.width == 64) {
            uint64_t b;
            std::memcpy(&b, &v, 8);
            return b;
        }
        const float f = static_cast<float>(v);
        uint32_t b;
        std::memcpy(&b, &f, 4);
        if (t.width == 32) return b;
        if (t.width == 8) return t.fp8 == 1 ? floatToE4M3Bits(f) : floatToE5M2Bits(f);
        if (t.bfloat) {  // round to nearest even on the upper 16 bits
            const uint32_t rounded = b + 0x7fffu + ((b >> 16) & 1u);
            return (std::isnan(f) ? (b | 0x400000u) : rounded) >> 16;
        }
        return floatToHalfBits(f);
    }
    fail(at, "literal of a non-numeric type");
}

void Module::declare(const Instruction &inst) {
    const auto &op = inst.opcode;
    const auto &a = inst.operands;
    const auto need = [&](size_t n) {
        if (a.size() < n) fail(inst, "expects at least " + std::to_string(n) + " operands");
    };
    if (op == "OpExtInstImport") {
        need(1);
        if (a[0] == "TOSA.001000.1") tosaImport = inst.result;
    } else if (op == "OpDecorate") {
        need(2);
        if (a[1] == "DescriptorSet" && a.size() >= 3) {
            variables[a[0]].set = static_cast<uint32_t>(std::strtoul(a[2].c_str(), nullptr, 0));
            variables[a[0]].hasSet = true;
        } else if (a[1] == "SpecId" && a.size() >= 3) {
            specIds[a[0]] = static_cast<uint32_t>(std::strtoul(a[2].c_str(), nullptr, 0));
        } else if (a[1] == "Binding" && a.size() >= 3) {
            variables[a[0]].binding = static_cast<uint32_t>(std::strtoul(a[2].c_str(), nullptr, 0));
            variables[a[0]].hasBinding = true;
        }
    } else if (op == "OpTypeInt") {
        need(1);
        Type t;
        t.kind = TypeKind::Int;
        t.width = std::atoi(a[0].c_str());
        types[inst.result] = t;
    } else if (op == "OpTypeFloat") {
        need(1);
        Type t;
        t.kind = TypeKind::Float;
        t.width = std::atoi(a[0].c_str());
        t.bfloat = a.size() >= 2 && a[1].find("BFloat16") != std::string::npos;
        if (a.size() >= 2 && a[1].find("Float8E4M3") != std::string::npos) t.fp8 = 1;
        if (a.size() >= 2 && a[1].find("Float8E5M2") != std::string::npos) t.fp8 = 2;
        if ((a.size() >= 2 && !t.bfloat && t.fp8 == 0) || (t.bfloat && t.width != 16) || ((t.fp8 != 0) != (t.width == 8)))
            fail(inst, "floating-point type of width " + a[0] + (a.size() >= 2 ? " and encoding " + a[1] : "") +
                           " is not supported");
        types[inst.result] = t;
    } else if (op == "OpTypeBool") {
        Type t;
        t.kind = TypeKind::Bool;
        types[inst.result] = t;
    } else if (op == "OpTypeArray") {
        need(2);
        Type t;
        t.kind = TypeKind::Array;
        t.element = a[0];
        t.length = scalarValue(inst, a[1]);
        types[inst.result] = t;
    } else if (op == "OpTypeTensorARM") {
        need(2);
        Type t;
        t.kind = TypeKind::Tensor;
        t.element = a[0];
        t.rank = static_cast<int>(scalarValue(inst, a[1]));
        if (t.rank < 0 || t.rank > MLEL_MAX_RANK) fail(inst, "tensor rank " + std::to_string(t.rank));
        if (a.size() >= 3) {
            const Constant &shape = constantOf(inst, a[2]);
            if (shape.kind != ConstKind::Composite || static_cast<int>(shape.members.size()) != t.rank)
                fail(inst, "tensor shape must be a composite of `rank` integers");
            for (const auto &m : shape.members) t.dims.push_back(scalarValue(inst, m));
            t.shaped = true;
        }
        types[inst.result] = t;
    } else if (op == "OpTypePointer") {
        need(2);
        Type t;
        t.kind = TypeKind::Pointer;
        t.element = a[1];
        types[inst.result] = t;
    } else if (op == "OpTypeGraphARM") {
        need(1);
        Type t;
        t.kind = TypeKind::Graph;
        t.numInputs = std::atoi(a[0].c_str());
        t.interfaceTypes.assign(a.begin() + 1, a.end());
        types[inst.result] = t;
    } else if (op == "OpTypeStruct") {
        Type t;
        t.kind = TypeKind::Struct;
        t.interfaceTypes = a;
        types[inst.result] = t;
    } else if (op.rfind("OpType", 0) == 0) {
        types[inst.result] = Type{};  // struct, vector, ...: only ever named, never inspected
    } else if (op == "OpConstant" || op == "OpSpecConstant") {
        need(2);
        Constant c;
        c.type = a[0];
        c.bits = parseLiteral(inst, typeOf(inst, a[0]), a[1]);
        uint64_t replaced = 0;
        if (op == "OpSpecConstant" && specialized(inst.result, &replaced)) {
            const Type &t = typeOf(inst, a[0]);
            c.bits = t.width >= 64 ? replaced : replaced & ((uint64_t(1) << t.width) - 1);
        }
        consts[inst.result] = c;
    } else if (op == "OpConstantTrue" || op == "OpConstantFalse" || op == "OpSpecConstantTrue" ||
               op == "OpSpecConstantFalse") {
        need(1);
        Constant c;
        c.type = a[0];
        c.bits = op.find("True") != std::string::npos ? 1 : 0;
        uint64_t replaced = 0;
        if (op.rfind("OpSpec", 0) == 0 && specialized(inst.result, &replaced)) c.bits = replaced != 0;
        consts[inst.result] = c;
    } else if (op == "OpConstantNull") {
        need(1);
        Constant c;
        c.kind = ConstKind::Null;
        c.type = a[0];
        consts[inst.result] = c;
    } else if (op == "OpConstantComposite" || op == "OpSpecConstantComposite") {
        need(1);
        Constant c;
        c.kind = ConstKind::Composite;
        c.type = a[0];
        c.members.assign(a.begin() + 1, a.end());
        consts[inst.result] = c;
    } else if (op == "OpConstantCompositeReplicateEXT" || op == "OpSpecConstantCompositeReplicateEXT") {
        need(2);
        Constant c;
        c.kind = ConstKind::Replicate;
        c.type = a[0];
        c.members = {a[1]};
        consts[inst.result] = c;
    } else if (op == "OpGraphConstantARM") {
        need(2);
        Constant c;
        c.kind = ConstKind::GraphConstant;
        c.type = a[0];
        c.graphConstantId = static_cast<uint32_t>(std::strtoul(a[1].c_str(), nullptr, 0));
        consts[inst.result] = c;
    } else if (op == "OpVariable") {
        need(2);
        variables[inst.result].pointerType = a[0];
        variableOrder.push_back(inst.result);
    }
    // everything else at module scope (capabilities, extensions, names, memory model, ...) carries nothing we use
}

int64_t Module::scalarValue(const Instruction &at, const std::string &id) const {
    const Constant &c = constantOf(at, id);
    if (c.kind == ConstKind::Null) return 0;
    if (c.kind != ConstKind::Scalar) fail(at, id + " is not a scalar constant");
    const Type &t = typeOf(at, c.type);
    if (t.kind == TypeKind::Bool) return c.bits != 0;
    if (t.kind != TypeKind::Int) fail(at, id + " is not an integer constant");
    if (t.width >= 64) return static_cast<int64_t>(c.bits);
    const uint64_t sign = uint64_t(1) << (t.width - 1);
    return static_cast<int64_t>((c.bits ^ sign)) - static_cast<int64_t>(sign);  // same-width signed reinterpretation
}

double Module::realFromBits(const Type &t, const uint64_t bits) const {
    if (t.width == 64) {
        double v;
        std::memcpy(&v, &bits, 8);
        return v;
    }
    uint32_t b = static_cast<uint32_t>(bits);
    if (t.width == 8 && t.fp8 == 1) return e4m3BitsToFloat(static_cast<uint8_t>(bits));
    if (t.width == 8) b <<= 8;  // e5m2 is the upper byte of a half
    if (t.width == 16 && t.bfloat) {
        b <<= 16;
    } else if (t.width == 16 || t.width == 8) {  // half -> float
        const uint32_t sign = (b & 0x8000u) << 16, e = (b >> 10) & 0x1f, m = b & 0x3ffu;
        if (e == 0) {
            const float v = std::ldexp(static_cast<float>(m), -24);
            return sign ? -v : v;
        }
        b = sign | ((e == 31 ? 255u : e - 15 + 127) << 23) | (m << 13);
    }
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}

double Module::scalarReal(const Instruction &at, const std::string &id) const {
    const Constant &c = constantOf(at, id);
    if (c.kind == ConstKind::Null) return 0.0;
    if (c.kind != ConstKind::Scalar) fail(at, id + " is not a scalar constant");
    const Type &t = typeOf(at, c.type);
    if (t.kind != TypeKind::Float) return static_cast<double>(scalarValue(at, id));
    return realFromBits(t, c.bits);
}

// Row-major bytes of a tensor constant.  Composites nest one rank per level; a replicated composite repeats its
// operand (a scalar or a lower-rank constant) until the tensor is full.
void Module::flatten(const Instruction &at, const std::string &id, const size_t elemSize, std::vector<uint8_t> &out) const {
    const Constant &c = constantOf(at, id);
    const Type &t = typeOf(at, c.type);
    if (t.kind != TypeKind::Tensor) {  // a scalar leaf
        if (c.kind != ConstKind::Scalar && c.kind != ConstKind::Null) fail(at, id + ": expected a scalar member");
        const uint64_t bits = c.kind == ConstKind::Null ? 0 : c.bits;
        for (size_t i = 0; i < elemSize; i++) out.push_back(static_cast<uint8_t>(bits >> (8 * i)));
        return;
    }
    if (!t.shaped) fail(at, id + ": a constant needs a shaped tensor type");
    size_t count = 1;
    for (const auto d : t.dims) count *= static_cast<size_t>(d);
    const size_t bytes = count * elemSize, start = out.size();
    switch (c.kind) {
    case ConstKind::Null: out.resize(start + bytes, 0); break;
    case ConstKind::Composite:
        for (const auto &m : c.members) flatten(at, m, elemSize, out);
        if (out.size() - start != bytes) fail(at, id + ": composite does not fill its tensor type");
        break;
    case ConstKind::Replicate: {
        std::vector<uint8_t> unit;
        flatten(at, c.members[0], elemSize, unit);
        if (unit.empty() || bytes % unit.size() != 0) fail(at, id + ": replicated operand does not tile the tensor");
        for (size_t i = 0; i < bytes; i += unit.size()) out.insert(out.end(), unit.begin(), unit.end());
        break;
    }
    default: fail(at, id + " cannot be evaluated at load time");
    }
}

// Elements of a small tensor constant (attributes, zero points) as numbers; a scalar id gives one element.
std::vector<double> Module::vectorReal(const Instruction &at, const std::string &id) const {
    const Constant &c = constantOf(at, id);
    const Type &t = typeOf(at, c.type);
    if (t.kind != TypeKind::Tensor) return {scalarReal(at, id)};
    const Type &elem = typeOf(at, t.element);
    if (elem.kind != TypeKind::Int && elem.kind != TypeKind::Bool && elem.kind != TypeKind::Float)
        fail(at, id + ": expected a numeric tensor constant");
    const size_t size = elem.kind == TypeKind::Bool ? 1 : static_cast<size_t>(elem.width / 8);
    std::vector<uint8_t> raw;
    flatten(at, id, size, raw);
    std::vector<double> out;
    for (size_t i = 0; i + size <= raw.size(); i += size) {
        uint64_t bits = 0;
        for (size_t b = 0; b < size; b++) bits |= static_cast<uint64_t>(raw[i + b]) << (8 * b);
        if (elem.kind == TypeKind::Float) {
            out.push_back(realFromBits(elem, bits));
        } else {  // integers are signed whatever their declared signedness
            const uint64_t sign = uint64_t(1) << (8 * size - 1);
            out.push_back(static_cast<double>(size == 8 ? static_cast<int64_t>(bits)
                                                        : static_cast<int64_t>(bits ^ sign) - static_cast<int64_t>(sign)));
        }
    }
    return out;
}

std::vector<int64_t> Module::vectorValue(const Instruction &at, const std::string &id) const {
    std::vector<int64_t> out;
    for (const double v : vectorReal(at, id)) out.push_back(static_cast<int64_t>(v));
    return out;
}

std::vector<int64_t> Module::bindingDims(const uint32_t set, const uint32_t binding, const uint32_t index) const {
    for (const auto &b : bindings)
        if (b.set == set && b.binding == binding && b.arrayIndex == index) return b.dims;
    return {};
}

// Every interface variable becomes an external tensor (reference: makeDescriptorSetBinding per resource).
void Module::registerVariables(const Instruction &at) {
    if (variablesRegistered) return;
    variablesRegistered = true;
    for (const auto &name : variableOrder) {
        const Variable &v = variables[name];
        if (!v.hasSet || !v.hasBinding) fail(at, name + " has no DescriptorSet/Binding decoration");
        const Type &ptr = typeOf(at, v.pointerType);
        if (ptr.kind != TypeKind::Pointer) fail(at, name + ": variable type is not a pointer");
        const Type *pointee = &typeOf(at, ptr.element);
        int64_t elements = 1;
        if (pointee->kind == TypeKind::Array) {
            elements = pointee->length;
            pointee = &typeOf(at, pointee->element);
        }
        if (pointee->kind != TypeKind::Tensor) fail(at, name + " is not a tensor or an array of tensors");
        const int32_t dtype = dtypeOfScalarType(at, typeOf(at, pointee->element));
        for (int64_t i = 0; i < elements; i++) {
            std::vector<int64_t> dims = pointee->shaped ? pointee->dims : bindingDims(v.set, v.binding, static_cast<uint32_t>(i));
            if (!pointee->shaped && dims.empty()) continue;  // never described by the caller: an error only if used
            if (static_cast<int>(dims.size()) != pointee->rank)
                fail(at, name + ": shape of set " + std::to_string(v.set) + " binding " + std::to_string(v.binding) +
                             " element " + std::to_string(i) + " does not have rank " + std::to_string(pointee->rank));
            pipeline.makeDescriptorSetBinding(v.set, v.binding, static_cast<uint32_t>(i), dtype, dims, {});
        }
    }
}

TensorPtr Module::tensorOperand(const Instruction &at, const std::string &id) {
    const auto known = values.find(id);
    if (known != values.end()) return known->second;
    const Constant &c = constantOf(at, id);
    const Type &t = typeOf(at, c.type);
    if (t.kind != TypeKind::Tensor) fail(at, id + " is not a tensor");
    const int32_t dtype = dtypeOfScalarType(at, typeOf(at, t.element));
    TensorPtr tensor;
    if (c.kind == ConstKind::GraphConstant) {
        const SpvConstant *data = nullptr;
        for (const auto &d : constantData)
            if (d.id == c.graphConstantId) data = &d;
        if (!data || !data->data) fail(at, "no data supplied for graph constant " + std::to_string(c.graphConstantId));
        const std::vector<int64_t> dims = t.shaped ? t.dims : data->dims;
        if (static_cast<int>(dims.size()) != t.rank) fail(at, "no shape for graph constant " + std::to_string(c.graphConstantId));
        pipeline.makeConstTensor(c.graphConstantId, dtype, dims, {}, data->data);
        tensor = pipeline.getConstTensor(c.graphConstantId);
    } else {
        std::vector<uint8_t> raw;
        flatten(at, id, dtypeSize(dtype), raw);
        tensor = pipeline.makeConstCompositeTensor(dtype, t.dims, raw.data());
    }
    values[id] = tensor;
    return tensor;
}

// The tensor an instruction result (or member `member` of a multi-result instruction) is written to: the graph
// output it is routed to, else a new session tensor of the declared type.
TensorPtr Module::resultTensor(const Instruction &inst, const int member) {
    std::string valueId = inst.result, typeId = inst.operands[0];
    if (member >= 0) {
        const Type &st = typeOf(inst, typeId);
        if (st.kind != TypeKind::Struct || static_cast<size_t>(member) >= st.interfaceTypes.size())
            fail(inst, "expected a result structure with at least " + std::to_string(member + 1) + " members");
        typeId = st.interfaceTypes[static_cast<size_t>(member)];
        const auto ex = extracts.find({inst.result, member});
        valueId = ex == extracts.end() ? std::string() : ex->second;
    }
    const auto routed = outputTargets.find(valueId);
    if (!valueId.empty() && routed != outputTargets.end()) return routed->second.front();
    const Type &t = typeOf(inst, typeId);
    if (t.kind != TypeKind::Tensor) fail(inst, "result is not a tensor");
    if (!t.shaped) fail(inst, "an intermediate result needs a shaped tensor type");
    return pipeline.makeTensor(dtypeOfScalarType(inst, typeOf(inst, t.element)), t.dims, {});
}

std::vector<int32_t> to32(const std::vector<int64_t> &v) { return std::vector<int32_t>(v.begin(), v.end()); }
std::vector<uint32_t> toU32(const std::vector<int64_t> &v) { return std::vector<uint32_t>(v.begin(), v.end()); }

// One TOSA.001000.1 instruction: `%r = OpExtInst %type %set NAME args...`; args in the order of the instruction set.
void Module::decodeTosa(const Instruction &inst) {
    const std::string &name = inst.operands[2];
    const std::vector<std::string> a(inst.operands.begin() + 3, inst.operands.end());
    const auto need = [&](size_t n) {
        if (a.size() < n) fail(inst, name + " expects " + std::to_string(n) + " arguments, got " + std::to_string(a.size()));
    };
    const auto T = [&](size_t i) { return tensorOperand(inst, a[i]); };
    const auto S = [&](size_t i) { return scalarValue(inst, a[i]); };
    const auto V = [&](size_t i) { return vectorValue(inst, a[i]); };
    const auto first = [&](size_t i) {  // a one-element tensor (zero points, shifts)
        const auto v = vectorValue(inst, a[i]);
        if (v.empty()) fail(inst, name + ": empty constant");
        return v[0];
    };
    const std::string dbg = inst.result.size() > 1 ? inst.result.substr(1) : name;
    // one line per decoded instruction, as the reference's handlers print (graph_tosa_1_0_ext_inst.cpp:453-457)
    MLEL_GRAPH_LOG(Info, "OpExtInst result=" << inst.result << ',' << dbg << ", " << name << [&] {
        std::string list;
        for (size_t i = 0; i < a.size(); i++) list += (i ? ", " : " ") + a[i];
        return list;
    }());
    if (name == "FFT2D" || name == "RFFT2D") {  // two results, picked apart by OpCompositeExtract
        const TensorPtr real = resultTensor(inst, 0), imag = resultTensor(inst, 1);
        if (name == "FFT2D") {
            need(4);  // inverse localBound real imag
            pipeline.makeFft2D(T(2), T(3), real, imag, S(0) != 0, dbg);
        } else {
            need(2);  // localBound input
            pipeline.makeRfft2D(T(1), real, imag, dbg);
        }
        members[inst.result] = {real, imag};
        return;
    }
    const TensorPtr out = resultTensor(inst);

    using Unary = void (GraphPipeline::*)(const TensorPtr &, const TensorPtr &, const std::string &);
    using Binary = void (GraphPipeline::*)(const TensorPtr &, const TensorPtr &, const TensorPtr &, const std::string &);
    static const std::map<std::string, Unary> unary = {
        {"ABS", &GraphPipeline::makeAbs}, {"BITWISE_NOT", &GraphPipeline::makeBitwiseNot},
        {"CEIL", &GraphPipeline::makeCeil}, {"CLZ", &GraphPipeline::makeClz}, {"COS", &GraphPipeline::makeCos},
        {"EXP", &GraphPipeline::makeExp}, {"FLOOR", &GraphPipeline::makeFloor}, {"LOG", &GraphPipeline::makeLog},
        {"LOGICAL_NOT", &GraphPipeline::makeLogicalNot}, {"RECIPROCAL", &GraphPipeline::makeReciprocal},
        {"RSQRT", &GraphPipeline::makeRsqrt}, {"SIGMOID", &GraphPipeline::makeSigmoid}, {"SIN", &GraphPipeline::makeSin},
        {"TANH", &GraphPipeline::makeTanh}, {"ERF", &GraphPipeline::makeErf}, {"CAST", &GraphPipeline::makeCast}};
    static const std::map<std::string, Binary> binary = {
        {"ADD", &GraphPipeline::makeAdd}, {"SUB", &GraphPipeline::makeSub},
        {"BITWISE_AND", &GraphPipeline::makeBitwiseAnd}, {"BITWISE_OR", &GraphPipeline::makeBitwiseOr},
        {"BITWISE_XOR", &GraphPipeline::makeBitwiseXor}, {"INTDIV", &GraphPipeline::makeIntdiv},
        {"LOGICAL_AND", &GraphPipeline::makeLogicalAnd}, {"LOGICAL_OR", &GraphPipeline::makeLogicalOr},
        {"LOGICAL_XOR", &GraphPipeline::makeLogicalXor}, {"LOGICAL_LEFT_SHIFT", &GraphPipeline::makeLogicalLeftShift},
        {"LOGICAL_RIGHT_SHIFT", &GraphPipeline::makeLogicalRightShift}, {"POW", &GraphPipeline::makePow},
        {"EQUAL", &GraphPipeline::makeEqual}, {"GREATER", &GraphPipeline::makeGreater},
        {"GREATER_EQUAL", &GraphPipeline::makeGreaterEqual}};

    if (const auto u = unary.find(name); u != unary.end()) {
        need(1);
        (pipeline.*(u->second))(T(0), out, dbg);
    } else if (const auto b = binary.find(name); b != binary.end()) {
        need(2);
        (pipeline.*(b->second))(T(0), T(1), out, dbg);
    } else if (name == "CONV2D" || name == "DEPTHWISE_CONV2D" || name == "CONV3D") {
        need(10);  // pad stride dilation accType localBound input weight bias inputZp weightZp
        const auto pad = to32(V(0)), stride = to32(V(1)), dilation = to32(V(2));
        const auto acc = static_cast<uint32_t>(S(3));
        const auto zi = static_cast<int8_t>(first(8)), zw = static_cast<int8_t>(first(9));
        if (name == "CONV2D")
            pipeline.makeConv2D(T(5), out, T(6), T(7), pad, stride, dilation, zi, zw, acc, dbg);
        else if (name == "DEPTHWISE_CONV2D")
            pipeline.makeDepthwiseConv2D(T(5), out, T(6), T(7), pad, stride, dilation, zi, zw, acc, dbg);
        else
            pipeline.makeConv3D(T(5), out, T(6), T(7), pad, stride, dilation, zi, zw, acc, dbg);
    } else if (name == "TRANSPOSE_CONV2D") {
        need(9);  // outPad stride accType localBound input weight bias inputZp weightZp
        pipeline.makeTransposeConv2D(T(4), out, T(5), T(6), to32(V(0)), to32(V(1)), static_cast<int8_t>(first(7)),
                                     static_cast<int8_t>(first(8)), static_cast<uint32_t>(S(2)), dbg);
    } else if (name == "MATMUL") {
        need(4);  // A B zpA zpB (read as int8)
        pipeline.makeMatmul(T(0), T(1), out, static_cast<int8_t>(first(2)), static_cast<int8_t>(first(3)), dbg);
    } else if (name == "AVG_POOL2D") {
        need(7);  // kernel stride pad accType input inputZp outputZp
        pipeline.makeAvgPool2D(T(4), out, to32(V(0)), to32(V(1)), to32(V(2)), static_cast<uint32_t>(S(3)),
                               static_cast<int8_t>(first(5)), static_cast<int8_t>(first(6)), dbg);
    } else if (name == "MAX_POOL2D") {
        need(5);  // kernel stride pad nanMode input
        pipeline.makeMaxPool2D(T(4), out, to32(V(0)), to32(V(1)), to32(V(2)), static_cast<uint32_t>(S(3)), dbg);
    } else if (name == "RESCALE") {
        need(10);  // scale32 roundingMode perChannel inputUnsigned outputUnsigned input multiplier shift inputZp outputZp
        const int64_t rounding = S(1);  // 1 single, 2 inexact, 3 double
        if (rounding != 1 && rounding != 3) fail(inst, "RESCALE rounding mode " + std::to_string(rounding) + " is not supported");
        pipeline.makeRescale(T(5), out, static_cast<int32_t>(first(8)), static_cast<int32_t>(first(9)), T(6), T(7),
                             S(0) != 0, rounding == 3, S(2) != 0, S(3) != 0, S(4) != 0, dbg);
    } else if (name == "CLAMP") {
        need(4);  // min max nanMode input
        pipeline.makeClamp(T(3), out, scalarReal(inst, a[0]), scalarReal(inst, a[1]), static_cast<uint32_t>(S(2)), dbg);
    } else if (name == "MAXIMUM" || name == "MINIMUM") {
        need(3);  // nanMode input1 input2
        if (name == "MAXIMUM")
            pipeline.makeMaximum(T(1), T(2), out, static_cast<uint32_t>(S(0)), dbg);
        else
            pipeline.makeMinimum(T(1), T(2), out, static_cast<uint32_t>(S(0)), dbg);
    } else if (name == "MUL") {
        need(3);  // input1 input2 shift
        pipeline.makeMul(T(0), T(1), out, static_cast<uint32_t>(first(2)) & 0xffu, dbg);
    } else if (name == "REDUCE_ALL" || name == "REDUCE_ANY" || name == "REDUCE_PRODUCT" || name == "REDUCE_SUM") {
        need(2);  // axis input
        const auto axis = static_cast<uint32_t>(S(0));
        if (name == "REDUCE_ALL") pipeline.makeReduceAll(T(1), out, axis, dbg);
        else if (name == "REDUCE_ANY") pipeline.makeReduceAny(T(1), out, axis, dbg);
        else if (name == "REDUCE_PRODUCT") pipeline.makeReduceProduct(T(1), out, axis, dbg);
        else pipeline.makeReduceSum(T(1), out, axis, dbg);
    } else if (name == "REDUCE_MAX" || name == "REDUCE_MIN" || name == "ARGMAX") {
        need(3);  // axis nanMode input
        const auto axis = static_cast<uint32_t>(S(0)), nan = static_cast<uint32_t>(S(1));
        if (name == "REDUCE_MAX") pipeline.makeReduceMax(T(2), out, axis, nan, dbg);
        else if (name == "REDUCE_MIN") pipeline.makeReduceMin(T(2), out, axis, nan, dbg);
        else pipeline.makeArgmax(T(2), out, axis, nan, dbg);
    } else if (name == "TABLE") {
        need(2);
        pipeline.makeTable(T(0), out, T(1), dbg);
    } else if (name == "NEGATE") {
        need(3);  // input inputZp outputZp (int32)
        pipeline.makeNegate(T(0), out, static_cast<int32_t>(first(1)), static_cast<int32_t>(first(2)), dbg);
    } else if (name == "ARITHMETIC_RIGHT_SHIFT") {
        need(3);  // round input1 input2
        pipeline.makeArithmeticRightShift(T(1), T(2), out, S(0) != 0, dbg);
    } else if (name == "RESHAPE") {
        need(1);  // input [shape]: the result type already carries the shape
        pipeline.makeReshape(T(0), out, dbg);
    } else if (name == "TRANSPOSE") {
        need(2);  // perms input
        pipeline.makeTranspose(T(1), out, toU32(V(0)), dbg);
    } else if (name == "SLICE") {
        need(3);  // input start size
        pipeline.makeSlice(T(0), out, toU32(V(1)), dbg);
    } else if (name == "CONCAT") {
        need(2);  // axis input0 input1 ...
        std::vector<TensorPtr> ins;
        for (size_t i = 1; i < a.size(); i++) ins.push_back(T(i));
        pipeline.makeConcat(ins, out, static_cast<uint32_t>(S(0)), dbg);
    } else if (name == "PAD") {
        need(3);  // input padding padConst
        const auto padValue = vectorReal(inst, a[2]);
        if (padValue.empty()) fail(inst, "PAD: empty pad constant");
        const double real = padValue[0];
        const int64_t integer = static_cast<int64_t>(real);
        pipeline.makePad(T(0), out, T(1), real, static_cast<int32_t>(integer), dbg);
    } else if (name == "REVERSE") {
        need(2);
        pipeline.makeReverse(T(1), out, static_cast<uint32_t>(S(0)), dbg);
    } else if (name == "SELECT") {
        need(3);
        pipeline.makeSelect(T(0), T(1), T(2), out, dbg);
    } else if (name == "TILE") {
        need(2);
        pipeline.makeTile(T(0), out, dbg);
    } else if (name == "GATHER") {
        need(2);
        pipeline.makeGather(T(0), T(1), out, dbg);
    } else if (name == "SCATTER") {
        need(3);  // valuesIn indices input
        pipeline.makeScatter(T(2), T(0), T(1), out, dbg);
    } else if (name == "RESIZE") {
        need(5);  // mode input scale offset border
        pipeline.makeResize(T(1), out, to32(V(2)), to32(V(3)), to32(V(4)), static_cast<uint32_t>(S(0)), dbg);
    } else {
        fail(inst, "TOSA operator " + name + " is not decoded by this front-end");
    }
    values[inst.result] = out;
}

SpvGraphInfo Module::build(const std::vector<Instruction> &program) {
    SpvGraphInfo info;
    // pass 1: everything outside graph bodies
    std::vector<const Instruction *> body;
    const Instruction *entry = nullptr, *graphDef = nullptr;
    bool inGraph = false, sawGraph = false;
    for (const auto &inst : program) {
        if (inst.opcode == "OpGraphEntryPointARM") {
            if (!entry) entry = &inst;
        } else if (inst.opcode == "OpGraphARM") {
            if (sawGraph) fail(inst, "more than one graph in a module is not supported");
            sawGraph = inGraph = true;
            graphDef = &inst;
        } else if (inst.opcode == "OpGraphEndARM") {
            inGraph = false;
        } else if (inGraph) {
            body.push_back(&inst);
        } else {
            declare(inst);
        }
    }
    if (!graphDef || !entry) throw std::runtime_error("SPIR-V graph: the module defines no graph entry point");
    if (tosaImport.empty()) fail(*graphDef, "the module does not import \"TOSA.001000.1\"");
    if (entry->operands.size() < 2 || entry->operands[0] != graphDef->result) fail(*entry, "entry point does not name the graph");
    info.entryPoint = entry->operands[1];
    const std::vector<std::string> iface(entry->operands.begin() + 2, entry->operands.end());
    const Type &gtype = typeOf(*graphDef, graphDef->operands.at(0));
    if (gtype.kind != TypeKind::Graph) fail(*graphDef, "not a graph type");
    registerVariables(*graphDef);

    const auto externalOf = [&](const Instruction &at, size_t ifaceIndex, uint32_t arrayIndex, std::array<uint32_t, 3> *key) {
        if (ifaceIndex >= iface.size()) fail(at, "interface index " + std::to_string(ifaceIndex) + " out of range");
        const auto v = variables.find(iface[ifaceIndex]);
        if (v == variables.end() || v->second.pointerType.empty()) fail(at, iface[ifaceIndex] + " is not a variable");
        *key = {v->second.set, v->second.binding, arrayIndex};
        TensorPtr tensor;
        try {
            tensor = pipeline.getTensor(v->second.set, v->second.binding, arrayIndex);
        } catch (const std::out_of_range &) {
        }
        if (!tensor)
            fail(at, iface[ifaceIndex] + ": no shape for set " + std::to_string(v->second.set) + " binding " +
                         std::to_string(v->second.binding) + " element " + std::to_string(arrayIndex));
        return tensor;
    };

    for (const auto *inst : body)
        if (inst->opcode == "OpCompositeExtract" && inst->operands.size() >= 3)
            extracts[{inst->operands[1], std::atoi(inst->operands[2].c_str())}] = inst->result;

    // pass 2: which values are routed to which outputs (an operator result routed to an output is written in place)
    struct Route {
        const Instruction *inst;
        std::string value;
        TensorPtr target;
    };
    std::vector<Route> routes;
    std::map<int64_t, std::array<uint32_t, 3>> outputKeys;
    std::map<int64_t, TensorPtr> outputTensors;
    for (const auto *inst : body) {
        if (inst->opcode != "OpGraphSetOutputARM") continue;
        if (inst->operands.size() < 2) fail(*inst, "expects a value and an output index");
        const int64_t index = scalarValue(*inst, inst->operands[1]);
        const auto arrayIndex = inst->operands.size() >= 3 ? static_cast<uint32_t>(scalarValue(*inst, inst->operands[2])) : 0u;
        std::array<uint32_t, 3> key{};
        TensorPtr target = externalOf(*inst, static_cast<size_t>(gtype.numInputs + index), arrayIndex, &key);
        outputTargets[inst->operands[0]].push_back(target);
        routes.push_back({inst, inst->operands[0], target});
        outputKeys[index] = key;
        outputTensors[index] = target;
    }

    // pass 3: the body
    std::map<int64_t, std::array<uint32_t, 3>> inputKeys;
    std::vector<const TensorDescriptor *> declaredInputs;
    for (const auto *inst : body) {
        if (inst->opcode == "OpGraphInputARM") {
            if (inst->operands.size() < 2) fail(*inst, "expects a type and an input index");
            const int64_t index = scalarValue(*inst, inst->operands[1]);
            const auto arrayIndex = inst->operands.size() >= 3 ? static_cast<uint32_t>(scalarValue(*inst, inst->operands[2])) : 0u;
            if (index < 0 || index >= gtype.numInputs) fail(*inst, "graph input index out of range");
            std::array<uint32_t, 3> key{};
            TensorPtr t = externalOf(*inst, static_cast<size_t>(index), arrayIndex, &key);
            values[inst->result] = t;
            inputKeys[index] = key;
            bool seen = false;
            for (const auto *d : declaredInputs) seen = seen || d == t.get();
            if (!seen) {
                pipeline.makeInput(t);
                declaredInputs.push_back(t.get());
            }
        } else if (inst->opcode == "OpExtInst") {
            if (inst->operands.size() < 3) fail(*inst, "expects a type, an instruction set and an instruction");
            if (inst->operands[1] != tosaImport) fail(*inst, "instruction set " + inst->operands[1] + " is not TOSA.001000.1");
            decodeTosa(*inst);
            info.instructions++;
        } else if (inst->opcode == "OpCompositeExtract") {
            if (inst->operands.size() < 3) fail(*inst, "expects a type, a composite and an index");
            const auto m = members.find(inst->operands[1]);
            const size_t index = static_cast<size_t>(std::atoi(inst->operands[2].c_str()));
            if (m == members.end() || index >= m->second.size()) fail(*inst, inst->operands[1] + " has no such member");
            values[inst->result] = m->second[index];
        } else if (inst->opcode == "OpGraphSetOutputARM") {
            continue;
        } else {
            fail(*inst, "only OpGraphInputARM, OpExtInst, OpCompositeExtract and OpGraphSetOutputARM may appear in a "
                        "graph body");
        }
    }

    // pass 4: outputs that are not written by their producer: inputs / constants routed to an output, and second
    // and later outputs of one operator result, are copies (the reference inserts a CAST for these)
    for (const auto &r : routes) {
        const auto produced = values.find(r.value);
        const bool isOperatorResult = produced != values.end() && produced->second.get() == outputTargets[r.value].front().get();
        if (isOperatorResult && r.target.get() == produced->second.get()) continue;
        const TensorPtr source = tensorOperand(*r.inst, r.value);
        pipeline.makeCast(source, r.target, "output_copy");
    }
    for (const auto &[index, tensor] : outputTensors) {
        pipeline.makeOutput(tensor);
        info.outputs.push_back(outputKeys[index]);
    }
    for (const auto &[index, key] : inputKeys) {
        (void)index;
        info.inputs.push_back(key);
    }
    return info;
}

}  // namespace

SpvGraphInfo loadSpirvAssembly(GraphPipeline &pipeline, const std::string &text, const std::vector<SpvBinding> &bindings,
                               const std::vector<SpvConstant> &constants,
                               const std::vector<SpvSpecialization> &specializations) {
    Module module(pipeline, bindings, constants, specializations);
    return module.build(tokenize(text));
}

SpvGraphInfo loadSpirvBinary(GraphPipeline &pipeline, const uint32_t *words, const size_t count,
                             const std::vector<SpvBinding> &bindings, const std::vector<SpvConstant> &constants,
                             const std::vector<SpvSpecialization> &specializations) {
    Module module(pipeline, bindings, constants, specializations);
    return module.build(decodeWords(words, count));
}

}  // namespace mlel::graph
