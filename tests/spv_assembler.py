"""Test helper: SPIR-V assembly text -> binary words, for the instructions data-graph modules use.

It exists so that the binary front-end (mlel_graph_load_spirv) can be fed the same modules as the text front-end:
the reference's own test modules (tests/shader/*.spvasm) and the ones tests/spvasm_writer.py writes.  The tables below
are typed from the published SPIR-V grammar independently of the decoder's tables in spirv_graph_loader.cpp, so a
slip in either shows up as a disagreement; neither is checked against SPIRV-Headers here (that package is not
available), which the tests' docstrings say.
"""
import struct

import numpy as np

MAGIC = 0x07230203
VERSION_1_6 = 0x00010600

CAPABILITY = {"Matrix": 0, "Shader": 1, "Float16": 9, "Float64": 10, "Int64": 11, "Int16": 22, "Int8": 39,
              "TensorsARM": 4174, "StorageTensorArrayDynamicIndexingARM": 4175,
              "StorageTensorArrayNonUniformIndexingARM": 4176, "GraphARM": 4191, "Float8EXT": 4212,
              "BFloat16TypeKHR": 5116, "VulkanMemoryModel": 5345, "ReplicatedCompositesEXT": 6024}
STORAGE_CLASS = {"UniformConstant": 0, "Input": 1, "Uniform": 2, "Output": 3, "Workgroup": 4, "Private": 6,
                 "Function": 7, "StorageBuffer": 12}
ADDRESSING = {"Logical": 0, "Physical32": 1, "Physical64": 2}
MEMORY_MODEL = {"Simple": 0, "GLSL450": 1, "OpenCL": 2, "Vulkan": 3}
DECORATION = {"SpecId": 1, "Block": 2, "ArrayStride": 6, "NonWritable": 24, "NonReadable": 25, "Binding": 33,
              "DescriptorSet": 34, "Offset": 35}
FP_ENCODING = {"BFloat16KHR": 0, "Float8E4M3EXT": 4214, "Float8E5M2EXT": 4215}

TOSA = ["ARGMAX", "AVG_POOL2D", "CONV2D", "CONV3D", "DEPTHWISE_CONV2D", "FFT2D", "MATMUL", "MAX_POOL2D", "RFFT2D",
        "TRANSPOSE_CONV2D",
        "CLAMP", "ERF", "SIGMOID", "TANH",
        "ADD", "ARITHMETIC_RIGHT_SHIFT", "BITWISE_AND", "BITWISE_OR", "BITWISE_XOR", "INTDIV", "LOGICAL_AND",
        "LOGICAL_LEFT_SHIFT", "LOGICAL_RIGHT_SHIFT", "LOGICAL_OR", "LOGICAL_XOR", "MAXIMUM", "MINIMUM", "MUL", "POW",
        "SUB", "TABLE",
        "ABS", "BITWISE_NOT", "CEIL", "CLZ", "COS", "EXP", "FLOOR", "LOG", "LOGICAL_NOT", "NEGATE", "RECIPROCAL",
        "RSQRT", "SIN",
        "SELECT",
        "EQUAL", "GREATER", "GREATER_EQUAL",
        "REDUCE_ALL", "REDUCE_ANY", "REDUCE_MAX", "REDUCE_MIN", "REDUCE_PRODUCT", "REDUCE_SUM",
        "CONCAT", "PAD", "RESHAPE", "REVERSE", "SLICE", "TILE", "TRANSPOSE",
        "GATHER", "SCATTER",
        "RESIZE",
        "CAST", "RESCALE"]

# opcode: (number, has result type, has result id, operand kinds)
OPCODES = {
    "OpName": (5, False, False, ["id", "str"]),
    "OpExtension": (10, False, False, ["str"]),
    "OpExtInstImport": (11, False, True, ["str"]),
    "OpExtInst": (12, True, True, ["id", "ext", "ids"]),
    "OpMemoryModel": (14, False, False, [ADDRESSING, MEMORY_MODEL]),
    "OpCapability": (17, False, False, [CAPABILITY]),
    "OpTypeVoid": (19, False, True, []),
    "OpTypeBool": (20, False, True, []),
    "OpTypeInt": (21, False, True, ["lit", "lit"]),
    "OpTypeFloat": (22, False, True, ["lit", "fpenc?"]),
    "OpTypeVector": (23, False, True, ["id", "lit"]),
    "OpTypeArray": (28, False, True, ["id", "id"]),
    "OpTypeRuntimeArray": (29, False, True, ["id"]),
    "OpTypeStruct": (30, False, True, ["ids"]),
    "OpTypePointer": (32, False, True, [STORAGE_CLASS, "id"]),
    "OpConstantTrue": (41, True, True, []),
    "OpConstantFalse": (42, True, True, []),
    "OpConstant": (43, True, True, ["const"]),
    "OpConstantComposite": (44, True, True, ["ids"]),
    "OpConstantNull": (46, True, True, []),
    "OpSpecConstantTrue": (48, True, True, []),
    "OpSpecConstantFalse": (49, True, True, []),
    "OpSpecConstant": (50, True, True, ["const"]),
    "OpSpecConstantComposite": (51, True, True, ["ids"]),
    "OpVariable": (59, True, True, [STORAGE_CLASS, "ids"]),
    "OpDecorate": (71, False, False, ["id", DECORATION, "lits"]),
    "OpCompositeExtract": (81, True, True, ["id", "lits"]),
    "OpTypeTensorARM": (4163, False, True, ["ids"]),
    "OpGraphConstantARM": (4181, True, True, ["lit"]),
    "OpGraphEntryPointARM": (4182, False, False, ["id", "str", "ids"]),
    "OpGraphARM": (4183, True, True, []),
    "OpGraphInputARM": (4184, True, True, ["ids"]),
    "OpGraphSetOutputARM": (4185, False, False, ["ids"]),
    "OpGraphEndARM": (4186, False, False, []),
    "OpTypeGraphARM": (4190, False, True, ["lit", "ids"]),
    "OpConstantCompositeReplicateEXT": (4461, True, True, ["id"]),
    "OpSpecConstantCompositeReplicateEXT": (4462, True, True, ["id"]),
}


def _tokens(line):
    out, i = [], 0
    while i < len(line):
        c = line[i]
        if c == ";":
            break
        if c in " \t\r":
            i += 1
        elif c == '"':
            j, text = i + 1, []
            while j < len(line) and line[j] != '"':
                if line[j] == "\\" and j + 1 < len(line):
                    j += 1
                text.append(line[j])
                j += 1
            out.append(("str", "".join(text)))
            i = j + 1
        else:
            j = i
            while j < len(line) and line[j] not in " \t\r;":
                j += 1
            out.append(("word", line[i:j]))
            i = j
    return out


def _string_words(text):
    raw = text.encode() + b"\0"
    raw += b"\0" * (-len(raw) % 4)
    return list(struct.unpack("<%dI" % (len(raw) // 4), raw))


def _float_bits(value, width, encoding):
    """Bits of `value` in the type's storage encoding, rounded to nearest even."""
    if width == 64:
        return struct.unpack("<Q", struct.pack("<d", value))[0]
    if width == 32:
        return struct.unpack("<I", struct.pack("<f", value))[0]
    if width == 16 and encoding is None:
        return int(np.array(value, np.float32).astype(np.float16).view(np.uint16))
    import torch
    kind = {(16, "BFloat16KHR"): torch.bfloat16, (8, "Float8E4M3EXT"): torch.float8_e4m3fn,
            (8, "Float8E5M2EXT"): torch.float8_e5m2}[(width, encoding)]
    t = torch.tensor([value], dtype=torch.float32).to(kind)
    return int(t.view(torch.uint8 if width == 8 else torch.int16).numpy().view(np.uint8 if width == 8 else np.uint16)[0])


def assemble(text, byte_swapped=False):
    """Returns the module as a numpy array of uint32 words."""
    ids, scalar_types = {}, {}

    def ident(word):
        assert word.startswith("%"), word
        if word not in ids:
            ids[word] = len(ids) + 1
        return ids[word]

    body = []
    for number, line in enumerate(text.splitlines(), 1):
        tok = _tokens(line)
        if not tok:
            continue
        result = None
        if len(tok) >= 3 and tok[1] == ("word", "="):
            result, tok = tok[0][1], tok[2:]
        name, args = tok[0][1], tok[1:]
        if name not in OPCODES:
            raise ValueError("line %d: %s is not known to this assembler" % (number, name))
        code, has_type, has_result, kinds = OPCODES[name]
        assert has_result == (result is not None), (number, line)
        words, k = [], 0
        type_word = None
        if has_type:
            type_word = args[k][1]
            words.append(ident(type_word))
            k += 1
        if has_result:
            words.append(ident(result))
        first_id = None
        for kind in kinds:
            if isinstance(kind, dict):
                words.append(kind[args[k][1]])
                k += 1
            elif kind == "id":
                if first_id is None:
                    first_id = args[k][1]
                words.append(ident(args[k][1]))
                k += 1
            elif kind == "ids":
                words += [ident(a[1]) for a in args[k:]]
                k = len(args)
            elif kind == "lit":
                words.append(int(args[k][1], 0) & 0xFFFFFFFF)
                k += 1
            elif kind == "lits":
                words += [int(a[1], 0) & 0xFFFFFFFF for a in args[k:]]
                k = len(args)
            elif kind == "str":
                assert args[k][0] == "str", (number, line)
                words += _string_words(args[k][1])
                k += 1
            elif kind == "fpenc?":
                if k < len(args):
                    words.append(FP_ENCODING[args[k][1]])
                    k += 1
            elif kind == "ext":
                word = args[k][1]
                words.append(TOSA.index(word) if word in TOSA else int(word, 0))
                k += 1
            elif kind == "const":
                what, width, extra = scalar_types[type_word]
                word = args[k][1]
                k += 1
                if word.startswith("!"):
                    bits = int(word[1:], 0)
                elif what == "int":
                    bits = int(word, 0) & ((1 << width) - 1)
                    if width < 32 and extra and bits >> (width - 1):  # signed: sign-extended to the word
                        bits |= 0xFFFFFFFF & ~((1 << width) - 1)
                else:
                    value = float.fromhex(word) if "0x" in word.lower() else float(word)
                    bits = _float_bits(value, width, extra)
                words += [bits & 0xFFFFFFFF] + ([bits >> 32] if width > 32 else [])
        assert k == len(args), "line %d: operands left over: %s" % (number, line)
        if name == "OpTypeInt":
            scalar_types[result] = ("int", int(args[0][1], 0), int(args[1][1], 0) != 0)
        elif name == "OpTypeFloat":
            scalar_types[result] = ("float", int(args[0][1], 0), args[1][1] if len(args) > 1 else None)
        body += [((len(words) + 1) << 16) | code] + words
    module = np.array([MAGIC, VERSION_1_6, 0, len(ids) + 1, 0] + body, dtype=np.uint32)
    return module.byteswap() if byte_swapped else module
