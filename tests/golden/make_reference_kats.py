"""Writes tests/golden/reference_kats.json: the known-answer vectors held by the reference's own tests.

Nothing from the reference is imported or executed: the numbers below are the literal inputs and expected
outputs of the reference's gtest cases (tests/vulkan.cpp, lines cited per case) and the operator attributes are
those of the SPIR-V graph each case loads (tests/shader/*.spvasm).  Run: python tests/golden/make_reference_kats.py
"""
import json
import os


def iota_u8(n):
    return [i & 0xFF for i in range(n)]


def s8(v):
    v &= 0xFF
    return v - 256 if v >= 128 else v


def s32(v):
    v &= 0xFFFFFFFF
    return v - (1 << 32) if v >= (1 << 31) else v


cases = {}

# tests/vulkan.cpp:998-1089 + tests/shader/conv2d.spvasm: CONV2D i8 -> i32, stride 2 (replicated), pad 0
conv_ref = [
    [0x000000ae, 0x000000f6, 0x0000013e, 0x00000186],
    [0x000002ee, 0x00000336, 0x0000037e, 0x000003c6],
    [0x0000052e, 0x00000176, 0xffffffbe, 0x00000006],
    [0xfffffb6e, 0xfffffbb6, 0xfffffbfe, 0xfffffc46],
]
cases["conv2d"] = {
    "source": "tests/vulkan.cpp:998-1089, tests/shader/conv2d.spvasm",
    "input": {"dtype": "i8", "shape": [1, 8, 8, 3], "data": [s8(v) for v in iota_u8(192)]},
    "weights": {"dtype": "i8", "shape": [3, 2, 2, 3], "data": [1] * 36},
    "bias": {"dtype": "i32", "shape": [3], "data": [0, 1, 2]},
    "attr": {"pad": [0, 0, 0, 0], "stride": [2, 2], "dilation": [1, 1], "input_zp": 0, "weight_zp": 0, "acc_type": 1},
    "expected": {"dtype": "i32", "shape": [1, 4, 4, 3],
                 "data": [s32(v + c) for row in conv_ref for v in row for c in range(3)]},
}

# tests/vulkan.cpp:1636-1678 + tests/shader/inlined-higher-rank-constant.spvasm: CONV2D (pad 1) then CAST i32->i8
cases["higher_rank_constant"] = {
    "source": "tests/vulkan.cpp:1636-1678, tests/shader/inlined-higher-rank-constant.spvasm",
    "input": {"dtype": "i8", "shape": [1, 3, 3, 1], "data": [1] * 9},
    "weights": {"dtype": "i8", "shape": [1, 3, 3, 1], "data": list(range(9))},
    "bias": {"dtype": "i32", "shape": [1], "data": [0]},
    "attr": {"pad": [1, 1, 1, 1], "stride": [1, 1], "dilation": [1, 1], "input_zp": 0, "weight_zp": 0, "acc_type": 1},
    "expected": {"dtype": "i8", "shape": [1, 3, 3, 1], "data": [24, 33, 20, 27, 36, 21, 12, 15, 8]},
}

# tests/vulkan.cpp:1158-1209 + tests/shader/conv2_acc_int64.spvasm: CONV2D i16 x i8 -> i64 accumulate
cases["conv2d_acc_int64"] = {
    "source": "tests/vulkan.cpp:1158-1209, tests/shader/conv2_acc_int64.spvasm",
    "input": {"dtype": "i16", "shape": [1, 2, 2, 4], "data": list(range(1, 17))},
    "weights": {"dtype": "i8", "shape": [4, 1, 1, 4], "data": [1, 2, 3, 4, -1, 0, 1, 2, 2, -3, 4, -5, -2, -1, 0, 1]},
    "bias": {"dtype": "i64", "shape": [4], "data": [10, -20, 30, -40]},
    "attr": {"pad": [0, 0, 0, 0], "stride": [1, 1], "dilation": [1, 1], "input_zp": 0, "weight_zp": 0, "acc_type": 4},
    "expected": {"dtype": "i64", "shape": [1, 2, 2, 4],
                 "data": [40, -10, 18, -40, 80, -2, 10, -48, 120, 6, 2, -56, 160, 14, -6, -64]},
}

# tests/vulkan.cpp:1211-1290 + tests/shader/conv3d_large_stride.spvasm: CONV3D i8 -> i32 with a kernel 8192 wide whose only
# non-zero taps are kx = 8190 and 8191 (weights[oc][kd][kh][8190 + j][ic] = relevant[((oc*2 + kd)*2 + kh)*8 + 4j + ic])
cases["conv3d_large_stride"] = {
    "source": "tests/vulkan.cpp:1211-1290, tests/shader/conv3d_large_stride.spvasm",
    "input": {"dtype": "i8", "shape": [1, 3, 2, 2, 4], "data": [-128] * 48},
    "weights_shape": [3, 2, 2, 8192, 4],
    "relevant_weights": [
        1, -1, 2, -1, 1, 0, -1, 0, 1, 2, 2, -1, 2, 2, 0, 1, 1, -2, -1, -2, 0, 2, -2, 0,
        1, 1, -2, 1, 0, -2, 2, -1, 1, 0, 0, 2, 2, 0, 0, -1, 0, 0, -1, -1, -1, 0, -1, -2,
        1, 1, -2, 2, -1, 1, 1, -2, 0, 0, 1, 2, 1, 2, 0, -2, 0, 2, 1, -2, 1, -1, -1, -1,
        0, -2, 2, -2, 0, -1, 0, -1, 0, 2, 0, -2, 2, 1, 1, 0, -1, 0, 1, -2, -2, 2, 1, 0],
    "attr": {"pad": [1, 0, 1, 0, 8190, 8192], "stride": [1, 1, 8192], "dilation": [1, 1, 1], "input_zp": 9,
             "weight_zp": 0, "acc_type": 1},
    "expected": {"dtype": "i32", "shape": [1, 3, 2, 2, 3], "data": [
        0, -548, 137, 0, 0, 0, 548, -685, -411, 0, 0, 0, -1233, 274, 685, 0, 0, 0,
        -822, -411, 274, 0, 0, 0, -1233, 274, 685, 0, 0, 0, -822, -411, 274, 0, 0, 0]},
}

# tests/vulkan.cpp:1091-1156: all-ones closed form, every output == IC (sizes reduced by the test that uses this)
cases["conv2d_all_ones"] = {
    "source": "tests/vulkan.cpp:1091-1156 (OC=262144 / H or W = 524281 in the reference)",
    "channels": 4,
    "large_oc": 262144,
    "large_spatial": 524281,
}

# tests/vulkan.cpp:611-658 + tests/shader/maxpool.spvasm: MAX_POOL2D 2x2 stride 2, channel 0 = -128 + pixel index
mp_in = [0] * (16 * 16 * 3)
for i in range(0, len(mp_in), 3):
    mp_in[i] = s8(-128 + i // 3)
mp_ref = [0x91, 0x93, 0x95, 0x97, 0x99, 0x9b, 0x9d, 0x9f, 0xb1, 0xb3, 0xb5, 0xb7, 0xb9, 0xbb, 0xbd, 0xbf,
          0xd1, 0xd3, 0xd5, 0xd7, 0xd9, 0xdb, 0xdd, 0xdf, 0xf1, 0xf3, 0xf5, 0xf7, 0xf9, 0xfb, 0xfd, 0xff,
          0x11, 0x13, 0x15, 0x17, 0x19, 0x1b, 0x1d, 0x1f, 0x31, 0x33, 0x35, 0x37, 0x39, 0x3b, 0x3d, 0x3f,
          0x51, 0x53, 0x55, 0x57, 0x59, 0x5b, 0x5d, 0x5f, 0x71, 0x73, 0x75, 0x77, 0x79, 0x7b, 0x7d, 0x7f]
cases["max_pool2d"] = {
    "source": "tests/vulkan.cpp:611-658, tests/shader/maxpool.spvasm",
    "input": {"dtype": "i8", "shape": [1, 16, 16, 3], "data": mp_in},
    "attr": {"kernel": [2, 2], "stride": [2, 2], "pad": [0, 0, 0, 0], "nan_mode": 1},
    "expected": {"dtype": "i8", "shape": [1, 8, 8, 3], "data": [x for v in mp_ref for x in (s8(v), 0, 0)]},
}

# tests/vulkan.cpp:752-792 + tests/shader/twolayer-maxpool.spvasm: two MAX_POOL2D 2x2 stride 2 in sequence
mp2_ref = [0xb3, 0xb7, 0xbb, 0xbf, 0xf3, 0xf7, 0xfb, 0xff, 0x33, 0x37, 0x3b, 0x3f, 0x73, 0x77, 0x7b, 0x7f]
cases["two_layer_max_pool2d"] = {
    "source": "tests/vulkan.cpp:752-792, tests/shader/twolayer-maxpool.spvasm",
    "input": {"dtype": "i8", "shape": [1, 16, 16, 3], "data": mp_in},
    "attr": {"kernel": [2, 2], "stride": [2, 2], "pad": [0, 0, 0, 0], "nan_mode": 1},
    "intermediate_shape": [1, 8, 8, 3],
    "expected": {"dtype": "i8", "shape": [1, 4, 4, 3], "data": [x for v in mp2_ref for x in (s8(v), 0, 0)]},
}

# tests/vulkan.cpp:1579-1634 + tests/shader/graph-constant-arm.spvasm:
# RESCALE(i8->i32, x2) + RESCALE(i8->i32, x3) -> ADD(i32) -> RESCALE(i32->i8, x4); shift 0, scale32, single round
cases["graph_constant_arm"] = {
    "source": "tests/vulkan.cpp:1579-1634, tests/shader/graph-constant-arm.spvasm",
    "input0": {"dtype": "i8", "shape": [5], "data": [0, 1, 2, 3, 4]},
    "input1": {"dtype": "i8", "shape": [5], "data": [0, 1, 2, 3, 4]},
    "multipliers": [2, 3, 4],
    "shifts": [0, 0, 0],
    "rescale": {"scale32": 1, "double_round": 0, "per_channel": 0, "input_unsigned": 0, "output_unsigned": 0,
                "input_zp": 0, "output_zp": 0},
    "expected": {"dtype": "i8", "shape": [5], "data": [0, 20, 40, 60, 80]},
}

# tests/vulkan.cpp:1333-1404 + tests/shader/concat.spvasm: CONCAT axis 1
cases["concat"] = {
    "source": "tests/vulkan.cpp:1333-1404, tests/shader/concat.spvasm",
    "input0": {"dtype": "i8", "shape": [1, 2, 2, 2], "data": list(range(8))},
    "input1": {"dtype": "i8", "shape": [1, 2, 2, 2], "data": list(range(8))},
    "axis": 1,
    "expected": {"dtype": "i8", "shape": [1, 4, 2, 2], "data": list(range(8)) * 2},
}

# tests/vulkan.cpp:1406-1439 + tests/shader/concat_interval.spvasm: ADD f32, CONCAT axis 1, RESHAPE
cases["concat_interval"] = {
    "source": "tests/vulkan.cpp:1406-1439, tests/shader/concat_interval.spvasm",
    "input": {"dtype": "f32", "shape": [3, 3], "data": [0, 1, 2, 3, 4, 5, 6, 7, 8]},
    "one": {"dtype": "f32", "shape": [3, 3], "data": [1] * 9},
    "zero": {"dtype": "f32", "shape": [3, 1], "data": [0] * 3},
    "expected": {"dtype": "f32", "shape": [12], "data": [1, 2, 3, 0, 4, 5, 6, 0, 7, 8, 9, 0]},
}

# tests/vulkan.cpp:1441-1492 + tests/shader/slice.spvasm: SLICE start (0,4,4,1) size (1,2,2,2)
cases["slice"] = {
    "source": "tests/vulkan.cpp:1441-1492, tests/shader/slice.spvasm",
    "input": {"dtype": "i8", "shape": [1, 8, 8, 3], "data": [s8(v) for v in iota_u8(192)]},
    "start": [0, 4, 4, 1],
    "size": [1, 2, 2, 2],
    "expected": {"dtype": "i8", "shape": [1, 2, 2, 2],
                 "data": [s8(v) for v in [0x6d, 0x6e, 0x70, 0x71, 0x85, 0x86, 0x88, 0x89]]},
}

# tests/vulkan.cpp:1494-1577 + tests/shader/nop-outputs.spvasm: pass-through outputs become CAST i8 -> i8
cases["nop_outputs"] = {
    "source": "tests/vulkan.cpp:1494-1577, tests/shader/nop-outputs.spvasm",
    "input": {"dtype": "i8", "shape": [1, 8, 8, 3], "data": [s8(v) for v in iota_u8(192)]},
    "constant": {"dtype": "i8", "shape": [1, 8, 8, 3], "data": [s8(v) for v in iota_u8(192)]},
}

# tests/vulkan.cpp:1680-1744 + tests/shader/maximum.spvasm: MAXIMUM i32
cases["maximum"] = {
    "source": "tests/vulkan.cpp:1680-1744, tests/shader/maximum.spvasm",
    "input0": {"dtype": "i32", "shape": [1, 2, 2, 2], "data": list(range(8))},
    "input1": {"dtype": "i32", "shape": [1, 2, 2, 2], "data": [-16 + 4 * i for i in range(8)]},
    "nan_mode": 1,
    "expected": {"dtype": "i32", "shape": [1, 2, 2, 2], "data": [0, 1, 2, 3, 4, 5, 8, 12]},
}

# tests/vulkan.cpp:1796-1842 + tests/shader/sin.spvasm: SIN f32 with an error bound
cases["sin"] = {
    "source": "tests/vulkan.cpp:1796-1842, tests/shader/sin.spvasm",
    "input": 0.000111731846,
    "reference": 0.00011173184588586903,
    "error_bound": 7.715463482888105e-08,
}

# tests/graph/interval_memory_planner_tests.cpp:17-106: {id, first, last, size, order}, unseen {id, size}
cases["interval_planner"] = [
    {"name": "NonOverlappingTensorsReuseMemory", "intervals": [[0, 0, 0, 64, 0], [1, 1, 1, 64, 1]], "unseen": [],
     "alignment": 16, "offsets": {"0": 0, "1": 0}, "memory_size": 64},
    {"name": "OverlappingTensorsDoNotAlias", "intervals": [[0, 0, 2, 64, 0], [1, 1, 3, 64, 1]], "unseen": [],
     "alignment": 16, "distinct": [[0, 1]], "memory_size": 128},
    {"name": "SplitsOversizedFreeBlocks", "intervals": [[0, 0, 0, 128, 0], [1, 1, 2, 64, 1], [2, 1, 2, 64, 2]],
     "unseen": [], "alignment": 16, "offsets": {"0": 0, "1": 0, "2": 64}, "memory_size": 128},
    {"name": "DoesNotCoalesceAdjacentFreeBlocks",
     "intervals": [[0, 0, 0, 64, 0], [1, 0, 0, 64, 1], [2, 1, 1, 128, 2]], "unseen": [], "alignment": 16,
     "offsets": {"0": 0, "1": 64, "2": 128}, "memory_size": 256},
    {"name": "UnseenTensorsReceiveUniqueStorage", "intervals": [[0, 0, 0, 64, 0]], "unseen": [[1, 32], [2, 32]],
     "alignment": 16, "offsets": {"0": 0, "1": 64, "2": 96}, "memory_size": 128},
    {"name": "ExternalTensorsAreNotIncludedInSessionAllocation", "intervals": [[0, 0, 0, 64, 0]],
     "unseen": [[1, 64]], "alignment": 16, "present": [0, 1], "absent": [2], "memory_size": 128},
]

here = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(here, "reference_kats.json"), "w") as f:
    json.dump(cases, f, indent=1, sort_keys=True)
print("wrote", len(cases), "cases")
