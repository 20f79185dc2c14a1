# writes tests/golden/reference_view_vectors.json (hand-transcribed from the reference's own tests in core/mod.rs)
import json
cases = []
def case(name, ref, inputs, program, expect, dtype="i32"):
    cases.append({"name": name, "ref": "core/mod.rs:" + ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
def T(shape, values): return {"shape": shape, "values": values}
def IDX(i): return {"range": [i, i]}
def G(*pairs): return [[list(i), v] for i, v in pairs]
r = lambda a, b: list(range(a, b + 1))

case("transpose_2d", "2056-2077", {"a": T([2, 3], r(1, 6))}, [["t", "transpose", "a"]],
     [{"t": "t", "shape": [3, 2], "strides": [1, 3], "get": G(((0, 0), 1), ((0, 1), 4), ((1, 0), 2), ((1, 1), 5), ((2, 0), 3), ((2, 1), 6))}])
case("transpose_3d", "2080-2106", {"a": T([2, 2, 2], r(1, 8))}, [["t", "transpose", "a"]],
     [{"t": "t", "shape": [2, 2, 2], "strides": [1, 2, 4], "get": G(((0, 0, 0), 1), ((1, 0, 0), 2), ((0, 1, 0), 3), ((0, 0, 1), 5), ((1, 1, 1), 8))}])
case("transpose_mut_2d", "2109-2131", {"a": T([2, 3], r(1, 6))},
     [["t", "transpose", "a"], ["t", "set", "t", [0, 0], 10], ["t", "set", "t", [1, 1], 50], ["t", "set", "t", [2, 1], 60]],
     [{"t": "t", "shape": [3, 2]}, {"t": "a", "get": G(((0, 0), 10), ((1, 1), 50), ((1, 2), 60)), "values": [10, 2, 3, 4, 50, 60]}])
case("transpose_mut_3d", "2134-2153", {"a": T([2, 2, 2], r(1, 8))},
     [["t", "transpose", "a"], ["t", "set", "t", [0, 0, 0], 100], ["t", "set", "t", [1, 0, 0], 200], ["t", "set", "t", [0, 0, 1], 500]],
     [{"t": "a", "get": G(((0, 0, 0), 100), ((0, 0, 1), 200), ((1, 0, 0), 500))}])
case("permute_2d_swap", "2156-2173", {"a": T([2, 3], r(1, 6))}, [["p", "permute", "a", [1, 0]]],
     [{"t": "p", "shape": [3, 2], "strides": [1, 3], "get": G(((0, 0), 1), ((1, 0), 2), ((2, 1), 6))}])
case("permute_3d_rotate", "2176-2204", {"a": T([2, 2, 3], r(1, 12))}, [["p", "permute", "a", [2, 0, 1]]],
     [{"t": "p", "shape": [3, 2, 2], "strides": [1, 6, 3], "get": G(((0, 0, 0), 1), ((1, 0, 0), 2), ((0, 0, 1), 4), ((2, 1, 1), 12))}])
case("permute_3d_partial_swap", "2207-2224", {"a": T([2, 2, 2], r(1, 8))}, [["p", "permute", "a", [1, 0, 2]]],
     [{"t": "p", "shape": [2, 2, 2], "strides": [2, 4, 1], "get": G(((0, 0, 0), 1), ((1, 0, 0), 3), ((0, 1, 1), 6))}])
case("permute_mut_with_write", "2227-2252", {"a": T([2, 2, 3], r(1, 12))},
     [["p", "permute", "a", [2, 0, 1]], ["p", "set", "p", [0, 0, 0], 100], ["p", "set", "p", [1, 0, 0], 200], ["p", "set", "p", [2, 1, 1], 1200]],
     [{"t": "p", "shape": [3, 2, 2]}, {"t": "a", "get": G(((0, 0, 0), 100), ((0, 0, 1), 200), ((1, 1, 2), 1200))}])
case("permute_identity", "2255-2268", {"a": T([2, 3], r(1, 6))}, [["p", "permute", "a", [0, 1]]],
     [{"t": "p", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((1, 2), 6))}])
case("permute_4d", "2271-2288", {"a": T([2, 2, 2, 2], r(1, 16))}, [["p", "permute", "a", [3, 2, 1, 0]]],
     [{"t": "p", "shape": [2, 2, 2, 2], "strides": [1, 2, 4, 8], "get": G(((0, 0, 0, 0), 1), ((1, 0, 0, 0), 2), ((1, 1, 1, 1), 16))}])
case("chained_permutations", "2339-2359", {"a": T([2, 2, 2], r(1, 8))}, [["p1", "permute", "a", [2, 0, 1]], ["p2", "permute", "p1", [1, 2, 0]]],
     [{"t": "p1", "shape": [2, 2, 2]}, {"t": "p2", "shape": [2, 2, 2], "get": G(((0, 0, 0), 1), ((1, 0, 0), 5), ((0, 1, 0), 3), ((1, 1, 1), 8))}])
case("permute_mut_chained", "2362-2379", {"a": T([2, 2, 2], r(1, 8))},
     [["p1", "permute", "a", [1, 0, 2]], ["p2", "permute", "p1", [2, 0, 1]], ["p2", "set", "p2", [0, 0, 0], 111]],
     [{"t": "a", "get": G(((0, 0, 0), 111))}])
case("permute_wrong_dims_short", "2382-2397", {"a": T([2, 3], r(1, 6))}, [["p", "permute", "a", [0]]], [{"error": "WrongDims"}])
case("permute_wrong_dims_long", "2382-2397", {"a": T([2, 3], r(1, 6))}, [["p", "permute", "a", [0, 1, 2]]], [{"error": "WrongDims"}])
case("permute_invalid_dim_a", "2400-2414", {"a": T([2, 3], r(1, 6))}, [["p", "permute", "a", [0, 3]]], [{"error": "InvalidDim"}])
case("permute_invalid_dim_b", "2400-2414", {"a": T([2, 3], r(1, 6))}, [["p", "permute", "a", [2, 1]]], [{"error": "InvalidDim"}])
case("transpose_then_slice", "2417-2434", {"a": T([2, 3], r(1, 6))}, [["t", "transpose", "a"], ["s", "slice", "t", 0, IDX(0)]],
     [{"t": "t", "shape": [3, 2]}, {"t": "s", "shape": [2], "get": G(((0,), 1), ((1,), 4))}])
case("slice_then_transpose_mut", "2437-2461", {"a": T([3, 4], r(1, 12))},
     [["s", "slice", "a", 0, {"range": [0, 2]}], ["t", "transpose", "s"], ["t", "set", "t", [0, 0], 100], ["t", "set", "t", [3, 1], 800]],
     [{"t": "a", "get": G(((0, 0), 100), ((1, 3), 800), ((2, 0), 9))}])
case("permute_write_compatibility_complex", "2464-2489", {"a": T([2, 3, 4], r(1, 24))},
     [["s", "slice", "a", 0, {"range": [1, 2]}], ["p", "permute", "s", [2, 0, 1]], ["p", "set", "p", [0, 0, 0], 1300], ["p", "set", "p", [3, 0, 2], 2400]],
     [{"t": "s", "shape": [1, 3, 4]}, {"t": "p", "shape": [4, 1, 3]}, {"t": "a", "get": G(((1, 0, 0), 1300), ((1, 2, 3), 2400), ((0, 0, 0), 1))}])
# ---- unsqueeze (2492-2945; `unsqueeze()` is unsqueeze_at(0)) ----
case("unsqueeze_scalar", "2492-2505", {"a": T([], [42])}, [["u", "unsqueeze", "a", 0]], [{"t": "u", "shape": [1], "strides": [1], "get": G(((0,), 42))}])
case("unsqueeze_1d", "2508-2527", {"a": T([5], r(1, 5))}, [["u", "unsqueeze", "a", 0]],
     [{"t": "u", "shape": [1, 5], "strides": [5, 1], "values": r(1, 5)}])
case("unsqueeze_2d", "2530-2550", {"a": T([2, 3], r(1, 6))}, [["u", "unsqueeze", "a", 0]],
     [{"t": "u", "shape": [1, 2, 3], "strides": [6, 3, 1], "values": r(1, 6)}])
case("double_unsqueeze", "2553-2571", {"a": T([3], [1, 2, 3])}, [["u1", "unsqueeze", "a", 0], ["u2", "unsqueeze", "u1", 0]],
     [{"t": "u1", "shape": [1, 3]}, {"t": "u2", "shape": [1, 1, 3], "strides": [3, 3, 1], "values": [1, 2, 3]}])
case("unsqueeze_after_slice", "2574-2594", {"a": T([2, 3], r(1, 6))}, [["s", "slice", "a", 0, IDX(0)], ["u", "unsqueeze", "s", 0]],
     [{"t": "s", "shape": [3]}, {"t": "u", "shape": [1, 3], "strides": [3, 1], "values": [1, 2, 3]}])
case("unsqueeze_after_column_slice", "2597-2617", {"a": T([2, 3], r(1, 6))}, [["s", "slice", "a", 1, IDX(0)], ["u", "unsqueeze", "s", 0]],
     [{"t": "s", "shape": [2], "strides": [3]}, {"t": "u", "shape": [1, 2], "strides": [6, 3], "values": [1, 4]}])
case("unsqueeze_at_beginning", "2794-2809", {"a": T([2, 3], r(1, 6))}, [["u", "unsqueeze", "a", 0]],
     [{"t": "u", "shape": [1, 2, 3], "strides": [6, 3, 1], "get": G(((0, 0, 0), 1), ((0, 0, 2), 3), ((0, 1, 0), 4), ((0, 1, 2), 6))}])
case("unsqueeze_at_middle", "2812-2827", {"a": T([2, 3], r(1, 6))}, [["u", "unsqueeze", "a", 1]],
     [{"t": "u", "shape": [2, 1, 3], "strides": [3, 3, 1], "get": G(((0, 0, 0), 1), ((0, 0, 2), 3), ((1, 0, 0), 4), ((1, 0, 2), 6))}])
case("unsqueeze_at_end", "2830-2845", {"a": T([2, 3], r(1, 6))}, [["u", "unsqueeze", "a", 2]],
     [{"t": "u", "shape": [2, 3, 1], "strides": [3, 1, 1], "get": G(((0, 0, 0), 1), ((0, 2, 0), 3), ((1, 0, 0), 4), ((1, 2, 0), 6))}])
case("unsqueeze_at_1d_tensor", "2848-2861", {"a": T([4], r(1, 4))}, [["u0", "unsqueeze", "a", 0], ["u1", "unsqueeze", "a", 1]],
     [{"t": "u0", "shape": [1, 4], "strides": [4, 1]}, {"t": "u1", "shape": [4, 1], "strides": [1, 1]}])
case("unsqueeze_at_3d_tensor", "2864-2890", {"a": T([2, 3, 4], r(1, 24))},
     [["u0", "unsqueeze", "a", 0], ["u1", "unsqueeze", "a", 1], ["u2", "unsqueeze", "a", 2], ["u3", "unsqueeze", "a", 3]],
     [{"t": "u0", "shape": [1, 2, 3, 4], "strides": [24, 12, 4, 1]}, {"t": "u1", "shape": [2, 1, 3, 4], "strides": [12, 12, 4, 1]},
      {"t": "u2", "shape": [2, 3, 1, 4], "strides": [12, 4, 4, 1]}, {"t": "u3", "shape": [2, 3, 4, 1], "strides": [12, 4, 1, 1]}])
case("unsqueeze_at_multiple_sequential", "2893-2912", {"a": T([2, 2], r(1, 4))},
     [["s1", "unsqueeze", "a", 0], ["s2", "unsqueeze", "s1", 1], ["s3", "unsqueeze", "s2", 2]],
     [{"t": "s1", "shape": [1, 2, 2]}, {"t": "s2", "shape": [1, 1, 2, 2]}, {"t": "s3", "shape": [1, 1, 1, 2, 2], "get": G(((0, 0, 0, 0, 0), 1), ((0, 0, 0, 1, 1), 4))}])
case("unsqueeze_at_multiple_different_positions", "2915-2940", {"a": T([2, 3], r(1, 6))},
     [["s1", "unsqueeze", "a", 2], ["s2", "unsqueeze", "s1", 0], ["s3", "unsqueeze", "s2", 2]],
     [{"t": "s1", "shape": [2, 3, 1]}, {"t": "s2", "shape": [1, 2, 3, 1]},
      {"t": "s3", "shape": [1, 2, 1, 3, 1], "get": G(((0, 0, 0, 0, 0), 1), ((0, 0, 0, 2, 0), 3), ((0, 1, 0, 0, 0), 4), ((0, 1, 0, 2, 0), 6))}])
# ---- squeeze (3501-3975) ----
case("squeeze_basic_2d", "3501-3512", {"a": T([1, 3], [1, 2, 3])}, [["q", "squeeze", "a"]], [{"t": "q", "shape": [3], "strides": [1], "values": [1, 2, 3]}])
case("squeeze_basic_3d", "3515-3526", {"a": T([1, 2, 1, 3], r(1, 6))}, [["q", "squeeze", "a"]],
     [{"t": "q", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((0, 2), 3), ((1, 0), 4), ((1, 2), 6))}])
case("squeeze_all_dimensions", "3529-3537", {"a": T([1, 1, 1], [42])}, [["q", "squeeze", "a"]], [{"t": "q", "shape": [], "strides": [], "values": [42]}])
case("squeeze_no_size_one_dims", "3540-3549", {"a": T([2, 3], r(1, 6))}, [["q", "squeeze", "a"]],
     [{"t": "q", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((1, 2), 6))}])
case("squeeze_at_specific_dim", "3552-3561", {"a": T([1, 2, 3], r(1, 6))}, [["q", "squeeze", "a", 0]],
     [{"t": "q", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((1, 2), 6))}])
case("squeeze_at_middle_dim", "3564-3573", {"a": T([2, 1, 3], r(1, 6))}, [["q", "squeeze", "a", 1]],
     [{"t": "q", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((1, 2), 6))}])
case("squeeze_at_end_dim", "3576-3585", {"a": T([2, 3, 1], r(1, 6))}, [["q", "squeeze", "a", 2]],
     [{"t": "q", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((1, 2), 6))}])
case("squeeze_after_slice", "3588-3604", {"a": T([2, 3], r(1, 6))}, [["s", "slice", "a", 0, IDX(0)], ["u", "unsqueeze", "s", 0], ["q", "squeeze", "u"]],
     [{"t": "s", "shape": [3]}, {"t": "u", "shape": [1, 3]}, {"t": "q", "shape": [3], "get": G(((0,), 1), ((2,), 3))}])
case("squeeze_after_column_slice", "3607-3625", {"a": T([2, 3], r(1, 6))}, [["s", "slice", "a", 1, IDX(1)], ["u", "unsqueeze", "s", 1], ["q", "squeeze", "u"]],
     [{"t": "s", "shape": [2], "get": G(((0,), 2), ((1,), 5))}, {"t": "u", "shape": [2, 1]}, {"t": "q", "shape": [2], "get": G(((0,), 2), ((1,), 5))}])
case("squeeze_after_3d_slice", "3628-3648", {"a": T([2, 3, 4], r(1, 24))}, [["s", "slice", "a", 0, IDX(1)], ["u", "unsqueeze", "s", 0], ["q", "squeeze", "u"]],
     [{"t": "s", "shape": [3, 4]}, {"t": "u", "shape": [1, 3, 4]}, {"t": "q", "shape": [3, 4], "get": G(((0, 0), 13), ((2, 3), 24))}])
case("squeeze_preserves_data_after_negative_stride", "3798-3818", {"a": T([6], r(1, 6))},
     [["v", "slice", "a", 0, {"slice": [None, None, -1]}], ["u", "unsqueeze", "v", 0], ["q", "squeeze", "u"]],
     [{"t": "v", "get": G(((0,), 6), ((5,), 1))}, {"t": "u", "shape": [1, 6]}, {"t": "q", "shape": [6], "get": G(((0,), 6), ((5,), 1))}])
case("squeeze_multiple_dims_2d", "3821-3831", {"a": T([1, 6, 1], r(1, 6))}, [["q", "squeeze", "a"]], [{"t": "q", "shape": [6], "strides": [1], "values": r(1, 6)}])
case("squeeze_multiple_dims_4d", "3834-3843", {"a": T([1, 2, 1, 3, 1], r(1, 6))}, [["q", "squeeze", "a"]],
     [{"t": "q", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((1, 2), 6))}])
case("squeeze_then_modify_mut", "3846-3870", {"a": T([1, 2, 4, 1], r(1, 8))},
     [["q", "squeeze", "a"]] + [["q", "set", "q", [0, i], i * 10] for i in range(4)],
     [{"t": "q", "shape": [2, 4], "get": G(((0, 0), 0), ((0, 1), 10), ((0, 2), 20), ((0, 3), 30), ((1, 0), 5), ((1, 3), 8))}])
case("squeeze_rank0", "3873-3880", {"a": T([], [42])}, [["q", "squeeze", "a"]], [{"t": "q", "shape": [], "values": [42]}])
case("squeeze_at_then_slice", "3883-3895", {"a": T([1, 3, 4], r(1, 12))}, [["q", "squeeze", "a", 0], ["s", "slice", "q", 0, IDX(1)]],
     [{"t": "q", "shape": [3, 4]}, {"t": "s", "shape": [4], "get": G(((0,), 5), ((3,), 8))}])
case("double_squeeze_at", "3898-3912", {"a": T([1, 2, 1, 2], r(1, 4))}, [["q1", "squeeze", "a", 0], ["q2", "squeeze", "q1", 1]],
     [{"t": "q1", "shape": [2, 1, 2]}, {"t": "q2", "shape": [2, 2], "values": [1, 2, 3, 4]}])
case("squeeze_unsqueeze_roundtrip", "3915-3936", {"a": T([2, 3], r(1, 6))}, [["u", "unsqueeze", "a", 0], ["q", "squeeze", "u", 0]],
     [{"t": "u", "shape": [1, 2, 3]}, {"t": "q", "shape": [2, 3], "strides": [3, 1], "get": G(((0, 0), 1), ((1, 2), 6))}])
case("squeeze_preserves_contiguity", "3962-3970", {"a": T([1, 2, 3], r(1, 6))}, [["q", "squeeze", "a"]], [{"t": "a", "contiguous": True}, {"t": "q", "shape": [2, 3], "contiguous": True}])
json.dump({"_comment": "Known-answer vectors transcribed from the reference's own #[test]s on views (transpose, permute, unsqueeze, squeeze, writes through views); "
                       "`ref` = file:lines under libs/rtensors/src/.  Program format: tests/golden_dsl.py.",
           "cases": cases}, open("tests/golden/reference_view_vectors.json", "w"), separators=(",", ":"))
print(len(cases), "cases")
