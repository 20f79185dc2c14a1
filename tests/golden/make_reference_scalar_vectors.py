# writes tests/golden/reference_scalar_vectors.json (hand-transcribed from the reference's own tests)
import json
R = "ops/mod.rs"
cases = []
def case(name, ref, dtype, inputs, program, expect):
    cases.append({"name": name, "ref": R + ":" + ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
def T(shape, values): return {"shape": shape, "values": values}
def ones(shape):
    n = 1
    for d in shape: n *= d
    return T(shape, [1.0] * n)
def IDX(i): return {"range": [i, i]}          # `a..a` selects one index and drops the dim
def inplace(name, ref, dtype, shape, values, steps, want, tol=None):
    prog = [["x", {"+": "iadd_scalar", "-": "isub_scalar", "*": "imul_scalar", "/": "idiv_scalar"}[op], "x", v] for op, v in steps]
    e = {"t": "x", "shape": shape, "values": want}
    if tol: e["tol"] = tol
    case(name, ref, dtype, {"x": T(shape, values)}, prog, [e])

# ---- in-place scalar ops on a whole tensor (ops/mod.rs:16-112) ----
inplace("scalar_add", "16-24", "i32", [3], [1, 2, 3], [("+", 5)], [6, 7, 8])
inplace("scalar_add_ref", "26-34", "i32", [3], [1, 2, 3], [("+", 10)], [11, 12, 13])
inplace("scalar_add_negative", "36-43", "i32", [3], [10, 20, 30], [("+", -5)], [5, 15, 25])
inplace("scalar_sub", "46-53", "i32", [3], [10, 20, 30], [("-", 5)], [5, 15, 25])
inplace("scalar_sub_ref", "55-63", "i32", [3], [10, 20, 30], [("-", 10)], [0, 10, 20])
inplace("scalar_sub_negative", "65-72", "i32", [3], [1, 2, 3], [("-", -5)], [6, 7, 8])
inplace("scalar_mul", "76-83", "i32", [3], [1, 2, 3], [("*", 5)], [5, 10, 15])
inplace("scalar_div_f32", "85-92", "f32", [3], [1., 2., 3.], [("/", 5.)], [0.2, 0.4, 0.6])
inplace("scalar_mul_ref", "94-102", "i32", [3], [1, 2, 3], [("*", 10)], [10, 20, 30])
inplace("scalar_mul_negative", "104-111", "i32", [3], [1, 2, 3], [("*", -5)], [-5, -10, -15])
# ---- in-place through slices (127-255) ----
case("scalar_add_after_slice", "127-143", "i32", {"x": T([2, 3], [1, 2, 3, 4, 5, 6])},
     [["s", "slice", "x", 0, IDX(1)], ["s", "iadd_scalar", "s", 100]],
     [{"t": "s", "shape": [3]}, {"t": "x", "values": [1, 2, 3, 104, 105, 106]}])
case("scalar_mul_after_slice", "170-187", "i32", {"x": T([2, 2, 2], [1, 2, 3, 4, 5, 6, 7, 8])},
     [["s", "slice", "x", 0, IDX(0)], ["s", "imul_scalar", "s", 10]],
     [{"t": "s", "shape": [2, 2]}, {"t": "x", "values": [10, 20, 30, 40, 5, 6, 7, 8]}])
case("scalar_mul_after_column_slice", "200-216", "i32", {"x": T([2, 3], [1, 2, 3, 4, 5, 6])},
     [["s", "slice", "x", 1, IDX(1)], ["s", "imul_scalar", "s", 3]],
     [{"t": "s", "shape": [2], "contiguous": False}, {"t": "x", "values": [1, 6, 3, 4, 15, 6]}])
case("scalar_add_ref_after_slice_chain", "230-255", "i32", {"x": T([2, 2, 2], [1, 2, 3, 4, 5, 6, 7, 8])},
     [["d", "slice", "x", 0, IDX(1)], ["r", "slice", "d", 0, IDX(0)], ["r", "iadd_scalar", "r", 1000]],
     [{"t": "d", "shape": [2, 2]}, {"t": "r", "shape": [2]}, {"t": "x", "values": [1, 2, 3, 4, 1005, 1006, 7, 8]}])
# ---- value-returning scalar ops (257-440, 443-600) ----
def notinplace(name, ref, dtype, shape, values, prog_view, op, v, want_shape, want):
    prog = list(prog_view) + [["r", {"+": "add_scalar", "-": "sub_scalar", "*": "mul_scalar"}[op], prog_view[-1][0] if prog_view else "x", v]]
    case(name, ref, dtype, {"x": T(shape, values)}, prog,
         [{"t": "r", "shape": want_shape, "values": want, "contiguous": True}, {"t": "x", "shape": shape, "values": values}])
notinplace("scalar_add_not_inplace_with_slice", "324-337", "i32", [2, 3], [1, 2, 3, 4, 5, 6], [["s", "slice", "x", 0, IDX(1)]], "+", 100, [3], [104, 105, 106])
notinplace("scalar_mul_not_inplace_noncontiguous_slice", "340-357", "i32", [2, 3], [1, 2, 3, 4, 5, 6], [["s", "slice", "x", 1, IDX(1)]], "*", 3, [2], [6, 15])
notinplace("scalar_add_not_inplace_negative", "375-382", "i32", [3], [10, 20, 30], [], "+", -5, [3], [5, 15, 25])
notinplace("scalar_mul_not_inplace_negative", "385-392", "i32", [3], [1, 2, 3], [], "*", -5, [3], [-5, -10, -15])
notinplace("scalar_add_not_inplace_chained_slices", "395-410", "i32", [2, 2, 2], [1, 2, 3, 4, 5, 6, 7, 8],
           [["d", "slice", "x", 0, IDX(1)], ["s", "slice", "d", 0, IDX(0)]], "+", 1000, [2], [1005, 1006])
notinplace("scalar_mul_not_inplace_matrix", "413-424", "i32", [2, 2], [1, 2, 3, 4], [], "*", 10, [2, 2], [10, 20, 30, 40])
notinplace("scalar_sub_not_inplace_rank0", "427-440", "i32", [], [100], [], "-", 50, [], [50])
notinplace("scalar_add_immutable_view", "443-453", "i32", [4], [1, 2, 3, 4], [], "+", 10, [4], [11, 12, 13, 14])
notinplace("scalar_add_immutable_view_ref", "456-465", "i32", [3], [5, 10, 15], [], "+", 100, [3], [105, 110, 115])
notinplace("scalar_sub_immutable_view", "468-477", "i32", [3], [100, 200, 300], [], "-", 50, [3], [50, 150, 250])
notinplace("scalar_sub_immutable_view_with_slice", "480-491", "i32", [2, 3], [10, 20, 30, 40, 50, 60], [["s", "slice", "x", 0, IDX(0)]], "-", 5, [3], [5, 15, 25])
notinplace("scalar_mul_immutable_view", "494-503", "i32", [4], [2, 4, 6, 8], [], "*", 3, [4], [6, 12, 18, 24])
notinplace("scalar_mul_immutable_view_matrix", "506-515", "i32", [2, 3], [1, 2, 3, 4, 5, 6], [], "*", 10, [2, 3], [10, 20, 30, 40, 50, 60])
notinplace("scalar_sub_immutable_view_rank0", "531-541", "i32", [], [999], [], "-", 99, [], [900])
notinplace("scalar_mul_immutable_view_noncontiguous_slice", "544-555", "i32", [2, 3], [1, 2, 3, 4, 5, 6], [["s", "slice", "x", 1, IDX(1)]], "*", 5, [2], [10, 25])
notinplace("scalar_sub_immutable_view_negative", "574-582", "i32", [3], [-10, -20, -30], [], "-", 5, [3], [-15, -25, -35])
notinplace("scalar_mul_immutable_view_with_ref", "585-600", "i32", [3], [7, 14, 21], [], "*", 2, [3], [14, 28, 42])
# ---- rank-0 and single-element tensors (603-683) ----
inplace("rank0_add", "603-609", "i32", [], [42], [("+", 10)], [52])
inplace("rank0_mul", "612-617", "i32", [], [7], [("*", 6)], [42])
inplace("rank0_sub", "620-625", "i32", [], [100], [("-", 58)], [42])
inplace("rank0_negative_value", "628-634", "i32", [], [-10], [("*", -3), ("+", 5)], [35])
inplace("rank0_zero_operations", "637-644", "i32", [], [0], [("+", 42), ("*", 0), ("+", 10)], [10])
notinplace("rank0_non_inplace", "647-655", "i32", [], [100], [], "+", 50, [], [150])
inplace("single_element_1d", "658-664", "i32", [1], [5], [("+", 10), ("*", 2)], [30])
inplace("single_element_2d", "667-672", "i32", [1, 1], [8], [("*", 5)], [40])
inplace("single_element_3d", "675-683", "i32", [1, 1, 1], [3], [("+", 7), ("*", 3)], [30])
# ---- matrix shapes (686-790) ----
inplace("tall_matrix", "686-691", "i32", [9, 1], list(range(1, 10)), [("*", 2)], [2 * v for v in range(1, 10)])
inplace("wide_matrix", "694-699", "i32", [1, 9], list(range(1, 10)), [("+", 10)], list(range(11, 20)))
inplace("rectangular_2x5", "702-713", "i32", [2, 5], list(range(1, 11)), [("*", 3)], [3 * v for v in range(1, 11)])
inplace("rectangular_5x2", "716-727", "i32", [5, 2], list(range(1, 11)), [("-", 1)], list(range(0, 10)))
inplace("rectangular_3d", "730-738", "i32", [2, 3, 4], list(range(1, 25)), [("+", 100)], list(range(101, 125)))
case("non_square_slice", "741-757", "i32", {"x": T([3, 4], list(range(1, 13)))},
     [["s", "slice", "x", 0, IDX(1)], ["s", "imul_scalar", "s", 10]],
     [{"t": "x", "values": [1, 2, 3, 4, 50, 60, 70, 80, 9, 10, 11, 12]}])
inplace("zero_tensor", "760-766", "i32", [4], [0, 0, 0, 0], [("+", 10), ("*", 2)], [20, 20, 20, 20])
inplace("resulting_in_zero", "769-774", "i32", [4], [5, 10, 15, 20], [("*", 0)], [0, 0, 0, 0])
inplace("mixed_positive_negative", "777-790", "i32", [6], [-5, 10, -15, 20, -25, 30], [("*", 2), ("+", 10)], [0, 30, -20, 50, -40, 70])
# ---- dtype coverage (793-880) ----
inplace("large_values_i32", "793-807", "i32", [3], [1000000, 2000000, 3000000], [("+", 500000)], [1500000, 2500000, 3500000])
inplace("f32_operations", "810-823", "f32", [4], [1.5, 2.5, 3.5, 4.5], [("*", 2.0), ("+", 1.0)], [4.0, 6.0, 8.0, 10.0], tol=1e-6)
inplace("f64_operations", "826-839", "f64", [4], [1.0, 2.0, 3.0, 4.0], [("+", 0.5), ("*", 2.0)], [3.0, 5.0, 7.0, 9.0], tol=1e-10)
inplace("i64_operations", "842-852", "i64", [4], [100, 200, 300, 400], [("-", 50), ("*", 3)], [150, 450, 750, 1050])
inplace("u32_operations", "855-865", "u32", [4], [10, 20, 30, 40], [("+", 5), ("*", 2)], [30, 50, 70, 90])
inplace("i16_operations", "868-880", "i16", [2, 3], [1, 2, 3, 4, 5, 6], [("*", 10), ("+", 5)], [15, 25, 35, 45, 55, 65])
# ---- non-contiguous and N-d (883-1017) ----
case("multiple_noncontiguous_operations", "883-900", "i32", {"x": T([4, 3], list(range(1, 13)))},
     [["c", "slice", "x", 1, IDX(1)], ["c", "iadd_scalar", "c", 100], ["c", "imul_scalar", "c", 2]],
     [{"t": "x", "values": [1, 204, 3, 4, 210, 6, 7, 216, 9, 10, 222, 12]}])
w = list(range(1, 25))
for i in (5, 6, 7, 8, 17, 18, 19, 20): w[i - 1] += 100
case("noncontiguous_slice_3d", "922-951", "i32", {"x": T([2, 3, 4], list(range(1, 25)))},
     [["s", "slice", "x", 1, IDX(1)], ["s", "iadd_scalar", "s", 100]],
     [{"t": "s", "shape": [2, 4], "strides": [12, 1], "offset": 4, "contiguous": False}, {"t": "x", "values": w}])
case("noncontiguous_slice_3d_view", "954-975", "i32", {"x": T([2, 3, 4], list(range(1, 25)))},
     [["s", "slice", "x", 1, IDX(1)]],
     [{"t": "s", "shape": [2, 4], "values": [5, 6, 7, 8, 17, 18, 19, 20]}])
inplace("tensor_4d", "978-986", "i32", [2, 2, 2, 2], list(range(1, 17)), [("+", 10)], list(range(11, 27)))
w = list(range(1, 25))
for i in range(12, 24): w[i] *= 10
case("slice_4d", "989-1003", "i32", {"x": T([2, 3, 2, 2], list(range(1, 25)))},
     [["s", "slice", "x", 0, IDX(1)], ["s", "imul_scalar", "s", 10]], [{"t": "x", "values": w}])
inplace("tensor_5d", "1006-1017", "i32", [2, 2, 2, 2, 2], list(range(1, 33)), [("*", 2), ("+", 5)], [2 * v + 5 for v in range(1, 33)])
inplace("long_operation_chain", "1020-1036", "i32", [4], [1, 2, 3, 4],
        [("+", 1), ("*", 2), ("-", 1), ("*", 3), ("+", 10), ("-", 5), ("*", 2), ("+", 2), ("-", 10), ("*", 1)], [20, 32, 44, 56])
case("alternating_inplace_noninplace", "1039-1060", "i32", {"x": T([3], [5, 10, 15])},
     [["x", "iadd_scalar", "x", 5], ["r1", "mul_scalar", "x", 2], ["x", "imul_scalar", "x", 3], ["r2", "add_scalar", "x", 10]],
     [{"t": "r1", "values": [20, 30, 40]}, {"t": "r2", "values": [40, 55, 70]}, {"t": "x", "values": [30, 45, 60]}])
case("multiple_views_different_ops", "1063-1090", "i32", {"x": T([2, 3], [1, 2, 3, 4, 5, 6])},
     [["r1", "slice", "x", 0, IDX(0)], ["r1", "iadd_scalar", "r1", 10], ["r2", "slice", "x", 0, IDX(1)], ["r2", "imul_scalar", "r2", 5]],
     [{"t": "x", "values": [11, 12, 13, 20, 25, 30]}])
inplace("f32_small_values", "1093-1105", "f32", [3], [0.0001, 0.0002, 0.0003], [("*", 1000.0)], [0.1, 0.2, 0.3], tol=1e-6)
inplace("f64_precision", "1108-1122", "f64", [3], [1.0 / 3.0, 2.0 / 3.0, 1.0], [("*", 3.0)], [1.0, 2.0, 3.0], tol=1e-10)
inplace("very_imbalanced_1000x2", "1125-1136", "i32", [1000, 2], list(range(1, 2001)), [("+", 5)], list(range(6, 2006)))
inplace("very_imbalanced_2x1000", "1139-1150", "i32", [2, 1000], list(range(1, 2001)), [("*", 2)], [2 * v for v in range(1, 2001)])

# ---- broadcasting of `ones` tensors: shapes and values (1564-1926) ----
def bshape(name, ref, sa, sb, out, full=True):
    n = 1
    for d in out: n *= d
    e = {"t": "c", "shape": out}
    if full: e["values"] = [2.0] * n
    case(name, ref, "f32", {"a": ones(sa), "b": ones(sb)}, [["c", "add", "a", "b"]], [e])
bshape("broadcast_identity", "1564-1577", [3, 4, 5], [3, 4, 5], [3, 4, 5])
bshape("broadcast_alternating_singletons", "1581-1590", [1, 4, 1, 6], [3, 1, 5, 1], [3, 4, 5, 6])
bshape("broadcast_trailing_singleton", "1593-1607", [3, 4, 1], [3, 4, 5], [3, 4, 5])
bshape("broadcast_leading_singleton", "1610-1624", [1, 4, 5], [3, 4, 5], [3, 4, 5])
bshape("broadcast_shape_2d_plus_3d", "1629-1637", [4, 5], [3, 4, 5], [3, 4, 5])
bshape("broadcast_shape_1d_plus_4d", "1640-1648", [7], [2, 3, 4, 7], [2, 3, 4, 7])
bshape("broadcast_shape_singleton_expansion", "1651-1659", [1, 5, 1], [4, 5, 6], [4, 5, 6])
bshape("broadcast_shape_prepending", "1662-1670", [5, 6], [2, 3, 4, 5, 6], [2, 3, 4, 5, 6])
bshape("broadcast_shape_both_expand", "1673-1681", [1, 4, 1, 6], [3, 1, 5, 6], [3, 4, 5, 6])
n = 2 * 3 * 4 * 5 * 6
case("broadcast_shape_scalar_expansion", "1684-1692", "f32", {"a": T([], [42.0]), "b": ones([2, 3, 4, 5, 6])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [2, 3, 4, 5, 6], "values": [43.0] * n}])
bshape("broadcast_shape_complex_5d", "1695-1703", [1, 1, 3, 1, 5], [2, 4, 3, 6, 5], [2, 4, 3, 6, 5])
case("broadcast_both_singletons_2d_pattern1", "1710-1727", "f32", {"a": T([1, 4], [5., 6., 1., 1.]), "b": ones([3, 1])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [3, 4], "values": [6., 7., 2., 2.] * 3}])
case("broadcast_both_singletons_2d_pattern2", "1730-1747", "f32", {"a": T([4, 1], [10., 20., 1., 1.]), "b": ones([1, 5])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [4, 5], "values": [11.] * 5 + [21.] * 5 + [2.] * 10}])
bshape("broadcast_both_singletons_3d_complementary", "1750-1765", [1, 3, 1], [2, 1, 4], [2, 3, 4])
a = [1.0] * 20; a[0] = 100.0
b = [1.0] * 15; b[0] = 200.0
case("broadcast_both_singletons_3d_alternating", "1768-1787", "f32", {"a": T([1, 4, 5], a), "b": T([3, 1, 5], b)}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [3, 4, 5], "get": [[[0, 0, 0], 300.0], [[1, 0, 0], 101.0], [[2, 0, 0], 101.0], [[0, 1, 0], 201.0], [[0, 2, 0], 201.0]]}])
bshape("broadcast_both_singletons_3d_partial_overlap", "1790-1806", [5, 1, 3], [1, 4, 3], [5, 4, 3])
bshape("broadcast_both_singletons_4d_zigzag", "1809-1820", [1, 3, 1, 5], [2, 1, 4, 1], [2, 3, 4, 5])
bshape("broadcast_both_singletons_4d_complex", "1823-1834", [1, 1, 6, 7], [5, 4, 1, 1], [5, 4, 6, 7])
bshape("broadcast_both_singletons_5d_checkerboard", "1837-1848", [1, 2, 1, 3, 1], [4, 1, 5, 1, 6], [4, 2, 5, 3, 6])
bshape("broadcast_both_singletons_5d_all_different", "1851-1863", [1, 3, 1, 1, 7], [2, 1, 4, 5, 1], [2, 3, 4, 5, 7])
bshape("broadcast_both_singletons_mixed_ranks", "1866-1881", [1, 5], [3, 1, 1], [3, 1, 5])
def bad(name, ref, sa, sb):
    case(name, ref, "f32", {"a": ones(sa), "b": ones(sb)}, [["c", "add", "a", "b"]], [{"error": "BroadcastError"}])
bad("broadcast_both_singletons_incompatible_2d", "1886-1894", [3, 4], [5, 1])
bad("broadcast_both_singletons_incompatible_3d", "1897-1905", [2, 1, 4], [1, 3, 5])
bad("broadcast_both_singletons_incompatible_4d", "1908-1916", [1, 3, 1, 6], [2, 1, 4, 7])
bad("broadcast_both_singletons_incompatible_middle", "1919-1927", [2, 4, 1], [3, 1, 5])
json.dump({"_comment": "Known-answer vectors transcribed from the reference's own #[test]s (scalar operators on tensors and views, dtype coverage, N-d shapes, "
                       "mutual broadcasting of singleton dims); `ref` = file:lines under libs/rtensors/src/.  Program format: tests/golden_dsl.py.",
           "cases": cases}, open("tests/golden/reference_scalar_vectors.json", "w"), indent=None, separators=(",", ":"))
print(len(cases), "cases")
