# appends slice / fill / owned cases to tests/golden/reference_view_vectors.json (hand-transcribed, core/mod.rs)
import json
path = "tests/golden/reference_view_vectors.json"
doc = json.load(open(path))
cases = [c for c in doc["cases"] if not c["name"].startswith(("fill_", "owned_", "slice_", "step_"))]
def case(name, ref, inputs, program, expect, dtype="i32"):
    cases.append({"name": name, "ref": "core/mod.rs:" + ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
def T(shape, values): return {"shape": shape, "values": values}
def IDX(i): return {"range": [i, i]}
def G(*pairs): return [[list(i) if isinstance(i, tuple) else [i], v] for i, v in pairs]
r = lambda a, b: list(range(a, b + 1))
S = lambda a, b, st: {"slice": [a, b, st]}

case("fill_contiguous", "1176-1186", {"a": T([3, 4], r(0, 11))}, [["a", "fill", "a", 42]], [{"t": "a", "values": [42] * 12}])
case("fill_contiguous_slice", "1189-1211", {"a": T([3, 4], r(0, 11))}, [["s", "slice", "a", 0, {"index": 1}], ["s", "fill", "s", 99]],
     [{"t": "a", "values": [0, 1, 2, 3, 99, 99, 99, 99, 8, 9, 10, 11]}])
case("fill_strided_column", "1214-1228", {"a": T([3, 4], r(0, 11))}, [["s", "slice", "a", 1, {"index": 2}], ["s", "fill", "s", 7]],
     [{"t": "a", "values": [0, 1, 7, 3, 4, 5, 7, 7, 8, 9, 7, 11]}])
w = r(0, 23)
for i in (1, 2):
    for j in (2, 3, 4): w[i * 6 + j] = 5
case("fill_2d_slice", "1231-1254", {"a": T([4, 6], r(0, 23))},
     [["s", "slice", "a", 0, {"range": [1, 3]}], ["s2", "slice", "s", 1, {"range": [2, 5]}], ["s2", "fill", "s2", 5]],
     [{"t": "s2", "shape": [2, 3]}, {"t": "a", "values": w, "get": G(((1, 2), 5), ((2, 4), 5), ((0, 2), 2), ((1, 1), 7), ((1, 5), 11), ((3, 2), 20))}])
case("owned_of_contiguous_view", "1486-1496", {"a": T([2, 3], r(1, 6))}, [["o", "owned", "a"]],
     [{"t": "o", "shape": [2, 3], "values": r(1, 6), "contiguous": True}])
case("owned_of_noncontiguous_column", "1499-1518", {"a": T([2, 3], r(1, 6))}, [["c", "slice", "a", 1, IDX(1)], ["o", "owned", "c"]],
     [{"t": "c", "shape": [2], "contiguous": False}, {"t": "o", "shape": [2], "values": [2, 5], "contiguous": True, "offset": 0, "strides": [1]}])
case("owned_of_row_slice", "1521-1533", {"a": T([2, 3], r(1, 6))}, [["s", "slice", "a", 0, IDX(1)], ["o", "owned", "s"]],
     [{"t": "s", "contiguous": True}, {"t": "o", "shape": [3], "values": [4, 5, 6], "offset": 0}])
case("owned_of_3d_slice", "1550-1561", {"a": T([2, 2, 2], r(1, 8))}, [["s", "slice", "a", 0, IDX(1)], ["o", "owned", "s"]],
     [{"t": "o", "shape": [2, 2], "values": [5, 6, 7, 8], "contiguous": True, "offset": 0}])
case("slice_matrix_column_with_mutation", "1914-1943", {"a": T([3, 4], r(1, 12))},
     [["s", "slice", "a", 1, {"range": [2, 3]}], ["s", "set", "s", [0, 0], 33], ["s", "set", "s", [2, 0], 111]],
     [{"t": "s", "shape": [3, 1]}, {"t": "a", "values": [1, 2, 33, 4, 5, 6, 7, 8, 9, 10, 111, 12]}])
case("slice_3d_depth_inclusive_with_mutation", "1946-1983", {"a": T([3, 2, 2], r(1, 12))},
     [["s", "slice", "a", 0, {"range_inclusive": [1, 1]}], ["s", "set", "s", [0, 0, 0], 55], ["s", "set", "s", [0, 1, 1], 88]],
     [{"t": "s", "shape": [1, 2, 2]}, {"t": "a", "values": [1, 2, 3, 4, 55, 6, 7, 88, 9, 10, 11, 12]}])
w = r(1, 24); w[1 * 6 + 3] = 999; w[2 * 6 + 4] = 1717
case("slice_chained_with_mutation", "1986-2021", {"a": T([4, 6], r(1, 24))},
     [["s1", "slice", "a", 0, {"range": [1, 3]}], ["s2", "slice", "s1", 1, {"range_inclusive": [2, 4]}], ["s2", "set", "s2", [0, 1], 999],
      ["s2", "set", "s2", [1, 2], 1717]],
     [{"t": "s1", "shape": [2, 6]}, {"t": "s2", "shape": [2, 3]}, {"t": "a", "values": w}])
case("step_2_with_mutation", "2024-2053", {"a": T([10], r(1, 10))},
     [["s", "slice", "a", 0, S(1, 9, 2)], ["s", "set", "s", [0], 22], ["s", "set", "s", [3], 88]],
     [{"t": "s", "shape": [4]}, {"t": "a", "values": [1, 22, 3, 4, 5, 6, 7, 88, 9, 10]}])
case("step_custom_positive", "609-650", {"a": T([16], r(0, 15))},
     [["s1", "slice", "a", 0, S(None, None, 2)], ["s2", "slice", "a", 0, S(1, 8, 3)], ["s3", "slice", "a", 0, S(None, 12, 4)],
      ["s4", "slice", "a", 0, S(3, None, 5)], ["s5", "slice", "a", 0, S(2, None, 10)]],
     [{"t": "s1", "shape": [8], "values": [0, 2, 4, 6, 8, 10, 12, 14]}, {"t": "s2", "shape": [3], "values": [1, 4, 7]},
      {"t": "s3", "shape": [3], "values": [0, 4, 8]}, {"t": "s4", "shape": [3], "values": [3, 8, 13]}, {"t": "s5", "shape": [2], "values": [2, 12]}])
case("step_custom_negative", "653-689", {"a": T([16], r(0, 15))},
     [["s1", "slice", "a", 0, S(None, None, -2)], ["s2", "slice", "a", 0, S(10, 1, -3)], ["s3", "slice", "a", 0, S(None, 2, -4)],
      ["s4", "slice", "a", 0, S(14, None, -5)]],
     [{"t": "s1", "shape": [8], "values": [15, 13, 11, 9, 7, 5, 3, 1]}, {"t": "s2", "shape": [3], "values": [10, 7, 4]},
      {"t": "s3", "shape": [4], "values": [15, 11, 7, 3]}, {"t": "s4", "shape": [3], "values": [14, 9, 4]}])
w = r(0, 15); w[0] = 100; w[2] = 102; w[14] = 114
case("step_custom_positive_mut", "692-716", {"a": T([16], r(0, 15))},
     [["s", "slice", "a", 0, S(None, None, 2)], ["s", "set", "s", [0], 100], ["s", "set", "s", [1], 102], ["s", "set", "s", [7], 114]],
     [{"t": "s", "shape": [8]}, {"t": "a", "values": w}])
w = r(0, 15); w[1] = 101; w[4] = 104; w[7] = 107
case("step_custom_positive_mut_with_range", "719-741", {"a": T([16], r(0, 15))},
     [["s", "slice", "a", 0, S(1, 10, 3)], ["s", "set", "s", [0], 101], ["s", "set", "s", [1], 104], ["s", "set", "s", [2], 107]],
     [{"t": "s", "shape": [3]}, {"t": "a", "values": w}])
w = r(0, 15); w[15] = 115; w[13] = 113; w[1] = 101
case("step_custom_negative_mut", "744-766", {"a": T([16], r(0, 15))},
     [["s", "slice", "a", 0, S(None, None, -2)], ["s", "set", "s", [0], 115], ["s", "set", "s", [1], 113], ["s", "set", "s", [7], 101]],
     [{"t": "s", "shape": [8]}, {"t": "a", "values": w}])
w = r(0, 15); w[12] = 212; w[9] = 209; w[6] = 206
case("step_custom_negative_mut_with_range", "769-791", {"a": T([16], r(0, 15))},
     [["s", "slice", "a", 0, S(12, 3, -3)], ["s", "set", "s", [0], 212], ["s", "set", "s", [1], 209], ["s", "set", "s", [2], 206]],
     [{"t": "s", "shape": [3]}, {"t": "a", "values": w}])
doc["cases"] = cases
doc["_comment"] = ("Known-answer vectors transcribed from the reference's own #[test]s on views (transpose, permute, unsqueeze, squeeze, slices with custom "
                   "steps, fill, owned, writes through views); `ref` = file:lines under libs/rtensors/src/.  Program format: tests/golden_dsl.py.")
json.dump(doc, open(path, "w"), separators=(",", ":"))
print(len(cases), "cases")
