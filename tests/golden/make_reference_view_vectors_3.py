# appends the slice-syntax / negative-step cases to tests/golden/reference_view_vectors.json (hand-transcribed, core/mod.rs)
import json
path = "tests/golden/reference_view_vectors.json"
doc = json.load(open(path))
cases = [c for c in doc["cases"] if not c["name"].startswith(("syntax_", "negstep_"))]
def case(name, ref, inputs, program, expect, dtype="i32"):
    cases.append({"name": name, "ref": "core/mod.rs:" + ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
def T(shape, values): return {"shape": shape, "values": values}
def G(*pairs): return [[list(i) if isinstance(i, tuple) else [i], v] for i, v in pairs]
S = lambda a, b, st: {"slice": [a, b, st]}
def sets(name, *pairs): return [[name, "set", name, [i] if not isinstance(i, tuple) else list(i), v] for i, v in pairs]
t10 = lambda n: [10 * (i + 1) for i in range(n)]

for nm, ref, spec in (("negstep_mut_full", "525-541", S(None, None, -1)), ("negstep_mut_from_range_full", "544-560", S(None, None, -1))):
    case(nm, ref, {"a": T([6], [1, 2, 3, 4, 5, 6])}, [["s", "slice", "a", 0, spec]] + sets("s", (0, 60), (5, 10)),
         [{"t": "a", "get": G((0, 10), (5, 60))}])
case("negstep_error_start_out_of_bounds", "563-571", {"a": T([6], [1, 2, 3, 4, 5, 6])}, [["s", "slice", "a", 0, S(10, 2, -1)]], [{"error": "IdxOutOfBounds"}])
case("negstep_error_end_out_of_bounds", "573-577", {"a": T([6], [1, 2, 3, 4, 5, 6])}, [["s", "slice", "a", 0, S(5, 10, -1)]], [{"error": "IdxOutOfBounds"}])
case("negstep_error_zero_step", "579-583", {"a": T([6], [1, 2, 3, 4, 5, 6])}, [["s", "slice", "a", 0, S(2, 5, 0)]], [{"error": "InvalidShape"}])
case("negstep_reverse_range_auto", "586-606", {"a": T([10], list(range(1, 11)))},
     [["s", "slice", "a", 0, {"range": [9, 0]}], ["u", "slice", "a", 0, {"range_inclusive": [9, 0]}]],
     [{"t": "s", "shape": [9], "get": G((0, 10), (1, 9), (8, 2))}, {"t": "u", "shape": [10], "get": G((0, 10), (9, 1))}])
case("syntax_range_to", "1585-1614", {"a": T([8], t10(8))},
     [["s", "slice", "a", 0, S(None, 5, 1)], ["o", "owned", "s"]] + sets("s", (0, 11), (2, 33), (4, 55)),
     [{"t": "s", "shape": [5]}, {"t": "o", "values": [10, 20, 30, 40, 50]}, {"t": "a", "get": G((0, 11), (2, 33), (4, 55), (5, 60))}])
case("syntax_range_from", "1617-1643", {"a": T([8], t10(8))},
     [["s", "slice", "a", 0, S(2, None, 1)], ["o", "owned", "s"]] + sets("s", (0, 333), (5, 888)),
     [{"t": "s", "shape": [6]}, {"t": "o", "get": G((0, 30), (1, 40), (5, 80))}, {"t": "a", "get": G((2, 333), (7, 888), (0, 10), (1, 20))}])
case("syntax_range_full", "1646-1671", {"a": T([4], t10(4))},
     [["s", "slice", "a", 0, S(None, None, 1)], ["o", "owned", "s"]] + sets("s", (0, 100), (3, 400)),
     [{"t": "s", "shape": [4]}, {"t": "o", "values": [10, 20, 30, 40]}, {"t": "a", "get": G((0, 100), (3, 400))}])
case("syntax_inclusive_range", "1674-1701", {"a": T([8], t10(8))},
     [["s", "slice", "a", 0, {"range_inclusive": [2, 5]}], ["o", "owned", "s"]] + sets("s", (0, 333), (3, 666)),
     [{"t": "s", "shape": [4]}, {"t": "o", "values": [30, 40, 50, 60]}, {"t": "a", "get": G((2, 333), (5, 666), (1, 20), (6, 70))}])
case("syntax_inclusive_range_zero_start", "1704-1726", {"a": T([5], t10(5))},
     [["s", "slice", "a", 0, {"range_inclusive": [0, 2]}], ["o", "owned", "s"]] + sets("s", (1, 222)),
     [{"t": "s", "shape": [3]}, {"t": "o", "values": [10, 20, 30]}, {"t": "a", "get": G((1, 222))}])
case("syntax_single_index", "1729-1754", {"a": T([2, 3], t10(6))},
     [["s", "slice", "a", 1, {"index": 1}], ["o", "owned", "s"]] + sets("s", (0, 222), (1, 555)),
     [{"t": "s", "shape": [2]}, {"t": "o", "values": [20, 50]}, {"t": "a", "get": G(((0, 1), 222), ((1, 1), 555), ((0, 0), 10), ((0, 2), 30))}])
case("syntax_reverse_range_exclusive", "1757-1783", {"a": T([8], t10(8))},
     [["s", "slice", "a", 0, {"range": [5, 2]}], ["o", "owned", "s"]] + sets("s", (0, 666), (2, 444)),
     [{"t": "s", "shape": [3]}, {"t": "o", "values": [60, 50, 40]}, {"t": "a", "get": G((5, 666), (3, 444), (2, 30), (6, 70))}])
case("syntax_from_with_negative_step", "1786-1811", {"a": T([10], t10(10))},
     [["s", "slice", "a", 0, S(8, None, -1)], ["o", "owned", "s"]] + sets("s", (0, 999), (8, 111)),
     [{"t": "s", "shape": [9]}, {"t": "o", "get": G((0, 90), (1, 80), (8, 10))}, {"t": "a", "get": G((8, 999), (0, 111), (9, 100))}])
case("syntax_to_with_negative_step", "1814-1841", {"a": T([8], t10(8))},
     [["s", "slice", "a", 0, S(None, 5, -1)], ["o", "owned", "s"]] + sets("s", (0, 888), (1, 777)),
     [{"t": "s", "shape": [2]}, {"t": "o", "values": [80, 70]}, {"t": "a", "get": G((7, 888), (6, 777), (5, 60), (4, 50))}])
case("syntax_reverse_first_n", "1844-1871", {"a": T([8], t10(8))},
     [["s", "slice", "a", 0, S(4, None, -1)], ["o", "owned", "s"]] + sets("s", (0, 555), (4, 111)),
     [{"t": "s", "shape": [5]}, {"t": "o", "values": [50, 40, 30, 20, 10]}, {"t": "a", "get": G((4, 555), (0, 111))}])
case("syntax_manual_negative_step_2", "1874-1899", {"a": T([10], t10(10))},
     [["s", "slice", "a", 0, S(8, 2, -2)], ["o", "owned", "s"]] + sets("s", (0, 999), (2, 555)),
     [{"t": "s", "shape": [3]}, {"t": "o", "values": [90, 70, 50]}, {"t": "a", "get": G((8, 999), (4, 555), (6, 70))}])
case("syntax_same_indices_collapse", "1902-1910", {"a": T([6], t10(6))}, [["s", "slice", "a", 0, {"range": [5, 5]}]], [{"t": "s", "shape": []}])
doc["cases"] = cases
json.dump(doc, open(path, "w"), separators=(",", ":"))
print(len(cases))

# ---- second batch: basic indexing, chained index slices, writes through chained / transposed mutable views
doc = json.load(open(path))
cases = [c for c in doc["cases"] if not c["name"].startswith("basic_")]
cube = [1, 2, 4, 5, 6, 7, 8, 9]
IDX = lambda i: {"range": [i, i]}
case("basic_slice_of_slice_cube", "794-817", {"a": T([2, 2, 2], cube)},
     [["s", "slice", "a", 0, IDX(1)], ["s2", "slice", "s", 1, IDX(0)], ["s3", "slice", "s2", 0, IDX(1)]],
     [{"t": "s", "shape": [2, 2], "get": G(((0, 0), 6), ((0, 1), 7), ((1, 0), 8), ((1, 1), 9))},
      {"t": "s2", "shape": [2], "get": G((0, 6), (1, 8))}, {"t": "s3", "shape": [], "get": [[[], 8]]}])
case("basic_mut_slices", "820-836", {"a": T([2, 3], [1, 2, 3, 4, 5, 6])},
     [["s", "slice", "a", 0, IDX(1)], ["o", "owned", "s"]] + sets("s", (1, 50)),
     [{"t": "s", "shape": [3], "get": G((1, 50))}, {"t": "o", "values": [4, 5, 6]}, {"t": "a", "get": G(((1, 1), 50))}])
case("basic_scalar", "859-867", {"a": T([], [42])}, [], [{"t": "a", "shape": [], "get": [[[], 42]]}])
case("basic_array", "870-881", {"a": T([3], [1, 2, 3])}, [["o", "owned", "a"]] + sets("a", (1, 1)),
     [{"t": "o", "values": [1, 2, 3]}, {"t": "a", "get": G((1, 1))}])
case("basic_matrix", "884-898", {"a": T([2, 3], [1, 2, 3, 4, 5, 6])}, [["o", "owned", "a"]] + sets("a", ((1, 2), 100)),
     [{"t": "o", "get": G(((0, 0), 1), ((0, 1), 2), ((0, 2), 3), ((1, 0), 4), ((1, 1), 5), ((1, 2), 6))}, {"t": "a", "get": G(((1, 2), 100))}])
case("basic_cube", "901-924", {"a": T([2, 2, 2], cube)}, [["o", "owned", "a"]] + sets("a", ((1, 0, 0), 67)),
     [{"t": "o", "get": G(((0, 0, 0), 1), ((0, 0, 1), 2), ((0, 1, 0), 4), ((0, 1, 1), 5), ((1, 0, 0), 6), ((1, 0, 1), 7), ((1, 1, 0), 8), ((1, 1, 1), 9))},
      {"t": "a", "get": G(((1, 0, 0), 67))}])
case("basic_slice_single_dim_to_scalar", "1318-1326", {"a": T([1], [42])}, [["s", "slice", "a", 0, IDX(0)]], [{"t": "s", "shape": [], "get": [[[], 42]]}])
case("basic_cube_slice_mut_chain", "1329-1346", {"a": T([2, 2, 2], cube)},
     [["d", "slice", "a", 0, IDX(1)], ["r", "slice", "d", 0, IDX(1)]] + sets("r", (0, 800)),
     [{"t": "d", "shape": [2, 2]}, {"t": "r", "shape": [2]}, {"t": "a", "get": G(((1, 1, 0), 800), ((1, 1, 1), 9))}])
case("basic_viewmut_to_owned", "1564-1572", {"a": T([2, 3], [1, 2, 3, 4, 5, 6])}, [["o", "owned", "a"]],
     [{"t": "o", "shape": [2, 3], "values": [1, 2, 3, 4, 5, 6]}])
case("basic_slice_then_transpose_mut", "2437-2462", {"a": T([3, 4], list(range(1, 13)))},
     [["s", "slice", "a", 0, {"range": [0, 2]}], ["t", "transpose", "s"]] + sets("t", ((0, 0), 100), ((3, 1), 800)),
     [{"t": "a", "get": G(((0, 0), 100), ((1, 3), 800), ((2, 0), 9))}])
doc["cases"] = cases
json.dump(doc, open(path, "w"), separators=(",", ":"))
print(len(cases))

# ---- third batch: writes through unsqueezed / squeezed mutable views
doc = json.load(open(path))
cases = [c for c in doc["cases"] if not c["name"].startswith(("unsq_", "sq_"))]
r = lambda a, b: list(range(a, b + 1))
U = lambda d, s, dim: [d, "unsqueeze", s, dim]
REV = S(None, None, -1)
case("unsq_mut_basic", "2620-2633", {"a": T([2, 2], [1, 2, 3, 4])}, [U("u", "a", 0)],
     [{"t": "u", "shape": [1, 2, 2], "strides": [4, 2, 1], "get": G(((0, 0, 0), 1), ((0, 1, 1), 4))}])
case("unsq_mut_with_write", "2641-2665", {"a": T([2, 3], r(1, 6))}, [U("u", "a", 0)] + sets("u", ((0, 0, 0), 100), ((0, 1, 2), 600)),
     [{"t": "u", "shape": [1, 2, 3]}, {"t": "a", "get": G(((0, 0), 100), ((1, 2), 600), ((0, 1), 2), ((1, 0), 4))}])
case("unsq_mut_after_slice", "2668-2694", {"a": T([2, 4], r(1, 8))},
     [["s", "slice", "a", 0, IDX(1)], U("u", "s", 0)] + sets("u", ((0, 0), 500), ((0, 3), 800)),
     [{"t": "s", "shape": [4]}, {"t": "u", "shape": [1, 4]}, {"t": "a", "get": G(((1, 0), 500), ((1, 3), 800), ((0, 0), 1), ((0, 3), 4))}])
case("unsq_scalar_mut", "2697-2717", {"a": T([], [99])}, [U("u", "a", 0), ["o", "owned", "u"]] + sets("u", (0, 77)),
     [{"t": "u", "shape": [1]}, {"t": "o", "values": [99]}, {"t": "a", "get": [[[], 77]]}])
case("unsq_indexing_comprehensive", "2720-2756", {"a": T([3, 4], t10(12))}, [U("u", "a", 0)],
     [{"t": "u", "shape": [1, 3, 4], "strides": [12, 4, 1], "values": t10(12)}, {"t": "a", "get": G(((0, 0), 10), ((1, 2), 70), ((2, 3), 120))}])
case("unsq_3d_indexing", "2759-2791", {"a": T([2, 3, 4], r(1, 24))}, [U("u", "a", 0)],
     [{"t": "u", "shape": [1, 2, 3, 4], "strides": [24, 12, 4, 1],
       "get": G(((0, 0, 0, 0), 1), ((0, 0, 0, 3), 4), ((0, 0, 2, 3), 12), ((0, 1, 0, 0), 13), ((0, 1, 2, 3), 24))}])
case("unsq_at_mut_basic", "2943-2962", {"a": T([2, 3], r(1, 6))}, [U("u", "a", 0)] + sets("u", ((0, 0, 0), 100), ((0, 1, 2), 200)),
     [{"t": "u", "shape": [1, 2, 3]}, {"t": "a", "get": G(((0, 0), 100), ((1, 2), 200))}])
case("unsq_at_mut_middle_dimension", "2965-2983", {"a": T([2, 3], r(1, 6))}, [U("u", "a", 1)] + sets("u", ((0, 0, 1), 10), ((1, 0, 0), 20)),
     [{"t": "u", "shape": [2, 1, 3]}, {"t": "a", "get": G(((0, 1), 10), ((1, 0), 20))}])
case("unsq_at_mut_end_dimension", "2986-3004", {"a": T([2, 2], r(1, 4))}, [U("u", "a", 2)] + sets("u", ((0, 0, 0), 99), ((1, 1, 0), 88)),
     [{"t": "u", "shape": [2, 2, 1]}, {"t": "a", "get": G(((0, 0), 99), ((1, 1), 88))}])
case("unsq_at_mut_chained", "3007-3028", {"a": T([2, 2], r(1, 4))},
     [U("u1", "a", 0), U("u2", "u1", 1)] + sets("u2", ((0, 0, 0, 0), 111), ((0, 0, 1, 1), 222)),
     [{"t": "u1", "shape": [1, 2, 2]}, {"t": "u2", "shape": [1, 1, 2, 2]}, {"t": "a", "get": G(((0, 0), 111), ((1, 1), 222))}])
case("unsq_at_mut_multiple_dims_in_row", "3031-3057", {"a": T([2, 4], r(1, 8))},
     [U("u1", "a", 2)] + sets("u1", ((0, 0, 0), 100)) + [U("u2", "a", 0)] + sets("u2", ((0, 1, 3), 200)) + [U("u3", "a", 1)] + sets("u3", ((1, 0, 2), 300)),
     [{"t": "u1", "shape": [2, 4, 1]}, {"t": "u2", "shape": [1, 2, 4]}, {"t": "u3", "shape": [2, 1, 4]},
      {"t": "a", "get": G(((0, 0), 100), ((1, 3), 200), ((1, 2), 300))}])
case("unsq_at_mut_complex_chaining", "3060-3087", {"a": T([2, 3], r(1, 6))},
     [U("v1", "a", 2)] + sets("v1", ((0, 0, 0), 10)) + [U("v2", "v1", 0)] + sets("v2", ((0, 0, 1, 0), 20)) + [U("v3", "v2", 2)] +
     sets("v3", ((0, 1, 0, 2, 0), 30)),
     [{"t": "v1", "shape": [2, 3, 1]}, {"t": "v2", "shape": [1, 2, 3, 1]}, {"t": "v3", "shape": [1, 2, 1, 3, 1]},
      {"t": "a", "get": G(((0, 0), 10), ((0, 1), 20), ((1, 2), 30))}])
case("unsq_at_mut_alternating_positions", "3090-3121", {"a": T([2, 2], r(1, 4))},
     [U("v1", "a", 2)] + sets("v1", ((0, 0, 0), 100)) + [U("v2", "v1", 0)] + sets("v2", ((0, 0, 1, 0), 200)) + [U("v3", "v2", 1)] +
     sets("v3", ((0, 0, 1, 0, 0), 300)) + [U("v4", "v3", 3)] + sets("v4", ((0, 0, 1, 0, 1, 0), 400)),
     [{"t": "v4", "shape": [1, 1, 2, 1, 2, 1]}, {"t": "a", "get": G(((0, 0), 100), ((0, 1), 200), ((1, 0), 300), ((1, 1), 400))}])
case("unsq_at_preserves_data_access", "3124-3157", {"a": T([3, 4], r(1, 12))}, [U("u0", "a", 0), U("u1", "a", 1), U("u2", "a", 2)],
     [{"t": "u0", "get": G(((0, 0, 0), 1), ((0, 2, 3), 12))}, {"t": "u1", "get": G(((0, 0, 0), 1), ((2, 0, 3), 12))},
      {"t": "u2", "get": G(((0, 0, 0), 1), ((2, 3, 0), 12))}])
case("unsq_at_after_slice", "3160-3177", {"a": T([4, 6], r(1, 24))}, [["s", "slice", "a", 0, {"range": [1, 3]}], U("u", "s", 0)],
     [{"t": "s", "shape": [2, 6]}, {"t": "u", "shape": [1, 2, 6], "get": G(((0, 0, 0), 7), ((0, 0, 5), 12), ((0, 1, 0), 13), ((0, 1, 5), 18))}])
case("unsq_at_after_column_slice", "3180-3196", {"a": T([3, 4], r(1, 12))}, [["s", "slice", "a", 1, {"range": [1, 3]}], U("u", "s", 2)],
     [{"t": "s", "shape": [3, 2]}, {"t": "u", "shape": [3, 2, 1], "get": G(((0, 0, 0), 2), ((0, 1, 0), 3), ((2, 1, 0), 11))}])
case("unsq_at_mut_after_slice", "3248-3272", {"a": T([4, 5], r(1, 20))},
     [["s", "slice", "a", 0, {"range": [1, 3]}], U("u", "s", 0)] + sets("u", ((0, 0, 0), 100), ((0, 1, 4), 200)),
     [{"t": "s", "shape": [2, 5]}, {"t": "u", "shape": [1, 2, 5]}, {"t": "a", "get": G(((1, 0), 100), ((2, 4), 200))}])
case("unsq_at_mut_negative_stride", "3275-3300", {"a": T([6], r(1, 6))},
     [["v", "slice", "a", 0, REV], ["o", "owned", "v"], U("u", "v", 1)] + sets("u", ((0, 0), 100), ((5, 0), 200)),
     [{"t": "v", "strides": [-1]}, {"t": "o", "get": G((0, 6))}, {"t": "u", "shape": [6, 1], "strides": [-1, 1]}, {"t": "a", "get": G((5, 100), (0, 200))}])
case("unsq_at_mut_negative_stride_2d", "3303-3328", {"a": T([3, 4], r(1, 12))},
     [["v1", "slice", "a", 0, REV], ["v2", "slice", "v1", 1, REV], U("u", "v2", 1)] + sets("u", ((0, 0, 0), 999), ((2, 0, 3), 888)),
     [{"t": "v2", "strides": [-4, -1]}, {"t": "u", "shape": [3, 1, 4]}, {"t": "a", "get": G(((2, 3), 999), ((0, 0), 888))}])
case("unsq_at_mut_complex_slice_pattern", "3331-3357", {"a": T([4, 5], r(0, 19))},
     [["s", "slice", "a", 0, S(3, None, -2)], ["o", "owned", "s"], U("u", "s", 2)] + sets("u", ((0, 0, 0), 300), ((1, 4, 0), 400)),
     [{"t": "s", "shape": [2, 5]}, {"t": "o", "get": G(((0, 0), 15), ((1, 0), 5))}, {"t": "u", "shape": [2, 5, 1]},
      {"t": "a", "get": G(((3, 0), 300), ((1, 4), 400))}])
case("unsq_at_mut_multiple_slices_then_unsqueeze", "3360-3387", {"a": T([5, 12], r(1, 60))},
     [["s1", "slice", "a", 0, {"range": [1, 4]}], ["s2", "slice", "s1", 1, {"range": [2, 7]}], U("u", "s2", 1)] +
     sets("u", ((0, 0, 0), 500), ((2, 0, 4), 600)),
     [{"t": "s2", "shape": [3, 5]}, {"t": "u", "shape": [3, 1, 5]}, {"t": "a", "get": G(((1, 2), 500), ((3, 6), 600))}])
case("unsq_at_mut_chained_with_negative_stride", "3390-3417", {"a": T([4, 6], r(1, 24))},
     [["v", "slice", "a", 0, REV], U("u1", "v", 0), U("u2", "u1", 3)] + sets("u2", ((0, 0, 0, 0), 700), ((0, 3, 5, 0), 800)),
     [{"t": "u1", "shape": [1, 4, 6]}, {"t": "u2", "shape": [1, 4, 6, 1]}, {"t": "a", "get": G(((3, 0), 700), ((0, 5), 800))}])
case("unsq_at_preserves_strides_after_slice", "3420-3445", {"a": T([5, 6], r(1, 30))},
     [["s", "slice", "a", 1, S(None, None, 2)], U("u", "s", 1)],
     [{"t": "s", "shape": [5, 3], "strides": [6, 2]},
      {"t": "u", "shape": [5, 1, 3], "strides": [6, 6, 2], "get": G(((0, 0, 0), 1), ((0, 0, 2), 5), ((4, 0, 2), 29))}])
case("unsq_at_out_of_bounds_too_large", "3450-3458", {"a": T([2, 3], r(1, 6))}, [U("u", "a", 4)], [{"error": "InvalidDim"}])
case("unsq_at_out_of_bounds_1d", "3461-3469", {"a": T([4], r(1, 4))}, [U("u", "a", 3)], [{"error": "InvalidDim"}])
case("unsq_at_mut_out_of_bounds", "3472-3480", {"a": T([3, 4], r(1, 12))}, [U("u", "a", 5)], [{"error": "InvalidDim"}])
case("unsq_at_out_of_bounds_after_slice", "3483-3495", {"a": T([4, 6], r(1, 24))}, [["s", "slice", "a", 0, {"range": [1, 3]}], U("u", "s", 4)],
     [{"error": "InvalidDim"}])
case("sq_mut_basic", "3651-3664", {"a": T([1, 3], [1, 2, 3])}, [["q", "squeeze", "a"]] + sets("q", (1, 20)),
     [{"t": "q", "shape": [3], "strides": [1], "get": G((1, 20))}])
case("sq_mut_after_modifications", "3667-3687", {"a": T([1, 2, 3], r(1, 6))},
     [["q", "squeeze", "a"]] + sets("q", ((0, 0), 10), ((0, 2), 30), ((1, 1), 50)),
     [{"t": "q", "shape": [2, 3], "get": G(((0, 0), 10), ((0, 2), 30), ((1, 1), 50), ((0, 1), 2), ((1, 0), 4))}])
case("sq_at_mut_basic", "3690-3703", {"a": T([2, 1, 3], r(1, 6))}, [["q", "squeeze", "a", 1]] + sets("q", ((0, 0), 10), ((1, 2), 60)),
     [{"t": "q", "shape": [2, 3], "get": G(((0, 0), 10), ((1, 2), 60))}])
case("sq_mut_after_slice", "3706-3731", {"a": T([3, 4], r(1, 12))},
     [["s", "slice", "a", 0, IDX(1)], U("u", "s", 0), ["q", "squeeze", "u"]] + sets("q", (0, 50), (3, 80)),
     [{"t": "s", "shape": [4]}, {"t": "u", "shape": [1, 4]}, {"t": "q", "shape": [4], "get": G((0, 50), (3, 80))}])
case("sq_mut_after_column_slice", "3734-3763", {"a": T([3, 3], r(1, 9))},
     [["s", "slice", "a", 1, IDX(1)], ["o", "owned", "s"], U("u", "s", 1), ["q", "squeeze", "u"]] + sets("q", (0, 20), (2, 80)),
     [{"t": "s", "shape": [3]}, {"t": "o", "values": [2, 5, 8]}, {"t": "q", "get": G((0, 20), (1, 5), (2, 80))}])
case("sq_chained_with_slices", "3766-3795", {"a": T([2, 3, 4], r(1, 24))},
     [["s1", "slice", "a", 0, IDX(0)], U("u1", "s1", 1), ["s2", "slice", "u1", 2, IDX(2)], U("u2", "s2", 0), ["q", "squeeze", "u2"]],
     [{"t": "s1", "shape": [3, 4]}, {"t": "u1", "shape": [3, 1, 4]}, {"t": "s2", "shape": [3, 1]}, {"t": "u2", "shape": [1, 3, 1]},
      {"t": "q", "shape": [3], "get": G((0, 3), (1, 7), (2, 11))}])
case("sq_at_non_singleton_dim", "3939-3943", {"a": T([2, 3], r(1, 6))}, [["q", "squeeze", "a", 0]], [{"error": "InvalidDim"}])
case("sq_at_invalid_dim", "3947-3951", {"a": T([1, 3], [1, 2, 3])}, [["q", "squeeze", "a", 5]], [{"error": "InvalidDim"}])
case("sq_at_mut_non_singleton_dim", "3955-3959", {"a": T([2, 3], r(1, 6))}, [["q", "squeeze", "a", 1]], [{"error": "InvalidDim"}])
case("sq_with_non_contiguous_slice", "3973-3999", {"a": T([3, 3], r(1, 9))},
     [["s", "slice", "a", 1, IDX(1)], U("u", "s", 1), ["q", "squeeze", "u"]],
     [{"t": "s", "shape": [3], "contiguous": False}, {"t": "u", "shape": [3, 1]}, {"t": "q", "shape": [3], "values": [2, 5, 8]}])
doc["cases"] = cases
json.dump(doc, open(path, "w"), separators=(",", ":"))
print(len(cases))

# ---- fourth batch: view_as / reshape
doc = json.load(open(path))
cases = [c for c in doc["cases"] if not c["name"].startswith("viewas_")]
case("viewas_owned_success", "927-943", {"a": T([2, 3], r(1, 6))}, [["v", "view_as", "a", [3, 2]]],
     [{"t": "v", "shape": [3, 2], "strides": [2, 1], "get": G(((0, 0), 1), ((0, 1), 2), ((1, 0), 3), ((1, 1), 4), ((2, 0), 5), ((2, 1), 6))}])
case("viewas_owned_error", "946-951", {"a": T([2, 3], r(1, 6))}, [["v", "view_as", "a", [4, 2]]], [{"error": "InvalidShape"}])
case("viewas_slice_success", "954-972", {"a": T([2, 3], r(1, 6))}, [["s", "slice", "a", 0, IDX(1)], ["v", "view_as", "s", [1, 3]]],
     [{"t": "s", "shape": [3]}, {"t": "v", "shape": [1, 3], "strides": [3, 1], "get": G(((0, 0), 4), ((0, 1), 5), ((0, 2), 6))}])
case("viewas_mut_view_modify", "975-987", {"a": T([2, 2], r(1, 4))}, sets("a", ((1, 0), 40)) + [["v", "view_as", "a", [4]]],
     [{"t": "v", "shape": [4], "strides": [1], "get": G((2, 40))}])
case("viewas_scalar", "990-1003", {"a": T([], [99])}, [["v", "view_as", "a", [1]], ["w", "view_as", "v", [1, 1, 1]]],
     [{"t": "a", "shape": []}, {"t": "v", "shape": [1], "strides": [1], "get": G((0, 99))}, {"t": "w", "get": G(((0, 0, 0), 99))}])
case("viewas_slice_error", "1278-1284", {"a": T([2, 3], r(1, 6))}, [["s", "slice", "a", 0, IDX(0)], ["v", "view_as", "s", [2, 2]]],
     [{"error": "InvalidShape"}])
case("viewas_mut_error", "1288-1292", {"a": T([2, 2], r(1, 4))}, [["v", "view_as", "a", [3, 2]]], [{"error": "InvalidShape"}])
case("viewas_to_owned_reshaped", "1536-1547", {"a": T([2, 3], r(1, 6))}, [["v", "view_as", "a", [3, 2]], ["o", "owned", "v"]],
     [{"t": "o", "shape": [3, 2], "values": r(1, 6), "contiguous": True}])
doc["cases"] = cases
json.dump(doc, open(path, "w"), separators=(",", ":"))
print(len(cases))
