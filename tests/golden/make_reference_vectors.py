# writes tests/golden/reference_vectors.json (hand-transcribed from the reference's own tests)
import json
R = "ops/mod.rs"
FULL_REV = {"slice": [None, None, -1]}
def seq(a, b): return [float(x) for x in range(a, b + 1)]
def iseq(a, b): return list(range(a, b + 1))
cases = []
def case(name, ref, dtype, inputs, program, expect):
    cases.append({"name": name, "ref": ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
def T(shape, values): return {"shape": shape, "values": values}
def ones(shape):
    n = 1
    for d in shape: n *= d
    return T(shape, [1.0] * n)

# ---- broadcasting through sliced / reversed views (ops/mod.rs:2435-2737) ----
case("broadcast_post_slice", R + ":2435-2452", "f32",
     {"a": ones([4, 3]), "b": T([2, 1], [2.0, 1.0])},
     [["c", "slice", "a", 0, {"slice": [0, 3, 2]}], ["d", "add", "c", "b"]],
     [{"t": "c", "shape": [2, 3]}, {"t": "d", "shape": [2, 3], "values": [3., 3., 3., 2., 2., 2.]}])
case("broadcast_with_negative_step_slice", R + ":2455-2479", "f32",
     {"a": T([4, 3], seq(1, 12)), "b": T([3], [10., 20., 30.])},
     [["s", "slice", "a", 0, FULL_REV], ["r", "add", "s", "b"]],
     [{"t": "s", "shape": [4, 3]},
      {"t": "r", "shape": [4, 3], "values": [20., 31., 42., 17., 28., 39., 14., 25., 36., 11., 22., 33.]}])
case("broadcast_with_column_slice_negative_step", R + ":2482-2504", "f32",
     {"a": T([2, 3], seq(1, 6)), "b": T([2, 1], [100., 200.])},
     [["s", "slice", "a", 1, FULL_REV], ["r", "add", "s", "b"]],
     [{"t": "r", "shape": [2, 3], "values": [103., 102., 101., 206., 205., 204.]}])
case("broadcast_with_step_2_slice", R + ":2507-2526", "f32",
     {"a": T([8], seq(1, 8)), "b": T([], [10.])},
     [["s", "slice", "a", 0, {"slice": [None, None, 2]}], ["r", "add", "s", "b"]],
     [{"t": "s", "shape": [4]}, {"t": "r", "shape": [4], "values": [11., 13., 15., 17.]}])
case("broadcast_with_negative_step_2_slice", R + ":2529-2547", "f32",
     {"a": T([8], seq(1, 8))},
     [["s", "slice", "a", 0, {"slice": [None, None, -2]}], ["r", "add_scalar", "s", 100.0]],
     [{"t": "s", "shape": [4]}, {"t": "r", "shape": [4], "values": [108., 106., 104., 102.]}])
case("broadcast_with_3d_negative_step", R + ":2550-2577", "f32",
     {"a": T([3, 2, 2], seq(1, 12)), "b": T([2, 2], [10., 20., 30., 40.])},
     [["s", "slice", "a", 0, FULL_REV], ["r", "add", "s", "b"]],
     [{"t": "r", "shape": [3, 2, 2], "values": [19., 30., 41., 52., 15., 26., 37., 48., 11., 22., 33., 44.]}])
case("broadcast_inplace_with_negative_step", R + ":2580-2601", "f32",
     {"a": T([2, 3], seq(1, 6)), "b": T([1, 1], [10.])},
     [["s", "slice", "a", 1, FULL_REV], ["s", "iadd", "s", "b"]],
     [{"t": "s", "shape": [2, 3]}, {"t": "a", "shape": [2, 3], "values": [11., 12., 13., 14., 15., 16.]}])
case("broadcast_chained_slices_with_negative_steps", R + ":2604-2635", "f32",
     {"a": T([4, 4], seq(1, 16)), "b": T([1, 2], [100., 200.])},
     [["s1", "slice", "a", 0, FULL_REV], ["s2", "slice", "s1", 1, {"slice": [None, None, 2]}], ["r", "add", "s2", "b"]],
     [{"t": "s2", "shape": [4, 2]}, {"t": "r", "shape": [4, 2], "values": [113., 215., 109., 211., 105., 207., 101., 203.]}])
case("broadcast_scalar_with_complex_negative_slice", R + ":2638-2656", "i32",
     {"a": T([10], iseq(1, 10))},
     [["s", "slice", "a", 0, {"slice": [8, 2, -2]}], ["r", "add_scalar", "s", 100]],
     [{"t": "s", "shape": [3]}, {"t": "r", "shape": [3], "values": [109, 107, 105]}])
case("broadcast_vector_to_negative_step_matrix_slice", R + ":2659-2681", "f32",
     {"a": T([4, 3], seq(1, 12)), "b": T([2, 1], [5., 10.])},
     [["s", "slice", "a", 0, {"slice": [3, None, -2]}], ["r", "add", "s", "b"]],
     [{"t": "s", "shape": [2, 3]}, {"t": "r", "shape": [2, 3], "values": [15., 16., 17., 14., 15., 16.]}])
case("broadcast_both_tensors_sliced_negative_steps", R + ":2684-2710", "f32",
     {"a": T([2, 3], seq(1, 6)), "b": T([1, 3], [10., 20., 30.])},
     [["sa", "slice", "a", 1, FULL_REV], ["sb", "slice", "b", 1, FULL_REV], ["r", "add", "sa", "sb"]],
     [{"t": "r", "shape": [2, 3], "values": [33., 22., 11., 36., 25., 14.]}])
case("broadcast_4d_with_negative_step_multiple_dims", R + ":2713-2737", "f32",
     {"a": T([2, 2, 2, 2], seq(1, 16)), "b": T([2], [100., 200.])},
     [["s1", "slice", "a", 0, FULL_REV], ["s2", "slice", "s1", 2, FULL_REV], ["r", "add", "s2", "b"]],
     [{"t": "s2", "shape": [2, 2, 2, 2]}, {"t": "r", "shape": [2, 2, 2, 2], "get": [[[0, 0, 0, 0], 111.], [[0, 0, 0, 1], 212.]]}])

# ---- plain broadcasting shapes (ops/mod.rs:1154-1420) ----
case("broadcast_flipped", R + ":1154-1171", "f32",
     {"a": T([1, 3], [22., 1., 1.]), "b": ones([3, 1])},
     [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [3, 3], "values": [23., 2., 2., 23., 2., 2., 23., 2., 2.]}])
case("broadcast_same", R + ":1173-1190", "f32",
     {"a": T([3, 1], [22., 1., 1.]), "b": ones([3, 1])},
     [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [3, 1], "values": [23., 2., 2.]}])
case("broadcast_3d_scalar_to_tensor", R + ":1199-1214", "f32",
     {"a": T([], [5.]), "b": ones([2, 3, 4])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [2, 3, 4], "values": [6.] * 24}])
case("broadcast_3d_vector_along_last_dim", R + ":1216-1232", "f32",
     {"a": T([3], [1., 2., 3.]), "b": ones([2, 4, 3])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [2, 4, 3], "values": [2., 3., 4.] * 8}])
case("broadcast_3d_singleton_dims", R + ":1252-1267", "f32",
     {"a": ones([1, 3, 1]), "b": ones([2, 3, 4])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [2, 3, 4], "values": [2.] * 24}])
case("broadcast_3d_prepend_dims", R + ":1269-1284", "f32",
     {"a": ones([3, 4]), "b": ones([5, 3, 4])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [5, 3, 4], "values": [2.] * 60}])
case("broadcast_4d_vector_to_tensor", R + ":1288-1305", "f32",
     {"a": T([2], [10., 20.]), "b": ones([3, 4, 5, 2])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [3, 4, 5, 2], "values": [11., 21.] * 60}])
case("broadcast_4d_complex_singletons", R + ":1307-1324", "f32",
     {"a": ones([1, 1, 5, 1]), "b": ones([2, 3, 5, 4])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [2, 3, 5, 4], "values": [2.] * 120}])
case("broadcast_5d_multiple_singletons", R + ":1370-1381", "f32",
     {"a": ones([1, 2, 1, 3, 1]), "b": ones([4, 2, 5, 3, 6])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [4, 2, 5, 3, 6], "get": [[[0, 0, 0, 0, 0], 2.], [[3, 1, 4, 2, 5], 2.]]}])
case("broadcast_1d_to_5d", R + ":1403-1424", "f32",
     {"a": T([3], [1., 2., 3.]), "b": ones([2, 4, 5, 6, 3])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [2, 4, 5, 6, 3], "values": [2., 3., 4.] * 240}])
case("broadcast_div_scalar_to_tensor", R + ":1430-1443", "f32",
     {"a": T([], [10.]), "b": T([2, 3], [2.] * 6)}, [["c", "div", "a", "b"]],
     [{"t": "c", "shape": [2, 3], "values": [5.] * 6}])
case("broadcast_div_3d_vector_along_last_dim", R + ":1445-1461", "f32",
     {"a": ones([2, 3, 4]), "b": T([4], [1., 2., 4., 8.])}, [["c", "div", "a", "b"]],
     [{"t": "c", "shape": [2, 3, 4], "values": [1., .5, .25, .125] * 6}])
case("broadcast_div_in_place", R + ":1463-1474", "f32",
     {"a": T([4], [10., 20., 30., 40.]), "b": T([], [2.])}, [["a", "idiv", "a", "b"]],
     [{"t": "a", "shape": [4], "values": [5., 10., 15., 20.]}])
case("broadcast_div_2d_matrices", R + ":1476-1488", "f32",
     {"a": T([2, 2], [100., 200., 300., 400.]), "b": T([1, 2], [10., 20.])}, [["c", "div", "a", "b"]],
     [{"t": "c", "shape": [2, 2], "values": [10., 10., 30., 20.]}])
for nm, ref, sa, sb in [
    ("broadcast_incompatible_dimensions_3d", ":1492-1499", [3, 4], [2, 5, 6]),
    ("broadcast_incompatible_inner_dim", ":1501-1508", [5], [2, 3, 7]),
    ("broadcast_incompatible_middle_dim", ":1510-1518", [2, 3, 4], [2, 5, 4]),
    ("broadcast_incompatible_4d", ":1520-1528", [2, 3, 4, 5], [2, 7, 4, 5]),
    ("broadcast_incompatible_5d_multiple", ":1530-1538", [1, 2, 3, 4, 5], [6, 2, 7, 4, 5]),
    ("broadcast_both_non_singleton_mismatch", ":1540-1548", [4, 5, 6], [4, 3, 6])]:
    case(nm, R + ref, "f32", {"a": ones(sa), "b": ones(sb)}, [["c", "add", "a", "b"]], [{"error": "BroadcastError"}])
case("broadcast_all_singletons", R + ":1552-1562", "f32",
     {"a": ones([1, 1, 1]), "b": ones([5, 6, 7])}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [5, 6, 7], "get": [[[0, 0, 0], 2.], [[4, 5, 6], 2.]]}])
# in-place
case("add_assign_broadcast", R + ":1930-1937", "i32",
     {"t": T([3, 3], [0] * 9), "u": T([3], [1, 1, 1])}, [["t", "iadd", "t", "u"]],
     [{"t": "t", "shape": [3, 3], "values": [1] * 9}])
case("add_assign_broadcast_incompatible", R + ":1939-1945", "i32",
     {"t": T([1, 3], [0] * 3), "u": T([4, 3], [1] * 12)}, [["t", "iadd", "t", "u"]], [{"error": "Panic"}])
case("sub_broadcast_basic", R + ":1951-1966", "f32",
     {"a": T([3, 3], [5., 1., 1., 1., 1., 1., 1., 1., 1.]), "b": ones([3, 1])}, [["c", "sub", "a", "b"]],
     [{"t": "c", "shape": [3, 3], "values": [4., 0., 0., 0., 0., 0., 0., 0., 0.]}])
case("sub_3d_broadcast", R + ":1968-1983", "f32",
     {"a": T([3], [10., 20., 30.]), "b": ones([2, 4, 3])}, [["c", "sub", "a", "b"]],
     [{"t": "c", "shape": [2, 4, 3], "values": [9., 19., 29.] * 8}])
case("sub_assign_broadcast", R + ":1985-1992", "i32",
     {"t": T([3], [5, 10, 15]), "u": T([3], [1, 1, 1])}, [["t", "isub", "t", "u"]],
     [{"t": "t", "shape": [3], "values": [4, 9, 14]}])
case("mul_broadcast_basic", R + ":2006-2020", "f32",
     {"a": T([3, 3], [5., 1., 1., 1., 1., 1., 1., 1., 1.]), "b": T([3, 1], [1., 2., 1.])}, [["c", "mul", "a", "b"]],
     [{"t": "c", "shape": [3, 3], "get": [[[0, 0], 5.], [[1, 0], 2.], [[2, 2], 1.]]}])
case("mul_scalar_broadcast", R + ":2038-2050", "f32",
     {"a": T([], [5.]), "b": T([2, 2], [1., 2., 3., 4.])}, [["c", "mul", "a", "b"]],
     [{"t": "c", "shape": [2, 2], "values": [5., 10., 15., 20.]}])
case("mul_assign_broadcast", R + ":2052-2059", "i32",
     {"t": T([3], [2, 4, 6]), "u": T([3], [3, 3, 3])}, [["t", "imul", "t", "u"]],
     [{"t": "t", "shape": [3], "values": [6, 12, 18]}])

# ---- reductions (backend/cpu.rs:1167-1279, backend/cuda.rs:2364-2374) ----
C = "backend/cpu.rs"
red = [0.2, 0.3, 0.1, 0.3, 0.3, -0.1, -0.3, 0.3]
case("reduce_total_sum_case1", C + ":1167-1172", "f64", {"x": T([4, 2], red)}, [["s", "sum", "x", None]],
     [{"t": "s", "shape": [], "values": [1.0999999999999999], "exact": True}])
case("reduce_total_max_case1", C + ":1175-1180", "f64", {"x": T([4, 2], red)}, [["s", "max", "x", None]],
     [{"t": "s", "shape": [], "values": [0.3], "exact": True}])
case("reduce_total_min_case1", C + ":1183-1188", "f64", {"x": T([4, 2], [0.2, 0.3, 0.1, -0.9, 0.3, -0.1, -0.3, 0.3])},
     [["s", "min", "x", None]], [{"t": "s", "shape": [], "values": [-0.9], "exact": True}])
case("reduce_total_prod_case1", C + ":1192-1197", "f64", {"x": T([4, 2], seq(1, 8))}, [["s", "prod", "x", None]],
     [{"t": "s", "shape": [], "values": [40320.], "exact": True}])
case("reduce_sum_case1", C + ":1200-1211", "f64", {"x": T([4, 2], [1., 0., 1., 0., 1., 1., 1., 0.])},
     [["s", "sum", "x", 0]], [{"t": "s", "shape": [1, 2], "values": [4., 1.], "exact": True}])
m = [3., 5., 6., 8., 1., 2., -1., 4.]
case("reduce_max_case1", C + ":1214-1224", "f64", {"x": T([4, 2], m)}, [["s", "max", "x", 0]],
     [{"t": "s", "shape": [1, 2], "values": [6., 8.], "exact": True}])
case("reduce_min_case1", C + ":1227-1238", "f64", {"x": T([4, 2], m)}, [["s", "min", "x", 0]],
     [{"t": "s", "shape": [1, 2], "values": [-1., 2.], "exact": True}])
case("reduce_prod_case1", C + ":1241-1250", "f64", {"x": T([4, 2], m)}, [["s", "prod", "x", 0]],
     [{"t": "s", "shape": [1, 2], "values": [-18., 320.], "exact": True}])
case("reduce_mean_case1", C + ":1253-1264", "f64", {"x": T([4, 2], seq(1, 8))}, [["s", "mean", "x", 0]],
     [{"t": "s", "shape": [1, 2], "values": [4., 5.], "exact": True}])
case("reduce_mean_case2", C + ":1268-1279", "f64", {"x": T([4, 2], seq(1, 8))}, [["s", "mean", "x", 1]],
     [{"t": "s", "shape": [4, 1], "values": [1.5, 3.5, 5.5, 7.5], "exact": True}])
case("reduce_total_mean", "backend/cuda.rs:2364-2374", "f64", {"x": T([4, 2], seq(1, 8))}, [["s", "mean", "x", None]],
     [{"t": "s", "shape": [], "values": [4.5], "exact": True}])

# ---- unary / scalar over the three layout fixtures (testing/mod.rs:6-195, ops/unary/mod.rs:407-450, ops/scalar/mod.rs:216-295)
U = "ops/unary/mod.rs"
relu16 = [-1.0, 1.0, 0.0, 2.0, 1.0, 2.3, -0.3, 0.4, 0.0, -0.3, 0.4, 0.5, -0.2, 0.1, 0.2, -0.5]
def nd_expected(vals, f):
    # (4,4,1) tensor, rows step 2, cols step 2 -> elements [0,2,8,10] are touched
    out = list(vals)
    for i in (0, 2, 8, 10): out[i] = f(vals[i])
    return out
case("unary_negate_contiguous", U + ":407-412", "f64", {"x": T([2, 1], [1., 1.])}, [["x", "unary_inplace", "x", "neg"]],
     [{"t": "x", "shape": [2, 1], "values": [-1., -1.], "path": "contiguous"}])
case("unary_negate_1d_strided", U + ":414-419", "f64", {"x": T([3, 1], [1., 1., 1.])},
     [["v", "slice", "x", 0, {"slice": [None, None, 2]}], ["v", "unary_inplace", "v", "neg"]],
     [{"t": "x", "shape": [3, 1], "values": [-1., 1., -1.]}, {"t": "v", "path": "1d_strided"}])
case("unary_negate_nd_strided", U + ":421-426", "f64", {"x": T([4, 4, 1], [1.] * 16)},
     [["v1", "slice", "x", 0, {"slice": [None, None, 2]}], ["v", "slice", "v1", 1, {"slice": [None, None, 2]}], ["v", "unary_inplace", "v", "neg"]],
     [{"t": "x", "shape": [4, 4, 1], "values": nd_expected([1.] * 16, lambda v: -v)}, {"t": "v", "path": "nd"}])
case("unary_relu_contiguous", U + ":428-431", "f64", {"x": T([2, 1], [-1., 1.])}, [["x", "unary_inplace", "x", "relu"]],
     [{"t": "x", "shape": [2, 1], "values": [0., 1.]}])
case("unary_relu_1d_strided", U + ":433-440", "f64", {"x": T([3, 1], [-1., 1., -1.])},
     [["v", "slice", "x", 0, {"slice": [None, None, 2]}], ["v", "unary_inplace", "v", "relu"]],
     [{"t": "x", "shape": [3, 1], "values": [0., 1., 0.]}])
case("unary_relu_nd_strided", U + ":442-450", "f64", {"x": T([4, 4, 1], relu16)},
     [["v1", "slice", "x", 0, {"slice": [None, None, 2]}], ["v", "slice", "v1", 1, {"slice": [None, None, 2]}], ["v", "unary_inplace", "v", "relu"]],
     [{"t": "x", "shape": [4, 4, 1], "values": nd_expected(relu16, lambda v: max(v, 0.0))}])
S = "ops/scalar/mod.rs"
lr16 = [-1, 2, -3, 4, -5, 6, -7, 8, -9, 10, -11, 12, -13, 14, -15, 16]
case("scalar_leaky_relu_1d_strided_i32", S + ":270-277", "i32", {"x": T([3, 1], [1, -2, 3])},
     [["v", "slice", "x", 0, {"slice": [None, None, 2]}], ["v", "scalar_inplace", "v", "leaky_relu", 1]],
     [{"t": "x", "shape": [3, 1], "values": [1, -2, 3]}])
case("scalar_leaky_relu_contiguous_i32", S + ":279-286", "i32", {"x": T([2, 1], [2, -1])},
     [["x", "scalar_inplace", "x", "leaky_relu", 1]], [{"t": "x", "shape": [2, 1], "values": [2, -1]}])
case("scalar_leaky_relu_nd_strided_i32", S + ":288-295", "i32", {"x": T([4, 4, 1], lr16)},
     [["v1", "slice", "x", 0, {"slice": [None, None, 2]}], ["v", "slice", "v1", 1, {"slice": [None, None, 2]}], ["v", "scalar_inplace", "v", "leaky_relu", 2]],
     [{"t": "x", "shape": [4, 4, 1], "values": nd_expected(lr16, lambda v: v if v > 0 else v * 2)}])
lrf = [float(v) for v in lr16]
import struct
def f32(x): return struct.unpack("f", struct.pack("f", x))[0]
case("scalar_leaky_relu_nd_strided_f32", S + ":232-239", "f32", {"x": T([4, 4, 1], lrf)},
     [["v1", "slice", "x", 0, {"slice": [None, None, 2]}], ["v", "slice", "v1", 1, {"slice": [None, None, 2]}], ["v", "scalar_inplace", "v", "leaky_relu", 0.2]],
     [{"t": "x", "shape": [4, 4, 1], "values": nd_expected(lrf, lambda v: v if v > 0 else f32(f32(v) * f32(0.2))), "tol": 1e-5}])
case("scalar_leaky_relu_contiguous_f32", S + ":224-230", "f32", {"x": T([2, 1], [2.0, -1.5])},
     [["x", "scalar_inplace", "x", "leaky_relu", 0.1]], [{"t": "x", "shape": [2, 1], "values": [2.0, f32(f32(-1.5) * f32(0.1))], "tol": 1e-5}])

# ---- large-N spot checks (ops/mod.rs:3115-3213) are generated in the tests from their closed forms ----
json.dump({"_comment": "Known-answer vectors transcribed from the reference's own #[test]s; `ref` = file:lines under libs/rtensors/src/.",
           "cases": cases}, open("tests/golden/reference_vectors.json", "w"), indent=1)
print(len(cases))

# ======================= second file: metadata-only vectors (core/mod.rs tests) =======================
cases2 = []
def mcase(name, ref, inputs, program, expect, dtype="i32"):
    cases2.append({"name": name, "ref": ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
M = "core/mod.rs"
mcase("negative_step_basic", M + ":332-345", {"a": T([8], iseq(1, 8))}, [["s", "slice", "a", 0, FULL_REV]],
      [{"t": "s", "shape": [8], "get": [[[0], 8], [[1], 7], [[7], 1]]}])
mcase("negative_step_with_range", M + ":348-362", {"a": T([8], iseq(1, 8))}, [["s", "slice", "a", 0, {"slice": [6, 2, -1]}]],
      [{"t": "s", "shape": [4], "get": [[[0], 7], [[1], 6], [[2], 5], [[3], 4]]}])
mcase("negative_step_skip_elements", M + ":365-378", {"a": T([8], iseq(1, 8))}, [["s", "slice", "a", 0, {"slice": [None, None, -2]}]],
      [{"t": "s", "shape": [4], "get": [[[0], 8], [[1], 6], [[2], 4], [[3], 2]]}])
mcase("negative_step_matrix_rows", M + ":381-406", {"a": T([4, 3], iseq(1, 12))}, [["s", "slice", "a", 0, FULL_REV]],
      [{"t": "s", "shape": [4, 3], "get": [[[0, 0], 10], [[0, 1], 11], [[0, 2], 12], [[3, 0], 1], [[3, 1], 2], [[3, 2], 3]]}])
mcase("negative_step_with_start_less_than_end", M + ":409-418", {"a": T([6], iseq(1, 6))}, [["s", "slice", "a", 0, {"slice": [2, 5, -1]}]],
      [{"t": "s", "shape": []}])
mcase("positive_step_with_start_greater_than_end", M + ":421-430", {"a": T([6], iseq(1, 6))}, [["s", "slice", "a", 0, {"slice": [5, 2, 1]}]],
      [{"t": "s", "shape": []}])
mcase("negative_step_partial_range", M + ":433-445", {"a": T([8], iseq(1, 8))}, [["s", "slice", "a", 0, {"slice": [5, None, -1]}]],
      [{"t": "s", "shape": [6], "get": [[[0], 6], [[5], 1]]}])
mcase("negative_step_partial_end", M + ":448-460", {"a": T([8], iseq(1, 8))}, [["s", "slice", "a", 0, {"slice": [None, 3, -1]}]],
      [{"t": "s", "shape": [4], "get": [[[0], 8], [[3], 5]]}])
mcase("negative_step_3d_tensor", M + ":463-486", {"a": T([4, 2, 2], iseq(1, 16))}, [["s", "slice", "a", 0, FULL_REV]],
      [{"t": "s", "shape": [4, 2, 2], "get": [[[0, 0, 0], 13], [[0, 1, 1], 16], [[3, 0, 0], 1], [[3, 1, 1], 4]]}])
mcase("negative_step_chained", M + ":489-506", {"a": T([10], iseq(1, 10))},
      [["s1", "slice", "a", 0, FULL_REV], ["s2", "slice", "s1", 0, {"slice": [None, None, 2]}]],
      [{"t": "s1", "get": [[[0], 10]]}, {"t": "s2", "shape": [5], "get": [[[0], 10], [[1], 8], [[4], 2]]}])
mcase("negative_step_funtax", M + ":509-522", {"a": T([10], iseq(1, 10))}, [["s", "slice", "a", 0, {"range_inclusive": [9, 0]}]],
      [{"t": "s", "shape": [10], "get": [[[0], 10], [[1], 9]]}])
mcase("meta_offsets_on_slices_2d", M + ":1382-1389", {"m": T([2, 2], [1, 2, 3, 4])}, [["s", "slice", "m", 0, {"range": [1, 1]}]],
      [{"t": "s", "offset": 2}])
mcase("meta_offsets_on_slices_3d", M + ":1391-1398", {"c": T([2, 2, 2], iseq(1, 8))},
      [["s1", "slice", "c", 0, {"range": [1, 1]}], ["s2", "slice", "s1", 1, {"range": [1, 1]}]],
      [{"t": "s1", "offset": 4}, {"t": "s2", "offset": 5}])
mcase("is_contiguous_owned_and_slices", M + ":1401-1417", {"mat": T([2, 3], iseq(1, 6))},
      [["row", "slice", "mat", 0, {"range": [1, 1]}], ["col", "slice", "mat", 1, {"range": [0, 0]}]],
      [{"t": "mat", "contiguous": True}, {"t": "row", "contiguous": True}, {"t": "col", "contiguous": False}])
mcase("permute_on_slice", M + ":2291-2312", {"a": T([3, 4], iseq(1, 12))},
      [["s", "slice", "a", 0, {"range": [1, 3]}], ["p", "permute", "s", [1, 0]]],
      [{"t": "s", "shape": [2, 4]}, {"t": "p", "shape": [4, 2], "get": [[[0, 0], 5], [[3, 1], 12]]}])
mcase("transpose_on_slice", M + ":2315-2336", {"a": T([4, 3], iseq(1, 12))},
      [["s", "slice", "a", 0, {"range": [1, 3]}], ["p", "transpose", "s"]],
      [{"t": "s", "shape": [2, 3]}, {"t": "p", "shape": [3, 2], "get": [[[0, 0], 4], [[2, 1], 9]]}])
mcase("unsqueeze_at_with_negative_stride", M + ":3199-3220", {"a": T([8], iseq(1, 8))},
      [["r", "slice", "a", 0, FULL_REV], ["u", "unsqueeze", "r", 0]],
      [{"t": "r", "shape": [8], "strides": [-1], "get": [[[0], 8], [[7], 1]]},
       {"t": "u", "shape": [1, 8], "strides": [-8, -1], "get": [[[0, 0], 8], [[0, 7], 1]]}])
mcase("unsqueeze_at_negative_stride_2d", M + ":3223-3246", {"a": T([3, 4], iseq(1, 12))},
      [["r", "slice", "a", 0, FULL_REV], ["u", "unsqueeze", "r", 1]],
      [{"t": "r", "shape": [3, 4], "strides": [-4, 1], "get": [[[0, 0], 9], [[2, 3], 4]]},
       {"t": "u", "shape": [3, 1, 4], "strides": [-4, 4, 1], "get": [[[0, 0, 0], 9], [[0, 0, 3], 12], [[2, 0, 0], 1]]}])
json.dump({"_comment": "View/metadata known answers transcribed from the reference's own #[test]s; `ref` = file:lines under libs/rtensors/src/.",
           "cases": cases2}, open("tests/golden/reference_meta_vectors.json", "w"), indent=1)
print(len(cases2))
