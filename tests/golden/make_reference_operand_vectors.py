# writes tests/golden/reference_operand_vectors.json (hand-transcribed from ops/mod.rs)
import json, itertools
from functools import reduce
cases = []
def prod(s): return reduce(lambda a, b: a * b, s, 1)
def T(shape, values): return {"shape": list(shape), "values": values}
def ones(*shape): return T(shape, [1.0] * prod(shape))
def case(name, ref, inputs, program, expect, dtype="f32"):
    cases.append({"name": name, "ref": "ops/mod.rs:" + ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
def allv(shape, v): return {"t": "c", "shape": list(shape), "values": [v] * prod(shape)}

case("broadcast_3d_matrix_to_tensor", "1235-1250", {"a": ones(3, 4), "b": ones(2, 3, 4)}, [["c", "add", "a", "b"]], [allv((2, 3, 4), 2.0)])
case("broadcast_4d_3d_to_4d", "1326-1345", {"a": ones(3, 5, 4), "b": ones(2, 3, 5, 4)}, [["c", "add", "a", "b"]], [allv((2, 3, 5, 4), 2.0)])
case("broadcast_5d_scalar_to_tensor", "1347-1366", {"a": T([], [100.0]), "b": ones(2, 2, 2, 2, 2)}, [["c", "add", "a", "b"]], [allv((2,) * 5, 101.0)])
case("broadcast_2d_to_4d", "1383-1400", {"a": ones(3, 4), "b": ones(2, 5, 3, 4)}, [["c", "add", "a", "b"]], [allv((2, 5, 3, 4), 2.0)])
case("broadcast_identity", "1564-1578", {"a": ones(3, 4, 5), "b": ones(3, 4, 5)}, [["c", "add", "a", "b"]], [allv((3, 4, 5), 2.0)])
case("broadcast_alternating_singletons", "1581-1590", {"a": ones(1, 4, 1, 6), "b": ones(3, 1, 5, 1)}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [3, 4, 5, 6], "get": [[[0, 0, 0, 0], 2.0], [[2, 3, 4, 5], 2.0]]}])
case("broadcast_trailing_singleton", "1593-1607", {"a": ones(3, 4, 1), "b": ones(3, 4, 5)}, [["c", "add", "a", "b"]], [allv((3, 4, 5), 2.0)])
case("broadcast_leading_singleton", "1610-1624", {"a": ones(1, 4, 5), "b": ones(3, 4, 5)}, [["c", "add", "a", "b"]], [allv((3, 4, 5), 2.0)])
for name, ref, sa, sb, sc in [
    ("broadcast_shape_2d_plus_3d", "1629-1637", (4, 5), (3, 4, 5), (3, 4, 5)),
    ("broadcast_shape_1d_plus_4d", "1640-1648", (7,), (2, 3, 4, 7), (2, 3, 4, 7)),
    ("broadcast_shape_singleton_expansion", "1651-1659", (1, 5, 1), (4, 5, 6), (4, 5, 6)),
    ("broadcast_shape_prepending", "1662-1670", (5, 6), (2, 3, 4, 5, 6), (2, 3, 4, 5, 6)),
    ("broadcast_shape_both_expand", "1673-1681", (1, 4, 1, 6), (3, 1, 5, 6), (3, 4, 5, 6)),
    ("broadcast_shape_complex_5d", "1695-1703", (1, 1, 3, 1, 5), (2, 4, 3, 6, 5), (2, 4, 3, 6, 5))]:
    case(name, ref, {"a": ones(*sa), "b": ones(*sb)}, [["c", "add", "a", "b"]], [{"t": "c", "shape": list(sc)}])
case("broadcast_shape_scalar_expansion", "1684-1692", {"a": T([], [42.0]), "b": ones(2, 3, 4, 5, 6)}, [["c", "add", "a", "b"]],
     [{"t": "c", "shape": [2, 3, 4, 5, 6]}])
case("sub_assign_broadcast_incompatible", "1995-2001", {"t": T([1, 3], [0, 0, 0]), "u": T([4, 3], [1] * 12)}, [["t", "isub", "t", "u"]],
     [{"error": "Panic"}], dtype="i32")
case("mul_assign_broadcast_incompatible", "2062-2068", {"t": T([1, 3], [0, 0, 0]), "u": T([4, 3], [1] * 12)}, [["t", "imul", "t", "u"]],
     [{"error": "Panic"}], dtype="i32")
case("mul_3d_broadcast", "2021-2036", {"a": T([3], [2.0, 3.0, 4.0]), "b": ones(2, 4, 3)}, [["c", "mul", "a", "b"]],
     [{"t": "c", "shape": [2, 4, 3], "values": [2.0, 3.0, 4.0] * 8}])

# every pairing of owner / view / mutable view / borrowed operands the reference's operator overloads accept: the operand kind does
# not change the kernel call, so each is the same program; the values differ per test
def ones_pair(name, ref, idx=(0, 0)):
    case(name, ref, {"a": ones(2, 3), "b": ones(2, 3)}, [["c", "add", "a", "b"]], [{"t": "c", "shape": [2, 3], "get": [[list(idx), 2.0]]}])
def vec_pair(name, ref, op, a, b, want):
    case(name, ref, {"a": T([2], a), "b": T([2], b)}, [["c", op, "a", "b"]], [{"t": "c", "values": want}])
ones_pair("tensorbase_add_tensorbase", "2074-2080")
vec_pair("tensorbase_sub_tensorbase", "2083-2089", "sub", [5.0, 3.0], [1.0, 1.0], [4.0, 2.0])
vec_pair("tensorbase_mul_tensorbase", "2092-2098", "mul", [2.0, 3.0], [4.0, 5.0], [8.0, 15.0])
ones_pair("tensorbase_add_tensorview", "2102-2107")
vec_pair("tensorbase_sub_tensorview", "2110-2116", "sub", [10.0, 20.0], [3.0, 7.0], [7.0, 13.0])
vec_pair("tensorbase_mul_tensorview", "2119-2125", "mul", [6.0, 7.0], [2.0, 3.0], [12.0, 21.0])
ones_pair("tensorbase_add_tensorviewmut", "2129-2134", (1, 2))
vec_pair("tensorbase_sub_tensorviewmut", "2137-2143", "sub", [8.0, 9.0], [3.0, 4.0], [5.0, 5.0])
vec_pair("tensorbase_mul_tensorviewmut", "2146-2152", "mul", [5.0, 6.0], [2.0, 2.0], [10.0, 12.0])
ones_pair("tensorbase_add_ref_tensorbase", "2156-2161")
vec_pair("tensorbase_sub_ref_tensorbase", "2164-2170", "sub", [15.0, 25.0], [5.0, 10.0], [10.0, 15.0])
vec_pair("tensorbase_mul_ref_tensorbase", "2173-2179", "mul", [3.0, 4.0], [5.0, 6.0], [15.0, 24.0])
ones_pair("ref_tensorbase_add_tensorbase", "2183-2188")
vec_pair("ref_tensorbase_sub_tensorbase", "2191-2197", "sub", [20.0, 30.0], [8.0, 12.0], [12.0, 18.0])
vec_pair("ref_tensorbase_mul_tensorbase", "2200-2206", "mul", [7.0, 8.0], [2.0, 3.0], [14.0, 24.0])
ones_pair("ref_tensorbase_add_ref_tensorbase", "2210-2215")
vec_pair("ref_tensorbase_sub_ref_tensorbase", "2218-2224", "sub", [100.0, 200.0], [30.0, 70.0], [70.0, 130.0])
vec_pair("ref_tensorbase_mul_ref_tensorbase", "2227-2233", "mul", [9.0, 10.0], [2.0, 4.0], [18.0, 40.0])
ones_pair("tensorview_add_tensorbase", "2237-2242")
vec_pair("tensorview_sub_tensorbase", "2245-2251", "sub", [50.0, 60.0], [20.0, 25.0], [30.0, 35.0])
vec_pair("tensorview_mul_tensorbase", "2254-2260", "mul", [11.0, 12.0], [3.0, 4.0], [33.0, 48.0])
ones_pair("tensorview_add_tensorview", "2264-2269")
vec_pair("tensorview_sub_tensorview", "2272-2278", "sub", [70.0, 80.0], [30.0, 35.0], [40.0, 45.0])
vec_pair("tensorview_mul_tensorview", "2281-2287", "mul", [13.0, 14.0], [2.0, 5.0], [26.0, 70.0])
ones_pair("tensorviewmut_add_tensorbase", "2291-2296")
vec_pair("tensorviewmut_sub_tensorbase", "2299-2305", "sub", [90.0, 100.0], [40.0, 45.0], [50.0, 55.0])
vec_pair("tensorviewmut_mul_tensorbase", "2308-2314", "mul", [15.0, 16.0], [2.0, 3.0], [30.0, 48.0])
ones_pair("tensorviewmut_add_tensorviewmut", "2318-2323")
vec_pair("tensorviewmut_sub_tensorviewmut", "2326-2332", "sub", [110.0, 120.0], [50.0, 60.0], [60.0, 60.0])
vec_pair("tensorviewmut_mul_tensorviewmut", "2335-2341", "mul", [17.0, 18.0], [3.0, 4.0], [51.0, 72.0])
ones_pair("ref_tensorview_add_ref_tensorview", "2345-2350")
vec_pair("ref_tensorview_sub_ref_tensorview", "2353-2359", "sub", [150.0, 200.0], [50.0, 100.0], [100.0, 100.0])
vec_pair("ref_tensorview_mul_ref_tensorview", "2362-2368", "mul", [19.0, 20.0], [2.0, 5.0], [38.0, 100.0])
ones_pair("ref_tensorviewmut_add_ref_tensorviewmut", "2372-2377")
vec_pair("ref_tensorviewmut_sub_ref_tensorviewmut", "2380-2386", "sub", [250.0, 300.0], [100.0, 150.0], [150.0, 150.0])
vec_pair("ref_tensorviewmut_mul_ref_tensorviewmut", "2389-2395", "mul", [21.0, 22.0], [3.0, 4.0], [63.0, 88.0])
case("tensorviewmut_add_assign_tensorbase", "2399-2407", {"a": ones(2, 3), "b": ones(2, 3)}, [["a", "iadd", "a", "b"]],
     [{"t": "a", "get": [[[0, 0], 2.0]]}])
case("tensorviewmut_sub_assign_tensorview", "2410-2419", {"a": T([2], [10.0, 20.0]), "b": T([2], [3.0, 7.0])}, [["a", "isub", "a", "b"]],
     [{"t": "a", "values": [7.0, 13.0]}])
case("tensorviewmut_mul_assign_tensorviewmut", "2422-2432", {"a": T([2], [5.0, 6.0]), "b": T([2], [2.0, 3.0])}, [["a", "imul", "a", "b"]],
     [{"t": "a", "values": [10.0, 18.0]}])
doc = {"_comment": "Known-answer vectors transcribed from the reference's own #[test]s (the broadcasts of every rank that the other fixtures "
                   "leave out, and every pairing of owner / view / mutable-view / borrowed operands of + - * and their assigning forms); "
                   "`ref` = file:lines under libs/rtensors/src/.", "cases": cases}
json.dump(doc, open("tests/golden/reference_operand_vectors.json", "w"), separators=(",", ":"))
print(len(cases))
