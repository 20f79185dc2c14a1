import json
def T(shape, values): return {"shape": shape, "values": values}
C=[]
def case(name, ref, dtype, inputs, program, expect): C.append({"name": name, "ref": ref, "dtype": dtype, "inputs": inputs, "program": program, "expect": expect})
case("matmul_2d_basic","ops/linalg/mod.rs:76-94","i32",{"a":T([2,3],[1,2,3,4,5,6]),"b":T([3,2],[7,8,9,10,11,12])},[["r","matmul","a","b"]],[{"t":"r","shape":[2,2],"values":[58,64,139,154]}])
case("matmul_2d_square","ops/linalg/mod.rs:96-113","i32",{"a":T([2,2],[1,2,3,4]),"b":T([2,2],[5,6,7,8])},[["r","matmul","a","b"]],[{"t":"r","shape":[2,2],"values":[19,22,43,50]}])
case("matmul_2d_identity","ops/linalg/mod.rs:115-129","i32",{"a":T([2,2],[1,2,3,4]),"i":T([2,2],[1,0,0,1])},[["r","matmul","a","i"]],[{"t":"r","shape":[2,2],"values":[1,2,3,4]}])
case("matmul_2d_float","ops/linalg/mod.rs:131-146","f32",{"a":T([2,2],[1.5,2.0,3.5,4.0]),"b":T([2,2],[2.0,1.0,3.0,4.0])},[["r","matmul","a","b"]],[{"t":"r","shape":[2,2],"values":[9.0,9.5,19.0,19.5]}])
case("matmul_f64_slice_then_transpose","ops/linalg/mod.rs:531-566","f64",{"full":T([3,4],[1.0,2.0,3.0,4.0,5.0,6.0,7.0,8.0,9.0,10.0,11.0,12.0]),"b":T([2,2],[1.0,0.0,0.0,1.0])},
     [["s1","slice","full",0,{"range":[0,2]}],["s","slice","s1",1,{"range":[1,3]}],["t","transpose","s"],["r","matmul","t","b"],["r2","matmul","b","t"]],
     [{"t":"r","shape":[2,2],"values":[2.0,6.0,3.0,7.0]},{"t":"r2","shape":[2,2],"values":[2.0,6.0,3.0,7.0]}])
case("matmul_3d_batched","ops/linalg/mod.rs:569-593","i32",{"a":T([2,2,2],[1,2,3,4,9,10,11,12]),"b":T([2,2,2],[5,6,7,8,13,14,15,16])},[["r","matmul","a","b"]],[{"t":"r","shape":[2,2,2],"values":[19,22,43,50,267,286,323,346]}])
case("matmul_3d_larger_batch","ops/linalg/mod.rs:596-628","i32",{"a":T([3,2,2],[1,0,0,1,2,0,0,2,3,0,0,3]),"b":T([3,2,2],[5,6,7,8]*3)},[["r","matmul","a","b"]],[{"t":"r","shape":[3,2,2],"values":[5,6,7,8,10,12,14,16,15,18,21,24]}])
case("matmul_dimension_mismatch","ops/linalg/mod.rs:631-639","i32",{"a":T([2,2],[1,2,3,4]),"b":T([3,2],[1,2,3,4,5,6])},[["r","matmul","a","b"]],[{"error":"SizeMismatch"}])
case("matmul_rank_mismatch","ops/linalg/mod.rs:642-650","i32",{"a":T([2,2],[1,2,3,4]),"b":T([2,2,2],[1,2,3,4,5,6,7,8])},[["r","matmul","a","b"]],[{"error":"InvalidShape"}])
case("matmul_batch_mismatch","ops/linalg/mod.rs:653-661","i32",{"a":T([2,2,2],[1,2,3,4,5,6,7,8]),"b":T([3,2,2],list(range(1,13)))},[["r","matmul","a","b"]],[{"error":"SizeMismatch"}])
case("matmul_2d_rectangular","ops/linalg/mod.rs:664-679","i32",{"a":T([3,4],list(range(1,13))),"b":T([4,2],list(range(1,9)))},[["r","matmul","a","b"]],[{"t":"r","shape":[3,2],"values":[50,60,114,140,178,220]}])
case("matmul_1d_array_fails","ops/linalg/mod.rs:691-699","i32",{"a":T([3],[1,2,3]),"b":T([3],[4,5,6])},[["r","matmul","a","b"]],[{"error":"InvalidShape"}])
case("matmul_1d_with_2d_fails","ops/linalg/mod.rs:702-710","i32",{"a":T([3],[1,2,3]),"b":T([3,2],[1,2,3,4,5,6])},[["r","matmul","a","b"]],[{"error":"InvalidShape"}])
case("matmul_scalar_fails","ops/linalg/mod.rs:713-721","i32",{"a":T([],[5]),"b":T([],[10])},[["r","matmul","a","b"]],[{"error":"InvalidShape"}])
case("matmul_4d_batch_squashing","ops/linalg/mod.rs:735-750","i32",{"a":T([2,2,2,1],list(range(1,9))),"b":T([2,2,1,2],list(range(1,9)))},[["r","matmul","a","b"]],[{"t":"r","shape":[2,2,2,2]}])
case("matmul_inner_dimension_mismatch_3d","ops/linalg/mod.rs:764-778","i32",{"a":T([2,2,3],list(range(1,13))),"b":T([2,2,2],list(range(1,9)))},[["r","matmul","a","b"]],[{"error":"SizeMismatch"}])
sq16=[float(x) for x in range(1,17)]
case("matmul_stride_rows","ops/linalg/mod.rs:809-843","f32",{"a":T([4,4],sq16),"b":T([4,2],[float(x) for x in range(1,9)])},[["as","slice","a",0,{"slice":[None,None,2]}],["r","matmul","as","b"]],[{"t":"r","shape":[2,2],"values":[50.0,60.0,178.0,220.0]}])
case("matmul_stride_rhs_i32","ops/linalg/mod.rs:883-915","i32",{"a":T([2,2],[1,2,3,4]),"b":T([4,4],list(range(1,17)))},[["bs","slice","b",0,{"slice":[None,None,2]}],["r","matmul","a","bs"]],[{"t":"r","shape":[2,4],"values":[19,22,25,28,39,46,53,60]}])
a_sb=[1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16, 91,92,93,94,95,96,97,98,99,910,911,912,913,914,915,916]
b_sb=list(range(1,33))+[91,92,93,94,95,96,97,98,99,910,911,912,913,914,915,916,917,918,919,920,921,922,923,924,925,926,927,928,929,930,931,932]
case("strided_batched_matmul_i32","ops/linalg/mod.rs:1143-1200","i32",{"a":T([2,4,4],a_sb),"b":T([2,8,4],b_sb)},
     [["as","slice","a",1,{"slice":[None,None,2]}],["bs","slice","b",1,{"slice":[None,None,2]}],["r","matmul","as","bs"]],
     [{"t":"r","shape":[2,2,4],"values":[170,180,190,200,586,628,670,712,189620,264510,264880,265250,1778086,2518018,2520850,2523682]}])
case("dot","ops/linalg/mod.rs:1392-1402","f32",{"a":T([3],[1.0,2.0,3.0]),"b":T([3],[4.0,5.0,6.0])},[["r","dot","a","b"]],[{"t":"r","shape":[],"values":[32.0],"tol":1e-6}])
case("both_column_major","ops/linalg/mod.rs:1452-1480","f32",{"a":T([2,2],[1.0,3.0,2.0,4.0]),"b":T([2,2],[5.0,7.0,6.0,8.0])},[["at","transpose","a"],["bt","transpose","b"],["r","matmul","at","bt"]],[{"t":"r","shape":[2,2],"values":[19.0,22.0,43.0,50.0]}])
case("both_column_major_column_stride","ops/linalg/mod.rs:1484-1526","f32",{"a":T([4,2],[1.0,3.0,8.0,8.0,2.0,4.0,8.0,8.0]),"b":T([4,2],[5.0,7.0,122.0,122.0,6.0,8.0,678.0,678.0])},
     [["as","slice","a",0,{"slice":[0,3,2]}],["at","transpose","as"],["bs","slice","b",0,{"slice":[0,3,2]}],["bt","transpose","bs"],["r","matmul","at","bt"]],
     [{"t":"r","shape":[2,2],"values":[19.0,22.0,43.0,50.0]}])
a_bs=[1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16, 21,22,23,24,25,26,27,28,29,210,211,212,213,214,215,216]
case("batched_i32_strided_rows","ops/linalg/mod.rs:1606-1654","i32",{"a":T([2,4,4],a_bs),"b":T([2,4,2],[1,2,3,4,5,6,7,8,11,12,13,14,15,16,17,18])},
     [["as","slice","a",1,{"slice":[None,None,2]}],["r","matmul","as","b"]],[{"t":"r","shape":[2,2,2],"values":[50,60,178,220,1270,1360,9818,10480]}])
a_mb=[1,2,3,4,5,6, 11,12,13,14,15,16, 21,22,23,24,25,26, 11,12,13,14,15,16, 1,2,3,4,5,6, 11,12,13,14,15,16]
b_mb=([7,8,9,10,11,12]+[17,18,19,20,21,22])*3
case("multibatch_non_contiguous_matmul","ops/linalg/mod.rs:1697-1779 (test body present, #[test] attribute commented out)","f32",
     {"a":T([3,2,2,3],[float(x) for x in a_mb]),"b":T([3,2,3,2],[float(x) for x in b_mb])},
     [["as","slice","a",0,{"slice":[None,None,2]}],["bs","slice","b",0,{"slice":[None,None,2]}],["r","matmul","as","bs"]],
     [{"t":"as","shape":[2,2,2,3]},{"t":"bs","shape":[2,2,3,2]},{"t":"r","shape":[2,2,2,2],"values":[58.0,64.0,139.0,154.0,688.0,724.0,859.0,904.0]*2}])
json.dump({"source":"transcribed by hand from the reference's own tests (libs/rtensors/src/ops/linalg/mod.rs); data only","cases":C}, open("tests/golden/reference_matmul_vectors.json","w"), indent=1)
print(len(C))
