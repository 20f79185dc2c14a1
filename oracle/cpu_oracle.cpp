// TEST INFRASTRUCTURE ONLY -- never linked into, loaded by, or called from the product path.
//
// CPU restatement of the rtensors `Cpu` backend (the parity oracle and the timed CPU baseline).
// Every function cites the reference lines it follows (paths relative to libs/rtensors/src/).
// Single threaded on purpose: the reference Cpu backend has no threading.
//
// Build: g++ -O2 -fno-fast-math -ffp-contract=off -fno-associative-math (see oracle/Makefile), so every
// float expression below is evaluated as written, one IEEE-754 operation at a time, in source order.
//
// Pinning status of each function (what fixes it besides this text) is listed in oracle/README.md and
// checked by tests/test_oracle_*.py:
//   broadcast / unary / scalar / fill / layouts : reference known-answer vectors + an independent numpy
//                                                 as_strided evaluation
//   reduce flat / nd (sum,prod,max,min,mean)    : reference known-answer vectors (incl. the order-sensitive
//                                                 f64 sum 1.0999999999999999) + numpy sequential accumulate
//   variance / stdev / logsumexp / norms / arg  : the Cuda backend's known-answer vectors (backend/cuda.rs:2321-2590) + numpy
//                                                 float64 var / logaddexp.reduce / norm / argmax (ties, NaN cases by hand)
//   integer reductions                          : not in the reference (WeightValue is f32/f64 only); pinned by
//                                                 the closed form "sum mod 2^w", min/max by numpy
//   transcendental unaries (exp, ln, sin ...)   : PARITY UNPINNED bit-for-bit (Rust std -> platform libm);
//                                                 held to the reference's own 1e-5 test tolerance only
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <cmath>
#include <limits>
#include <type_traits>
#include <vector>

namespace {

// ---- status codes -------------------------------------------------------------------------------------------
enum : int {
    ORC_OK = 0,
    ORC_E_DTYPE = 1,        // dtype/op combination the reference trait bounds do not admit
    ORC_E_OOB = 2,          // the reference would panic with an index-out-of-bounds
    ORC_E_ARITH = 3,        // the reference would panic (integer divide by zero / MIN / -1, bool division todo!())
    ORC_E_WRONG_DIMS = 4,   // TensorError::WrongDims (non-contiguous reduce), backend/mod.rs:386-390
    ORC_E_OP = 5,           // accumulator not implemented (reduction/mod.rs:185) / unknown op code
};

// ---- dtype codes: core/value.rs:567-581 ---------------------------------------------------------------------
enum : int { U8 = 0, I8 = 1, U16 = 2, I16 = 3, U32 = 4, U128 = 5, I32 = 6, U64 = 7, I64 = 8, I128 = 9, F32 = 10, F64 = 11, BOOL = 12 };

typedef unsigned __int128 u128_t;
typedef __int128 i128_t;

// `types::boolean` (core/value.rs:650-765): one byte holding 0/1; + is OR, - is XOR, * is AND, / is todo!().
struct boolean { uint8_t v; };

template <class T> struct is_float : std::integral_constant<bool, std::is_same<T, float>::value || std::is_same<T, double>::value> {};
template <class T> struct is_bool : std::is_same<T, boolean> {};
template <class T> struct is_sint : std::integral_constant<bool, std::is_same<T, int8_t>::value || std::is_same<T, int16_t>::value ||
                                                                     std::is_same<T, int32_t>::value || std::is_same<T, int64_t>::value ||
                                                                     std::is_same<T, i128_t>::value> {};
template <class T> struct is_uint : std::integral_constant<bool, std::is_same<T, uint8_t>::value || std::is_same<T, uint16_t>::value ||
                                                                     std::is_same<T, uint32_t>::value || std::is_same<T, uint64_t>::value ||
                                                                     std::is_same<T, u128_t>::value> {};

// Unsigned carrier wide enough that +,-,* never hit C++ signed-overflow UB; the final cast truncates, which
// is Rust's release-mode wrapping behaviour (the reference uses plain `+ - *`, ops/base.rs:27-37).
template <class T, class = void> struct carrier;
template <class T> struct carrier<T, typename std::enable_if<(is_sint<T>::value || is_uint<T>::value) && sizeof(T) <= 4>::type> { typedef uint32_t type; };
template <class T> struct carrier<T, typename std::enable_if<(is_sint<T>::value || is_uint<T>::value) && sizeof(T) == 8>::type> { typedef uint64_t type; };
template <class T> struct carrier<T, typename std::enable_if<(is_sint<T>::value || is_uint<T>::value) && sizeof(T) == 16>::type> { typedef u128_t type; };

// ---- TypeConstants: core/value.rs:317-323, 496-508 ----------------------------------------------------------
template <class T> struct consts {
    static T zero() { return T(0); }
    static T one() { return T(1); }
    static T min() { return std::numeric_limits<T>::lowest(); }  // f32::MIN is the lowest *finite* value
    static T max() { return std::numeric_limits<T>::max(); }
};
template <> struct consts<i128_t> {
    static i128_t zero() { return 0; }
    static i128_t one() { return 1; }
    static i128_t min() { return (i128_t)((u128_t)1 << 127); }
    static i128_t max() { return (i128_t)(~((u128_t)1 << 127)); }
};
template <> struct consts<u128_t> {
    static u128_t zero() { return 0; }
    static u128_t one() { return 1; }
    static u128_t min() { return 0; }
    static u128_t max() { return ~(u128_t)0; }
};
template <> struct consts<boolean> {
    static boolean zero() { return boolean{0}; }
    static boolean one() { return boolean{1}; }
    static boolean min() { return boolean{0}; }
    static boolean max() { return boolean{1}; }
};

// ---- scalar arithmetic exactly as `a + b`, `a - b`, `a * b`, `a / b` on T (ops/base.rs:27-37) -----------------
struct arith_fault { bool hit = false; };

template <class T> inline typename std::enable_if<is_float<T>::value, T>::type add(T a, T b) { return a + b; }
template <class T> inline typename std::enable_if<is_float<T>::value, T>::type sub(T a, T b) { return a - b; }
template <class T> inline typename std::enable_if<is_float<T>::value, T>::type mul(T a, T b) { return a * b; }
template <class T> inline typename std::enable_if<is_float<T>::value, T>::type dvd(T a, T b, arith_fault&) { return a / b; }

template <class T> inline typename std::enable_if<is_sint<T>::value || is_uint<T>::value, T>::type add(T a, T b) {
    typedef typename carrier<T>::type W; return (T)(W)((W)a + (W)b);
}
template <class T> inline typename std::enable_if<is_sint<T>::value || is_uint<T>::value, T>::type sub(T a, T b) {
    typedef typename carrier<T>::type W; return (T)(W)((W)a - (W)b);
}
template <class T> inline typename std::enable_if<is_sint<T>::value || is_uint<T>::value, T>::type mul(T a, T b) {
    typedef typename carrier<T>::type W; return (T)(W)((W)a * (W)b);
}
// Integer `/` truncates toward zero; Rust panics on a zero divisor and on MIN / -1 in every build profile.
template <class T> inline typename std::enable_if<is_uint<T>::value, T>::type dvd(T a, T b, arith_fault& f) {
    if (b == 0) { f.hit = true; return 0; }
    return (T)(a / b);
}
template <class T> inline typename std::enable_if<is_sint<T>::value, T>::type dvd(T a, T b, arith_fault& f) {
    if (b == 0 || (a == consts<T>::min() && b == (T)-1)) { f.hit = true; return 0; }
    return (T)(a / b);
}
inline boolean add(boolean a, boolean b) { return boolean{(uint8_t)(a.v || b.v)}; }   // core/value.rs:708-713
inline boolean sub(boolean a, boolean b) { return boolean{(uint8_t)(a.v != b.v)}; }   // core/value.rs:715-720
inline boolean mul(boolean a, boolean b) { return boolean{(uint8_t)(a.v && b.v)}; }   // core/value.rs:722-727
inline boolean dvd(boolean, boolean, arith_fault& f) { f.hit = true; return boolean{0}; }  // todo!(), core/value.rs:759-764

template <class T> inline bool gt(T a, T b) { return a > b; }
template <class T> inline bool lt(T a, T b) { return a < b; }
inline bool gt(boolean a, boolean b) { return a.v > b.v; }
inline bool lt(boolean a, boolean b) { return a.v < b.v; }

// `Absolute` (core/value.rs:515-557): signed ints / floats call `.abs()`, unsigned and boolean are identity.
template <class T> inline typename std::enable_if<is_float<T>::value, T>::type absolute(T x) { return std::fabs(x); }
template <class T> inline typename std::enable_if<is_sint<T>::value, T>::type absolute(T x) {
    typedef typename carrier<T>::type W; return x < 0 ? (T)(W)((W)0 - (W)x) : x;   // MIN.abs() wraps to MIN in release
}
template <class T> inline typename std::enable_if<is_uint<T>::value, T>::type absolute(T x) { return x; }
inline boolean absolute(boolean x) { return x; }

// ---- layouts ------------------------------------------------------------------------------------------------
struct Meta {
    size_t offset;
    int rank;
    const size_t* shape;
    const int64_t* strides;
    size_t size() const { size_t n = 1; for (int i = 0; i < rank; ++i) n *= shape[i]; return n; }   // core/meta.rs:186
};

// core/meta.rs:526-541 (is_contiguous_relaxed): |stride| is compared, so reversed views count as contiguous.
bool is_contiguous_relaxed(const Meta& m) {
    if (m.rank == 0) return true;
    for (int i = 0; i < m.rank; ++i) if (m.shape[i] == 0) return true;
    size_t expected = 1;
    for (int i = m.rank - 1; i >= 0; --i) {
        size_t dim = m.shape[i];
        int64_t s = m.strides[i];
        if (dim != 1) {
            size_t a = s < 0 ? (size_t)(-(s + 1)) + 1 : (size_t)s;
            if (a != expected) return false;
            size_t prod;
            if (__builtin_mul_overflow(expected, dim, &prod)) prod = SIZE_MAX;   // saturating_mul
            expected = prod;
        }
    }
    return true;
}

// core/meta.rs:368-430 (TensorOffsetIterator): odometer over `shape`, last dim fastest, offset recomputed
// from the index vector on every step.
struct OffsetIter {
    const Meta& m;
    std::vector<size_t> index;
    bool started = false, done = false;
    explicit OffsetIter(const Meta& meta) : m(meta), index((size_t)meta.rank, 0) {}
    bool next(int64_t& phys) {
        if (done) return false;
        if (m.rank == 0) {
            if (started) { done = true; return false; }
            started = true; phys = (int64_t)m.offset; return true;
        }
        started = true;
        int64_t off = (int64_t)m.offset;
        for (int d = 0; d < m.rank; ++d) off += (int64_t)index[(size_t)d] * m.strides[d];
        phys = off;
        for (int d = m.rank - 1; d >= 0; --d) {
            index[(size_t)d] += 1;
            if (index[(size_t)d] < m.shape[d]) return true;
            index[(size_t)d] = 0;
        }
        done = true;
        return true;
    }
};

// core/meta.rs:432-486 (CoordIter): yields a fresh coordinate vector per element.
struct CoordIter {
    const Meta& m;
    std::vector<size_t> coords;
    bool started = false, done = false;
    explicit CoordIter(const Meta& meta) : m(meta), coords((size_t)meta.rank, 0) {}
    bool next(std::vector<size_t>& out) {
        if (done) return false;
        if (m.rank == 0) {
            if (started) { done = true; return false; }
            started = true; out = std::vector<size_t>(); return true;
        }
        if (!started) { started = true; out = coords; return true; }   // .clone()
        for (int d = m.rank - 1; d >= 0; --d) {
            coords[(size_t)d] += 1;
            if (coords[(size_t)d] < m.shape[d]) { out = coords; return true; }
            coords[(size_t)d] = 0;
        }
        done = true;
        return false;
    }
};

// backend/mod.rs:15-213, 239-268: which of the three loop shapes the default trait method picks.
enum : int { PATH_CONTIGUOUS = 0, PATH_1D_STRIDED = 1, PATH_ND = 2 };

// Runs `f(T&)` over every element the view addresses, through the same three loops as
// backend/cpu.rs:10-42 (slice loop, 1-D strided loop with bounds-checked index, N-d offset iterator).
template <class T, class F>
int visit(T* buf, size_t buflen, const Meta& m, int* path, F f) {
    if (is_contiguous_relaxed(m)) {
        if (path) *path = PATH_CONTIGUOUS;
        size_t start = m.offset, len = m.size();
        if (start > buflen || len > buflen - start) return ORC_E_OOB;   // &mut buf[start..start+len] panics
        for (size_t i = 0; i < len; ++i) f(buf[start + i]);
        return ORC_OK;
    }
    int nns = 0, which = -1;
    for (int d = 0; d < m.rank; ++d) if (m.shape[d] > 1) { ++nns; which = d; }   // core/meta.rs:618-625
    if (nns == 1) {
        if (path) *path = PATH_1D_STRIDED;
        int64_t idx = (int64_t)m.offset;
        for (size_t k = 0; k < m.shape[which]; ++k) {
            if (idx < 0 || (size_t)idx >= buflen) return ORC_E_OOB;
            f(buf[idx]);
            idx += m.strides[which];
        }
        return ORC_OK;
    }
    if (path) *path = PATH_ND;
    OffsetIter it(m);
    int64_t phys;
    while (it.next(phys)) {
        if (phys < 0 || (size_t)phys >= buflen) return ORC_E_OOB;
        f(buf[phys]);
    }
    return ORC_OK;
}

// ---- unary functions: backend/cpu.rs:485-675 ------------------------------------------------------------------
enum : int {  // numbering = declaration order of UnaryOp, backend/remote/protocol.rs:213-224
    U_NEG = 0, U_RELU, U_SIGMOID, U_SILU, U_TANH, U_ABS, U_SQRT, U_LN, U_EXPM1, U_LN1P, U_FLOOR, U_CEIL, U_ROUND, U_TRUNC,
    U_SIN, U_COS, U_TAN, U_ASIN, U_ACOS, U_ATAN, U_SINH, U_COSH, U_ASINH, U_ACOSH, U_ATANH, U_RSQRT, U_RECIPROCAL, U_SQUARE,
    U_CUBE, U_EXP, U_SIGN, U_COUNT
};

template <class T> inline T relu(T x) { return gt(x, consts<T>::zero()) ? x : consts<T>::zero(); }   // cpu.rs:650-657

template <class T> inline T fexp(T x) { return std::exp(x); }
template <class T> inline T finvexp(T x) { return std::exp(-x); }   // core/primops/exp.rs:26-31

template <class T> T unary_float(int op, T x) {
    const T one = 1;
    switch (op) {
        case U_NEG: return -x;                                                   // cpu.rs:644-647
        case U_RELU: return relu(x);
        case U_SIGMOID: return one / (one + finvexp(x));                         // cpu.rs:661-667
        case U_SILU: return x * (one / (one + finvexp(x)));                      // cpu.rs:669-675
        case U_TANH: { T a = fexp(x), b = finvexp(x); return (a - b) / (a + b); }  // cpu.rs:624-629
        case U_ABS: return absolute(x);
        case U_SQRT: return std::sqrt(x);
        case U_LN: return std::log(x);
        case U_EXPM1: return std::expm1(x);
        case U_LN1P: return std::log1p(x);
        case U_FLOOR: return std::floor(x);
        case U_CEIL: return std::ceil(x);
        case U_ROUND: return std::round(x);                                      // half away from zero, like Rust
        case U_TRUNC: return std::trunc(x);
        case U_SIN: return std::sin(x);
        case U_COS: return std::cos(x);
        case U_TAN: return std::tan(x);
        case U_ASIN: return std::asin(x);
        case U_ACOS: return std::acos(x);
        case U_ATAN: return std::atan(x);
        case U_SINH: { T a = fexp(x), b = finvexp(x); return (a - b) / (one + one); }   // cpu.rs:485-490
        case U_COSH: { T a = fexp(x), b = finvexp(x); return (a + b) / (one + one); }   // cpu.rs:492-497
        case U_ASINH: { T sq = x * x; return std::log(x + std::sqrt(sq + one)); }        // cpu.rs:499-505
        case U_ACOSH: { T sq = x * x; return std::log(x + std::sqrt(sq - one)); }        // cpu.rs:507-513
        case U_ATANH: { T two = one + one; return std::log((one + x) / (one - x)) / two; }  // cpu.rs:515-521
        case U_RSQRT: return one / std::sqrt(x);                                 // cpu.rs:523-526
        case U_RECIPROCAL: return one / x;                                       // cpu.rs:528-531
        case U_SQUARE: return x * x;                                             // cpu.rs:533-536
        case U_CUBE: return x * x * x;                                           // cpu.rs:538-541 (left assoc)
        case U_EXP: return fexp(x);
        case U_SIGN: return x < T(0) ? -one : (x > T(0) ? one : T(0));           // cpu.rs:548-557 (NaN -> 0)
    }
    return x;
}

template <class T>
typename std::enable_if<is_float<T>::value, int>::type
unary_impl(int op, T* buf, size_t buflen, const Meta& m, int* path) {
    if (op < 0 || op >= U_COUNT) return ORC_E_OP;
    return visit(buf, buflen, m, path, [op](T& x) { x = unary_float<T>(op, x); });
}

// Non-float dtypes: the trait admits `relu` and `abs` for every TensorValue and `neg` for types with
// `Neg` (signed ints); everything else is bounded on WeightValue = {f32, f64} (backend/mod.rs:311-355).
template <class T>
typename std::enable_if<!is_float<T>::value, int>::type
unary_impl(int op, T* buf, size_t buflen, const Meta& m, int* path) {
    if (op == U_RELU) return visit(buf, buflen, m, path, [](T& x) { x = relu(x); });
    if (op == U_ABS) return visit(buf, buflen, m, path, [](T& x) { x = absolute(x); });
    if (op == U_NEG) {
        if (!is_sint<T>::value) return ORC_E_DTYPE;
        return visit(buf, buflen, m, path, [](T& x) { x = sub(consts<T>::zero(), x); });   // -x wraps for MIN
    }
    return ORC_E_DTYPE;
}

// ---- scalar functions: backend/cpu.rs:677-724 -------------------------------------------------------------------
enum : int { S_ADD = 0, S_SUB, S_MUL, S_DIV, S_LOG, S_LOG1P, S_LEAKY_RELU, S_ELU, S_LEAKY_GRAD, S_COUNT };   // protocol.rs:226-232; S_LEAKY_GRAD: ops/scalar/mod.rs:149-166

template <class T> inline typename std::enable_if<is_float<T>::value, bool>::type
scalar_float_only(int op, T& x, T v) {
    switch (op) {
        case S_LOG: x = std::log(x) / std::log(v); return true;                       // f32::log(base) = ln(x)/ln(base); value.rs vlog
        case S_LOG1P: x = std::log1p(x) / std::log(v); return true;                   // core/value.rs vlog1p
        case S_ELU: x = (x >= T(0)) ? x : v * std::expm1(x); return true;             // cpu.rs:717-724
    }
    return false;
}
template <class T> inline typename std::enable_if<!is_float<T>::value, bool>::type
scalar_float_only(int, T&, T) { return false; }

template <class T>
int scalar_impl(int op, T* buf, size_t buflen, T v, const Meta& m, int* path) {
    arith_fault fault;
    int rc;
    switch (op) {
        case S_ADD: rc = visit(buf, buflen, m, path, [v](T& x) { x = add(x, v); }); break;
        case S_SUB: rc = visit(buf, buflen, m, path, [v](T& x) { x = sub(x, v); }); break;
        case S_MUL: rc = visit(buf, buflen, m, path, [v](T& x) { x = mul(x, v); }); break;
        case S_DIV: rc = visit(buf, buflen, m, path, [v, &fault](T& x) { x = dvd(x, v, fault); }); break;
        case S_LEAKY_RELU:                                                            // cpu.rs:708-715
            rc = visit(buf, buflen, m, path, [v](T& x) { x = gt(x, consts<T>::zero()) ? x : mul(x, v); });
            break;
        case S_LEAKY_GRAD:                                                            // ops/scalar/mod.rs:152-160: 1 where input > 0, else the slope
            rc = visit(buf, buflen, m, path, [v](T& x) { x = gt(x, consts<T>::zero()) ? consts<T>::one() : v; });
            break;
        case S_LOG: case S_LOG1P: case S_ELU:
            if (!is_float<T>::value) return ORC_E_DTYPE;
            rc = visit(buf, buflen, m, path, [op, v](T& x) { scalar_float_only<T>(op, x, v); });
            break;
        default: return ORC_E_OP;
    }
    if (rc == ORC_OK && fault.hit) return ORC_E_ARITH;
    return rc;
}

// ---- fill: backend/cpu.rs:245-289 -----------------------------------------------------------------------------
template <class T>
int fill_impl(T* buf, size_t buflen, T v, const Meta& m, int* path) {
    return visit(buf, buflen, m, path, [v](T& x) { x = v; });
}

// ---- broadcast: backend/cpu.rs:292-352 --------------------------------------------------------------------------
// The coordinate iterator hands out one coordinate vector per element; the three running offsets are advanced by
// the per-dim deltas against the previous coordinate, last dim first.
enum : int { B_ADD = 0, B_SUB = 1, B_MUL = 2, B_DIV = 3 };   // ops/base.rs:7-12

template <class T>
int broadcast_impl(int op, const T* l, size_t llen, const Meta& lm, const T* r, size_t rlen, const Meta& rm,
                   T* d, size_t dlen, const Meta& dm) {
    if (op < 0 || op > 3) return ORC_E_OP;
    const int rank = dm.rank;
    int64_t ol = (int64_t)lm.offset, orr = (int64_t)rm.offset, od = (int64_t)dm.offset;
    std::vector<size_t> coords((size_t)rank, 0), nc;
    bool first = true;
    arith_fault fault;
    CoordIter it(dm);
    while (it.next(nc)) {
        if (first) {
            first = false;
        } else {
            for (int k = rank - 1; k >= 0; --k) {
                if (nc[(size_t)k] != coords[(size_t)k]) {
                    int64_t delta = (int64_t)nc[(size_t)k] - (int64_t)coords[(size_t)k];
                    ol += delta * lm.strides[k];
                    orr += delta * rm.strides[k];
                    od += delta * dm.strides[k];
                }
            }
        }
        coords = nc;
        if (ol < 0 || (size_t)ol >= llen || orr < 0 || (size_t)orr >= rlen || od < 0 || (size_t)od >= dlen) return ORC_E_OOB;
        T a = l[ol], b = r[orr], out;
        switch (op) {
            case B_ADD: out = add(a, b); break;
            case B_SUB: out = sub(a, b); break;
            case B_MUL: out = mul(a, b); break;
            default: out = dvd(a, b, fault); break;
        }
        if (fault.hit) return ORC_E_ARITH;
        d[od] = out;
    }
    return ORC_OK;
}

// ---- reductions: ops/reduction/mod.rs:3-137 (accumulators), backend/cpu.rs:397-449 ------------------------------
enum : int { R_SUM = 1, R_PROD = 2, R_MAX = 3, R_MIN = 4, R_MEAN = 5 };   // ReductionOpTypes::get_code, reduction/mod.rs:161-175

// WeightValue::from_usize (core/value.rs:54-56) goes through f32: `from_f32(value as f32)`.
template <class T> inline typename std::enable_if<is_float<T>::value, T>::type from_usize(size_t n) { return (T)(float)n; }
// Integers are outside WeightValue in the reference; the same route (usize -> f32 -> T, Rust `as` saturating)
// is kept so that the definition is a single one.
template <class T> inline typename std::enable_if<!is_float<T>::value && !is_bool<T>::value, T>::type from_usize(size_t n) {
    float f = (float)n;
    if (f >= (float)consts<T>::max()) return consts<T>::max();
    return (T)f;
}
template <class T> inline typename std::enable_if<is_bool<T>::value, T>::type from_usize(size_t n) { return boolean{(uint8_t)(n != 0)}; }

template <class T> struct Accum {
    int op;
    T acc;
    explicit Accum(int o) : op(o) {
        switch (o) {
            case R_SUM: case R_MEAN: acc = consts<T>::zero(); break;
            case R_PROD: acc = consts<T>::one(); break;
            case R_MAX: acc = consts<T>::min(); break;
            default: acc = consts<T>::max(); break;
        }
    }
    inline void accumulate(T v) {
        switch (op) {
            case R_SUM: case R_MEAN: acc = add(acc, v); break;      // self.sum += value
            case R_PROD: acc = mul(acc, v); break;                  // self.prod *= value
            case R_MAX: if (gt(v, acc)) acc = v; break;             // NaN never wins; first of equals stays
            default: if (lt(v, acc)) acc = v; break;
        }
    }
    inline int finalize(size_t count, T& out) const {
        if (op == R_MEAN) {
            arith_fault f;
            out = dvd(acc, from_usize<T>(count), f);                // self.sum / T::from_usize(count)
            return f.hit ? ORC_E_ARITH : ORC_OK;
        }
        out = acc;
        return ORC_OK;
    }
};

template <class T>
int reduce_flat_impl(int op, const T* src, size_t srclen, T* dst, size_t dstlen, size_t start, size_t len) {
    if (op < R_SUM || op > R_MEAN) return ORC_E_OP;
    if (start > srclen || len > srclen - start || dstlen == 0) return ORC_E_OOB;
    Accum<T> a(op);
    for (size_t i = 0; i < len; ++i) a.accumulate(src[start + i]);
    return a.finalize(len, dst[0]);
}

// backend/cpu.rs:413-449.  `honour_offset == 0` reproduces the reference literally (the base index has no
// offset term, which the reference itself calls a known CPU-backend bug, backend/remote/server.rs:327-330);
// `honour_offset == 1` adds meta.offset, which is what the Cuda backend does (cuda.rs:1934).
template <class T>
int reduce_nd_impl(int op, const T* src, size_t srclen, const Meta& sm, T* dst, size_t dstlen, int dim, int honour_offset) {
    if (op < R_SUM || op > R_MEAN) return ORC_E_OP;
    if (!is_contiguous_relaxed(sm)) return ORC_E_WRONG_DIMS;             // backend/mod.rs:386-390
    if (dim < 0 || dim >= sm.rank) return ORC_E_OOB;
    size_t inner = 1;                                                    // core/meta.rs:209-218
    for (int i = dim + 1; i < sm.rank; ++i) inner *= sm.shape[i];
    if (inner < 1) inner = 1;
    size_t outer = 1;                                                    // core/meta.rs:220-235
    for (int i = 0; i < dim; ++i) outer *= sm.shape[i];
    const size_t r = sm.shape[dim];
    const size_t r_stride = (size_t)sm.strides[dim];                     // `k * r_stride as usize`
    const size_t left_stride = r * inner;
    const size_t base0 = honour_offset ? sm.offset : 0;
    for (size_t i = 0; i < inner; ++i) {
        for (size_t o = 0; o < outer; ++o) {
            size_t base = base0 + o * left_stride + i;
            size_t out_idx = o * inner + i;
            Accum<T> a(op);
            for (size_t k = 0; k < r; ++k) {
                size_t idx = base + k * r_stride;
                if (idx >= srclen) return ORC_E_OOB;
                a.accumulate(src[idx]);
            }
            if (out_idx >= dstlen) return ORC_E_OOB;
            int rc = a.finalize(r, dst[out_idx]);
            if (rc != ORC_OK) return rc;
        }
    }
    return ORC_OK;
}

// ---- statistics and index reductions -------------------------------------------------------------------------------------
// The reference's Cpu backend has no accumulator for these (ops/reduction/mod.rs:185 panics, backend/cpu.rs:451-471 is todo!());
// its Cuda backend defines them in cuda/kernels/reduction/reduce.cu.  Restated here are that file's per-element rules, applied
// in ascending index order by one thread (the Cuda kernels combine the same states in tree order):
//   variance / stdev  welford_update 181-189, finalize 385-402: m2 / (n - 1 | n), optional sqrt
//   logsumexp         lse_from_value / lse_combine 654-673, result m + log(s) 731-733; x == max counts as exp(0) = 1, so that
//                     infinite inputs give +-inf instead of the NaN of exp(inf - inf)
//   norms             L1SumOp 66-75 (sum |x|), L2SumOp 88-97 + PostSqrt 143-152 (sqrt(sum x^2))
//   argmax / argmin   strict comparison starting from lowest() / max() with index 0, 893-905: the first extremum wins, NaN never
// The source is viewed as (outer, R, inner) from `offset`, as apply_reduce_contiguous_nd does (backend/cpu.rs:413-449).
enum : int { R_VARIANCE = 6, R_LOGSUMEXP = 7, R_NORM = 8, R_ARGMAX = 9, R_ARGMIN = 10, RF_UNBIASED = 0x100, RF_STD = 0x200, RF_L1 = 0x100, RF_L2 = 0x200 };

template <class T>
int reduce_stat_impl(int op, const T* src, size_t srclen, size_t offset, size_t outer, size_t r, size_t inner, T* dst, size_t dstlen) {
    const int code = op & 0xff, flags = op & ~0xff;
    if (code == R_VARIANCE) { if (flags & ~(RF_UNBIASED | RF_STD)) return ORC_E_OP; }
    else if (code == R_LOGSUMEXP) { if (flags) return ORC_E_OP; }
    else if (code == R_NORM) { if (flags != RF_L1 && flags != RF_L2) return ORC_E_OP; }
    else return ORC_E_OP;
    if (outer * inner > dstlen) return ORC_E_OOB;
    if (outer * r * inner > 0 && (offset > srclen || outer * r * inner > srclen - offset)) return ORC_E_OOB;
    for (size_t o = 0; o < outer; ++o) {
        for (size_t i = 0; i < inner; ++i) {
            const T* base = src + offset + o * r * inner + i;
            T out;
            if (code == R_VARIANCE) {
                T mean = (T)0, m2 = (T)0;
                long count = 0;
                for (size_t k = 0; k < r; ++k) {
                    const T x = base[k * inner];
                    count += 1;
                    const T delta = x - mean;
                    mean += delta / (T)count;
                    const T delta2 = x - mean;
                    m2 += delta * delta2;
                }
                const T denom = (flags & RF_UNBIASED) ? (T)(count - 1) : (T)count;
                out = m2 / denom;
                if (flags & RF_STD) out = std::sqrt(out);
            } else if (code == R_LOGSUMEXP) {
                T m = -std::numeric_limits<T>::infinity(), sum = (T)0;
                for (size_t k = 0; k < r; ++k) {
                    const T x = base[k * inner];
                    const T top = (x > m) ? x : m;                                   // NaN never becomes the maximum
                    const T keep = (m == top) ? (T)1 : std::exp(m - top);
                    const T add = (x == top) ? (T)1 : std::exp(x - top);
                    sum = sum * keep + add;
                    m = top;
                }
                out = (sum == (T)0) ? m : m + std::log(sum);
            } else {
                T sum = (T)0;
                for (size_t k = 0; k < r; ++k) {
                    const T x = base[k * inner];
                    sum += (flags == RF_L1) ? std::fabs(x) : x * x;
                }
                out = (flags == RF_L1) ? sum : std::sqrt(sum);
            }
            dst[o * inner + i] = out;
        }
    }
    return ORC_OK;
}

template <class T, class E = void> struct arg_ok : std::false_type {};
template <class T> struct arg_ok<T, typename std::enable_if<std::is_arithmetic<T>::value && sizeof(T) <= 8>::type> : std::true_type {};

template <class T>
typename std::enable_if<arg_ok<T>::value, int>::type
argmax_impl(int op, const T* src, size_t srclen, size_t offset, size_t outer, size_t r, size_t inner, uint64_t* dst, size_t dstlen) {
    if (op != R_ARGMAX && op != R_ARGMIN) return ORC_E_OP;
    if (outer * inner > dstlen) return ORC_E_OOB;
    if (outer * r * inner > 0 && (offset > srclen || outer * r * inner > srclen - offset)) return ORC_E_OOB;
    for (size_t o = 0; o < outer; ++o) {
        for (size_t i = 0; i < inner; ++i) {
            const T* base = src + offset + o * r * inner + i;
            T best = op == R_ARGMAX ? std::numeric_limits<T>::lowest() : std::numeric_limits<T>::max();
            uint64_t at = 0;
            for (size_t k = 0; k < r; ++k) {
                const T x = base[k * inner];
                if (op == R_ARGMAX ? x > best : x < best) { best = x; at = k; }
            }
            dst[o * inner + i] = at;
        }
    }
    return ORC_OK;
}
template <class T>
typename std::enable_if<!arg_ok<T>::value, int>::type
argmax_impl(int, const T*, size_t, size_t, size_t, size_t, size_t, uint64_t*, size_t) { return ORC_E_DTYPE; }

// ---- view_to_contiguous: core/tensor.rs:299-325 with core/meta.rs:263-307, 506-521 ------------------------------
// Copies forward-contiguous runs (negative strides never form a run) into a fresh row-major buffer.
template <class T>
int gather_impl(const T* src, size_t srclen, const Meta& m, T* dst, size_t dstlen) {
    size_t n = m.size();
    if (n > dstlen) return ORC_E_OOB;
    size_t j = 0;
    OffsetIter it(m);
    int64_t phys;
    if (n == 0) return ORC_OK;
    while (it.next(phys)) {
        if (phys < 0 || (size_t)phys >= srclen) return ORC_E_OOB;
        dst[j++] = src[phys];
    }
    return ORC_OK;
}

// ---- Buf equality (Box<[T]> PartialEq): elementwise `==`, so NaN != NaN and -0.0 == 0.0 --------------------------
template <class T> inline bool eq1(T a, T b) { return a == b; }
inline bool eq1(boolean a, boolean b) { return a.v == b.v; }
template <class T> int equal_impl(const T* a, const T* b, size_t n) {
    for (size_t i = 0; i < n; ++i) if (!eq1(a[i], b[i])) return 0;
    return 1;
}

// ---- dtype dispatch -------------------------------------------------------------------------------------------
#define ORC_DISPATCH(dtype, CALL)                               \
    switch (dtype) {                                            \
        case U8: { typedef uint8_t T; CALL; }                   \
        case I8: { typedef int8_t T; CALL; }                    \
        case U16: { typedef uint16_t T; CALL; }                 \
        case I16: { typedef int16_t T; CALL; }                  \
        case U32: { typedef uint32_t T; CALL; }                 \
        case U128: { typedef u128_t T; CALL; }                  \
        case I32: { typedef int32_t T; CALL; }                  \
        case U64: { typedef uint64_t T; CALL; }                 \
        case I64: { typedef int64_t T; CALL; }                  \
        case I128: { typedef i128_t T; CALL; }                  \
        case F32: { typedef float T; CALL; }                    \
        case F64: { typedef double T; CALL; }                   \
        case BOOL: { typedef boolean T; CALL; }                 \
        default: return ORC_E_DTYPE;                            \
    }

// ---- matmul: backend/cpu.rs:857-939 (generic_backend_matmul) -------------------------------------------------------------------
// dst[batch][row][col] = sum over inner, ascending, of lhs * rhs with `sum += a * b` on T (wrapping integers, OR/AND for
// boolean); dst is row-major from element 0.  The reference writes the loop twice, for two row-major and for two
// column-major operands (lhs_idx = batch + row*lda + inner / batch + row + inner*lda, ...); with (row stride, column stride)
// per operand both are the one loop below.  For f32/f64 the reference calls OpenBLAS gemm (backend/cpu.rs:725-855; OpenBLAS
// 0.3.30, build.rs:76-169, not vendored), whose summation order is not part of its interface: for those two dtypes this loop
// is the textbook definition, exact whenever every partial sum is representable (all of the reference's own test vectors)
// and otherwise only a tolerance reference -- bit parity for float matmul is unpinned.
template <class T>
int matmul_impl(const T* lhs, size_t lhs_len, size_t l_off, int64_t l_rs, int64_t l_cs, int64_t l_bs,
                const T* rhs, size_t rhs_len, size_t r_off, int64_t r_rs, int64_t r_cs, int64_t r_bs,
                T* dst, size_t dst_len, size_t b, size_t m, size_t k, size_t n) {
    if (l_rs < 0 || l_cs < 0 || l_bs < 0 || r_rs < 0 || r_cs < 0 || r_bs < 0) return ORC_E_OOB;
    if (b * m * n > dst_len) return ORC_E_OOB;
    if (b && m && k && l_off + (b - 1) * (size_t)l_bs + (m - 1) * (size_t)l_rs + (k - 1) * (size_t)l_cs >= lhs_len) return ORC_E_OOB;
    if (b && k && n && r_off + (b - 1) * (size_t)r_bs + (k - 1) * (size_t)r_rs + (n - 1) * (size_t)r_cs >= rhs_len) return ORC_E_OOB;
    for (size_t batch = 0; batch < b; ++batch) {
        const size_t lhs_batch = l_off + batch * (size_t)l_bs, rhs_batch = r_off + batch * (size_t)r_bs, out_batch = batch * m * n;
        for (size_t row = 0; row < m; ++row) {
            for (size_t col = 0; col < n; ++col) {
                T sum = consts<T>::zero();
                for (size_t inner = 0; inner < k; ++inner) {
                    const T a = lhs[lhs_batch + row * (size_t)l_rs + inner * (size_t)l_cs];
                    const T c = rhs[rhs_batch + inner * (size_t)r_rs + col * (size_t)r_cs];
                    sum = add(sum, mul(a, c));
                }
                dst[out_batch + row * n + col] = sum;
            }
        }
    }
    return ORC_OK;
}

template <class T> inline T load_value(const void* p) { T v; std::memcpy(&v, p, sizeof(T)); return v; }

}  // namespace

extern "C" {

int orc_dtype_size(int dtype) {
    switch (dtype) {
        case U8: case I8: case BOOL: return 1;
        case U16: case I16: return 2;
        case U32: case I32: case F32: return 4;
        case U64: case I64: case F64: return 8;
        case U128: case I128: return 16;
    }
    return 0;
}

int orc_is_contiguous(size_t offset, int rank, const size_t* shape, const int64_t* strides) {
    Meta m{offset, rank, shape, strides};
    return is_contiguous_relaxed(m) ? 1 : 0;
}

int orc_unary(int dtype, int op, void* buf, size_t buflen, size_t offset, int rank, const size_t* shape,
              const int64_t* strides, int* path) {
    Meta m{offset, rank, shape, strides};
    ORC_DISPATCH(dtype, return unary_impl<T>(op, (T*)buf, buflen, m, path));
}

int orc_scalar(int dtype, int op, void* buf, size_t buflen, const void* value, size_t offset, int rank,
               const size_t* shape, const int64_t* strides, int* path) {
    Meta m{offset, rank, shape, strides};
    ORC_DISPATCH(dtype, return scalar_impl<T>(op, (T*)buf, buflen, load_value<T>(value), m, path));
}

int orc_fill(int dtype, void* buf, size_t buflen, const void* value, size_t offset, int rank, const size_t* shape,
             const int64_t* strides, int* path) {
    Meta m{offset, rank, shape, strides};
    ORC_DISPATCH(dtype, return fill_impl<T>((T*)buf, buflen, load_value<T>(value), m, path));
}

int orc_broadcast(int dtype, int op, int rank, const size_t* shape,
                  const void* l, size_t llen, size_t loff, const int64_t* lstrides,
                  const void* r, size_t rlen, size_t roff, const int64_t* rstrides,
                  void* d, size_t dlen, size_t doff, const int64_t* dstrides) {
    Meta lm{loff, rank, shape, lstrides}, rm{roff, rank, shape, rstrides}, dm{doff, rank, shape, dstrides};
    ORC_DISPATCH(dtype, return broadcast_impl<T>(op, (const T*)l, llen, lm, (const T*)r, rlen, rm, (T*)d, dlen, dm));
}

int orc_reduce_flat(int dtype, int op, const void* src, size_t srclen, void* dst, size_t dstlen, size_t start, size_t len) {
    ORC_DISPATCH(dtype, return reduce_flat_impl<T>(op, (const T*)src, srclen, (T*)dst, dstlen, start, len));
}

int orc_reduce_nd(int dtype, int op, const void* src, size_t srclen, size_t offset, int rank, const size_t* shape,
                  const int64_t* strides, void* dst, size_t dstlen, int dim, int honour_offset) {
    Meta m{offset, rank, shape, strides};
    ORC_DISPATCH(dtype, return reduce_nd_impl<T>(op, (const T*)src, srclen, m, (T*)dst, dstlen, dim, honour_offset));
}

int orc_reduce_stat(int dtype, int op, const void* src, size_t srclen, size_t offset, size_t outer, size_t r, size_t inner, void* dst, size_t dstlen) {
    if (dtype == F32) return reduce_stat_impl<float>(op, (const float*)src, srclen, offset, outer, r, inner, (float*)dst, dstlen);
    if (dtype == F64) return reduce_stat_impl<double>(op, (const double*)src, srclen, offset, outer, r, inner, (double*)dst, dstlen);
    return ORC_E_DTYPE;                                                  // T: WeightValue
}

int orc_argmax(int dtype, int op, const void* src, size_t srclen, size_t offset, size_t outer, size_t r, size_t inner, uint64_t* dst, size_t dstlen) {
    ORC_DISPATCH(dtype, return argmax_impl<T>(op, (const T*)src, srclen, offset, outer, r, inner, dst, dstlen));
}

int orc_gather(int dtype, const void* src, size_t srclen, size_t offset, int rank, const size_t* shape,
               const int64_t* strides, void* dst, size_t dstlen) {
    Meta m{offset, rank, shape, strides};
    ORC_DISPATCH(dtype, return gather_impl<T>((const T*)src, srclen, m, (T*)dst, dstlen));
}

int orc_matmul(int dtype, const void* lhs, size_t lhs_len, size_t l_off, int64_t l_rs, int64_t l_cs, int64_t l_bs,
               const void* rhs, size_t rhs_len, size_t r_off, int64_t r_rs, int64_t r_cs, int64_t r_bs,
               void* dst, size_t dst_len, size_t b, size_t m, size_t k, size_t n) {
    ORC_DISPATCH(dtype, return matmul_impl<T>((const T*)lhs, lhs_len, l_off, l_rs, l_cs, l_bs, (const T*)rhs, rhs_len, r_off, r_rs, r_cs, r_bs,
                                              (T*)dst, dst_len, b, m, k, n));
}

int orc_equal(int dtype, const void* a, const void* b, size_t n) {
    ORC_DISPATCH(dtype, return equal_impl<T>((const T*)a, (const T*)b, n));
}

}  // extern "C"
