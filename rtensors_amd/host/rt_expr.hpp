// `Expr`: a pending elementwise expression over tensors -- the operators of `Tensor` recorded instead of run, then issued as few
// passes over memory as the backend allows.
//
// The reference runs every operator of an expression such as `c = relu(a * 3.0 + b); c -= 1.0` as its own backend call, with a clone
// before each value-returning scalar / unary op (ops/scalar/add.rs:84-113, ops/unary/mod.rs:114-126, ops/broadcast/add.rs:173-208):
// four kernels and two copies, 13 passes over a tensor.  `Expr` records the same steps in the same order and hands runs of up to
// RT_CHAIN_MAX_STEPS of them to rt_fused_chain: every operand read once, the result written once.  Each step is the same operation on
// T as the separate call, so the values are bit for bit those of the reference's sequence.  Operands that do not fit the fused form
// (shapes that need broadcasting, views that are not forward contiguous runs, steps the chain kernel does not have) go through the
// ordinary operators of `Tensor`, step by step.
#pragma once

#include "rt_tensor.hpp"

namespace rt {

class Expr {
  public:
    explicit Expr(const Tensor& start) { inputs_.push_back(start); }

    Expr unary(int op) const { return with(Step{RT_CHAIN_UNARY, op, 0, Scalar{}}); }
    Expr scalar(int op, const Scalar& v) const { return with(Step{RT_CHAIN_SCALAR, op, 0, v}); }
    Expr scalar(int op, double v) const { return scalar(op, Scalar::from_double(inputs_[0].dtype(), v)); }
    // acc op rhs / lhs op acc
    Expr binary(BinaryOpType op, const Tensor& rhs) const { return with_operand(RT_CHAIN_BINARY, op, rhs); }
    Expr binary_rev(BinaryOpType op, const Tensor& lhs) const { return with_operand(RT_CHAIN_BINARY_REV, op, lhs); }

    Expr operator+(double s) const { return scalar(RT_S_ADD, s); }
    Expr operator-(double s) const { return scalar(RT_S_SUB, s); }
    Expr operator*(double s) const { return scalar(RT_S_MUL, s); }
    Expr operator/(double s) const { return scalar(RT_S_DIV, s); }
    Expr operator+(const Tensor& t) const { return binary(BinaryOpType::Add, t); }
    Expr operator-(const Tensor& t) const { return binary(BinaryOpType::Sub, t); }
    Expr operator*(const Tensor& t) const { return binary(BinaryOpType::Mul, t); }
    Expr operator/(const Tensor& t) const { return binary(BinaryOpType::Div, t); }
    Expr relu() const { return unary(RT_U_RELU); }
    Expr abs() const { return unary(RT_U_ABS); }
    Expr neg() const { return unary(RT_U_NEG); }
    Expr leaky_relu(double slope) const { return scalar(RT_S_LEAKY_RELU, slope); }

    size_t steps() const { return steps_.size(); }

    // The value of the expression as a new row-major tensor.  `fused_launches` (optional) receives the number of rt_fused_chain
    // launches that were issued: 0 means every step went through the ordinary operators.
    Tensor eval(int* fused_launches = nullptr) const {
        int launches = 0;
        Tensor cur = inputs_[0];
        bool owned = false;                                   // `cur` is a temporary of this evaluation: later steps may overwrite it
        size_t s = 0;
        while (s < steps_.size()) {
            size_t taken = 0;
            if (try_fused(cur, owned, s, &taken)) {
                launches += 1;
                owned = true;
                s += taken;
                continue;
            }
            apply_one(cur, owned, steps_[s]);
            owned = true;
            s += 1;
        }
        if (!owned) cur = cur.owned();                        // an expression without steps is a copy
        if (fused_launches) *fused_launches = launches;
        return cur;
    }

  private:
    struct Step { int kind, op, operand; Scalar value; };

    Expr with(const Step& st) const {
        Expr e = *this;
        e.steps_.push_back(st);
        return e;
    }
    Expr with_operand(int kind, BinaryOpType op, const Tensor& t) const {
        if (t.dtype() != inputs_[0].dtype()) throw TensorError(ErrorKind::UnsupportedOperation, "operands of one expression share a dtype");
        Expr e = *this;
        int k = -1;
        for (size_t i = 0; i < e.inputs_.size(); ++i)
            if (e.inputs_[i].buf().get() == t.buf().get() && e.inputs_[i].meta().shape == t.meta().shape && e.inputs_[i].meta().strides == t.meta().strides &&
                e.inputs_[i].offset() == t.offset())
                k = (int)i;
        if (k < 0) { e.inputs_.push_back(t); k = (int)e.inputs_.size() - 1; }
        e.steps_.push_back(Step{kind, (int)op, k, Scalar{}});
        return e;
    }

    static bool is_run(const Tensor& t) { return t.size() > 0 && t.meta().is_forward_contiguous(); }

    // Steps [s, s + taken) as one rt_fused_chain launch from `cur`; false when the next step does not fit the fused form.
    bool try_fused(Tensor& cur, bool owned, size_t s, size_t* taken) const {
        if (!is_run(cur)) return false;
        const int dtype = cur.dtype();
        if (dtype == RT_BOOL || dtype == RT_U128 || dtype == RT_I128) return false;
        std::vector<const Tensor*> ins{&cur};
        std::vector<rt_chain_step> prog;
        std::vector<size_t> ins_after;                        // inputs in use after each step: they are appended in order of first use
        size_t k = s;
        for (; k < steps_.size() && prog.size() < RT_CHAIN_MAX_STEPS; ++k) {
            const Step& st = steps_[k];
            rt_chain_step cs;
            std::memset(&cs, 0, sizeof(cs));
            cs.kind = st.kind;
            cs.op = st.op;
            if (st.kind == RT_CHAIN_BINARY || st.kind == RT_CHAIN_BINARY_REV) {
                const Tensor& other = inputs_[(size_t)st.operand];
                // same shape, no broadcasting, a forward run: otherwise the step needs the broadcast kernel
                if (other.meta().shape != cur.meta().shape || !is_run(other)) break;
                int idx = -1;
                for (size_t i = 1; i < ins.size(); ++i)
                    if (ins[i] == &other) idx = (int)i;
                // operand 0 of the expression is `cur` only while no step has run yet
                if (idx < 0 && st.operand == 0 && s == 0 && !owned) idx = 0;
                if (idx < 0) {
                    if (ins.size() == RT_CHAIN_MAX_INPUTS) break;
                    ins.push_back(&other);
                    idx = (int)ins.size() - 1;
                }
                cs.operand = idx;
            } else if (st.kind == RT_CHAIN_SCALAR) {
                std::memcpy(cs.value, st.value.bytes, 8);
            }
            prog.push_back(cs);
            ins_after.push_back(ins.size());
        }
        if (prog.empty()) return false;
        // the first launch of an expression writes a fresh tensor; later ones overwrite the temporary in place
        Tensor dst = owned ? cur : cur.like_row_major();
        while (!prog.empty()) {
            ins.resize(ins_after[prog.size() - 1]);           // an input that only dropped steps name is not read
            std::vector<const void*> ptrs;
            std::vector<uint64_t> lens, starts;
            for (const Tensor* t : ins) { ptrs.push_back(t->buf()->ptr()); lens.push_back(t->buf()->len()); starts.push_back(t->offset()); }
            const int32_t st = rt_fused_chain(cur.backend().raw(), dtype, (int32_t)ins.size(), ptrs.data(), lens.data(), starts.data(), cur.size(),
                                              (int32_t)prog.size(), prog.data(), dst.buf()->ptr(), dst.buf()->len(), dst.offset());
            if (st == RT_OK) {
                cur = dst;
                *taken = prog.size();
                return true;
            }
            if (st != RT_E_DTYPE) check(st);
            prog.pop_back();                                  // the last step is not available in a chain: fuse the steps before it
        }
        return false;
    }

    // one step through the ordinary operators (value-returning the first time, in place on the temporary afterwards)
    void apply_one(Tensor& cur, bool owned, const Step& st) const {
        switch (st.kind) {
            case RT_CHAIN_UNARY:
                if (owned) cur.unary_inplace(st.op); else cur = cur.unary(st.op);
                break;
            case RT_CHAIN_SCALAR:
                if (owned) cur.scalar_assign(st.op, st.value); else cur = cur.scalar(st.op, st.value);
                break;
            case RT_CHAIN_BINARY:
                cur = cur.binary(inputs_[(size_t)st.operand], (BinaryOpType)st.op);
                break;
            default:
                cur = inputs_[(size_t)st.operand].binary(cur, (BinaryOpType)st.op);
                break;
        }
    }

    std::vector<Tensor> inputs_;          // inputs_[0] is where the expression starts
    std::vector<Step> steps_;
};

inline Expr lazy(const Tensor& t) { return Expr(t); }

}  // namespace rt
