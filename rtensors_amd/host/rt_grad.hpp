// Reverse-mode tape for the broadcast/reduce training step (no matmul): y = relu(x + bias), loss = mean_l1_loss(y, t),
// backward to d(bias), SGD update.  Follows the reference's engine: grad/mod.rs:269-308 (context, attach), 432-495
// (backwards: toposort, upstream accumulation), grad/backwards.rs:7-42, 148-161, 229-239, 516-538 (node rules),
// ops/broadcast/l1.rs:16-84 (L1 loss and its gradient map), ops/unary/mod.rs:234-252 (ReLU gradient map),
// grad/optim.rs:28-50 (SGD).  Every arithmetic step is a backend call issued through rt::Tensor.
#pragma once

#include <map>
#include <memory>
#include <set>
#include <vector>

#include "rt_tensor.hpp"

namespace rt {
namespace grad {

// How `inverse_broadcast_gradient` treats a broadcast dim.
//   Sum              : d(operand) = sum of the upstream gradient over the dim (what the function's own doc comment and
//                      the maths say).
//   ReferenceLiteral : what grad/backwards.rs:527 executes -- `grad.meta = grad.sum_at(dim)?.meta`: the sum is computed,
//                      its buffer dropped, and only its metadata kept, so the stored gradient is the first slice of the
//                      upstream buffer.  Kept so the divergence can be shown in a test.
enum class BroadcastGradMode { Sum, ReferenceLiteral };

enum class NodeKind { None, Leaf, BroadcastAdd, BroadcastSub, ReLU, L1, MatMul };

struct Node {
    NodeKind kind = NodeKind::None;
    std::vector<int> parents;            // -1 = no gradient flows there (GradNode::None sentinel)
    Strides lhs_strides, rhs_strides;    // BroadcastAdd / BroadcastSub
    Shape lhs_shape, rhs_shape;
    Tensor grad_map;                     // ReLU, L1
    Tensor left_input, right_input;      // MatMul (row-major copies, ops/linalg/matmul.rs:126-130)
    Tensor loss;                         // L1
    std::shared_ptr<Tensor> grad;        // Leaf: accumulated gradient (null until the first backward pass)
};

struct Var {
    Tensor t;
    int node = -1;
};

class GradContext {
  public:
    BroadcastGradMode mode = BroadcastGradMode::Sum;
    bool seed_with_loss = true;   // grad/mod.rs:442-447 seeds the root with the loss tensor itself, not with 1

    Var input(const Tensor& t) { return Var{t, -1}; }
    Var param(const Tensor& t) {                        // TensorBase::param + GradNode::Leaf
        Node n;
        n.kind = NodeKind::Leaf;
        nodes_.push_back(n);
        return Var{t, (int)nodes_.size() - 1};
    }

    // ops/broadcast/add.rs:173-208 + attach_broadcast_add_grad (586-607)
    Var add(const Var& a, const Var& b) { return broadcast(a, b, BinaryOpType::Add, NodeKind::BroadcastAdd); }
    Var sub(const Var& a, const Var& b) { return broadcast(a, b, BinaryOpType::Sub, NodeKind::BroadcastSub); }

    // ops/unary/mod.rs:114-126 (relu = owned + relu_inplace) with the gradient map of 234-252: 1 where input > 0
    Var relu(const Var& a) {
        Tensor result = a.t.relu();
        if (a.node < 0) return Var{result, -1};
        Tensor gmap = a.t.unary(RT_U_STEP);
        Node n;
        n.kind = NodeKind::ReLU;
        n.parents = {a.node};
        n.grad_map = gmap;
        nodes_.push_back(n);
        return Var{result, (int)nodes_.size() - 1};
    }

    // ops/scalar/mod.rs:149-166: leaky_relu shares GradNode::ReLU; its map is 1 where input > 0 and the slope elsewhere
    Var leaky_relu(const Var& a, double slope) {
        Tensor result = a.t.scalar(RT_S_LEAKY_RELU, slope);
        if (a.node < 0) return Var{result, -1};
        return map_node(result, a.t.scalar(RT_S_LEAKY_GRAD, slope), a.node);
    }

    // ops/unary/mod.rs:213-232: Abs keeps a map of +1 where input > 0 and -1 elsewhere; backwards_abs (backwards.rs:267-276)
    // multiplies it into the upstream gradient exactly as backwards_relu does
    Var abs(const Var& a) {
        Tensor result = a.t.abs();
        if (a.node < 0) return Var{result, -1};
        return map_node(result, a.t.unary(RT_U_ABS_GRAD), a.node);
    }

    // ops/linalg/matmul.rs:5-139 + attach_matmul_grad (182-198): the node keeps contiguous copies of both inputs
    Var matmul(const Var& a, const Var& b) {
        Tensor result = a.t.matmul(b.t);
        if (a.node < 0 && b.node < 0) return Var{result, -1};
        Node n;
        n.kind = NodeKind::MatMul;
        n.parents = {a.node, b.node};
        n.left_input = a.t.contiguous();
        n.right_input = b.t.contiguous();
        nodes_.push_back(n);
        return Var{result, (int)nodes_.size() - 1};
    }

    // ops/broadcast/l1.rs:49-84 with ReductionType::Mean
    Var mean_l1_loss(const Var& y, const Var& target) {
        Tensor diff = y.t - target.t;
        Tensor gmap = diff.sign();
        diff.abs_inplace();
        Tensor loss = diff.mean();
        // attach_l1_grad (l1.rs:16-46): grad_map = sign(gmap) / T::from_usize(N), from_usize going through f32.  gmap is
        // already a sign map and sign(sign(x)) == sign(x) bit for bit (-1, +0, +1; NaN and -0.0 went to +0 the first time),
        // so the second sign pass is not issued.
        Tensor grad_map = gmap / (double)(float)diff.size();
        Node n;
        n.kind = NodeKind::L1;
        n.parents = {y.node, target.node};
        n.grad_map = grad_map;
        n.loss = loss;
        nodes_.push_back(n);
        return Var{loss, (int)nodes_.size() - 1};
    }

    // grad/mod.rs:432-495
    void backwards(const Var& root) {
        if (root.node < 0 || nodes_[(size_t)root.node].kind != NodeKind::L1)
            throw TensorError(ErrorKind::GradError, "Root node does not contain a loss.");
        std::vector<int> order;
        std::set<int> seen;
        toposort(root.node, seen, order);
        std::map<int, std::vector<Tensor>> acc;
        const Tensor& loss = nodes_[(size_t)root.node].loss;
        acc[root.node].push_back(seed_with_loss ? loss.owned() : Tensor::ones(loss.backend(), loss.dtype(), loss.shape()));
        for (size_t i = order.size(); i-- > 0;) {
            const int key = order[i];
            std::vector<Tensor>& ups = acc[key];
            if (ups.empty()) continue;
            Tensor dldy = ups[0];
            for (size_t k = 1; k < ups.size(); ++k) dldy = dldy + ups[k];
            Node& n = nodes_[(size_t)key];
            std::vector<Tensor> down = node_backwards(n, dldy);
            for (size_t p = 0; p < n.parents.size() && p < down.size(); ++p)
                if (n.parents[p] >= 0) acc[n.parents[p]].push_back(down[p]);
            acc.erase(key);
        }
    }

    std::shared_ptr<Tensor> grad_of(const Var& v) const { return v.node >= 0 ? nodes_[(size_t)v.node].grad : nullptr; }
    void clear_grad(const Var& v) { if (v.node >= 0) nodes_[(size_t)v.node].grad.reset(); }

  private:
    Var broadcast(const Var& a, const Var& b, BinaryOpType op, NodeKind kind) {
        Tensor result = a.t.binary(b.t, op);
        if (a.node < 0 && b.node < 0) return Var{result, -1};
        BroadcastParams p = compute_broadcasted_params(a.t.meta(), b.t.meta());
        Node n;
        n.kind = kind;
        n.parents = {a.node, b.node};
        n.lhs_strides = p.a;
        n.rhs_strides = p.b;
        n.lhs_shape = a.t.shape();
        n.rhs_shape = b.t.shape();
        nodes_.push_back(n);
        return Var{result, (int)nodes_.size() - 1};
    }

    void toposort(int key, std::set<int>& seen, std::vector<int>& order) {
        if (key < 0 || seen.count(key)) return;
        seen.insert(key);
        for (int p : nodes_[(size_t)key].parents) toposort(p, seen, order);
        order.push_back(key);
    }

    // grad/backwards.rs:516-538
    void inverse_broadcast_gradient(Tensor& g, const Strides& strides, const Shape& shape) const {
        const size_t differential = g.rank() - shape.size();
        for (size_t dim = 0; dim < strides.size(); ++dim) {
            if (strides[dim] != 0) continue;
            Tensor summed = g.sum_at(dim);
            if (mode == BroadcastGradMode::Sum) g = summed;
            else g.set_meta(summed.meta());
        }
        for (size_t dim = strides.size(); dim-- > 0;) {
            if (strides[dim] == 0 && (dim < differential || shape[dim - differential] != 1)) {
                Tensor sq = g.squeeze_at(dim);
                g.set_meta(sq.meta());
            }
        }
    }

    Var map_node(const Tensor& result, const Tensor& gmap, int parent) {
        Node n;
        n.kind = NodeKind::ReLU;
        n.parents = {parent};
        n.grad_map = gmap;
        nodes_.push_back(n);
        return Var{result, (int)nodes_.size() - 1};
    }

    std::vector<Tensor> node_backwards(Node& n, const Tensor& up) {
        switch (n.kind) {
            case NodeKind::Leaf:                                         // accumulate_grad, backwards.rs:7-25
                if (n.grad) *n.grad += up;
                else n.grad = std::make_shared<Tensor>(up.owned());
                return {};
            case NodeKind::L1: {                                         // backwards_l1, backwards.rs:148-161
                std::vector<Tensor> out(2);
                if (n.parents[0] >= 0) out[0] = n.grad_map * up;
                if (n.parents[1] >= 0) out[1] = (-n.grad_map) * up;
                return out;
            }
            case NodeKind::ReLU:                                         // backwards_relu, backwards.rs:229-239
                return {n.grad_map * up};
            case NodeKind::BroadcastAdd:                                 // backwards_add / backwards_sub, backwards.rs:27-60
            case NodeKind::BroadcastSub: {
                std::vector<Tensor> out(2);
                // The reference clones the upstream gradient first (backwards.rs:36-37).  Nothing downstream writes into a
                // gradient it was handed (the leaf accumulates into its own buffer), so the handle is shared instead.
                if (n.parents[0] >= 0) { out[0] = up; inverse_broadcast_gradient(out[0], n.lhs_strides, n.lhs_shape); }
                if (n.parents[1] >= 0) {
                    out[1] = n.kind == NodeKind::BroadcastSub ? -up : up;
                    inverse_broadcast_gradient(out[1], n.rhs_strides, n.rhs_shape);
                }
                return out;
            }
            case NodeKind::MatMul: {                                     // backwards_matmul, backwards.rs:493-510
                // d(lhs) = upstream @ rhs^T, d(rhs) = lhs^T @ upstream; only the last two dims are swapped
                auto swap_last_two = [](const Tensor& t) {
                    std::vector<size_t> dims(t.rank());
                    for (size_t i = 0; i < dims.size(); ++i) dims[i] = i;
                    std::swap(dims[dims.size() - 1], dims[dims.size() - 2]);
                    return t.permute(dims);
                };
                std::vector<Tensor> out(2);
                if (n.parents[0] >= 0) out[0] = up.matmul(swap_last_two(n.right_input));
                if (n.parents[1] >= 0) out[1] = swap_last_two(n.left_input).matmul(up);
                return out;
            }
            default:
                return {};
        }
    }

    std::vector<Node> nodes_;
};

// The training step y = relu(x + bias), loss = mean_l1_loss(y, target), backward to d(bias) in three fused passes instead of the
// eleven the tape above issues (one per arithmetic step, each with a full-size temporary): 7 x the tensor size of traffic instead
// of about 22 x.  The element-wise results and the products that are summed are bit for bit those of the tape; the loss and d(bias)
// are tree sums of the same terms.  Takes whole row-major tensors (x and target (rows, cols), bias (cols)); anything else -- views,
// other dtypes than f32 / f64, rows that are not whole 16-byte vectors -- is for the tape.
struct FusedStep {
    Tensor y, loss, dbias;
};
inline bool fused_step_applies(const Tensor& x, const Tensor& bias, const Tensor& target) {
    const int dt = x.dtype();
    if ((dt != RT_F32 && dt != RT_F64) || bias.dtype() != dt || target.dtype() != dt) return false;
    if (x.rank() != 2 || bias.rank() != 1 || target.shape() != x.shape() || bias.shape()[0] != x.shape()[1]) return false;
    const uint64_t vec = dt == RT_F32 ? 4 : 2;
    if (x.shape()[1] % vec != 0 || x.size() == 0) return false;
    auto whole = [](const Tensor& t) { return t.offset() == 0 && t.is_contiguous() && t.strides().back() == 1 && t.size() == t.buf()->len(); };
    return whole(x) && whole(bias) && whole(target);
}
// passes == 3: y, then the loss and the stored gradient map, then d(bias) from the map (7 passes over a tensor).  passes == 2 (default):
// y and the loss together, then d(bias) from y and the target with the map's elements formed in registers (5 passes).  The map is a
// temporary of the tape (ops/broadcast/l1.rs:58-60), not a result; every value that is summed is the same bits either way.
inline FusedStep fused_bias_relu_l1_step(const Tensor& x, const Tensor& bias, const Tensor& target, bool seed_with_loss, int passes = 2) {
    const Hip& be = x.backend();
    const int dt = x.dtype();
    const uint64_t rows = x.shape()[0], cols = x.shape()[1], n = rows * cols;
    FusedStep out;
    Buf y = be.alloc_uninit(dt, n), loss = be.alloc_uninit(dt, 1), gmap;
    if (passes == 3) {
        be.fused_bias_relu(*x.buf(), *bias.buf(), *y, rows, cols);
        gmap = be.alloc_uninit(dt, n);
        be.fused_l1_forward(*y, *target.buf(), *gmap, *loss, n);
    } else {
        be.fused_bias_relu_l1(*x.buf(), *bias.buf(), *target.buf(), *y, *loss, rows, cols);
    }
    out.y = Tensor(be, y, MetaTensor::row_major(x.shape()));
    out.loss = Tensor(be, loss, MetaTensor::row_major(Shape{}));
    // grad/mod.rs:442-447 seeds the root with the loss tensor itself
    Tensor seed = seed_with_loss ? out.loss : Tensor::ones(be, dt, Shape{});
    Buf dbias = be.alloc_uninit(dt, cols);
    if (passes == 3) be.fused_l1_relu_backward(*gmap, *y, *seed.buf(), *dbias, rows, cols);
    else be.fused_l1_relu_backward_t(*y, *target.buf(), *seed.buf(), *dbias, rows, cols);
    out.dbias = Tensor(be, dbias, MetaTensor::row_major(Shape{cols}));
    return out;
}

// grad/optim.rs:14-50
class SGD {
  public:
    explicit SGD(double learning_rate) : lr_(learning_rate) {}
    void register_parameter(GradContext& ctx, Var& param) {
        if (param.node < 0) throw TensorError(ErrorKind::GradError, "Only leaf tensors can be registered as parameters.");
        ctx_ = &ctx;
        params_.push_back(&param);
    }
    void step() {
        for (Var* p : params_) {
            std::shared_ptr<Tensor> g = ctx_->grad_of(*p);
            if (!g) continue;
            Tensor update = *g * lr_;           // grad * lr: owned copy + in-place scalar mul, rounded to T
            ctx_->clear_grad(*p);
            Tensor v = p->t.view();
            v -= update;                        // in-place broadcast sub through a mutable view
        }
    }
  private:
    double lr_;
    GradContext* ctx_ = nullptr;
    std::vector<Var*> params_;
};

}  // namespace grad
}  // namespace rt
