// C entry points over the C++ host layer (rt::Tensor, rt::grad) so that it can be driven from a test harness in
// another language.  Handles are heap-allocated rt::Tensor / rt::Hip objects.  Every function returns 0 on success or
// 1 + ErrorKind on failure; rth_last_error() has the message.  The rth_meta_* functions are pure host arithmetic.
#include <cstring>
#include <string>

#include "rt_expr.hpp"
#include "rt_grad.hpp"

using namespace rt;

static thread_local std::string g_err;

template <class F> static int guarded(F f) {
    try {
        f();
        return 0;
    } catch (const TensorError& e) {
        g_err = e.what();
        return 1 + (int)e.kind;
    } catch (const std::exception& e) {
        g_err = e.what();
        return 1 + (int)ErrorKind::HipError;
    }
}

static Slice make_slice(int has_start, uint64_t start, int has_end, uint64_t end, int64_t step) {
    Slice s;
    if (has_start) s.start = start;
    if (has_end) s.end = end;
    s.step = step;
    return s;
}

static MetaTensor make_meta(int rank, const uint64_t* shape, const int64_t* strides, uint64_t offset) {
    return MetaTensor(Shape(shape, shape + rank), Strides(strides, strides + rank), offset);
}

static void put_meta(const MetaTensor& m, int* rank, uint64_t* shape, int64_t* strides, uint64_t* offset) {
    *rank = (int)m.rank();
    for (size_t i = 0; i < m.rank(); ++i) { shape[i] = m.shape[i]; strides[i] = m.strides[i]; }
    *offset = m.offset;
}

extern "C" {

const char* rth_last_error() { return g_err.c_str(); }

// ---- metadata only ----------------------------------------------------------------------------------------------------
int rth_meta_slice(int rank, const uint64_t* shape, const int64_t* strides, uint64_t offset, uint64_t dim, int has_start, uint64_t start,
                   int has_end, uint64_t end, int64_t step, int* orank, uint64_t* oshape, int64_t* ostrides, uint64_t* ooffset) {
    return guarded([&] { put_meta(compute_sliced_parameters(make_meta(rank, shape, strides, offset), dim, make_slice(has_start, start, has_end, end, step)),
                                  orank, oshape, ostrides, ooffset); });
}
int rth_meta_permute(int rank, const uint64_t* shape, const int64_t* strides, uint64_t offset, int ndims, const uint64_t* dims,
                     int* orank, uint64_t* oshape, int64_t* ostrides, uint64_t* ooffset) {
    return guarded([&] { put_meta(compute_permuted_parameters(make_meta(rank, shape, strides, offset), std::vector<size_t>(dims, dims + ndims)),
                                  orank, oshape, ostrides, ooffset); });
}
int rth_meta_unsqueeze(int rank, const uint64_t* shape, const int64_t* strides, uint64_t offset, uint64_t dim,
                       int* orank, uint64_t* oshape, int64_t* ostrides, uint64_t* ooffset) {
    return guarded([&] { put_meta(compute_unsqueezed_parameters(make_meta(rank, shape, strides, offset), dim), orank, oshape, ostrides, ooffset); });
}
int rth_meta_squeeze(int rank, const uint64_t* shape, const int64_t* strides, uint64_t offset, int64_t dim,
                     int* orank, uint64_t* oshape, int64_t* ostrides, uint64_t* ooffset) {
    return guarded([&] {
        put_meta(compute_squeezed_parameters(make_meta(rank, shape, strides, offset), dim < 0 ? std::nullopt : std::optional<size_t>((size_t)dim)),
                 orank, oshape, ostrides, ooffset);
    });
}
int rth_meta_broadcast(int ranka, const uint64_t* shapea, const int64_t* stridesa, int rankb, const uint64_t* shapeb, const int64_t* stridesb,
                       int* orank, uint64_t* oshape, int64_t* ostra, int64_t* ostrb) {
    return guarded([&] {
        BroadcastParams p = compute_broadcasted_params(make_meta(ranka, shapea, stridesa, 0), make_meta(rankb, shapeb, stridesb, 0));
        *orank = (int)p.shape.size();
        for (size_t i = 0; i < p.shape.size(); ++i) { oshape[i] = p.shape[i]; ostra[i] = p.a[i]; ostrb[i] = p.b[i]; }
    });
}
int rth_meta_contiguity_type(int rank, const uint64_t* shape, const int64_t* strides) { return (int)contiguity_type(make_meta(rank, shape, strides, 0)); }
int rth_meta_is_contiguous(int rank, const uint64_t* shape, const int64_t* strides) { return make_meta(rank, shape, strides, 0).is_contiguous() ? 1 : 0; }

// ---- backend / tensors ---------------------------------------------------------------------------------------------------
int rth_backend_create(int device, void** out) { return guarded([&] { *out = new Hip(device); }); }
void rth_backend_destroy(void* b) { delete (Hip*)b; }
int rth_backend_sync(void* b) { return guarded([&] { ((Hip*)b)->sync(); }); }

int rth_from_buf(void* backend, int dtype, const void* host, uint64_t len, int rank, const uint64_t* shape, void** out) {
    return guarded([&] { *out = new Tensor(Tensor::from_buf(*(Hip*)backend, dtype, host, len, Shape(shape, shape + rank))); });
}
int rth_zeros(void* backend, int dtype, int rank, const uint64_t* shape, void** out) {
    return guarded([&] { *out = new Tensor(Tensor::zeros(*(Hip*)backend, dtype, Shape(shape, shape + rank))); });
}
int rth_ones(void* backend, int dtype, int rank, const uint64_t* shape, void** out) {
    return guarded([&] { *out = new Tensor(Tensor::ones(*(Hip*)backend, dtype, Shape(shape, shape + rank))); });
}
int rth_limit(void* backend, int dtype, int highest, int rank, const uint64_t* shape, void** out) {
    return guarded([&] {
        Shape sh(shape, shape + rank);
        *out = new Tensor(highest ? Tensor::max(*(Hip*)backend, dtype, sh) : Tensor::min(*(Hip*)backend, dtype, sh));
    });
}
int rth_into_dtype(void* t, int dtype, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)t)->into_dtype(dtype)); }); }
void rth_free(void* t) { delete (Tensor*)t; }

int rth_info(void* t, int* rank, uint64_t* shape, int64_t* strides, uint64_t* offset, int* dtype, int* is_view, int* contiguous, uint64_t* buf_len) {
    return guarded([&] {
        Tensor* x = (Tensor*)t;
        put_meta(x->meta(), rank, shape, strides, offset);
        *dtype = x->dtype(); *is_view = x->is_view(); *contiguous = x->is_contiguous(); *buf_len = x->buf()->len();
    });
}
int rth_slice(void* t, uint64_t dim, int has_start, uint64_t start, int has_end, uint64_t end, int64_t step, void** out) {
    return guarded([&] { *out = new Tensor(((Tensor*)t)->slice(dim, make_slice(has_start, start, has_end, end, step))); });
}
int rth_permute(void* t, int n, const uint64_t* dims, void** out) {
    return guarded([&] { *out = new Tensor(((Tensor*)t)->permute(std::vector<size_t>(dims, dims + n))); });
}
int rth_transpose(void* t, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)t)->transpose()); }); }
int rth_unsqueeze(void* t, uint64_t dim, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)t)->unsqueeze_at(dim)); }); }
int rth_squeeze(void* t, int64_t dim, void** out) {
    return guarded([&] { *out = new Tensor(dim < 0 ? ((Tensor*)t)->squeeze() : ((Tensor*)t)->squeeze_at((size_t)dim)); });
}
int rth_view_as(void* t, int rank, const uint64_t* shape, void** out) {
    return guarded([&] { *out = new Tensor(((Tensor*)t)->view_as(Shape(shape, shape + rank))); });
}
int rth_reshape(void* t, int rank, const uint64_t* shape, void** out) {
    return guarded([&] { *out = new Tensor(((Tensor*)t)->reshape(Shape(shape, shape + rank))); });
}
int rth_owned(void* t, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)t)->owned()); }); }
int rth_contiguous(void* t, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)t)->contiguous()); }); }

int rth_binary(void* a, void* b, int op, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)a)->binary(*(Tensor*)b, (BinaryOpType)op)); }); }
int rth_binary_assign(void* a, void* b, int op) { return guarded([&] { ((Tensor*)a)->binary_assign(*(Tensor*)b, (BinaryOpType)op); }); }
int rth_matmul(void* a, void* b, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)a)->matmul(*(Tensor*)b)); }); }
int rth_dot(void* a, void* b, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)a)->dot(*(Tensor*)b)); }); }
int rth_outer(void* a, void* b, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)a)->outer(*(Tensor*)b)); }); }
int rth_scalar(void* a, int op, double v, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)a)->scalar(op, v)); }); }
int rth_scalar_assign(void* a, int op, double v) { return guarded([&] { ((Tensor*)a)->scalar_assign(op, v); }); }
int rth_unary(void* a, int op, void** out) { return guarded([&] { *out = new Tensor(((Tensor*)a)->unary(op)); }); }
int rth_unary_inplace(void* a, int op) { return guarded([&] { ((Tensor*)a)->unary_inplace(op); }); }
int rth_reduce(void* a, int op, int64_t axis, void** out) {
    return guarded([&] { *out = new Tensor(((Tensor*)a)->reduce((ReductionOpTypes)op, axis < 0 ? std::nullopt : std::optional<size_t>((size_t)axis))); });
}
int rth_fill(void* a, double v) { return guarded([&] { Tensor* t = (Tensor*)a; t->fill(Scalar::from_double(t->dtype(), v)); }); }
int rth_get(void* a, int n, const uint64_t* idx, double* out) {
    return guarded([&] { *out = ((Tensor*)a)->get(std::vector<uint64_t>(idx, idx + n)).to_double(); });
}
int rth_set(void* a, int n, const uint64_t* idx, double v) {
    return guarded([&] { Tensor* t = (Tensor*)a; t->set(std::vector<uint64_t>(idx, idx + n), Scalar::from_double(t->dtype(), v)); });
}
int rth_to_host(void* a, void* dst) { return guarded([&] { ((Tensor*)a)->to_host(dst); }); }
int rth_dump_buffer(void* a, void* dst) { return guarded([&] { ((Tensor*)a)->dump_buffer(dst); }); }
int rth_equals(void* a, void* b, int* out) { return guarded([&] { *out = ((Tensor*)a)->equals(*(Tensor*)b) ? 1 : 0; }); }

// ---- expressions -----------------------------------------------------------------------------------------------------------
// An elementwise expression starting at `first`: step k is (kinds[k], ops[k]) with values[k] for a scalar step and operands[k] (a tensor
// handle) for a binary one; kinds are rt_chain_kind.  Evaluated through rt::Expr: fused launches where the operands allow, the ordinary
// operators elsewhere.  *out_fused receives the number of fused launches.
int rth_expr_eval(void* first, int nsteps, const int* kinds, const int* ops, const double* values, void* const* operands, void** out, int* out_fused) {
    return guarded([&] {
        Expr e(*(Tensor*)first);
        for (int k = 0; k < nsteps; ++k) {
            switch (kinds[k]) {
                case RT_CHAIN_UNARY: e = e.unary(ops[k]); break;
                case RT_CHAIN_SCALAR: e = e.scalar(ops[k], values[k]); break;
                case RT_CHAIN_BINARY: e = e.binary((BinaryOpType)ops[k], *(Tensor*)operands[k]); break;
                case RT_CHAIN_BINARY_REV: e = e.binary_rev((BinaryOpType)ops[k], *(Tensor*)operands[k]); break;
                default: throw TensorError(ErrorKind::UnsupportedOperation, "unknown step kind");
            }
        }
        int fused = 0;
        *out = new Tensor(e.eval(&fused));
        if (out_fused) *out_fused = fused;
    });
}

// ---- the training step of the autograd configuration -----------------------------------------------------------------------
// y = relu(x + bias); loss = mean_l1_loss(y, target); backward; SGD(lr) on bias (updated in place).
// mode: 0 = sum over the broadcast dim, 1 = reference-literal metadata rewrite.  seed_with_loss: 1 = the reference's
// root seed (the loss value), 0 = seed 1.  Outputs: loss tensor and the gradient that was applied to bias.
int rth_train_step(void* x, void* bias, void* target, double lr, int mode, int seed_with_loss, void** out_loss, void** out_grad) {
    return guarded([&] {
        grad::GradContext ctx;
        ctx.mode = mode == 0 ? grad::BroadcastGradMode::Sum : grad::BroadcastGradMode::ReferenceLiteral;
        ctx.seed_with_loss = seed_with_loss != 0;
        grad::Var vx = ctx.input(*(Tensor*)x);
        grad::Var vb = ctx.param(*(Tensor*)bias);
        grad::Var vt = ctx.input(*(Tensor*)target);
        grad::SGD opt(lr);
        opt.register_parameter(ctx, vb);
        grad::Var y = ctx.relu(ctx.add(vx, vb));
        grad::Var loss = ctx.mean_l1_loss(y, vt);
        ctx.backwards(loss);
        std::shared_ptr<Tensor> g = ctx.grad_of(vb);
        if (!g) throw TensorError(ErrorKind::GradError, "no gradient reached the parameter");
        *out_grad = new Tensor(g->contiguous());
        *out_loss = new Tensor(loss.t);
        opt.step();
    });
}

// The same step through the fused passes, two or three of them (seed_with_loss as above; the broadcast gradient is the sum).  Returns 1 through
// *out_used when the operands fit the fused form, else runs the tape and returns 0 there.
int rth_train_step_fused(void* x, void* bias, void* target, double lr, int seed_with_loss, int passes, void** out_loss, void** out_grad, int* out_used) {
    if (!grad::fused_step_applies(*(Tensor*)x, *(Tensor*)bias, *(Tensor*)target)) {
        *out_used = 0;
        return rth_train_step(x, bias, target, lr, 0, seed_with_loss, out_loss, out_grad);
    }
    *out_used = 1;
    return guarded([&] {
        grad::FusedStep st = grad::fused_bias_relu_l1_step(*(Tensor*)x, *(Tensor*)bias, *(Tensor*)target, seed_with_loss != 0, passes == 3 ? 3 : 2);
        *out_grad = new Tensor(st.dbias);
        *out_loss = new Tensor(st.loss);
        // SGD::step (grad/optim.rs:28-50): update = grad * lr, rounded to T, then an in-place broadcast sub through a mutable view
        Tensor update = st.dbias * lr;
        Tensor v = ((Tensor*)bias)->view();
        v -= update;
    });
}

// y = x @ w; loss = mean_l1_loss(y, target); backward; SGD(lr) on w (updated in place).  Outputs: loss and d(w).
int rth_linear_step(void* x, void* w, void* target, double lr, int seed_with_loss, void** out_loss, void** out_grad) {
    return guarded([&] {
        grad::GradContext ctx;
        ctx.seed_with_loss = seed_with_loss != 0;
        grad::Var vx = ctx.input(*(Tensor*)x);
        grad::Var vw = ctx.param(*(Tensor*)w);
        grad::Var vt = ctx.input(*(Tensor*)target);
        grad::SGD opt(lr);
        opt.register_parameter(ctx, vw);
        grad::Var loss = ctx.mean_l1_loss(ctx.matmul(vx, vw), vt);
        ctx.backwards(loss);
        std::shared_ptr<Tensor> g = ctx.grad_of(vw);
        if (!g) throw TensorError(ErrorKind::GradError, "no gradient reached the parameter");
        *out_grad = new Tensor(g->contiguous());
        *out_loss = new Tensor(loss.t);
        opt.step();
    });
}

}  // extern "C"
