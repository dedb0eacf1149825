// Host side of the device-resident tape: see tape.h. Plain C++ driving the
// kernels of elementwise.hip and the attention entry points of the C ABI.
#include "tape.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <unordered_map>

namespace pk {

namespace detail {
std::atomic<size_t> g_live_vars{0};
}
size_t live_variables() { return detail::g_live_vars.load(); }

// compute-dtype copies of a context's fp32 parameters, valid until the next optimizer step
struct TapeContext::Shadows {
    struct Cat {
        Tensor t;
        std::vector<const Variable*> ws;
    };
    std::unordered_map<const Variable*, Tensor> single;  // one weight
    std::unordered_map<const Variable*, Cat> cat;        // [W_0 | W_1 | ...], keyed by the first weight
};

// Weight-gradient products dW += X^T dY that the Linear closures of a running backward pass have handed in instead
// of multiplying at once. Each is a few dozen output tiles over a contraction as long as the token count; several
// of them fill the chip as one launch where each alone would have to cut its contraction into slices and add partial
// products afterwards. They are multiplied when eight have gathered and whenever a backward pass (a checkpointed
// segment's included) ends, so every parameter's gradient is complete when backward() returns.
struct TapeContext::Pending {
    struct Job {
        Tensor x, dy;           // [tokens, in], [tokens, columns of all the weights multiplied together]
        int64_t col0, ncols;    // this weight's columns of dy
        Var W;
    };
    std::vector<Job> jobs;
    int depth = 0;  // run_backward calls in progress
};

namespace {
thread_local bool g_recomputing = false;  // inside a checkpointed segment's re-run at backward time
thread_local bool g_grad_enabled = true;
thread_local TapeContext g_own_context;            // what a thread works on outside any ContextScope
thread_local TapeContext* g_context = nullptr;

TapeContext::Shadows& shadows() {
    TapeContext& c = tape_context();
    if (!c.shadows) c.shadows = std::make_shared<TapeContext::Shadows>();
    return *c.shadows;
}

const Tensor& shadow_of(const Var& W) {
    const int compute = tape_context().compute;
    if (compute == PK_F32 || W->data.dtype != PK_F32) return W->data;
    auto& map = shadows().single;
    auto it = map.find(W.get());
    if (it == map.end()) {
        Tensor t = Tensor::make(W->data.rows, W->data.cols, compute);
        k_cast(W->data, t);
        it = map.emplace(W.get(), std::move(t)).first;
    }
    return it->second;
}

const Tensor& shadow_cat(const std::vector<Var>& Ws) {
    auto& map = shadows().cat;
    auto it = map.find(Ws[0].get());
    if (it == map.end()) {
        const int64_t d = Ws[0]->data.cols;
        Tensor t = Tensor::make(Ws[0]->data.rows, d * static_cast<int64_t>(Ws.size()), tape_context().compute);
        std::vector<const Variable*> ws;
        for (size_t k = 0; k < Ws.size(); ++k) {
            k_cast_cols(Ws[k]->data, t, static_cast<int64_t>(k) * d);
            ws.push_back(Ws[k].get());
        }
        it = map.emplace(Ws[0].get(), TapeContext::Shadows::Cat{std::move(t), std::move(ws)}).first;
    }
    return it->second.t;
}

// The order the backward closures run in: the root first, every other node once all the nodes that consume it
// have run, so its gradient is complete by then. The reference gets such an order by reversing a depth-first
// post-order (src/autograd.cpp:31-45, 58-65); here the consumers of each node are counted first and a node is
// released when its count reaches zero, which needs no recursion either and visits each edge twice.
std::vector<Variable*> backward_order(const Var& root) {
    std::unordered_map<Variable*, int> consumers_left;
    std::vector<Variable*> frontier{root.get()};
    consumers_left[root.get()] = 0;
    while (!frontier.empty()) {
        Variable* n = frontier.back();
        frontier.pop_back();
        for (const Var& p : n->parents) {
            auto found = consumers_left.try_emplace(p.get(), 0);
            ++found.first->second;
            if (found.second) frontier.push_back(p.get());
        }
    }
    std::vector<Variable*> order;
    order.reserve(consumers_left.size());
    std::vector<Variable*> ready{root.get()};
    while (!ready.empty()) {
        Variable* n = ready.back();
        ready.pop_back();
        order.push_back(n);
        for (const Var& p : n->parents)
            if (--consumers_left[p.get()] == 0) ready.push_back(p.get());
    }
    return order;
}

TapeContext::Pending& pending() {
    TapeContext& c = tape_context();
    if (!c.pending) c.pending = std::make_shared<TapeContext::Pending>();
    return *c.pending;
}

void flush_weight_gradients() {
    auto& jobs = pending().jobs;
    size_t i = 0;
    while (i < jobs.size()) {
        // a run of jobs with one token count
        size_t j = i;
        GroupedProduct gp[8];
        while (j < jobs.size() && j - i < 8 && jobs[j].x.rows == jobs[i].x.rows) {
            const auto& job = jobs[j];
            Tensor& g = job.W->ensure_grad();
            gp[j - i] = GroupedProduct{job.x.ptr(), job.x.cols,
                                       static_cast<const char*>(job.dy.ptr()) + job.col0 * static_cast<int64_t>(job.dy.esize()),
                                       job.dy.cols, static_cast<float*>(g.ptr()), g.cols, job.x.cols, job.ncols};
            ++j;
        }
        const int64_t K = jobs[i].x.rows;
        if (!gemm_mfma_grouped_tn(gp, static_cast<int>(j - i), K, tape_stream())) {
            for (size_t k = 0; k < j - i; ++k)
                if (!gemm_mfma_bf16(gp[k].a, true, gp[k].lda, gp[k].b, false, gp[k].ldb, gp[k].c, PK_F32, gp[k].M, gp[k].N, K,
                                    gp[k].ldc, 1.0f, tape_stream()))
                    throw std::runtime_error("a deferred weight-gradient product was refused by the kernel it was queued for");
        }
        i = j;
    }
    jobs.clear();
}

// Whether dW += x^T dy[:, col0 : col0 + ncols] can wait in the queue: a backward pass is running and the product is one
// the hand-written kernel takes (bf16 operands, fp32 parameter gradient, aligned, a contraction worth grouping).
bool weight_gradient_can_wait(const Tensor& x, const Tensor& dy, int64_t col0, int64_t ncols, const Var& W) {
    if (pending().depth == 0 || gemm_backend() != 1) return false;
    if (x.dtype != PK_BF16 || dy.dtype != PK_BF16 || !W->is_param || x.rows != dy.rows || x.rows < 2048) return false;
    if (x.cols % 8 || dy.cols % 8 || col0 % 8 || ncols % 8 || W->data.rows != x.cols || W->data.cols != ncols) return false;
    return W->grad.empty() || W->grad.dtype == PK_F32;
}
void hold_weight_gradient(const Tensor& x, const Tensor& dy, int64_t col0, int64_t ncols, const Var& W) {
    auto& pd = pending();
    // a weight that is used twice must not meet itself in one launch: its two products would add into the same
    // gradient tiles at the same time
    bool again = false;
    for (const auto& job : pd.jobs) again = again || job.W.get() == W.get();
    if (again || pd.jobs.size() == 8) flush_weight_gradients();
    pd.jobs.push_back(TapeContext::Pending::Job{x, dy, col0, ncols, W});
}
bool defer_weight_gradient(const Tensor& x, const Tensor& dy, int64_t col0, int64_t ncols, const Var& W) {
    if (!weight_gradient_can_wait(x, dy, col0, ncols, W)) return false;
    hold_weight_gradient(x, dy, col0, ncols, W);
    return true;
}

void run_backward(const Var& root) {
    auto& pd = pending();
    ++pd.depth;
    try {
        for (Variable* n : backward_order(root))
            if (n->backward_fn && !n->grad.empty()) n->backward_fn();
        flush_weight_gradients();
    } catch (...) {
        pd.jobs.clear();
        --pd.depth;
        throw;
    }
    --pd.depth;
}

float scalar_to_host(const Tensor& t) {
    float h = 0.0f;
    if (t.dtype == PK_F32) {
        hip_check(hipMemcpyAsync(&h, t.ptr(), 4, hipMemcpyDeviceToHost, tape_stream()), "hipMemcpyAsync");
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
    } else {
        uint16_t u = 0;
        hip_check(hipMemcpyAsync(&u, t.ptr(), 2, hipMemcpyDeviceToHost, tape_stream()), "hipMemcpyAsync");
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
        uint32_t w = static_cast<uint32_t>(u) << 16;
        std::memcpy(&h, &w, 4);
    }
    return h;
}

// The gradient of a [1,1] node as a host value: 1 without asking the device where backward() seeded it and nothing
// has been added since (the usual case: the loss is the root), a copy back and a wait otherwise.
float upstream_scalar(const Variable* v) { return v->grad_is_unit ? 1.0f : scalar_to_host(v->grad); }

pk_tensor4 view4(const void* base, int64_t elem_off, size_t esize, int64_t sb, int64_t st, int64_t sh) {
    pk_tensor4 t;
    t.ptr = const_cast<char*>(static_cast<const char*>(base)) + elem_off * static_cast<int64_t>(esize);
    t.stride_b = sb;
    t.stride_t = st;
    t.stride_h = sh;
    return t;
}
void attn_check(int rc) {
    if (rc != PK_OK) throw Error(rc, pk_last_error());
}

}  // namespace

Tensor upload(const float* host, int64_t rows, int64_t cols, int dtype) {
    if (!host) throw Error(PK_ERR_ARGUMENT, "upload: null host pointer");
    Tensor staged = Tensor::make(rows, cols, PK_F32);
    hip_check(hipMemcpyAsync(staged.ptr(), host, sizeof(float) * rows * cols, hipMemcpyHostToDevice, tape_stream()),
              "hipMemcpyAsync");
    Tensor out = staged;
    if (dtype != PK_F32) {
        out = Tensor::make(rows, cols, dtype);
        k_cast(staged, out);
    }
    hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
    return out;
}

void download(const Tensor& t, float* host) {
    if (t.empty() || !host) throw Error(PK_ERR_ARGUMENT, "download: empty tensor or null host pointer");
    Tensor f = t;
    if (t.dtype != PK_F32) {
        f = Tensor::make(t.rows, t.cols, PK_F32);
        k_cast(t, f);
    }
    hip_check(hipMemcpyAsync(host, f.ptr(), sizeof(float) * t.rows * t.cols, hipMemcpyDeviceToHost, tape_stream()),
              "hipMemcpyAsync");
    hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
}

TapeContext& tape_context() { return g_context ? *g_context : g_own_context; }
ContextScope::ContextScope(TapeContext& c) : prev_(g_context) { g_context = &c; }
ContextScope::~ContextScope() { g_context = prev_; }

void set_compute_dtype(int dtype) {
    if (dtype != PK_F32 && dtype != PK_BF16) throw std::runtime_error("compute dtype must be PK_F32 or PK_BF16");
    tape_context().compute = dtype;
    tape_context().shadows.reset();
}
int compute_dtype() { return tape_context().compute; }
void invalidate_shadows() { tape_context().shadows.reset(); }
// The copies are brought up to date where they lie instead of being dropped and rebuilt at their next use: one
// launch for all of them (a model's dozens of weights would otherwise each be a cast kernel of a few microseconds
// after every optimizer step). The parameters they were made from must still be alive.
void refresh_shadows() {
    TapeContext& c = tape_context();
    if (!c.shadows) return;
    std::vector<CastJob> jobs;
    for (auto& kv : c.shadows->single) jobs.push_back(CastJob{kv.first->data, kv.second, 0});
    for (auto& kv : c.shadows->cat) {
        int64_t off = 0;
        for (const Variable* w : kv.second.ws) {
            jobs.push_back(CastJob{w->data, kv.second.t, off});
            off += w->data.cols;
        }
    }
    if (jobs.empty()) return;
    if (!k_cast_many(jobs)) c.shadows.reset();  // not casts the batched kernel takes: rebuilt at their next use
}
void prepare_shadow(const Var& W) { (void)shadow_of(W); }
void prepare_shadow_cat(const std::vector<Var>& Ws) { (void)shadow_cat(Ws); }

Tensor& Variable::ensure_grad() {
    if (grad.empty()) {
        grad = Tensor::make(data.rows, data.cols, is_param ? PK_F32 : data.dtype);
        k_fill(grad, 0.0f);
    }
    return own_grad();
}

Tensor& Variable::own_grad() {
    if (grad_shared && !grad.empty()) {
        Tensor mine = Tensor::make(grad.rows, grad.cols, grad.dtype);
        k_scale(grad, 1.0f, mine);
        grad = std::move(mine);
    }
    grad_shared = false;
    grad_is_unit = false;  // the caller is about to write
    return grad;
}

void Variable::accumulate(const Tensor& g, float a) {
    if (g.rows != data.rows || g.cols != data.cols) shape_fail("accumulate: gradient shape mismatch");
    grad_is_unit = false;
    if (grad.empty()) {
        grad = Tensor::make(data.rows, data.cols, is_param ? PK_F32 : data.dtype);
        grad_shared = false;
        k_scale(g, a, grad);  // first contribution: grad = a * g, no zero fill
        return;
    }
    if (grad_shared && a == 1.0f && g.dtype == grad.dtype) {  // the sum goes into a tensor of this Variable's own
        Tensor sum = Tensor::make(grad.rows, grad.cols, grad.dtype);
        k_add(grad, g, sum);
        grad = std::move(sum);
        grad_shared = false;
        return;
    }
    k_axpy(own_grad(), a, g);
}

void Variable::accumulate_owned(Tensor&& g, bool shared) {
    const int want = is_param ? PK_F32 : data.dtype;
    const bool whole = g.buf && g.off_bytes == 0 && (shared || g.buf.use_count() == 1) &&
                       g.buf->bytes == static_cast<size_t>(g.rows) * g.cols * g.esize();
    if (grad.empty() && whole && g.dtype == want && g.rows == data.rows && g.cols == data.cols) {
        grad = std::move(g);
        grad_shared = shared;
        grad_is_unit = false;
        return;
    }
    accumulate(g);
}

bool grad_enabled() { return g_grad_enabled; }
bool recomputing() { return g_recomputing; }
NoGrad::NoGrad() : prev_(g_grad_enabled) { g_grad_enabled = false; }
NoGrad::~NoGrad() { g_grad_enabled = prev_; }

Var record(Tensor result, std::vector<Var> parents, std::function<void(Variable*)> bw) {
    bool needs = false;
    if (grad_enabled())
        for (const auto& p : parents) needs = needs || p->requires_grad;
    Var out = make_var(std::move(result), needs);
    if (needs) {
        out->parents = std::move(parents);
        Variable* self = out.get();
        out->backward_fn = [self, bw]() { bw(self); };
    }
    return out;
}

void backward(const Var& root) {
    if (root->data.rows != 1 || root->data.cols != 1)
        throw std::runtime_error("backward: root must be a [1,1] scalar (compose with mean/sum)");
    Tensor seed = Tensor::make(1, 1, root->data.dtype);
    k_fill(seed, 1.0f);
    const bool fresh = root->grad.empty();
    root->accumulate(seed);
    root->grad_is_unit = fresh;
    run_backward(root);
}

void zero_grad(const std::vector<Var>& vars) {
    for (const auto& v : vars) {
        if (v->grad.empty()) continue;
        if (v->grad_shared) {  // a tensor of its own instead of zeroing the other holder's gradient
            v->grad = Tensor::make(v->grad.rows, v->grad.cols, v->grad.dtype);
            v->grad_shared = false;
        }
        k_fill(v->grad, 0.0f);
        v->grad_is_unit = false;
    }
}

Var checkpoint(const std::function<Var(const Var&)>& fn, const Var& x) {
    if (!grad_enabled()) return fn(x);  // eval: nothing to rematerialise
    Tensor boundary;
    {
        NoGrad tape_off;
        boundary = fn(x)->data;  // only the segment's output survives this scope
    }
    Var node = make_var(std::move(boundary), true);
    node->parents = {x};
    Variable* raw = node.get();
    node->backward_fn = [raw, segment = fn]() {
        const Var& input = raw->parents[0];
        // Rebuild the segment's tape from a fresh leaf that shares the input's storage (no op writes into a
        // tensor it did not produce, so the reference's copy of x, autograd.cpp:86, is not needed), hand it this
        // node's gradient -- nobody else reads it -- and run the rebuilt tape. Parameters used inside the
        // segment are the model's own Variables, so their gradients land where they belong.
        Var leaf = make_var(input->data, /*requires_grad=*/true);
        const bool outer = g_recomputing;
        g_recomputing = true;  // the segment may skip what only its own result needs (recomputing())
        Var rebuilt;
        try {
            rebuilt = segment(leaf);
        } catch (...) {
            g_recomputing = outer;
            throw;
        }
        g_recomputing = outer;
        if (rebuilt->data.rows != raw->grad.rows || rebuilt->data.cols != raw->grad.cols)
            shape_fail("checkpoint: recomputed output shape mismatch");
        rebuilt->accumulate_owned(std::move(raw->grad), raw->grad_shared);
        raw->grad_shared = false;
        run_backward(rebuilt);
        if (input->requires_grad && !leaf->grad.empty()) input->accumulate_owned(std::move(leaf->grad), leaf->grad_shared);
    };
    return node;
}

namespace ops {

Var linear(const Var& x, const Var& W) {
    if (x->data.cols != W->data.rows) shape_fail("matmul: inner dimensions disagree");
    const Tensor& Wc = shadow_of(W);
    Tensor y = Tensor::make(x->data.rows, W->data.cols, x->data.dtype);
    gemm(x->data, false, Wc, false, y.ptr(), y.dtype, y.rows, y.cols, y.cols, 0.0f);
    return record(std::move(y), {x, W}, [](Variable* self) {
        const Var& x = self->parents[0];
        const Var& W = self->parents[1];
        if (x->requires_grad) {  // dX = dY W^T  (ops.cpp:48-51)
            Tensor dx = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
            gemm(self->grad, false, shadow_of(W), true, dx.ptr(), dx.dtype, dx.rows, dx.cols, dx.cols, 0.0f);
            x->accumulate_owned(std::move(dx));
        }
        if (W->requires_grad && !defer_weight_gradient(x->data, self->grad, 0, W->data.cols, W)) {
            Tensor& g = W->ensure_grad();  // dW += X^T dY (ops.cpp:52-55), straight into the fp32 grad
            gemm(x->data, true, self->grad, false, g.ptr(), g.dtype, g.rows, g.cols, g.cols, 1.0f);
        }
    });
}

// y = r + x W: a Linear whose output joins a residual stream (o_proj and the MLP's down projection,
// llama.cpp:47-59), the sum formed in the product's epilogue where the library's own GEMM takes the operands (one
// rounding of r + x W instead of two, and no pass over y and r afterwards), by an add otherwise. One node with
// the gradients of both ops: dr is the node's gradient itself.
Var linear_add(const Var& x, const Var& W, const Var& r, bool result_needed) {
    if (x->data.cols != W->data.rows) shape_fail("matmul: inner dimensions disagree");
    if (r->data.rows != x->data.rows || r->data.cols != W->data.cols || r->data.dtype != x->data.dtype)
        shape_fail("add: shape mismatch");
    const Tensor& Wc = shadow_of(W);
    Tensor y = Tensor::make(x->data.rows, W->data.cols, x->data.dtype);
    const bool contiguous = r->data.off_bytes % 16 == 0;
    // result_needed = false: the caller only wants the node (the last op of a segment that is being re-run for its
    // tape: the backward closure reads x, W and the node's gradient, never the node's value), so nothing is multiplied
    if (!result_needed && grad_enabled()) {
        // y stays as allocated: its shape is what the tape needs
    } else if (!(x->data.dtype == PK_BF16 && Wc.dtype == PK_BF16 && gemm_backend() != 0 && contiguous &&
          gemm_mfma_bf16(x->data.ptr(), false, x->data.cols, Wc.ptr(), false, Wc.cols, y.ptr(), y.dtype, y.rows, y.cols,
                         x->data.cols, y.cols, 1.0f, tape_stream(), r->data.ptr()))) {
        gemm(x->data, false, Wc, false, y.ptr(), y.dtype, y.rows, y.cols, y.cols, 0.0f);
        k_add(r->data, y, y);
    }
    return record(std::move(y), {x, W, r}, [](Variable* self) {
        const Var& x = self->parents[0];
        const Var& W = self->parents[1];
        const Var& r = self->parents[2];
        if (x->requires_grad) {
            Tensor dx = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
            gemm(self->grad, false, shadow_of(W), true, dx.ptr(), dx.dtype, dx.rows, dx.cols, dx.cols, 0.0f);
            x->accumulate_owned(std::move(dx));
        }
        bool held = false;  // a held-back product still reads this node's gradient
        if (W->requires_grad) {
            held = defer_weight_gradient(x->data, self->grad, 0, W->data.cols, W);
            if (!held) {
                Tensor& g = W->ensure_grad();
                gemm(x->data, true, self->grad, false, g.ptr(), g.dtype, g.rows, g.cols, g.cols, 1.0f);
            }
        }
        if (r->requires_grad) {
            const bool was_shared = self->grad_shared;  // the products above have read it; r takes the tensor itself
            self->grad_shared = false;
            r->accumulate_owned(std::move(self->grad), was_shared || held);
        }
    });
}

// y = x [W_0 | W_1 | ...]: several Linear layers that read the same input (q/k/v projections,
// gate/up projections) as ONE GEMM against the column-wise concatenation of their weights, which
// is kept as a compute-dtype copy like any other shadow. Backward is one GEMM for dX and one for
// all the weight gradients, whose column blocks are scattered to the separate gradient tensors.
Var linear_cat(const Var& x, const std::vector<Var>& Ws) {
    if (Ws.empty() || Ws.size() > 4) throw std::runtime_error("linear_cat: 1 to 4 weights");
    const int64_t N = x->data.rows, d = Ws[0]->data.cols;
    for (const Var& W : Ws)
        if (W->data.cols != d || W->data.rows != x->data.cols) shape_fail("matmul: inner dimensions disagree");
    const int n = static_cast<int>(Ws.size());
    Tensor y = Tensor::make(N, n * d, x->data.dtype);
    gemm(x->data, false, shadow_cat(Ws), false, y.ptr(), y.dtype, N, n * d, n * d, 0.0f);
    std::vector<Var> parents{x};
    parents.insert(parents.end(), Ws.begin(), Ws.end());
    return record(std::move(y), std::move(parents), [n](Variable* self) {
        const Var& x = self->parents[0];
        const std::vector<Var> Ws(self->parents.begin() + 1, self->parents.end());
        if (x->requires_grad) {  // dX = dY [W_0 | W_1 | ...]^T
            Tensor dx = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
            gemm(self->grad, false, shadow_cat(Ws), true, dx.ptr(), dx.dtype, dx.rows, dx.cols, dx.cols, 0.0f);
            x->accumulate_owned(std::move(dx));
        }
        bool any = false;
        for (const Var& W : Ws) any = any || W->requires_grad;
        if (any) {  // held back, one product per weight, if every one of them can wait
            bool all = true;
            const int64_t d = Ws[0]->data.cols;
            for (int k = 0; k < n; ++k)
                all = all && (!Ws[k]->requires_grad || weight_gradient_can_wait(x->data, self->grad, k * d, d, Ws[k]));
            if (all) {
                for (int k = 0; k < n; ++k)
                    if (Ws[k]->requires_grad) hold_weight_gradient(x->data, self->grad, k * d, d, Ws[k]);
                any = false;
            }
        }
        if (any) {  // dW_k += X^T dY[:, block k]
            float* dst[4] = {nullptr, nullptr, nullptr, nullptr};
            std::vector<Tensor> unused;
            for (int k = 0; k < n; ++k) {
                if (Ws[k]->requires_grad) {
                    Tensor& g = Ws[k]->ensure_grad();
                    if (g.dtype != PK_F32) throw std::runtime_error("linear_cat: weight gradients must be fp32");
                    dst[k] = static_cast<float*>(g.ptr());
                } else {
                    unused.push_back(Tensor::make(Ws[k]->data.rows, Ws[k]->data.cols, PK_F32));
                    dst[k] = static_cast<float*>(unused.back().ptr());
                }
            }
            gemm_tn_split(x->data, self->grad, dst, n, 1.0f);
        }
    });
}

Var linear3(const Var& x, const Var& Wq, const Var& Wk, const Var& Wv) { return linear_cat(x, {Wq, Wk, Wv}); }

Var add(const Var& a, const Var& b) {
    Tensor y = Tensor::make(a->data.rows, a->data.cols, a->data.dtype);
    k_add(a->data, b->data, y);
    return record(std::move(y), {a, b}, [](Variable* self) {
        // Both parents take the tensor itself where they can: it is the gradient of either, shared and read-only
        // until one of them has to write (a parameter, or a parent that has a gradient already, gets a copy or
        // an axpy instead).
        const Var& a = self->parents[0];
        const Var& b = self->parents[1];
        const bool both = a->requires_grad && b->requires_grad && a != b;
        const bool share = both && !a->is_param && !b->is_param && a->grad.empty() && b->grad.empty() &&
                           a->data.dtype == self->grad.dtype && b->data.dtype == self->grad.dtype;
        const bool was_shared = self->grad_shared;
        self->grad_shared = false;
        if (share) {
            a->accumulate_owned(Tensor(self->grad), true);
            b->accumulate_owned(std::move(self->grad), true);
            return;
        }
        if (a->requires_grad) a->accumulate(self->grad);
        if (b->requires_grad) b->accumulate_owned(std::move(self->grad), was_shared);
    });
}

Var mul(const Var& a, const Var& b) {
    Tensor y = Tensor::make(a->data.rows, a->data.cols, a->data.dtype);
    k_mul(a->data, b->data, y);
    return record(std::move(y), {a, b}, [](Variable* self) {
        const Var& a = self->parents[0];
        const Var& b = self->parents[1];
        if (a->requires_grad) {
            Tensor t = Tensor::make(a->data.rows, a->data.cols, a->data.dtype);
            k_mul(self->grad, b->data, t);
            a->accumulate_owned(std::move(t));
        }
        if (b->requires_grad) {
            Tensor t = Tensor::make(a->data.rows, a->data.cols, a->data.dtype);
            k_mul(self->grad, a->data, t);
            b->accumulate_owned(std::move(t));
        }
    });
}

Var scale(const Var& x, float s) {
    Tensor y = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
    k_scale(x->data, s, y);
    return record(std::move(y), {x}, [s](Variable* self) {
        if (self->parents[0]->requires_grad) self->parents[0]->accumulate(self->grad, s);
    });
}

Var silu(const Var& x) {
    Tensor y = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
    k_silu_fwd(x->data, y);
    return record(std::move(y), {x}, [](Variable* self) {
        const Var& x = self->parents[0];
        if (!x->requires_grad) return;
        Tensor dx = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
        k_silu_bwd(x->data, self->grad, dx);
        x->accumulate_owned(std::move(dx));
    });
}

Var silu_mul(const Var& gate, const Var& up) {
    if (gate->data.rows != up->data.rows || gate->data.cols != up->data.cols) shape_fail("mul: shape mismatch");
    Tensor y = Tensor::make(gate->data.rows, gate->data.cols, gate->data.dtype);
    k_silu_mul_fwd(gate->data, up->data, y);
    return record(std::move(y), {gate, up}, [](Variable* self) {
        const Var& gate = self->parents[0];
        const Var& up = self->parents[1];
        if (!gate->requires_grad && !up->requires_grad) return;
        Tensor dg = Tensor::make(gate->data.rows, gate->data.cols, gate->data.dtype);
        Tensor du = Tensor::make(gate->data.rows, gate->data.cols, gate->data.dtype);
        k_silu_mul_bwd(gate->data, up->data, self->grad, dg, du);
        if (gate->requires_grad) gate->accumulate_owned(std::move(dg));
        if (up->requires_grad) up->accumulate_owned(std::move(du));
    });
}

Var silu_mul_cat(const Var& gu) {
    if (gu->data.cols % 2 != 0) shape_fail("mul: shape mismatch");
    Tensor y = Tensor::make(gu->data.rows, gu->data.cols / 2, gu->data.dtype);
    k_silu_mul_cat_fwd(gu->data, y);
    return record(std::move(y), {gu}, [](Variable* self) {
        const Var& gu = self->parents[0];
        if (!gu->requires_grad) return;
        Tensor dgu = Tensor::make(gu->data.rows, gu->data.cols, gu->data.dtype);
        k_silu_mul_cat_bwd(gu->data, self->grad, dgu);
        gu->accumulate_owned(std::move(dgu));
    });
}

Var rmsnorm(const Var& x, const Var& w) {
    if (w->data.rows != 1 || w->data.cols != x->data.cols) shape_fail("rmsnorm: w must be [1, cols(x)]");
    auto rinv = std::make_shared<Buffer>(sizeof(float) * x->data.rows);
    Tensor y = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
    k_rmsnorm_fwd(x->data, w->data, 1e-5f, y, static_cast<float*>(rinv->p));
    return record(std::move(y), {x, w}, [rinv](Variable* self) {
        const Var& x = self->parents[0];
        const Var& w = self->parents[1];
        Tensor dx;
        if (x->requires_grad) dx = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
        Tensor* dw = w->requires_grad ? &w->ensure_grad() : nullptr;
        // x usually has the residual branch's gradient already: the kernel adds it on the way out (one rounding of
        // the sum instead of two) and the result replaces it, which also leaves a shared tensor untouched
        const bool onto = x->requires_grad && !x->is_param && !x->grad.empty() && x->grad.dtype == dx.dtype;
        k_rmsnorm_bwd(self->grad, x->data, static_cast<const float*>(rinv->p), w->data, dw,
                      x->requires_grad ? &dx : nullptr, onto ? &x->grad : nullptr);
        if (onto) {
            x->grad = std::move(dx);
            x->grad_shared = false;
        } else if (x->requires_grad) {
            x->accumulate_owned(std::move(dx));
        }
    });
}

Var apply_rope(const Var& qkv, const std::shared_ptr<Buffer>& pos, float theta, int head_dim, int rot_heads, bool in_place) {
    if (qkv->data.cols % 3 != 0) shape_fail("apply_rope: cols must be divisible by 3");
    const int d = static_cast<int>(qkv->data.cols / 3);
    if (in_place) {
        // The caller hands over a projection nobody else reads (a Linear's backward needs its input and weight, not
        // its output): the rotation is applied where the data lies and the node shares the storage; the backward
        // turns this node's gradient back in place and passes it on whole.
        k_rope_inplace(qkv->data, static_cast<const int*>(pos->p), theta, d, head_dim, rot_heads, false);
        return record(Tensor(qkv->data), {qkv}, [pos, theta, head_dim, rot_heads, d](Variable* self) {
            const Var& x = self->parents[0];
            if (!x->requires_grad) return;
            k_rope_inplace(self->own_grad(), static_cast<const int*>(pos->p), theta, d, head_dim, rot_heads, true);
            x->accumulate_owned(std::move(self->grad));
            self->grad = Tensor();
        });
    }
    Tensor y = Tensor::make(qkv->data.rows, qkv->data.cols, qkv->data.dtype);
    k_rope(qkv->data, static_cast<const int*>(pos->p), theta, d, head_dim, rot_heads, false, y);
    return record(std::move(y), {qkv}, [pos, theta, head_dim, rot_heads, d](Variable* self) {
        const Var& x = self->parents[0];
        if (!x->requires_grad) return;
        Tensor dx = Tensor::make(x->data.rows, x->data.cols, x->data.dtype);
        k_rope(self->grad, static_cast<const int*>(pos->p), theta, d, head_dim, rot_heads, true, dx);
        x->accumulate_owned(std::move(dx));
    });
}

Var embedding(const Var& table, const std::shared_ptr<Buffer>& ids, int64_t n) {
    Tensor y = Tensor::make(n, table->data.cols, compute_dtype());
    k_embedding_fwd(table->data, static_cast<const int*>(ids->p), y);
    return record(std::move(y), {table}, [ids](Variable* self) {
        const Var& t = self->parents[0];
        if (!t->requires_grad) return;
        k_embedding_bwd(self->grad, static_cast<const int*>(ids->p), t->ensure_grad());  // scatter-add, ops.cpp:338-347
    });
}

namespace {

struct AttnGeom {
    int64_t B, T;
    int H, dk;
    float scale;
    bool causal;
    int window, sinks;
};

pk_attn_shape shape_of(const AttnGeom& g, int dtype) {
    pk_attn_shape s;
    s.B = static_cast<int32_t>(g.B);
    s.T = static_cast<int32_t>(g.T);
    s.Hq = s.Hkv = g.H;
    s.dk = g.dk;
    s.causal = g.causal;
    s.window = g.window;
    s.sinks = g.sinks;
    s.scale = g.scale;
    s.dtype = s.grad_dtype = dtype;
    return s;
}

}  // namespace

Var attention_qkv(const Var& qkv, int n_heads, float scale, int64_t seq_len, bool causal, int window, int sinks) {
    const int64_t N = qkv->data.rows, d3 = qkv->data.cols;
    if (d3 % 3 != 0 || (d3 / 3) % n_heads != 0) shape_fail("fused_attention: shape mismatch");
    const int64_t d = d3 / 3, sl = seq_len == 0 ? N : seq_len;
    if (N % sl != 0) shape_fail("fused_attention: rows not a multiple of seq_len");
    AttnGeom g{N / sl, sl, n_heads, static_cast<int>(d / n_heads), scale, causal, window, sinks};
    const int dt = qkv->data.dtype;
    const size_t es = qkv->data.esize();
    Tensor o = Tensor::make(N, d, dt);
    auto lse = std::make_shared<Buffer>(sizeof(float) * g.B * g.H * g.T);
    const pk_attn_shape sh = shape_of(g, dt);
    const pk_tensor4 q4 = view4(qkv->data.ptr(), 0, es, sl * d3, d3, g.dk), k4 = view4(qkv->data.ptr(), d, es, sl * d3, d3, g.dk),
                     v4 = view4(qkv->data.ptr(), 2 * d, es, sl * d3, d3, g.dk), o4 = view4(o.ptr(), 0, es, sl * d, d, g.dk);
    attn_check(pk_attn_fwd(&sh, &q4, &k4, &v4, &o4, static_cast<float*>(lse->p), tape_stream()));
    // The node keeps O (its own data) and LSE; P is rebuilt from Q, K and LSE in backward.
    return record(std::move(o), {qkv}, [g, lse](Variable* self) {
        const Var& qkv = self->parents[0];
        if (!qkv->requires_grad) return;
        const int64_t N = qkv->data.rows, d3 = qkv->data.cols, d = d3 / 3, sl = g.T;
        const int dt = qkv->data.dtype;
        const size_t es = qkv->data.esize();
        Tensor dqkv = Tensor::make(N, d3, dt);
        const pk_attn_shape sh = shape_of(g, dt);
        Buffer ws(pk_attn_bwd_workspace_bytes(&sh));
        const pk_tensor4 q4 = view4(qkv->data.ptr(), 0, es, sl * d3, d3, g.dk), k4 = view4(qkv->data.ptr(), d, es, sl * d3, d3, g.dk),
                         v4 = view4(qkv->data.ptr(), 2 * d, es, sl * d3, d3, g.dk),
                         o4 = view4(self->data.ptr(), 0, es, sl * d, d, g.dk), g4 = view4(self->grad.ptr(), 0, es, sl * d, d, g.dk),
                         dq4 = view4(dqkv.ptr(), 0, es, sl * d3, d3, g.dk), dk4 = view4(dqkv.ptr(), d, es, sl * d3, d3, g.dk),
                         dv4 = view4(dqkv.ptr(), 2 * d, es, sl * d3, d3, g.dk);
        attn_check(pk_attn_bwd(&sh, &q4, &k4, &v4, &o4, static_cast<const float*>(lse->p), &g4, &dq4, &dk4, &dv4, ws.p,
                               ws.bytes, tape_stream()));
        qkv->accumulate_owned(std::move(dqkv));
    });
}

namespace {
Var head_attention(const Var& q, const Var& k, const Var& v, float scale, int64_t seq_len, bool causal, int window,
                   int sinks, const char* who) {
    const int64_t T = q->data.rows;
    if (k->data.rows != T || v->data.rows != T || q->data.cols != k->data.cols || v->data.cols != k->data.cols)
        shape_fail(std::string(who) + ": shape mismatch");
    const int64_t sl = seq_len == 0 ? T : seq_len;
    if (T % sl != 0) shape_fail(std::string(who) + ": rows not a multiple of seq_len");
    const int dk = static_cast<int>(q->data.cols);
    AttnGeom g{T / sl, sl, 1, dk, scale, causal, window, sinks};
    const int dt = q->data.dtype;
    const size_t es = q->data.esize();
    Tensor o = Tensor::make(T, dk, dt);
    auto lse = std::make_shared<Buffer>(sizeof(float) * T);
    const pk_attn_shape sh = shape_of(g, dt);
    auto v4of = [&](const Tensor& t) { return view4(t.ptr(), 0, es, sl * dk, dk, dk); };
    const pk_tensor4 q4 = v4of(q->data), k4 = v4of(k->data), vv4 = v4of(v->data), o4 = v4of(o);
    attn_check(pk_attn_fwd(&sh, &q4, &k4, &vv4, &o4, static_cast<float*>(lse->p), tape_stream()));
    return record(std::move(o), {q, k, v}, [g, lse](Variable* self) {
        const Var& q = self->parents[0];
        const Var& k = self->parents[1];
        const Var& v = self->parents[2];
        if (!q->requires_grad && !k->requires_grad && !v->requires_grad) return;
        const int dt = q->data.dtype, dk = g.dk;
        const size_t es = q->data.esize();
        const int64_t T = q->data.rows, sl = g.T;
        Tensor dq = Tensor::make(T, dk, dt), dkk = Tensor::make(T, dk, dt), dv = Tensor::make(T, dk, dt);
        const pk_attn_shape sh = shape_of(g, dt);
        Buffer ws(pk_attn_bwd_workspace_bytes(&sh));
        auto v4of = [&](const Tensor& t) { return view4(t.ptr(), 0, es, sl * dk, dk, dk); };
        const pk_tensor4 q4 = v4of(q->data), k4 = v4of(k->data), vv4 = v4of(v->data), o4 = v4of(self->data),
                         g4 = v4of(self->grad), dq4 = v4of(dq), dk4 = v4of(dkk), dv4 = v4of(dv);
        attn_check(pk_attn_bwd(&sh, &q4, &k4, &vv4, &o4, static_cast<const float*>(lse->p), &g4, &dq4, &dk4, &dv4, ws.p,
                               ws.bytes, tape_stream()));
        if (q->requires_grad) q->accumulate_owned(std::move(dq));
        if (k->requires_grad) k->accumulate_owned(std::move(dkk));
        if (v->requires_grad) v->accumulate_owned(std::move(dv));
    });
}
}  // namespace

Var fused_attention(const Var& q, const Var& k, const Var& v, float scale, int64_t seq_len, bool causal) {
    return head_attention(q, k, v, scale, seq_len, causal, 0, 0, "fused_attention");
}
Var swa_attention(const Var& q, const Var& k, const Var& v, float scale, int64_t window, int64_t sinks, int64_t seq_len) {
    if (window == 0) throw std::runtime_error("swa_attention: window must be >= 1");  // ops.cpp:954
    return head_attention(q, k, v, scale, seq_len, true, static_cast<int>(window), static_cast<int>(sinks), "swa_attention");
}

Var matmul_nt(const Var& h, const Var& E) {
    if (h->data.cols != E->data.cols) shape_fail("matmul: inner dimensions disagree");
    Tensor y = Tensor::make(h->data.rows, E->data.rows, PK_F32);  // logits stay fp32, as in the reference
    gemm(h->data, false, shadow_of(E), true, y.ptr(), y.dtype, y.rows, y.cols, y.cols, 0.0f);
    return record(std::move(y), {h, E}, [](Variable* self) {
        const Var& h = self->parents[0];
        const Var& E = self->parents[1];
        Tensor dl = self->grad;
        if (dl.dtype != h->data.dtype) {
            dl = Tensor::make(self->grad.rows, self->grad.cols, h->data.dtype);
            k_cast(self->grad, dl);
        }
        if (h->requires_grad) {
            Tensor dh = Tensor::make(h->data.rows, h->data.cols, h->data.dtype);
            gemm(dl, false, shadow_of(E), false, dh.ptr(), dh.dtype, dh.rows, dh.cols, dh.cols, 0.0f);
            h->accumulate_owned(std::move(dh));
        }
        if (E->requires_grad) {
            Tensor& g = E->ensure_grad();
            gemm(dl, true, h->data, false, g.ptr(), g.dtype, g.rows, g.cols, g.cols, 1.0f);
        }
    });
}

Var cross_entropy(const Var& logits, const std::shared_ptr<Buffer>& targets) {
    const int64_t R = logits->data.rows;
    // softmax copy for the fused backward, as the reference caches P (ops.cpp:357)
    auto P = std::make_shared<Tensor>(Tensor::make(R, logits->data.cols, logits->data.dtype));
    k_cast(logits->data, *P);
    Buffer nll(sizeof(float) * R);
    k_ce_rows(*P, static_cast<const int*>(targets->p), 1.0f / static_cast<float>(R), static_cast<float*>(nll.p));
    Tensor out = Tensor::make(1, 1, PK_F32);
    k_mean_f32(static_cast<const float*>(nll.p), R, out);
    return record(std::move(out), {logits}, [P](Variable* self) {
        const Var& l = self->parents[0];
        if (!l->requires_grad) return;
        l->accumulate(*P, upstream_scalar(self));  // (P - onehot) * g / R, ops.cpp:371-374
    });
}

Var linear_cross_entropy(const Var& h, const Var& E, const std::shared_ptr<Buffer>& targets, int64_t chunk_rows,
                         bool loss_is_root) {
    const int64_t N = h->data.rows, V = E->data.rows, d = h->data.cols;
    if (d != E->data.cols) shape_fail("matmul: inner dimensions disagree");
    const int* tg = static_cast<const int*>(targets->p);
    const size_t hes = h->data.esize();
    // One pass over row chunks. The loss is a scalar, so its gradient with respect to the logits is known up to
    // the upstream factor as soon as a chunk's softmax is: when a gradient will be asked for, the same pass also
    // produces dh and dE for an upstream gradient of 1 (dlogits = (P - onehot) / N), and the backward closure only
    // scales them. Nothing of size [N, vocab] outlives its chunk, and no chunk's logits are computed twice.
    const bool want_dh = grad_enabled() && h->requires_grad, want_dE = grad_enabled() && E->requires_grad;
    // loss_is_root: the caller will seed this loss with 1 and nothing else, so E's share is added to E's gradient as
    // the chunks go by instead of being kept beside it until the backward closure runs ([V, d] fp32 less at the peak,
    // one pass over it less); the closure then insists on a unit seed.
    const bool dE_in_place = want_dE && loss_is_root && E->is_param;
    Tensor dh1, dE1;
    if (want_dh) dh1 = Tensor::make(N, d, h->data.dtype);
    if (want_dE) {
        if (dE_in_place) {
            dE1 = E->ensure_grad();
            if (dE1.dtype != PK_F32) throw std::runtime_error("linear_cross_entropy: the embedding's gradient must be fp32");
        } else {
            dE1 = Tensor::make(V, d, PK_F32);
        }
    }
    const Tensor& Ec = shadow_of(E);
    Buffer nll(sizeof(float) * N);
    const float g1 = 1.0f / static_cast<float>(N);
    const bool grads = want_dh || want_dE;
    // bf16 operands the library's own GEMM takes: the cross-entropy runs inside the logits product, which forms
    // every tile twice (row statistics and loss, then dlogits) instead of storing [rows, V] logits for a row kernel
    bool in_product = h->data.dtype == PK_BF16 && Ec.dtype == PK_BF16 && head_kernel() != 0 && gemm_backend() != 0 &&
                      gemm_head_takes(h->data.ptr(), d, Ec.ptr(), d, std::min<int64_t>(N, chunk_rows > 0 ? chunk_rows : 4096), V, d);
    // default chunk: the same scratch either way (4096 rows of bf16 dlogits, or 2048 of fp32 logits: 262 MB at 32000 words)
    if (chunk_rows <= 0) chunk_rows = in_product ? 4096 : 2048;
    for (int64_t r0 = 0; r0 < N; r0 += chunk_rows) {
        const int64_t rows = std::min(chunk_rows, N - r0);
        const Tensor hview = h->data.row_range(r0, rows);
        float* nll_r = static_cast<float*>(nll.p) + r0;
        Tensor dl;
        int64_t dl_ld = V;
        if (in_product) {
            Buffer stats(sizeof(float) * 2 * static_cast<size_t>(gemm_head_spans(V)) * rows), rowf(sizeof(float) * 3 * rows);
            float* zt = static_cast<float*>(rowf.p);
            float* row_max = zt + rows;
            float* row_inv = row_max + rows;
            in_product = gemm_head_rows(hview.ptr(), d, Ec.ptr(), d, rows, V, d, tg + r0, stats.p, zt, row_max, row_inv, nll_r,
                                        tape_stream());
            if (in_product && grads) {
                dl = Tensor::make(rows, V, PK_BF16);
                if (!gemm_head_dlogits(hview.ptr(), d, Ec.ptr(), d, rows, V, d, tg + r0, row_max, row_inv, g1, dl.ptr(), V,
                                       tape_stream()))
                    throw std::runtime_error("linear_cross_entropy: the head's second pass refused what its first took");
            }
        }
        if (!in_product) {
            Tensor logits = Tensor::make(rows, V, PK_F32);
            gemm(hview, false, Ec, true, logits.ptr(), PK_F32, rows, V, V, 0.0f);
            // dlogits takes the place of the logits it came from: in fp32 the same matrix, in bf16 the first half of
            // every fp32 row (row pitch 2V bf16 elements), so a chunk holds one [rows, V] fp32 buffer and nothing else.
            if (grads) {
                dl = logits;
                if (h->data.dtype != PK_F32) {
                    dl.dtype = h->data.dtype;
                    dl_ld = 2 * V;
                }
            }
            if (!k_ce_rows_once(logits, tg + r0, g1, nll_r, grads ? &dl : nullptr, dl_ld)) {
                k_ce_rows(logits, tg + r0, g1, nll_r);  // generic row kernel: dlogits in place as fp32
                if (grads && h->data.dtype != PK_F32) {
                    dl = Tensor::make(rows, V, h->data.dtype);
                    dl_ld = V;
                    k_cast(logits, dl);
                }
            }
        }
        if (want_dh)
            gemm(dl, false, Ec, false, static_cast<char*>(dh1.ptr()) + r0 * d * hes, dh1.dtype, rows, d, d, 0.0f, dl_ld);
        if (want_dE) gemm(dl, true, hview, false, dE1.ptr(), PK_F32, V, d, d, r0 == 0 && !dE_in_place ? 0.0f : 1.0f, dl_ld);
    }
    Tensor out = Tensor::make(1, 1, PK_F32);
    k_mean_f32(static_cast<const float*>(nll.p), N, out);  // the loss stays on the device: no wait in mid-step
    if (dE_in_place) dE1 = Tensor();
    return record(std::move(out), {h, E}, [dh1, dE1, dE_in_place](Variable* self) mutable {
        const Var& h = self->parents[0];
        const Var& E = self->parents[1];
        const float g = upstream_scalar(self);  // upstream gradient of the scalar loss
        if (dE_in_place && g != 1.0f)
            throw std::runtime_error("linear_cross_entropy: built with loss_is_root, but its gradient is not the unit seed");
        if (h->requires_grad && !dh1.empty()) {
            if (g == 1.0f)
                h->accumulate_owned(std::move(dh1));
            else
                h->accumulate(dh1, g);
        }
        if (E->requires_grad && !dE1.empty()) {
            if (g == 1.0f)
                E->accumulate_owned(std::move(dE1));
            else
                E->accumulate(dE1, g);
        }
        dh1 = Tensor();
        dE1 = Tensor();
    });
}

double clip_grad_norm(const std::vector<Var>& params, float max_norm) {
    // double accumulation as the reference (ops.cpp:1047-1053); one host round trip for all parameters
    Buffer parts(sizeof(double) * SUMSQ_MAX_PARTS * std::max<size_t>(params.size(), 1));
    int64_t n = 0;
    for (const auto& p : params)
        if (!p->grad.empty()) n += k_sumsq_parts(p->grad, static_cast<double*>(parts.p) + n);
    const double sq = n ? k_sum_f64_to_host(static_cast<const double*>(parts.p), n) : 0.0;
    const double total = std::sqrt(sq);
    if (total > max_norm && total > 0.0) {
        const float s = static_cast<float>(max_norm / total);
        for (const auto& p : params)
            if (!p->grad.empty()) k_scale(p->own_grad(), s, p->grad);
    }
    return total;
}

}  // namespace ops
}  // namespace pk
