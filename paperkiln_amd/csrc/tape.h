// The autograd tape, device-resident. Same shape as the reference's
// (paperkiln include/microtorch/autograd.hpp:28-104, src/autograd.cpp): a
// Variable owns its data, a lazily created grad, its parents and the closure
// that scatters its gradient to them; backward() runs closures in reverse
// topological order; checkpoint() rematerialises a segment. What changes is
// where the numbers live (HBM, via pk::Tensor) and what the attention node
// keeps: O (its own data) and the per-row logsumexp, never a [T,T] matrix.
#pragma once
#include <atomic>
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "tensor.h"

namespace pk {

class Variable;
using Var = std::shared_ptr<Variable>;

namespace detail {
extern std::atomic<size_t> g_live_vars;
}

class Variable {
public:
    Tensor data;
    Tensor grad;  // allocated and zeroed on first accumulate(); fp32 for parameters, data's dtype otherwise
    bool requires_grad = false;
    bool is_param = false;
    std::vector<Var> parents;
    std::function<void()> backward_fn;

    explicit Variable(Tensor d, bool rg = false) : data(std::move(d)), requires_grad(rg) { ++detail::g_live_vars; }
    ~Variable() { --detail::g_live_vars; }
    Variable(const Variable&) = delete;
    Variable& operator=(const Variable&) = delete;

    bool is_leaf() const { return parents.empty(); }
    void accumulate(const Tensor& g, float a = 1.0f);  // grad += a * g (autograd.cpp:16-24)
    // The same for a temporary the caller is done with: the first contribution takes the buffer over instead of
    // copying it (the reference's lazily sized grad, autograd.cpp:17-19, makes that first += a copy as well).
    void accumulate_owned(Tensor&& g);
    Tensor& ensure_grad();                             // zero-filled grad of data's shape
};

size_t live_variables();  // autograd.hpp:61-64

inline Var make_var(Tensor data, bool requires_grad = false) {
    return std::make_shared<Variable>(std::move(data), requires_grad);
}

void backward(const Var& root);                 // root must be [1,1] (autograd.cpp:51-66)
void zero_grad(const std::vector<Var>& vars);   // autograd.cpp:104-108
// Runs fn(x) without recording; on backward re-runs it under grad on a detached
// copy of x and pushes the output gradient through the fresh subgraph
// (autograd.cpp:68-102). fn must be recomputation-deterministic.
Var checkpoint(const std::function<Var(const Var&)>& fn, const Var& x);

bool grad_enabled();
class NoGrad {
public:
    NoGrad();
    ~NoGrad();
    NoGrad(const NoGrad&) = delete;
    NoGrad& operator=(const NoGrad&) = delete;

private:
    bool prev_;
};

// Attach a tape node unless grad is off or no parent requires grad (ops.cpp:17-29).
Var record(Tensor result, std::vector<Var> parents, std::function<void(Variable*)> bw);

namespace ops {

// y = x W for a parameter W [in, out] kept in fp32 with a compute-dtype shadow
// (ops::matmul + nn::Linear::forward, ops.cpp:33-58, nn.cpp:106-109).
Var linear(const Var& x, const Var& W);
// Three projections of the same input written side by side into one [N, 3*out]
// matrix: the concat_cols({q, k, v}) of llama.cpp:30-36 without the copies.
Var linear3(const Var& x, const Var& Wq, const Var& Wk, const Var& Wv);
Var linear_cat(const Var& x, const std::vector<Var>& Ws);  // y = x [W_0 | W_1 | ...], equal widths, 1..4 weights
Var add(const Var& a, const Var& b);                // ops.cpp:60-65
Var mul(const Var& a, const Var& b);                // ops.cpp:76-83
Var scale(const Var& x, float s);                   // ops.cpp:843-861
Var silu(const Var& x);                             // ops.cpp:404-424
Var silu_mul(const Var& gate, const Var& up);        // mul(silu(gate), up) as one node (llama.cpp:55-58)
Var silu_mul_cat(const Var& gate_up);                // the same on the halves of one [N, 2*d_ff] projection [gate | up]
Var rmsnorm(const Var& x, const Var& w);            // ops.cpp:426-479, eps fixed at 1e-5 (:435)
// ops::apply_rope on the fused [N, 3d] matrix (ops.cpp:481-537). rot_heads = 1 is the
// reference as written (only the first head of q and of k is rotated, :498-499 with the
// call at llama.cpp:36); rot_heads = n_heads rotates every head.
Var apply_rope(const Var& qkv, const std::shared_ptr<Buffer>& pos_dev, float theta, int head_dim, int rot_heads,
               bool in_place = false);  // in_place: qkv is a projection nobody else reads; rotate it where it lies
Var embedding(const Var& table, const std::shared_ptr<Buffer>& ids_dev, int64_t n);  // ops.cpp:329-348
// All heads of llama.cpp:47-53 in one node: heads are read in place from the fused
// [N, 3d] matrix (q | k | v thirds, head h at columns h*dk) and written side by side
// into [N, d]. window == 0: ops::fused_attention; window >= 1: ops::swa_attention.
Var attention_qkv(const Var& qkv, int n_heads, float scale, int64_t seq_len, bool causal, int window, int sinks);
// One head as [rows, dk] matrices: ops::fused_attention / ops::swa_attention (ops.cpp:863-1027).
Var fused_attention(const Var& q, const Var& k, const Var& v, float scale, int64_t seq_len, bool causal);
Var swa_attention(const Var& q, const Var& k, const Var& v, float scale, int64_t window, int64_t sinks, int64_t seq_len);
// Tied head + loss: mean cross-entropy of logits = h E^T (llama.cpp:88 + ops.cpp:350-376),
// evaluated in row chunks so that the [N, vocab] logits and their softmax copy never
// exist as a whole. The chunk's dlogits feed dh and dE immediately; backward scales them.
Var linear_cross_entropy(const Var& h, const Var& E, const std::shared_ptr<Buffer>& targets_dev, int64_t chunk_rows);
// The unfused pair, for parity at sizes where the logits fit: logits = h E^T, then ops::cross_entropy.
Var matmul_nt(const Var& h, const Var& E);
Var cross_entropy(const Var& logits, const std::shared_ptr<Buffer>& targets_dev);
double clip_grad_norm(const std::vector<Var>& params, float max_norm);  // ops.cpp:1046-1064

}  // namespace ops

// Element type of activations and GEMM operands on the current context (PK_F32 or PK_BF16; the reference's
// device::set, device.cpp:41-46, is the nearest counterpart), and the compute-dtype shadows of its parameters,
// which go stale with every optimizer step.
void set_compute_dtype(int dtype);
int compute_dtype();
void invalidate_shadows();

}  // namespace pk
