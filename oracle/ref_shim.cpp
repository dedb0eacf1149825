// TEST INFRASTRUCTURE ONLY. A thin extern "C" driver around the *compiled
// reference* (paperkiln / namespace microtorch). It is linked against the
// reference's own translation units where they lie under /root/reference and
// lands in oracle/_ref/libpk_ref.so. It is used (a) to pin oracle/pk_oracle.c
// against the real thing, (b) to write the golden fixtures under
// tests/golden/, (c) optionally as the timed CPU baseline. The product
// library never links or loads it.
//
// Every entry takes row-major fp32 host buffers, exactly the reference's
// Matrix layout (third_party/transformer_cpp/include/matrix.hpp:32-43).
#include <cmath>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "microtorch/autograd.hpp"
#include "microtorch/llama.hpp"
#include "microtorch/nn.hpp"
#include "microtorch/ops.hpp"

using namespace microtorch;

namespace {

thread_local std::string g_err;

Matrix from_buf(const float* p, size_t r, size_t c) {
    Matrix m(r, c);
    std::memcpy(m.data(), p, r * c * sizeof(float));
    return m;
}
void to_buf(const Matrix& m, float* p) {
    if (p && m.rows() != 0) std::memcpy(p, m.data(), m.rows() * m.cols() * sizeof(float));
}
void grad_to_buf(const Var& v, float* p) {
    if (!p) return;
    if (v->grad.rows() == 0) {
        std::memset(p, 0, v->data.rows() * v->data.cols() * sizeof(float));
    } else {
        to_buf(v->grad, p);
    }
}

// Push an arbitrary upstream gradient through one tape node: the reference's
// backward() insists on a [1,1] root (src/autograd.cpp:51-55), so seed the
// node's grad and fire its closure directly, which is all backward() does for
// a single node (src/autograd.cpp:61-65).
void fire(const Var& y, const Matrix& dy) {
    y->accumulate(dy);
    if (y->backward_fn) y->backward_fn();
}

template <typename F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        g_err = e.what();
        return 1;
    }
}

struct LlamaHandle {
    std::unique_ptr<nn::Llama> model;
    std::vector<std::pair<std::string, Var>> named;
    std::unique_ptr<nn::AdamW> opt;
};

}  // namespace

extern "C" {

const char* pkref_last_error() { return g_err.c_str(); }

// ops::fused_attention (src/ops.cpp:863-934). v may have any column count dv
// (the op only requires q.cols == k.cols, :866), which lets the caller pass an
// identity V to read back the attention weights A themselves.
int pkref_fused_attention(const float* q, const float* k, const float* v, const float* dy,
                          size_t rows, size_t dk, size_t dv, float scale, size_t seq_len,
                          int causal, float* y, float* dq, float* dk_out, float* dv_out) {
    return guarded([&] {
        Var Q = make_var(from_buf(q, rows, dk), true);
        Var K = make_var(from_buf(k, rows, dk), true);
        Var V = make_var(from_buf(v, rows, dv), true);
        Var Y = ops::fused_attention(Q, K, V, scale, seq_len, causal != 0);
        to_buf(Y->data, y);
        if (dy) {
            fire(Y, from_buf(dy, rows, dv));
            grad_to_buf(Q, dq);
            grad_to_buf(K, dk_out);
            grad_to_buf(V, dv_out);
        }
    });
}

// ops::swa_attention (src/ops.cpp:948-1027).
int pkref_swa_attention(const float* q, const float* k, const float* v, const float* dy,
                        size_t rows, size_t dk, size_t dv, float scale, size_t window,
                        size_t sinks, size_t seq_len, float* y, float* dq, float* dk_out,
                        float* dv_out) {
    return guarded([&] {
        Var Q = make_var(from_buf(q, rows, dk), true);
        Var K = make_var(from_buf(k, rows, dk), true);
        Var V = make_var(from_buf(v, rows, dv), true);
        Var Y = ops::swa_attention(Q, K, V, scale, window, sinks, seq_len);
        to_buf(Y->data, y);
        if (dy) {
            fire(Y, from_buf(dy, rows, dv));
            grad_to_buf(Q, dq);
            grad_to_buf(K, dk_out);
            grad_to_buf(V, dv_out);
        }
    });
}

// ops::attention_mask (src/ops.cpp:1029-1044).
int pkref_attention_mask(size_t rows, size_t seq_len, int causal, float* out) {
    return guarded([&] { to_buf(ops::attention_mask(rows, seq_len, causal != 0), out); });
}

// ops::rmsnorm (src/ops.cpp:426-479).
int pkref_rmsnorm(const float* x, const float* w, const float* dy, size_t R, size_t C, float* y,
                  float* dx, float* dw) {
    return guarded([&] {
        Var X = make_var(from_buf(x, R, C), true);
        Var W = make_var(from_buf(w, 1, C), true);
        Var Y = ops::rmsnorm(X, W);
        to_buf(Y->data, y);
        if (dy) {
            fire(Y, from_buf(dy, R, C));
            grad_to_buf(X, dx);
            grad_to_buf(W, dw);
        }
    });
}

// ops::silu (src/ops.cpp:404-424).
int pkref_silu(const float* x, const float* dy, size_t R, size_t C, float* y, float* dx) {
    return guarded([&] {
        Var X = make_var(from_buf(x, R, C), true);
        Var Y = ops::silu(X);
        to_buf(Y->data, y);
        if (dy) {
            fire(Y, from_buf(dy, R, C));
            grad_to_buf(X, dx);
        }
    });
}

// ops::apply_rope (src/ops.cpp:481-537) on a fused [T, 3d] matrix.
int pkref_apply_rope(const float* qkv, const int* pos, const float* dy, size_t T, size_t d3,
                     float theta, size_t head_dim, float* y, float* dqkv) {
    return guarded([&] {
        Var X = make_var(from_buf(qkv, T, d3), true);
        std::vector<int> p(pos, pos + T);
        Var Y = ops::apply_rope(X, p, theta, head_dim);
        to_buf(Y->data, y);
        if (dy) {
            fire(Y, from_buf(dy, T, d3));
            grad_to_buf(X, dqkv);
        }
    });
}

// ops::cross_entropy (src/ops.cpp:350-376); dlogits is d(loss)/d(logits).
int pkref_cross_entropy(const float* logits, const int* targets, size_t R, size_t C, float* loss,
                        float* dlogits) {
    return guarded([&] {
        Var L = make_var(from_buf(logits, R, C), true);
        std::vector<int> t(targets, targets + R);
        Var out = ops::cross_entropy(L, t);
        *loss = out->data(0, 0);
        if (dlogits) {
            backward(out);
            grad_to_buf(L, dlogits);
        }
    });
}

// ops::embedding (src/ops.cpp:329-348): gather forward, scatter-add backward.
int pkref_embedding(const float* table, const int* ids, const float* dy, size_t V, size_t d,
                    size_t n, float* y, float* dtable) {
    return guarded([&] {
        Var E = make_var(from_buf(table, V, d), true);
        std::vector<int> id(ids, ids + n);
        Var Y = ops::embedding(E, id);
        to_buf(Y->data, y);
        if (dy) {
            fire(Y, from_buf(dy, n, d));
            grad_to_buf(E, dtable);
        }
    });
}

// ops::matmul (src/ops.cpp:33-58) -> device::gemm -> matmul_optimized.
int pkref_matmul(const float* a, const float* b, size_t M, size_t K, size_t N, float* c) {
    return guarded([&] {
        Var A = make_var(from_buf(a, M, K));
        Var B = make_var(from_buf(b, K, N));
        to_buf(ops::matmul(A, B)->data, c);
    });
}

// ---- nn::Llama (src/llama.cpp) ------------------------------------------

void* pkref_llama_create(size_t vocab, size_t d, size_t n_layers, size_t n_heads, size_t d_ff,
                         size_t n_ctx, float rope_theta, int tie, unsigned seed) {
    LlamaHandle* h = nullptr;
    int rc = guarded([&] {
        nn::LlamaConfig cfg;
        cfg.vocab = vocab;
        cfg.d = d;
        cfg.n_layers = n_layers;
        cfg.n_heads = n_heads;
        cfg.d_ff = d_ff;
        cfg.n_ctx = n_ctx;
        cfg.rope_theta = rope_theta;
        cfg.tie_embeddings = tie != 0;
        h = new LlamaHandle;
        h->model = std::make_unique<nn::Llama>(cfg, seed);
        h->named = h->model->named_parameters();
    });
    return rc == 0 ? h : nullptr;
}

void pkref_llama_destroy(void* hv) { delete static_cast<LlamaHandle*>(hv); }

size_t pkref_llama_num_params(void* hv) { return static_cast<LlamaHandle*>(hv)->named.size(); }

const char* pkref_llama_param_name(void* hv, size_t i) {
    return static_cast<LlamaHandle*>(hv)->named[i].first.c_str();
}
void pkref_llama_param_shape(void* hv, size_t i, size_t* r, size_t* c) {
    const Var& p = static_cast<LlamaHandle*>(hv)->named[i].second;
    *r = p->data.rows();
    *c = p->data.cols();
}
void pkref_llama_get_param(void* hv, size_t i, float* out) {
    to_buf(static_cast<LlamaHandle*>(hv)->named[i].second->data, out);
}
void pkref_llama_set_param(void* hv, size_t i, const float* in) {
    Var& p = static_cast<LlamaHandle*>(hv)->named[i].second;
    std::memcpy(p->data.data(), in, p->data.rows() * p->data.cols() * sizeof(float));
}
void pkref_llama_get_grad(void* hv, size_t i, float* out) {
    grad_to_buf(static_cast<LlamaHandle*>(hv)->named[i].second, out);
}

// zero_grad -> forward -> cross_entropy -> backward, the step shape of
// tools/mtstudio.cpp:456-471 (accum = 1). live_after_fwd is the reference's
// own memory receipt (tests/test_checkpointing.cpp:46-60).
int pkref_llama_loss_backward(void* hv, const int* ids, const int* targets, size_t n,
                              size_t seq_len, int checkpoint_blocks, int do_backward,
                              float* loss, size_t* live_after_fwd, float* logits_out) {
    return guarded([&] {
        auto* h = static_cast<LlamaHandle*>(hv);
        h->model->checkpoint_blocks = checkpoint_blocks != 0;
        auto params = h->model->parameters();
        zero_grad(params);
        std::vector<int> x(ids, ids + n), y(targets, targets + n);
        const size_t live0 = live_variables();
        Var logits = h->model->forward(x, seq_len);
        Var l = ops::cross_entropy(logits, y);
        if (live_after_fwd) *live_after_fwd = live_variables() - live0;
        if (logits_out) to_buf(logits->data, logits_out);
        *loss = l->data(0, 0);
        if (do_backward) backward(l);
    });
}

// clip_grad_norm (src/ops.cpp:1046-1064) then AdamW::step (src/nn.cpp:301-321).
int pkref_llama_adamw_step(void* hv, float lr, float b1, float b2, float eps, float wd,
                           float max_norm, float* total_norm) {
    return guarded([&] {
        auto* h = static_cast<LlamaHandle*>(hv);
        auto params = h->model->parameters();
        if (!h->opt) h->opt = std::make_unique<nn::AdamW>(params, lr, b1, b2, eps, wd);
        h->opt->lr = lr;
        float tn = 0.0f;
        if (max_norm > 0.0f) tn = ops::clip_grad_norm(params, max_norm);
        if (total_norm) *total_norm = tn;
        h->opt->step();
    });
}

}  // extern "C"
