// Llama-family model, AdamW and the training step on the device-resident
// tape, plus their C ABI. Mirrors paperkiln src/llama.cpp (LlamaBlock::forward
// :25-60, Llama::forward :71-89), nn::AdamW (src/nn.cpp:301-321) and the step
// shape of tools/mtstudio.cpp:456-480. The per-block activation checkpoint is
// the reference's checkpoint() (src/autograd.cpp:68-102) on HBM tensors; its
// receipt here is bytes from the allocator's high-water mark, not a node count.
#include <cmath>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "pk_internal.h"
#include "tape.h"

namespace pk {
namespace {

// splitmix64 + Box-Muller, the same stream as paperkiln_amd/synth.py randn():
// the reference initialises from libstdc++'s mt19937 + normal_distribution
// (nn.cpp:14-21), which is not reproducible outside libstdc++.
struct Rng {
    uint64_t seed;
    static uint64_t mix(uint64_t z) {
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double u01(uint64_t idx) const {  // idx is 1-based
        const uint64_t z = mix(seed + idx * 0x9E3779B97F4A7C15ull);
        return (static_cast<double>(z >> 11) + 0.5) * (1.0 / 9007199254740992.0);
    }
};
std::vector<float> randn_host(uint64_t seed, size_t n, float std_) {
    const size_t m = (n + 1) / 2;
    Rng r{seed};
    std::vector<float> out(2 * m);
    for (size_t i = 0; i < m; ++i) {
        const double u1 = r.u01(i + 1), u2 = r.u01(m + i + 1);
        const double rad = std::sqrt(-2.0 * std::log(u1)), th = 2.0 * M_PI * u2;
        out[2 * i] = static_cast<float>(rad * std::cos(th) * std_);
        out[2 * i + 1] = static_cast<float>(rad * std::sin(th) * std_);
    }
    out.resize(n);
    return out;
}

Var make_param(int64_t r, int64_t c, const std::vector<float>& host) {
    Tensor t = Tensor::make(r, c, PK_F32);
    hip_check(hipMemcpy(t.ptr(), host.data(), sizeof(float) * r * c, hipMemcpyHostToDevice), "hipMemcpy");
    Var v = make_var(std::move(t), true);
    v->is_param = true;
    return v;
}

struct Block {
    Var ln1_w, ln2_w, q, k, v, o, gate, up, down;
};

struct Model {
    pk_llama_config cfg;
    // The model's own tape state (stream, element type, parameter shadows) and the lock that keeps two host
    // threads from running the same model at once; every C entry holds both for the length of the call.
    TapeContext ctx;
    std::mutex mu;
    int64_t head_chunk_rows = 0;  // rows of the tied head evaluated at a time (linear_cross_entropy); 0 = its default
    Var embed, norm_w;
    std::vector<Block> blocks;
    std::vector<std::pair<std::string, Var>> named;
    bool checkpoint_blocks = false;
    // Master weights, gradients and the two AdamW moments (nn.cpp:293-299) each live in ONE
    // allocation, [1, slab_len] fp32, with every parameter's tensors as views at the same offset:
    // zero_grad, the clip norm and the optimiser step are then one launch each, not one per parameter.
    Tensor pslab, gslab, mslab, vslab;
    long t = 0;
    // Pinned staging for what a pass sends up (ids, targets, positions): one host copy and asynchronous transfers
    // instead of three transfers from pageable memory with a wait each. Written only between passes (a pass ends
    // with a wait for its stream).
    int* stage = nullptr;
    size_t stage_cap = 0;
    ~Model() {
        if (stage) (void)hipHostFree(stage);
    }
    int* staging(size_t n_ints) {
        if (n_ints > stage_cap) {
            if (stage) hip_check(hipHostFree(stage), "hipHostFree");
            stage = nullptr;
            stage_cap = 0;
            void* p = nullptr;
            hip_check(hipHostMalloc(&p, sizeof(int) * n_ints, hipHostMallocDefault), "hipHostMalloc");
            stage = static_cast<int*>(p);
            stage_cap = n_ints;
        }
        return stage;
    }

    void reg(const std::string& name, const Var& p) { named.emplace_back(name, p); }

    Model(const pk_llama_config& c, unsigned seed) : cfg(c) {
        if (c.d % c.n_heads != 0) shape_fail("llama: d must divide by n_heads");
        const int64_t d = c.d, ff = c.d_ff;
        auto lin = [&](int64_t in, int64_t out, unsigned s) {
            return make_param(in, out, randn_host(static_cast<uint64_t>(s) * 7919u + 1u, in * out, 0.02f));
        };
        const std::vector<float> ones(d, 1.0f);
        embed = make_param(c.vocab, d, randn_host(static_cast<uint64_t>(seed + 11) * 104729u + 3u, c.vocab * d, 0.02f));
        reg("embed_tokens.weight", embed);
        for (int i = 0; i < c.n_layers; ++i) {
            const unsigned s = seed + 100u * static_cast<unsigned>(i + 1);
            const std::string p = "layers." + std::to_string(i) + ".";
            Block b;
            b.ln1_w = make_param(1, d, ones);
            b.ln2_w = make_param(1, d, ones);
            b.q = lin(d, d, s + 1);
            b.k = lin(d, d, s + 2);
            b.v = lin(d, d, s + 3);
            b.o = lin(d, d, s + 4);
            b.gate = lin(d, ff, s + 5);
            b.up = lin(d, ff, s + 6);
            b.down = lin(ff, d, s + 7);
            reg(p + "input_layernorm.weight", b.ln1_w);
            reg(p + "post_attention_layernorm.weight", b.ln2_w);
            reg(p + "self_attn.q_proj.weight", b.q);
            reg(p + "self_attn.k_proj.weight", b.k);
            reg(p + "self_attn.v_proj.weight", b.v);
            reg(p + "self_attn.o_proj.weight", b.o);
            reg(p + "mlp.gate_proj.weight", b.gate);
            reg(p + "mlp.up_proj.weight", b.up);
            reg(p + "mlp.down_proj.weight", b.down);
            blocks.push_back(b);
        }
        norm_w = make_param(1, d, ones);
        reg("norm.weight", norm_w);
        if (!c.tie_embeddings) throw std::runtime_error("llama: only the tied head (lm_head = embed_tokens) is built");
        build_slabs();
    }

    void build_slabs() {
        std::vector<int64_t> off;
        int64_t total = 0;
        for (const auto& kv : named) {  // 256-byte granules keep every view aligned for the GEMMs
            off.push_back(total);
            total += (kv.second->data.numel() + 63) / 64 * 64;
        }
        pslab = Tensor::make(1, total, PK_F32);
        gslab = Tensor::make(1, total, PK_F32);
        k_fill(pslab, 0.0f);
        k_fill(gslab, 0.0f);
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
        for (size_t i = 0; i < named.size(); ++i) {
            Variable& p = *named[i].second;
            auto view = [&](const Tensor& slab) {
                Tensor t = slab;
                t.rows = p.data.rows;
                t.cols = p.data.cols;
                t.off_bytes = off[i] * static_cast<int64_t>(sizeof(float));
                return t;
            };
            Tensor w = view(pslab);
            hip_check(hipMemcpy(w.ptr(), p.data.ptr(), sizeof(float) * p.data.numel(), hipMemcpyDeviceToDevice), "hipMemcpy");
            p.data = w;
            p.grad = view(gslab);
        }
    }

    std::vector<Var> parameters() const {
        std::vector<Var> out;
        for (const auto& kv : named) out.push_back(kv.second);
        return out;
    }

    // LlamaBlock::forward, llama.cpp:25-60. The 3H slice_cols + H fused_attention +
    // concat_cols nodes of :47-53 are one attention node reading heads in place.
    Var block_forward(const Block& b, const Var& x, const std::shared_ptr<Buffer>& pos, int64_t seq_len) const {
        const int dk = cfg.d / cfg.n_heads;
        Var h = ops::rmsnorm(x, b.ln1_w);
        Var qkv = ops::linear3(h, b.q, b.k, b.v);
        qkv = ops::apply_rope(qkv, pos, cfg.rope_theta, dk, cfg.rope_all_heads ? cfg.n_heads : 1, /*in_place=*/true);
        const float sc = 1.0f / std::sqrt(static_cast<float>(dk));
        Var x1 = ops::linear_add(ops::attention_qkv(qkv, cfg.n_heads, sc, seq_len, true, cfg.window, cfg.sinks), b.o, x);
        Var h2 = ops::rmsnorm(x1, b.ln2_w);
        // re-run at backward time, the block's own output is not needed again (the gradient arrives from outside): the
        // down projection is recorded but not multiplied
        return ops::linear_add(ops::silu_mul_cat(ops::linear_cat(h2, {b.gate, b.up})), b.down, x1, !recomputing());
    }

    // Llama::forward (llama.cpp:71-89) up to the final norm; positions restart per sequence.
    Var hidden(const std::shared_ptr<Buffer>& ids, const std::shared_ptr<Buffer>& pos_dev, int64_t n, int64_t seq_len) const {
        Var h = ops::embedding(embed, ids, n);
        for (const Block& blk : blocks) {
            if (checkpoint_blocks && grad_enabled()) {
                const Block* bp = &blk;
                h = checkpoint([this, bp, pos_dev, seq_len](const Var& in) { return block_forward(*bp, in, pos_dev, seq_len); },
                               h);
            } else {
                h = block_forward(blk, h, pos_dev, seq_len);
            }
        }
        return ops::rmsnorm(h, norm_w);
    }
};

thread_local std::string g_llama_err;
template <typename F>
int guarded(F&& f) {
    try {
        f();
        return PK_OK;
    } catch (const std::exception& e) {
        g_llama_err = e.what();
        set_error(g_llama_err);
        return status_of(e);
    }
}

Model* model_of(void* handle) {
    if (!handle) throw Error(PK_ERR_ARGUMENT, "null model handle");
    return static_cast<Model*>(handle);
}
// Runs f(model) as the model's own tape: its lock held, its context current on this thread.
template <typename F>
int with_model(void* handle, F&& f) {
    return guarded([&] {
        Model* m = model_of(handle);
        std::lock_guard<std::mutex> lk(m->mu);
        ContextScope scope(m->ctx);
        f(m);
    });
}

}  // namespace
}  // namespace pk

using namespace pk;

extern "C" {

int pk_alloc(size_t bytes, void** out) {
    return guarded([&] {
        if (!out) throw Error(PK_ERR_ARGUMENT, "pk_alloc: null result pointer");
        *out = dev_alloc(bytes);
    });
}
int pk_free(void* p) {
    return guarded([&] {
        if (!dev_free(p)) throw Error(PK_ERR_ARGUMENT, "pk_free: not a pointer pk_alloc returned (or already freed)");
    });
}
size_t pk_live_bytes(void) { return dev_live_bytes(); }
size_t pk_peak_bytes(void) { return dev_peak_bytes(); }
void pk_reset_peak(void) { dev_reset_peak(); }
void pk_trim(void) { dev_trim(); }

int pk_llama_create(const pk_llama_config* cfg, unsigned seed, void** handle) {
    return guarded([&] {
        if (!cfg || !handle) throw Error(PK_ERR_ARGUMENT, "pk_llama_create: null argument");
        // the parameters are created under a context of the model's element type, which the model then keeps
        TapeContext ctx;
        ContextScope scope(ctx);
        set_compute_dtype(cfg->compute_dtype);
        Model* m = new Model(*cfg, seed);
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
        m->ctx = ctx;
        *handle = m;
    });
}
int pk_llama_destroy(void* h) {
    return guarded([&] {
        if (!h) return;
        Model* m = static_cast<Model*>(h);
        {
            std::lock_guard<std::mutex> lk(m->mu);
            ContextScope scope(m->ctx);
            hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
            m->ctx.shadows.reset();  // the shadows' memory goes back tagged with the model's stream
        }
        TapeContext last = m->ctx;  // parameters and slabs are freed under the model's stream as well
        ContextScope scope(last);
        delete m;
    });
}
int pk_llama_num_params(void* h) { return h ? static_cast<int>(static_cast<Model*>(h)->named.size()) : -1; }
int pk_llama_param_info(void* h, int i, char* name, size_t name_len, int64_t* rows, int64_t* cols) {
    return with_model(h, [&](Model* m) {
        if (i < 0 || i >= static_cast<int>(m->named.size())) throw Error(PK_ERR_ARGUMENT, "parameter index out of range");
        if (name && name_len) std::snprintf(name, name_len, "%s", m->named[i].first.c_str());
        if (rows) *rows = m->named[i].second->data.rows;
        if (cols) *cols = m->named[i].second->data.cols;
    });
}
int pk_llama_set_param(void* h, int i, const float* host) {
    return with_model(h, [&](Model* m) {
        if (i < 0 || i >= static_cast<int>(m->named.size()) || !host) throw Error(PK_ERR_ARGUMENT, "parameter index out of range or null data");
        const Tensor& t = m->named[i].second->data;
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
        hip_check(hipMemcpy(t.ptr(), host, sizeof(float) * t.numel(), hipMemcpyHostToDevice), "hipMemcpy");
        invalidate_shadows();
    });
}
int pk_llama_get_param(void* h, int i, float* host) {
    return with_model(h, [&](Model* m) {
        if (i < 0 || i >= static_cast<int>(m->named.size()) || !host) throw Error(PK_ERR_ARGUMENT, "parameter index out of range or null data");
        const Tensor& t = m->named[i].second->data;
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
        hip_check(hipMemcpy(host, t.ptr(), sizeof(float) * t.numel(), hipMemcpyDeviceToHost), "hipMemcpy");
    });
}
int pk_llama_get_grad(void* h, int i, float* host) {
    return with_model(h, [&](Model* m) {
        if (i < 0 || i >= static_cast<int>(m->named.size()) || !host) throw Error(PK_ERR_ARGUMENT, "parameter index out of range or null data");
        const Var& p = m->named[i].second;
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
        if (p->grad.empty())
            std::memset(host, 0, sizeof(float) * p->data.numel());
        else
            hip_check(hipMemcpy(host, p->grad.ptr(), sizeof(float) * p->data.numel(), hipMemcpyDeviceToHost), "hipMemcpy");
    });
}
int pk_llama_set_head_chunk(void* h, int64_t rows) {
    return with_model(h, [&](Model* m) {
        if (rows <= 0) throw Error(PK_ERR_ARGUMENT, "pk_llama_set_head_chunk: rows must be positive");
        m->head_chunk_rows = rows;
    });
}

int pk_llama_loss_backward(void* h, const int* host_ids, const int* host_targets, int64_t n, int64_t seq_len,
                           int checkpoint_blocks, int do_backward, int fused_head, float* loss, pk_llama_stats* stats,
                           void* stream) {
    return with_model(h, [&](Model* m) {
        if (!host_ids || !host_targets || !loss || n <= 0) throw Error(PK_ERR_ARGUMENT, "pk_llama_loss_backward: null or empty argument");
        set_tape_stream(static_cast<hipStream_t>(stream));  // the model keeps it: the optimiser step runs there too
        for (int64_t i = 0; i < n; ++i)
            if (host_ids[i] < 0 || host_ids[i] >= m->cfg.vocab) throw std::runtime_error("embedding: id out of range");
        for (int64_t i = 0; i < n; ++i)
            if (host_targets[i] < 0 || host_targets[i] >= m->cfg.vocab)
                throw std::runtime_error("cross_entropy: target out of range");
        m->checkpoint_blocks = checkpoint_blocks != 0;
        const int64_t sl = seq_len == 0 ? n : seq_len;
        if (n % sl != 0) shape_fail("ids not a multiple of seq_len");
        k_fill(m->gslab, 0.0f);  // zero_grad: every parameter's gradient is a view of this slab
        // ids, targets and positions (which restart per sequence, llama.cpp:73-76) go up from pinned memory behind
        // the fill, without a wait
        int* st = m->staging(static_cast<size_t>(3 * n + 1));
        std::memcpy(st, host_ids, sizeof(int) * n);
        std::memcpy(st + n, host_targets, sizeof(int) * n);
        for (int64_t i = 0; i < n; ++i) st[2 * n + i] = static_cast<int>(i % sl);
        auto up = [&](const int* src) {
            auto b = std::make_shared<Buffer>(sizeof(int) * n);
            hip_check(hipMemcpyAsync(b->p, src, sizeof(int) * n, hipMemcpyHostToDevice, tape_stream()), "hipMemcpyAsync");
            return b;
        };
        auto ids = up(st);
        auto tg = up(st + n);
        auto pos_dev = up(st + 2 * n);
        // Everything allocated from here on, until backward returns, is activation memory.
        if (compute_dtype() != PK_F32) {  // build the bf16 parameter shadows first: they are not activations
            for (const auto& b : m->blocks) {
                prepare_shadow_cat({b.q, b.k, b.v});
                prepare_shadow(b.o);
                prepare_shadow_cat({b.gate, b.up});
                prepare_shadow(b.down);
            }
            prepare_shadow(m->embed);
        }
        const size_t base = dev_live_bytes();  // the allocator's host-side counters: nothing to wait for
        dev_reset_peak();
        const size_t live0 = live_variables();
        Var hid = m->hidden(ids, pos_dev, n, seq_len);
        Var l = fused_head ? ops::linear_cross_entropy(hid, m->embed, tg, m->head_chunk_rows, do_backward != 0)
                           : ops::cross_entropy(ops::matmul_nt(hid, m->embed), tg);
        hid.reset();
        // the allocator's counters move when the host allocates and frees, not when the GPU gets there: no wait here
        if (stats) {
            stats->live_vars_after_forward = static_cast<int64_t>(live_variables() - live0);
            stats->activation_bytes_after_forward = static_cast<int64_t>(dev_live_bytes() - base);
        }
        if (do_backward) backward(l);
        // the loss comes back into the pinned staging's spare word behind the last kernel: one wait ends the pass
        float* hl = reinterpret_cast<float*>(st + 3 * n);
        hip_check(hipMemcpyAsync(hl, l->data.ptr(), 4, hipMemcpyDeviceToHost, tape_stream()), "hipMemcpyAsync");
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
        if (stats) stats->peak_activation_bytes = static_cast<int64_t>(dev_peak_bytes() - base);
        *loss = *hl;
    });
}

int pk_llama_adamw_step(void* h, float lr, float b1, float b2, float eps, float wd, float max_norm, float* total_norm) {
    return with_model(h, [&](Model* m) {
        if (m->mslab.empty()) {
            m->mslab = Tensor::make(1, m->pslab.cols, PK_F32);
            m->vslab = Tensor::make(1, m->pslab.cols, PK_F32);
            k_fill(m->mslab, 0.0f);
            k_fill(m->vslab, 0.0f);
        }
        // ops::clip_grad_norm over the slab (the padding between parameters is zero): double
        // accumulation as the reference (ops.cpp:1047-1053), one host round trip.
        double tn = 0.0;
        float clip = 1.0f;
        if (max_norm > 0.0f) {
            Buffer parts(sizeof(double) * SUMSQ_MAX_PARTS);
            const int nb = k_sumsq_parts(m->gslab, static_cast<double*>(parts.p));
            tn = std::sqrt(k_sum_f64_to_host(static_cast<const double*>(parts.p), nb));
            if (tn > max_norm && tn > 0.0) clip = static_cast<float>(max_norm / tn);  // applied by the AdamW pass
        }
        if (total_norm) *total_norm = static_cast<float>(tn);
        ++m->t;
        const float c1 = 1.0f - std::pow(b1, static_cast<float>(m->t));
        const float c2 = 1.0f - std::pow(b2, static_cast<float>(m->t));
        // every parameter of this model receives a gradient each step, so the reference's "skip a
        // parameter that never accumulated" (nn.cpp:309) never applies; padding stays at zero
        k_adamw(m->pslab, m->gslab, m->mslab, m->vslab, lr, b1, b2, eps, wd, c1, c2, clip);
        refresh_shadows();  // the bf16 copies of the weights follow them, in one launch
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
    });
}

}  // extern "C"
