// Python module over the device-resident tape (include/paperkiln_amd.hpp): the additions to the reference's
// `_microtorch` surface (paperkiln python/bindings.cpp:41-192) that its hot path lacks -- the reference binds
// neither fused_attention nor swa_attention, checkpoint or Llama (bindings.cpp:70-90, 121-146). Same shape as
// that module: a Variable class with data / grad / requires_grad / shape, tensor(), backward(), zero_grad(), an
// `ops` submodule, numpy float32 copies at the boundary and no views (bindings.cpp:1-7, 21-37). Strictly
// additive: nothing of the existing surface is renamed or changed.
#include <pybind11/functional.h>
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <map>
#include <string>
#include <vector>

#include "paperkiln_amd.hpp"

namespace py = pybind11;
using pk::Var;
using pk::Variable;
using farray = py::array_t<float, py::array::c_style | py::array::forcecast>;

namespace {

py::array_t<float> to_numpy(const pk::Tensor& t) {
    py::array_t<float> out({t.rows, t.cols});
    pk::download(t, out.mutable_data());
    return out;
}
pk::Tensor from_numpy(const farray& a, int dtype) {
    if (a.ndim() != 2) throw std::runtime_error("expected a 2-D float32 array");
    return pk::upload(a.data(), a.shape(0), a.shape(1), dtype);
}
int dtype_of(const std::string& name) {
    if (name == "fp32" || name == "float32") return PK_F32;
    if (name == "bf16" || name == "bfloat16") return PK_BF16;
    throw std::runtime_error("dtype must be 'fp32' or 'bf16'");
}
std::shared_ptr<pk::Buffer> ints_on_device(const std::vector<int>& h) {
    static_assert(sizeof(int) == sizeof(float), "ids travel as 4-byte words");
    return pk::upload(reinterpret_cast<const float*>(h.data()), 1, static_cast<int64_t>(h.size()), PK_F32).buf;
}
void must(int rc) {
    if (rc != PK_OK) throw pk::Error(rc, pk_last_error());
}

// nn::Llama + AdamW behind the C ABI (the model itself lives inside the library)
struct LlamaModel {
    void* handle = nullptr;
    pk_llama_config cfg{};
    LlamaModel(int vocab, int d, int n_layers, int n_heads, int d_ff, float rope_theta, const std::string& compute_dtype,
               bool rope_all_heads, int window, int sinks, unsigned seed) {
        cfg.vocab = vocab, cfg.d = d, cfg.n_layers = n_layers, cfg.n_heads = n_heads, cfg.d_ff = d_ff;
        cfg.rope_theta = rope_theta, cfg.tie_embeddings = 1, cfg.compute_dtype = dtype_of(compute_dtype);
        cfg.rope_all_heads = rope_all_heads, cfg.window = window, cfg.sinks = sinks;
        must(pk_llama_create(&cfg, seed, &handle));
    }
    ~LlamaModel() { pk_llama_destroy(handle); }
    LlamaModel(const LlamaModel&) = delete;
    LlamaModel& operator=(const LlamaModel&) = delete;
    std::map<std::string, py::array_t<float>> fetch(int (*get)(void*, int, float*)) {
        std::map<std::string, py::array_t<float>> out;
        char name[256];
        for (int i = 0; i < pk_llama_num_params(handle); ++i) {
            int64_t r = 0, c = 0;
            must(pk_llama_param_info(handle, i, name, sizeof name, &r, &c));
            py::array_t<float> a({r, c});
            must(get(handle, i, a.mutable_data()));
            out.emplace(name, std::move(a));
        }
        return out;
    }
};

}  // namespace

PYBIND11_MODULE(_paperkiln, mod) {
    mod.doc() = "paperkiln_amd: the device-resident tape of libpaperkiln_amd.so (MI355X)";
    py::register_exception<pk::Error>(mod, "PkError", PyExc_RuntimeError);
    mod.def("init", [](int device) {
        char arch[64] = {0};
        must(pk_init(device, arch, sizeof arch));
        return std::string(arch);
    }, py::arg("device") = 0, "Bring the library up on a GPU; returns its architecture name.");

    // ---- tape ----
    py::class_<Variable, Var>(mod, "Variable")
        .def_property_readonly("data", [](const Variable& v) { return to_numpy(v.data); })
        .def_property_readonly("grad", [](const Variable& v) {
            if (v.grad.empty()) throw std::runtime_error("grad not populated; call backward()");
            return to_numpy(v.grad);
        })
        .def_readonly("requires_grad", &Variable::requires_grad)
        .def_property_readonly("shape", [](const Variable& v) { return py::make_tuple(v.data.rows, v.data.cols); })
        .def_property_readonly("dtype", [](const Variable& v) { return v.data.dtype == PK_F32 ? "fp32" : "bf16"; })
        .def("__repr__", [](const Variable& v) {
            return "<Variable [" + std::to_string(v.data.rows) + ", " + std::to_string(v.data.cols) + "] " +
                   (v.data.dtype == PK_F32 ? "fp32" : "bf16") + " requires_grad=" + (v.requires_grad ? "True" : "False") + ">";
        });
    mod.def("tensor", [](const farray& a, bool requires_grad, const std::string& dtype, bool is_param) {
        Var v = pk::make_var(from_numpy(a, dtype_of(dtype)), requires_grad);
        v->is_param = is_param;
        return v;
    }, py::arg("array"), py::arg("requires_grad") = false, py::arg("dtype") = "fp32", py::arg("is_param") = false,
       "Create a Variable on the GPU from a 2-D numpy float32 array (copies).");
    mod.def("backward", &pk::backward, "Reverse pass from a scalar [1,1] root.");
    mod.def("zero_grad", &pk::zero_grad);
    mod.def("live_variables", &pk::live_variables, "Variables currently alive: the reference's checkpointing receipt.");
    mod.def("live_bytes", &pk_live_bytes);
    mod.def("peak_bytes", &pk_peak_bytes);
    mod.def("reset_peak", &pk_reset_peak);
    mod.def("checkpoint", [](const std::function<Var(const Var&)>& fn, const Var& x) { return pk::checkpoint(fn, x); },
            py::arg("fn"), py::arg("x"),
            "y = fn(x) keeping only x and y; fn is run again in the backward pass (it must be deterministic).");
    mod.def("set_grad_enabled", [](bool on) {
        // the tape's switch is a scoped object in C++; Python gets the flag itself
        static thread_local std::unique_ptr<pk::NoGrad> off;
        if (on)
            off.reset();
        else if (!off)
            off = std::make_unique<pk::NoGrad>();
    });
    mod.def("grad_enabled", &pk::grad_enabled);

    // ---- ops ----
    auto ops = mod.def_submodule("ops", "tape ops of the attention hot path");
    ops.def("fused_attention", [](const Var& q, const Var& k, const Var& v, float scale, size_t seq_len, bool causal) {
        return pk::ops::fused_attention(q, k, v, scale, static_cast<int64_t>(seq_len), causal);
    }, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("scale"), py::arg("seq_len") = 0, py::arg("causal") = true);
    ops.def("swa_attention", [](const Var& q, const Var& k, const Var& v, float scale, size_t window, size_t sinks, size_t seq_len) {
        return pk::ops::swa_attention(q, k, v, scale, static_cast<int64_t>(window), static_cast<int64_t>(sinks),
                                      static_cast<int64_t>(seq_len));
    }, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("scale"), py::arg("window"), py::arg("sinks") = 0, py::arg("seq_len") = 0);
    ops.def("attention_qkv", &pk::ops::attention_qkv, py::arg("qkv"), py::arg("n_heads"), py::arg("scale"),
            py::arg("seq_len") = 0, py::arg("causal") = true, py::arg("window") = 0, py::arg("sinks") = 0,
            "All heads of a fused [N, 3d] projection in one node (heads read in place).");
    ops.def("linear", &pk::ops::linear, "y = x W for a weight W [in, out]");
    ops.def("add", &pk::ops::add);
    ops.def("mul", &pk::ops::mul);
    ops.def("scale", &pk::ops::scale);
    ops.def("silu", &pk::ops::silu);
    ops.def("rmsnorm", &pk::ops::rmsnorm);
    ops.def("cross_entropy", [](const Var& logits, const std::vector<int>& targets) {
        if (static_cast<int64_t>(targets.size()) != logits->data.rows) throw std::runtime_error("cross_entropy: one target per row");
        for (int t : targets)
            if (t < 0 || t >= logits->data.cols) throw std::runtime_error("cross_entropy: target out of range");
        return pk::ops::cross_entropy(logits, ints_on_device(targets));
    });

    // ---- model ----
    py::class_<LlamaModel>(mod, "Llama")
        .def(py::init<int, int, int, int, int, float, const std::string&, bool, int, int, unsigned>(), py::arg("vocab"),
             py::arg("d"), py::arg("n_layers"), py::arg("n_heads"), py::arg("d_ff"), py::arg("rope_theta") = 10000.0f,
             py::arg("compute_dtype") = "fp32", py::arg("rope_all_heads") = false, py::arg("window") = 0,
             py::arg("sinks") = 0, py::arg("seed") = 0)
        .def("state_dict", [](LlamaModel& m) { return m.fetch(&pk_llama_get_param); })
        .def("grads", [](LlamaModel& m) { return m.fetch(&pk_llama_get_grad); })
        .def("load_state_dict", [](LlamaModel& m, const std::map<std::string, farray>& sd) {
            char name[256];
            for (int i = 0; i < pk_llama_num_params(m.handle); ++i) {
                int64_t r = 0, c = 0;
                must(pk_llama_param_info(m.handle, i, name, sizeof name, &r, &c));
                auto it = sd.find(name);
                if (it == sd.end()) throw std::runtime_error(std::string("load_state_dict: missing ") + name);
                if (it->second.size() != r * c) throw std::runtime_error(std::string("load_state_dict: shape of ") + name);
                must(pk_llama_set_param(m.handle, i, it->second.data()));
            }
        })
        .def("loss_backward", [](LlamaModel& m, const std::vector<int>& ids, const std::vector<int>& targets, int64_t seq_len,
                                 bool checkpoint_blocks, bool backward, bool fused_head) {
            if (ids.size() != targets.size()) throw std::runtime_error("cross_entropy: one target per row");
            float loss = 0.0f;
            pk_llama_stats st{};
            must(pk_llama_loss_backward(m.handle, ids.data(), targets.data(), static_cast<int64_t>(ids.size()), seq_len,
                                        checkpoint_blocks, backward, fused_head, &loss, &st, nullptr));
            py::dict stats;
            stats["live_vars_after_forward"] = st.live_vars_after_forward;
            stats["activation_bytes_after_forward"] = st.activation_bytes_after_forward;
            stats["peak_activation_bytes"] = st.peak_activation_bytes;
            return py::make_tuple(loss, stats);
        }, py::arg("ids"), py::arg("targets"), py::arg("seq_len") = 0, py::arg("checkpoint_blocks") = false,
           py::arg("backward") = true, py::arg("fused_head") = true,
           "zero_grad -> forward -> mean cross-entropy -> backward; returns (loss, stats).")
        .def("adamw_step", [](LlamaModel& m, float lr, float b1, float b2, float eps, float wd, float max_norm) {
            float tn = 0.0f;
            must(pk_llama_adamw_step(m.handle, lr, b1, b2, eps, wd, max_norm, &tn));
            return tn;
        }, py::arg("lr"), py::arg("b1") = 0.9f, py::arg("b2") = 0.999f, py::arg("eps") = 1e-8f, py::arg("wd") = 0.01f,
           py::arg("max_norm") = 0.0f, "clip_grad_norm (when max_norm > 0) then AdamW; returns the gradient norm.");
}
