// See microtorch_hip_seam.hpp. Plain C++ over the C ABI of libpaperkiln_amd.so (include/paperkiln_amd.h): no
// HIP header, no kernel code. Host data goes up, the library runs, results come down -- the write-through
// contract of the reference's op set (docs/CUDA_PHASE_B2.md section 4; src/cuda_ops.cu:398-609), so host
// storage is never stale. Operands of device::gemm that belong to a Variable are kept on the device inside
// a step window, as the reference's step residency does (src/cuda_resident.cu:102-134, 226-263).
#include "microtorch_hip_seam.hpp"

#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <unordered_map>

#include "microtorch/device.hpp"
#include "microtorch/ops.hpp"
#include "paperkiln_amd.h"

namespace microtorch {
namespace device {

// A Variable's device copy: the buffer and the window that stamped it.
struct DevState {
    void* ptr = nullptr;
    size_t bytes = 0;
    unsigned long long stamp = 0;
};

namespace {

Device g_where = Device::CPU;
bool g_ops_on = false, g_step_on = false, g_window_open = false, g_ready = false, g_resident_on = false;
unsigned long long g_stamp = 0;

// Explicit residency (include/microtorch/device_cache.hpp:19-25; the reference's table is src/cuda_resident.cu:175-207):
// device copies of host matrices the caller asked to keep, keyed by the host data pointer. Nothing enters it
// implicitly and nothing detects a stale copy: the caller invalidates or refreshes after mutating host data.
struct Resident {
    void* ptr;
    size_t rows, cols;
};
std::unordered_map<const float*, Resident> g_resident;

void must(int rc, const char* what) {
    if (rc != PK_OK) throw std::runtime_error(std::string(what) + ": " + pk_last_error());
}
void bring_up() {
    if (g_ready) return;
    must(pk_init(0, nullptr, 0), "device::set");
    g_ready = true;
}
bool ops_active() { return g_ops_on && g_where == Device::CUDA; }

// Device memory for the length of one call; freed on every exit path.
class Temp {
public:
    explicit Temp(size_t floats) : bytes_(floats * sizeof(float)) { must(pk_alloc(bytes_ ? bytes_ : 4, &p_), "pk_alloc"); }
    Temp(const float* host, size_t floats) : Temp(floats) { must(pk_memcpy_h2d(p_, host, bytes_, nullptr), "upload"); }
    explicit Temp(const Matrix& m) : Temp(m.get_data(), m.rows() * m.cols()) {}
    ~Temp() { pk_free(p_); }
    Temp(const Temp&) = delete;
    Temp& operator=(const Temp&) = delete;
    void* get() const { return p_; }
    float* f() const { return static_cast<float*>(p_); }
    void to(float* host) const { must(pk_memcpy_d2h(host, p_, bytes_, nullptr), "download"); }
    void to(Matrix& m) const { to(m.get_data()); }

private:
    void* p_ = nullptr;
    size_t bytes_;
};

void same_shape(const Matrix& a, const Matrix& b, const char* who) {
    if (a.rows() != b.rows() || a.cols() != b.cols()) throw std::runtime_error(std::string(who) + ": shape mismatch");
}
int64_t count(const Matrix& m) { return static_cast<int64_t>(m.rows() * m.cols()); }

// The device copy of a gemm operand: the Variable's cached one when a step window is open and the slot was
// stamped in this window, a fresh upload into the slot otherwise, a temporary when there is no slot.
struct Operand {
    void* ptr = nullptr;
    bool temp = false;
    ~Operand() {
        if (temp) pk_free(ptr);
    }
};
void stage(const Matrix& m, DevState** slot, Operand& out) {
    const size_t bytes = m.rows() * m.cols() * sizeof(float);
    const bool cache = slot && g_step_on && g_window_open;
    if (!cache && g_resident_on) {  // an operand the caller made resident: its device copy as it stands
        const auto it = g_resident.find(m.get_data());
        if (it != g_resident.end() && it->second.rows == m.rows() && it->second.cols == m.cols()) {
            out.ptr = it->second.ptr;
            return;
        }
    }
    if (!cache) {
        must(pk_alloc(bytes, &out.ptr), "pk_alloc");
        out.temp = true;
        must(pk_memcpy_h2d(out.ptr, m.get_data(), bytes, nullptr), "upload");
        return;
    }
    if (!*slot) *slot = new DevState;
    DevState& s = **slot;
    if (s.ptr && s.bytes != bytes) {
        pk_free(s.ptr);
        s.ptr = nullptr;
    }
    if (!s.ptr) {
        must(pk_alloc(bytes, &s.ptr), "pk_alloc");
        s.bytes = bytes;
        s.stamp = 0;
    }
    if (s.stamp != g_stamp) {  // host data may have changed between windows: upload again
        must(pk_memcpy_h2d(s.ptr, m.get_data(), bytes, nullptr), "upload");
        s.stamp = g_stamp;
    }
    out.ptr = s.ptr;
}

pk_attn_shape head_shape(const Matrix& q, float scale, size_t seq_len, bool causal, size_t window, size_t sinks) {
    const size_t rows = q.rows(), sl = seq_len == 0 ? rows : seq_len;
    pk_attn_shape s;
    s.B = static_cast<int32_t>(rows / sl);
    s.T = static_cast<int32_t>(sl);
    s.Hq = s.Hkv = 1;
    s.dk = static_cast<int32_t>(q.cols());
    s.causal = causal ? 1 : 0;
    // size_t arguments beyond the sequence mean "everything": the library clamps, int32 must not wrap first
    s.window = static_cast<int32_t>(window > sl ? sl : window);
    s.sinks = static_cast<int32_t>(sinks > sl ? sl : sinks);
    s.scale = scale;
    s.dtype = s.grad_dtype = PK_F32;
    return s;
}
pk_tensor4 one_head(void* p, const pk_attn_shape& s) {
    pk_tensor4 t;
    t.ptr = p;
    t.stride_b = static_cast<int64_t>(s.T) * s.dk;
    t.stride_t = s.dk;
    t.stride_h = s.dk;
    return t;
}
void check_heads(const Matrix& q, const Matrix& k, const Matrix& v, size_t seq_len, const char* who) {
    const size_t T = q.rows();
    if (k.rows() != T || v.rows() != T || q.cols() != k.cols() || v.cols() != k.cols())
        throw std::runtime_error(std::string(who) + ": shape mismatch");
    const size_t sl = seq_len == 0 ? T : seq_len;
    if (T % sl != 0) throw std::runtime_error(std::string(who) + ": rows not a multiple of seq_len");
}

}  // namespace

// ---- include/microtorch/device.hpp ----------------------------------------------------------------------
Device get() { return g_where; }
bool cuda_compiled() { return true; }  // "a GPU build": the enum value CUDA names the GPU device here
void set(Device d) {
    if (d == Device::CUDA) bring_up();  // throws when no gfx950 device is visible: nothing falls back silently
    g_where = d;
}
void set_device_ops(bool on) { g_ops_on = on; }
bool device_ops_enabled() { return g_ops_on; }
void set_from_env() {
    auto is = [](const char* name, const char* want) {
        const char* v = std::getenv(name);
        return v && std::strcmp(v, want) == 0;
    };
    if (is("MICROTORCH_STEP_RESIDENCY", "1")) set_step_residency(true);
    if (is("MICROTORCH_DEVICE_OPS", "1")) set_device_ops(true);
    const char* v = std::getenv("MICROTORCH_DEVICE");
    if (!v) return;
    if (is("MICROTORCH_DEVICE", "cuda") || is("MICROTORCH_DEVICE", "hip"))
        set(Device::CUDA);
    else if (is("MICROTORCH_DEVICE", "cpu"))
        set(Device::CPU);
    else
        throw std::runtime_error("MICROTORCH_DEVICE must be cpu, cuda or hip");
}

Matrix gemm(const Matrix& A, DevState** devA, Trans tA, const Matrix& B, DevState** devB, Trans tB) {
    const bool ta = tA == Trans::T, tb = tB == Trans::T;
    const size_t M = ta ? A.cols() : A.rows(), Ka = ta ? A.rows() : A.cols();
    const size_t Kb = tb ? B.cols() : B.rows(), N = tb ? B.rows() : B.cols();
    if (Ka != Kb) throw std::runtime_error("gemm: inner dimensions disagree");
    if (g_where != Device::CUDA) {  // the host path, exactly as before: materialised transposes, blocked AVX2 product
        return matmul_optimized(ta ? A.transpose() : A, tb ? B.transpose() : B);
    }
    Operand a, b;
    stage(A, devA, a);
    stage(B, devB, b);
    Temp c(M * N);
    must(pk_op_gemm(a.ptr, ta, b.ptr, tb, c.get(), static_cast<int64_t>(M), static_cast<int64_t>(N),
                    static_cast<int64_t>(Ka), PK_F32, PK_F32, 0, nullptr),
         "gemm");
    Matrix C(M, N);
    c.to(C);
    return C;
}
Matrix matmul(const Matrix& a, const Matrix& b) { return gemm(a, nullptr, Trans::N, b, nullptr, Trans::N); }

// ---- include/microtorch/device_cache.hpp: residency -----------------------------------------------------
void set_residency(bool on) { g_resident_on = on; }
bool residency_enabled() { return g_resident_on; }
void make_resident(const Matrix& m) {  // upload now, or refresh in place when the shape still matches
    bring_up();
    const float* key = m.get_data();
    const size_t bytes = m.rows() * m.cols() * sizeof(float);
    auto it = g_resident.find(key);
    if (it != g_resident.end() && (it->second.rows != m.rows() || it->second.cols != m.cols())) {
        pk_free(it->second.ptr);
        g_resident.erase(it);
        it = g_resident.end();
    }
    if (it == g_resident.end()) {
        void* d = nullptr;
        must(pk_alloc(bytes ? bytes : 4, &d), "pk_alloc");
        it = g_resident.emplace(key, Resident{d, m.rows(), m.cols()}).first;
    }
    const int rc = pk_memcpy_h2d(it->second.ptr, key, bytes, nullptr);
    if (rc != PK_OK) {  // no half-made entry stays behind
        pk_free(it->second.ptr);
        g_resident.erase(it);
        must(rc, "upload");
    }
}
void invalidate(const Matrix& m) {
    const auto it = g_resident.find(m.get_data());
    if (it == g_resident.end()) return;
    pk_free(it->second.ptr);
    g_resident.erase(it);
}
void evict_all() {
    for (auto& kv : g_resident) pk_free(kv.second.ptr);
    g_resident.clear();
}
size_t resident_count() { return g_resident.size(); }

void set_step_residency(bool on) { g_step_on = on; }
bool step_residency_enabled() { return g_step_on; }
void step_begin() {
    ++g_stamp;  // copies stamped by an earlier window are uploaded again before use
    g_window_open = true;
}
void step_end() { g_window_open = false; }
namespace detail {
void release_devstate_impl(DevState* s) {
    if (!s) return;
    if (s->ptr) pk_free(s->ptr);
    delete s;
}
}  // namespace detail

// ---- include/microtorch/device_cache.hpp: op set ----------------------------------------------------------
namespace devops {

bool add(const Matrix& a, const Matrix& b, Matrix& y) {
    if (!ops_active()) return false;
    same_shape(a, b, "add");
    Temp da(a), db(b), dy(a.rows() * a.cols());
    must(pk_op_add(da.get(), db.get(), dy.get(), count(a), PK_F32, nullptr), "add");
    dy.to(y);
    return true;
}
bool sub(const Matrix& a, const Matrix& b, Matrix& y) {  // a + (-1) b on the device
    if (!ops_active()) return false;
    same_shape(a, b, "sub");
    Temp dy(a), db(b);
    must(pk_op_axpy(dy.get(), -1.0f, db.get(), count(a), PK_F32, nullptr), "sub");
    dy.to(y);
    return true;
}
bool mul(const Matrix& a, const Matrix& b, Matrix& y) {
    if (!ops_active()) return false;
    same_shape(a, b, "mul");
    Temp da(a), db(b), dy(a.rows() * a.cols());
    must(pk_op_mul(da.get(), db.get(), dy.get(), count(a), PK_F32, nullptr), "mul");
    dy.to(y);
    return true;
}
bool scale(const Matrix& a, float s, Matrix& y) {
    if (!ops_active()) return false;
    Temp da(a), dy(a.rows() * a.cols());
    must(pk_op_scale(da.get(), s, dy.get(), count(a), PK_F32, nullptr), "scale");
    dy.to(y);
    return true;
}
bool axpy(Matrix& y, float a, const Matrix& x) {
    if (!ops_active()) return false;
    same_shape(y, x, "axpy");
    Temp dy(y), dx(x);
    must(pk_op_axpy(dy.get(), a, dx.get(), count(y), PK_F32, nullptr), "axpy");
    dy.to(y);
    return true;
}
bool fill(Matrix& y, float v) {
    if (!ops_active()) return false;
    Temp dy(y.rows() * y.cols());
    must(pk_op_fill(dy.get(), v, count(y), PK_F32, nullptr), "fill");
    dy.to(y);
    return true;
}

// Outside the accelerated path (GPT-2's operators): not handled, the caller's host loop runs.
bool sigmoid_fwd(const Matrix&, Matrix&) { return false; }
bool sigmoid_bwd(const Matrix&, const Matrix&, Matrix&) { return false; }
bool gelu_fwd(const Matrix&, Matrix&) { return false; }
bool gelu_bwd(const Matrix&, const Matrix&, Matrix&) { return false; }
bool softmax_fwd(const Matrix&, Matrix&) { return false; }
bool softmax_bwd(const Matrix&, const Matrix&, Matrix&) { return false; }
bool layernorm_fwd(const Matrix&, const Matrix&, const Matrix&, float, Matrix&, Matrix&, std::vector<float>&) {
    return false;
}
bool layernorm_bwd(const Matrix&, const Matrix&, const std::vector<float>&, const Matrix&, bool, Matrix*, Matrix*, bool,
                   Matrix*) {
    return false;
}

bool rmsnorm_fwd(const Matrix& x, const Matrix& w, float eps, Matrix& y, std::vector<float>& rms_inv) {
    if (!ops_active()) return false;
    if (w.rows() != 1 || w.cols() != x.cols()) throw std::runtime_error("rmsnorm: w must be [1, cols(x)]");
    Temp dx(x), dw(w), dy(x.rows() * x.cols()), dr(x.rows());
    must(pk_op_rmsnorm_fwd(dx.get(), dw.f(), eps, dy.get(), dr.f(), static_cast<int64_t>(x.rows()),
                           static_cast<int64_t>(x.cols()), PK_F32, nullptr),
         "rmsnorm_fwd");
    dy.to(y);
    rms_inv.resize(x.rows());
    dr.to(rms_inv.data());
    return true;
}
bool rmsnorm_bwd(const Matrix& dY, const Matrix& x, const std::vector<float>& rms_inv, const Matrix& w, bool want_dw,
                 Matrix* dw, bool want_dx, Matrix* dx) {
    if (!ops_active()) return false;
    same_shape(dY, x, "rmsnorm_bwd");
    Temp ddy(dY), dxin(x), dr(rms_inv.data(), rms_inv.size()), dwin(w);
    Temp ddw(want_dw ? x.cols() : 1), ddx(want_dx ? x.rows() * x.cols() : 1);
    must(pk_op_rmsnorm_bwd(ddy.get(), dxin.get(), dr.f(), dwin.f(), want_dw ? ddw.f() : nullptr,
                           want_dx ? ddx.get() : nullptr, static_cast<int64_t>(x.rows()),
                           static_cast<int64_t>(x.cols()), PK_F32, nullptr),
         "rmsnorm_bwd");
    if (want_dw && dw) ddw.to(*dw);
    if (want_dx && dx) ddx.to(*dx);
    return true;
}

bool silu_fwd(const Matrix& x, Matrix& y) {
    if (!ops_active()) return false;
    Temp dx(x), dy(x.rows() * x.cols());
    must(pk_op_silu_fwd(dx.get(), dy.get(), count(x), PK_F32, nullptr), "silu_fwd");
    dy.to(y);
    return true;
}
bool silu_bwd(const Matrix& x, const Matrix& dy, Matrix& dx) {
    if (!ops_active()) return false;
    same_shape(x, dy, "silu_bwd");
    Temp a(x), g(dy), out(x.rows() * x.cols());
    must(pk_op_silu_bwd(a.get(), g.get(), out.get(), count(x), PK_F32, nullptr), "silu_bwd");
    out.to(dx);
    return true;
}

bool attention_fwd(const Matrix& q, const Matrix& k, const Matrix& v, float scale, size_t seq_len, bool causal,
                   size_t window, size_t sinks, Matrix& y, std::vector<float>& lse) {
    if (!ops_active()) return false;
    check_heads(q, k, v, seq_len, "fused_attention");
    const pk_attn_shape s = head_shape(q, scale, seq_len, causal, window, sinks);
    Temp dq(q), dk(k), dv(v), dy(q.rows() * q.cols()), dl(q.rows());
    const pk_tensor4 tq = one_head(dq.get(), s), tk = one_head(dk.get(), s), tv = one_head(dv.get(), s),
                     ty = one_head(dy.get(), s);
    must(pk_attn_fwd(&s, &tq, &tk, &tv, &ty, dl.f(), nullptr), "fused_attention");
    dy.to(y);
    lse.resize(q.rows());
    dl.to(lse.data());
    return true;
}
bool attention_bwd(const Matrix& q, const Matrix& k, const Matrix& v, const Matrix& y, const std::vector<float>& lse,
                   const Matrix& dy, float scale, size_t seq_len, bool causal, size_t window, size_t sinks, Matrix* dq,
                   Matrix* dk, Matrix* dv) {
    if (!ops_active()) return false;
    check_heads(q, k, v, seq_len, "fused_attention");
    same_shape(y, dy, "fused_attention backward");
    const pk_attn_shape s = head_shape(q, scale, seq_len, causal, window, sinks);
    const size_t n = q.rows() * q.cols();
    Temp a(q), b(k), c(v), o(y), g(dy), l(lse.data(), lse.size()), gq(n), gk(n), gv(n);
    Temp ws(pk_attn_bwd_workspace_bytes(&s) / sizeof(float) + 1);
    const pk_tensor4 tq = one_head(a.get(), s), tk = one_head(b.get(), s), tv = one_head(c.get(), s),
                     to = one_head(o.get(), s), tg = one_head(g.get(), s), tdq = one_head(gq.get(), s),
                     tdk = one_head(gk.get(), s), tdv = one_head(gv.get(), s);
    must(pk_attn_bwd(&s, &tq, &tk, &tv, &to, l.f(), &tg, &tdq, &tdk, &tdv, ws.get(), pk_attn_bwd_workspace_bytes(&s),
                     nullptr),
         "fused_attention backward");
    if (dq) gq.to(*dq);
    if (dk) gk.to(*dk);
    if (dv) gv.to(*dv);
    return true;
}

}  // namespace devops
}  // namespace device

// ---- the tape nodes over the seam ------------------------------------------------------------------------
namespace ops {
namespace {

Var attention_node(const Var& q, const Var& k, const Var& v, float scale, size_t seq_len, bool causal, size_t window,
                   size_t sinks) {
    Matrix y(q->data.rows(), q->data.cols());
    auto lse = std::make_shared<std::vector<float>>();
    if (!device::devops::attention_fwd(q->data, k->data, v->data, scale, seq_len, causal, window, sinks, y, *lse)) {
        // not handled: the host loops of src/ops.cpp, unchanged
        return window > 0 ? swa_attention(q, k, v, scale, window, sinks, seq_len)
                          : fused_attention(q, k, v, scale, seq_len, causal);
    }
    const bool needs = grad_enabled() && (q->requires_grad || k->requires_grad || v->requires_grad);
    Var out = make_var(std::move(y), needs);
    if (!needs) return out;
    out->parents = {q, k, v};
    Variable* self = out.get();
    out->backward_fn = [self, lse, scale, seq_len, causal, window, sinks]() {
        const Var& q = self->parents[0];
        const Var& k = self->parents[1];
        const Var& v = self->parents[2];
        Matrix dq(q->data.rows(), q->data.cols()), dk(k->data.rows(), k->data.cols()), dv(v->data.rows(), v->data.cols());
        if (!device::devops::attention_bwd(q->data, k->data, v->data, self->data, *lse, self->grad, scale, seq_len, causal,
                                           window, sinks, &dq, &dk, &dv))
            throw std::runtime_error("fused_attention: the device went away between forward and backward");
        if (q->requires_grad) q->accumulate(dq);
        if (k->requires_grad) k->accumulate(dk);
        if (v->requires_grad) v->accumulate(dv);
    };
    return out;
}

}  // namespace

Var fused_attention_hip(const Var& q, const Var& k, const Var& v, float scale, size_t seq_len, bool causal) {
    return attention_node(q, k, v, scale, seq_len, causal, 0, 0);
}
Var swa_attention_hip(const Var& q, const Var& k, const Var& v, float scale, size_t window, size_t sinks,
                      size_t seq_len) {
    if (window == 0) throw std::runtime_error("swa_attention: window must be >= 1");
    return attention_node(q, k, v, scale, seq_len, true, window, sinks);
}

}  // namespace ops
}  // namespace microtorch
