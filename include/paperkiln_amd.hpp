// paperkiln_amd -- the C++ side of the boundary: the device-resident autograd tape.
//
// Same shape as the reference's tape (paperkiln include/microtorch/autograd.hpp:28-104 and
// include/microtorch/ops.hpp:141-150): Variable / Var / make_var / record / backward / zero_grad /
// checkpoint / NoGrad / live_variables and the tape ops, by the reference's names and argument order. What
// differs is where the numbers live: a Variable's data and grad are pk::Tensor, row-major matrices in HBM
// (the reference's Matrix moved to the device), and the attention node keeps O and the per-row logsumexp,
// never a [T,T] matrix. Link against libpaperkiln_amd.so; every failure is a pk::Error (a
// std::runtime_error, as in the reference). The plain-C entry points are in paperkiln_amd.h.
#pragma once
#include <stdint.h>

#include <atomic>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "paperkiln_amd.h"

// HIP's own stream handle type, redeclared so that this header needs no HIP header.
struct ihipStream_t;
typedef struct ihipStream_t* hipStream_t;

namespace pk {


// What the host side throws. It is a std::runtime_error, as every failure of the reference is (shape faults,
// src/ops.cpp:866-870; runtime-API faults, src/cuda_ops.cu:34-38), and carries the status the C ABI returns.
struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string& msg) : std::runtime_error(msg), code(c) {}
};
[[noreturn]] inline void shape_fail(const std::string& msg) { throw Error(PK_ERR_SHAPE, msg); }
// The status of an exception caught at the C ABI: an Error's own code, PK_ERR_OOM for bad_alloc, else PK_ERR_ARGUMENT.
int status_of(const std::exception& e);

// ---- allocator -------------------------------------------------------------
// Caching device allocator with a byte-level high-water mark. It replaces the
// per-call cudaMalloc / cudaFree of the reference's device seam (paperkiln
// src/cuda_resident.cu:226-263, src/cuda_ops.cu:63-72) and supplies the memory
// receipt the reference can only give as a node count (live_variables(),
// include/microtorch/autograd.hpp:61-64). Blocks are recycled in stream order:
// a block remembers the stream that used it last (the stream it was allocated
// for, or the stream of the last C-ABI call that was handed it: dev_touch) and,
// once freed, is handed out again at once, but only to a request made for that
// same stream, whose later work is ordered after the work that last used the
// block; a request for another stream may take it over only when that stream
// has nothing queued any more.
void* dev_alloc(size_t bytes);
bool dev_free(void* p);       // false: not a block this allocator has handed out (nothing is done then)
void dev_touch(const void* p, void* stream);  // a block of this allocator is about to be used on `stream` (no-op for other pointers)
bool dev_owns(const void* p);  // a block this allocator handed out and has not been given back
size_t dev_live_bytes();
size_t dev_peak_bytes();
void dev_reset_peak();
void dev_trim();  // return cached blocks to the driver

struct Buffer {
    void* p = nullptr;
    size_t bytes = 0;
    bool owned = true;
    explicit Buffer(size_t n) : p(dev_alloc(n)), bytes(n) {}
    Buffer(void* caller_memory, size_t n) : p(caller_memory), bytes(n), owned(false) {}  // a view of caller memory
    ~Buffer() {
        if (owned) (void)dev_free(p);
    }
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
};

// Row-major [rows, cols] matrix, the reference's Matrix
// (third_party/transformer_cpp/include/matrix.hpp:32-43) moved to the device.
struct Tensor {
    std::shared_ptr<Buffer> buf;
    int64_t rows = 0, cols = 0;
    int dtype = PK_F32;
    int64_t off_bytes = 0;  // a row-range view shares the buffer of the whole matrix
    bool empty() const { return !buf; }
    void* ptr() const { return buf ? static_cast<char*>(buf->p) + off_bytes : nullptr; }
    int64_t numel() const { return rows * cols; }
    size_t esize() const { return dtype == PK_F32 ? 4 : 2; }
    static Tensor make(int64_t r, int64_t c, int dt) {
        if (r <= 0 || c <= 0) shape_fail("Matrix: zero dimension");  // components.cpp:29-58
        Tensor t;
        t.rows = r;
        t.cols = c;
        t.dtype = dt;
        t.buf = std::make_shared<Buffer>(static_cast<size_t>(r) * c * (dt == PK_F32 ? 4 : 2));
        return t;
    }
    static Tensor borrow(const void* p, int64_t r, int64_t c, int dt) {  // caller-owned device memory, never freed here
        if (!p) throw std::runtime_error("null device pointer");
        if (r <= 0 || c <= 0) shape_fail("Matrix: zero dimension");
        if (dt != PK_F32 && dt != PK_BF16) throw std::runtime_error("unknown element type");
        Tensor t;
        t.rows = r;
        t.cols = c;
        t.dtype = dt;
        t.buf = std::make_shared<Buffer>(const_cast<void*>(p), static_cast<size_t>(r) * c * (dt == PK_F32 ? 4 : 2));
        return t;
    }
    Tensor row_range(int64_t r0, int64_t n) const {  // rows [r0, r0+n) of this matrix, no copy
        Tensor t = *this;
        t.rows = n;
        t.off_bytes = off_bytes + r0 * cols * static_cast<int64_t>(esize());
        return t;
    }
};


// ---- per-tape state ---------------------------------------------------------
// Everything a tape needs besides its Variables: the stream its kernels are
// enqueued on and the element type activations and GEMM operands are held in.
// The reference keeps the like in process-wide globals (device::set,
// src/device.cpp:22,41-46); here a model owns one, and the C ABI makes it the
// calling thread's current context for the length of each call, so two models
// of different element types, or on different streams, do not see each other.
// A thread that never entered a scope works on a context of its own.
struct TapeContext {
    hipStream_t stream = nullptr;
    int compute = PK_F32;
    struct Shadows;  // compute-dtype copies of fp32 parameters (tape.hip)
    std::shared_ptr<Shadows> shadows;
    struct Pending;  // weight-gradient products a backward pass has held back to run several as one launch (tape.hip)
    std::shared_ptr<Pending> pending;
};
TapeContext& tape_context();
class ContextScope {
public:
    explicit ContextScope(TapeContext& c);
    ~ContextScope();
    ContextScope(const ContextScope&) = delete;
    ContextScope& operator=(const ContextScope&) = delete;

private:
    TapeContext* prev_;
};
inline hipStream_t tape_stream() { return tape_context().stream; }
inline void set_tape_stream(hipStream_t s) { tape_context().stream = s; }

// Host <-> device copies of a whole matrix as float32 (bf16 storage is converted on the way), the counterpart
// of the numpy float32 copies at the reference's Python boundary (python/bindings.cpp:21-37). Both wait for
// the tape's stream.
Tensor upload(const float* host, int64_t rows, int64_t cols, int dtype = PK_F32);
void download(const Tensor& t, float* host);

// ---- the tape -----------------------------------------------------------------
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
    // grad's storage is also another Variable's grad (both parents of an add take the same tensor): it is read-only
    // until own_grad() has given this Variable a copy of its own. accumulate(), ensure_grad() and zero_grad() do so.
    bool grad_shared = false;
    // grad is exactly 1: backward() seeded this [1,1] root and nothing has been added since (lets a scalar loss's
    // backward skip reading its upstream gradient back from the device). Code that writes grad directly clears it.
    bool grad_is_unit = false;
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
    void accumulate_owned(Tensor&& g, bool shared = false);
    Tensor& ensure_grad();                             // zero-filled grad of data's shape
    Tensor& own_grad();                                // grad, after un-sharing it (call before writing into it in place)
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
// True while checkpoint() re-runs a segment at backward time: the segment's own result is not needed then, only its tape.
bool recomputing();

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
// r + x W: a Linear whose output joins the residual stream (llama.cpp:47, 59), the add done in the product's epilogue
// result_needed = false (only under grad): the node is recorded but its value is not computed -- for the last op of a
// checkpointed segment while it is re-run at backward time (recomputing()), whose value nobody reads.
Var linear_add(const Var& x, const Var& W, const Var& r, bool result_needed = true);
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
// loss_is_root: the caller promises to call backward() on this loss itself (a unit seed); E's gradient share is then
// added to E->grad chunk by chunk during the forward instead of being held until the closure runs.
Var linear_cross_entropy(const Var& h, const Var& E, const std::shared_ptr<Buffer>& targets_dev, int64_t chunk_rows,
                         bool loss_is_root = false);
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
// The same effect for a caller whose parameters outlive the copies (a model that owns both): every copy is
// re-cast from its parameter where it lies, all of them in one launch.
void refresh_shadows();
// Builds the compute-dtype copy of a parameter (or of the side-by-side concatenation linear_cat multiplies by) now
// instead of at its first use, so that a caller measuring activation memory can have them allocated beforehand.
void prepare_shadow(const Var& W);
void prepare_shadow_cat(const std::vector<Var>& Ws);

}  // namespace pk
