// Device tensors, the caching allocator and the kernel launchers used by the
// host-side tape (tape.h). Everything here lives in HBM; there is no host copy
// of an activation and no CPU code path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <memory>
#include <stdexcept>
#include <string>

#include "paperkiln_amd.h"

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
// a freed block remembers the stream of the thread that freed it (tape_stream())
// and is handed out again at once, but only to a request made for that same
// stream, whose later work is ordered after the work that last used the block.
void* dev_alloc(size_t bytes);
bool dev_free(void* p);       // false: not a block this allocator has handed out (nothing is done then)
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

void hip_check(hipError_t e, const char* what);  // throws Error(PK_ERR_HIP), as cuda_check throws (cuda_ops.cu:34-38)

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

// ---- kernel launchers (elementwise.hip) -----------------------------------
// All take row-major contiguous tensors; T = fp32 or bf16 storage, fp32 math.
void k_fill(const Tensor& y, float v);
void k_cast(const Tensor& src, const Tensor& dst);                      // dtype conversion / copy
void k_cast_cols(const Tensor& src, const Tensor& dst, int64_t col_off);  // dst[:, off:off+src.cols] = src
void k_add(const Tensor& a, const Tensor& b, const Tensor& y);          // y = a + b      (ops.cpp:60-65)
void k_mul(const Tensor& a, const Tensor& b, const Tensor& y);          // y = a .* b     (ops.cpp:76-83)
void k_scale(const Tensor& a, float s, const Tensor& y);                // y = a * s
void k_axpy(const Tensor& y, float a, const Tensor& x);                 // y += a * x     (autograd.cpp:16-24)
void k_silu_fwd(const Tensor& x, const Tensor& y);                      // ops.cpp:404-411
void k_silu_bwd(const Tensor& x, const Tensor& dy, const Tensor& dx);   // ops.cpp:412-423
void k_silu_mul_fwd(const Tensor& gate, const Tensor& up, const Tensor& y);  // silu(gate) .* up, llama.cpp:55-58
void k_silu_mul_bwd(const Tensor& gate, const Tensor& up, const Tensor& dy, const Tensor& dgate, const Tensor& dup);
// the same on the two halves of one [rows, 2*cols] matrix [gate | up]
void k_silu_mul_cat_fwd(const Tensor& gu, const Tensor& y);
void k_silu_mul_cat_bwd(const Tensor& gu, const Tensor& dy, const Tensor& dgu);
void k_rmsnorm_fwd(const Tensor& x, const Tensor& w, float eps, const Tensor& y, float* rinv);  // ops.cpp:437-445
void k_rmsnorm_bwd(const Tensor& dy, const Tensor& x, const float* rinv, const Tensor& w, const Tensor* dw_f32,
                   const Tensor* dx);                                   // ops.cpp:447-478
// apply_rope on a fused [N, 3d] matrix (ops.cpp:481-537): rotates adjacent pairs of the
// first `rot_heads` heads of the q third and of the k third; inverse = backward.
void k_rope(const Tensor& x, const int* pos, float theta, int d, int head_dim, int rot_heads, bool inverse,
            const Tensor& y);
void k_rope_inplace(const Tensor& x, const int* pos, float theta, int d, int head_dim, int rot_heads, bool inverse);
void k_embedding_fwd(const Tensor& table_f32, const int* ids, const Tensor& y);       // ops.cpp:329-337
void k_embedding_bwd(const Tensor& dy, const int* ids, const Tensor& dtable_f32);     // scatter-add, ops.cpp:338-347
// Row-wise softmax cross-entropy on a block of logits (ops.cpp:350-376): writes
// dlogits = (P - onehot) * gscale in place and the per-row nll (fp32) with the
// reference's max(p, 1e-12) clamp.
void k_ce_rows(const Tensor& logits, const int* targets, float gscale, float* nll_rows);
// The same on fp32 logits that are read once and left untouched: dl == nullptr computes only the nll, otherwise
// dlogits go to *dl (fp32 or bf16). Returns false when the shape does not fit (the caller then uses k_ce_rows).
bool k_ce_rows_once(const Tensor& logits, const int* targets, float gscale, float* nll_rows, const Tensor* dl,
                    int64_t dl_ld = 0);  // dl_ld: row pitch of dl in its own elements (0 = cols)
double k_sum_f32_to_host(const float* x, int64_t n);                   // double accumulation, ops.cpp:360-367
double k_sumsq_to_host(const Tensor& g);                               // clip_grad_norm's sum, ops.cpp:1046-1052
// The same in two halves, so that many gradients cost one host round trip: per-block partial sums (at most
// SUMSQ_MAX_PARTS doubles) into device memory, then one copy and a host sum over all of them.
constexpr int SUMSQ_MAX_PARTS = 1024;
int k_sumsq_parts(const Tensor& g, double* part_dev);
double k_sum_f64_to_host(const double* part_dev, int64_t n);
void k_adamw(const Tensor& p, const Tensor& g, const Tensor& m, const Tensor& v, float lr, float b1, float b2,
             float eps, float wd, float c1, float c2);                 // nn.cpp:301-321

// C[M,N] (+)= op(A) . op(B), row-major, bf16 or fp32 operands, fp32 accumulate
// (device::gemm, src/device.cpp:91-125). C may be a column slice of a wider
// matrix (ldc). beta is 0 or 1.
void gemm(const Tensor& A, bool tA, const Tensor& B, bool tB, void* C, int c_dtype, int64_t M, int64_t N, int64_t ldc,
          float beta, int64_t lda = 0);
// dst[k] ([A.cols, B.cols/nsplit] fp32, contiguous) = beta * dst[k] + A^T B[:, k-th column block], k < nsplit <= 4
void gemm_tn_split(const Tensor& A, const Tensor& B, float* const* dst, int nsplit, float beta);

}  // namespace pk
