// C ABI of the Llama block operators: the HIP counterparts of the reference's
// devops entry points (paperkiln include/microtorch/device_cache.hpp:97-127)
// and of the operators the reference still runs as host loops (silu, rope,
// embedding, cross-entropy, AdamW, clip). Device pointers in, device pointers
// out, row-major contiguous matrices, fp32 or bf16 storage with fp32 math.
// Every call only enqueues on `stream` unless it says it returns a host value.
#include <cmath>
#include <stdexcept>
#include <string>

#include "paperkiln_amd.h"
#include "pk_internal.h"
#include "tensor.h"

namespace pk {
namespace {

struct StreamScope {  // the launchers enqueue on the tape's stream
    hipStream_t prev;
    explicit StreamScope(void* s) : prev(tape_stream()) { set_tape_stream(static_cast<hipStream_t>(s)); }
    ~StreamScope() { set_tape_stream(prev); }
};

thread_local std::string g_op_err;
template <typename F>
int op_guard(void* stream, F&& f) {
    try {
        StreamScope sc(stream);
        f();
        return PK_OK;
    } catch (const std::exception& e) {
        g_op_err = e.what();
        set_error(g_op_err);
        return status_of(e);
    }
}

// a caller's matrix as a borrowed tensor; if it is a block of the library's allocator, the allocator learns which
// stream uses it now
Tensor mat(const void* p, int64_t r, int64_t c, int dt) {
    dev_touch(p, tape_stream());
    return Tensor::borrow(p, r, c, dt);
}
Tensor vec(const void* p, int64_t n, int dt) { return mat(p, 1, n, dt); }

}  // namespace
}  // namespace pk

using namespace pk;

extern "C" {

int pk_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes, void* stream) {
    return op_guard(stream, [&] {
        if (bytes == 0) return;
        if (!dst_device || !src_host) throw Error(PK_ERR_ARGUMENT, "pk_memcpy_h2d: null pointer");
        hip_check(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, tape_stream()), "hipMemcpyAsync");
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
    });
}
int pk_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream) {
    return op_guard(stream, [&] {
        if (bytes == 0) return;
        if (!dst_host || !src_device) throw Error(PK_ERR_ARGUMENT, "pk_memcpy_d2h: null pointer");
        hip_check(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, tape_stream()), "hipMemcpyAsync");
        hip_check(hipStreamSynchronize(tape_stream()), "hipStreamSynchronize");
    });
}

int pk_op_add(const void* a, const void* b, void* y, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_add(vec(a, n, dtype), vec(b, n, dtype), vec(y, n, dtype)); });
}
int pk_op_mul(const void* a, const void* b, void* y, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_mul(vec(a, n, dtype), vec(b, n, dtype), vec(y, n, dtype)); });
}
int pk_op_scale(const void* a, float s, void* y, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_scale(vec(a, n, dtype), s, vec(y, n, dtype)); });
}
int pk_op_axpy(void* y, float a, const void* x, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_axpy(vec(y, n, dtype), a, vec(x, n, dtype)); });
}
int pk_op_fill(void* y, float v, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_fill(vec(y, n, dtype), v); });
}
int pk_op_silu_fwd(const void* x, void* y, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_silu_fwd(vec(x, n, dtype), vec(y, n, dtype)); });
}
int pk_op_silu_bwd(const void* x, const void* dy, void* dx, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_silu_bwd(vec(x, n, dtype), vec(dy, n, dtype), vec(dx, n, dtype)); });
}
int pk_op_silu_mul_fwd(const void* gate, const void* up, void* y, int64_t n, int dtype, void* stream) {
    return op_guard(stream, [&] { k_silu_mul_fwd(vec(gate, n, dtype), vec(up, n, dtype), vec(y, n, dtype)); });
}
int pk_op_silu_mul_bwd(const void* gate, const void* up, const void* dy, void* dgate, void* dup, int64_t n, int dtype,
                       void* stream) {
    return op_guard(stream, [&] {
        k_silu_mul_bwd(vec(gate, n, dtype), vec(up, n, dtype), vec(dy, n, dtype), vec(dgate, n, dtype), vec(dup, n, dtype));
    });
}
int pk_op_rmsnorm_fwd(const void* x, const float* w, float eps, void* y, float* rms_inv, int64_t rows, int64_t cols,
                      int dtype, void* stream) {
    return op_guard(stream, [&] {
        if (!rms_inv) throw std::runtime_error("rmsnorm: rms_inv is required");
        k_rmsnorm_fwd(mat(x, rows, cols, dtype), mat(w, 1, cols, PK_F32), eps,
                      mat(y, rows, cols, dtype), rms_inv);
    });
}
int pk_op_rmsnorm_bwd(const void* dy, const void* x, const float* rms_inv, const float* w, float* dw, void* dx,
                      int64_t rows, int64_t cols, int dtype, void* stream) {
    return op_guard(stream, [&] {
        if (!rms_inv) throw std::runtime_error("rmsnorm: rms_inv is required");
        Tensor tdw, tdx;
        if (dw) {
            tdw = mat(dw, 1, cols, PK_F32);
            k_fill(tdw, 0.0f);  // the launcher accumulates, as the tape's grad does; this entry point overwrites
        }
        if (dx) tdx = mat(dx, rows, cols, dtype);
        k_rmsnorm_bwd(mat(dy, rows, cols, dtype), mat(x, rows, cols, dtype), rms_inv,
                      mat(w, 1, cols, PK_F32), dw ? &tdw : nullptr, dx ? &tdx : nullptr);
    });
}
int pk_op_rope(const void* qkv, const int* pos, float theta, int64_t rows, int64_t d, int head_dim, int all_heads,
               int inverse, void* y, int dtype, void* stream) {
    return op_guard(stream, [&] {
        if (!pos) throw std::runtime_error("apply_rope: positions are required");
        if (d <= 0 || head_dim <= 0) throw std::runtime_error("apply_rope: head_dim must be even and <= d");
        const int rot = all_heads ? static_cast<int>(d / head_dim) : 1;
        k_rope(mat(qkv, rows, 3 * d, dtype), pos, theta, static_cast<int>(d), head_dim, rot, inverse != 0,
               mat(y, rows, 3 * d, dtype));
    });
}
int pk_op_embedding_fwd(const float* table, const int* ids, void* y, int64_t n, int64_t vocab, int64_t d, int dtype,
                        void* stream) {
    return op_guard(stream, [&] {
        if (!ids) throw std::runtime_error("embedding: ids are required");
        k_embedding_fwd(mat(table, vocab, d, PK_F32), ids, mat(y, n, d, dtype));
    });
}
int pk_op_embedding_bwd(const void* dy, const int* ids, float* dtable, int64_t n, int64_t vocab, int64_t d, int dtype,
                        void* stream) {
    return op_guard(stream, [&] {
        if (!ids) throw std::runtime_error("embedding: ids are required");
        k_embedding_bwd(mat(dy, n, d, dtype), ids, mat(dtable, vocab, d, PK_F32));
    });
}
int pk_op_cross_entropy(void* logits, const int* targets, int64_t rows, int64_t vocab, float upstream, float* nll_rows,
                        float* loss, int dtype, void* stream) {
    return op_guard(stream, [&] {
        if (!targets || !nll_rows) throw std::runtime_error("cross_entropy: one target per row");
        k_ce_rows(mat(logits, rows, vocab, dtype), targets, upstream / static_cast<float>(rows), nll_rows);
        if (loss) *loss = static_cast<float>(k_sum_f32_to_host(nll_rows, rows) / static_cast<double>(rows));
    });
}
int pk_op_adamw(float* p, const float* g, float* m, float* v, int64_t n, float lr, float b1, float b2, float eps,
                float wd, int t, void* stream) {
    return op_guard(stream, [&] {
        if (t < 1) throw std::runtime_error("AdamW: step count starts at 1");
        const float c1 = 1.0f - powf(b1, static_cast<float>(t)), c2 = 1.0f - powf(b2, static_cast<float>(t));
        k_adamw(vec(p, n, PK_F32), vec(g, n, PK_F32), vec(m, n, PK_F32), vec(v, n, PK_F32), lr, b1, b2, eps, wd, c1, c2);
    });
}
int pk_op_sumsq(const float* g, int64_t n, double* host_out, void* stream) {
    return op_guard(stream, [&] {
        if (!host_out) throw std::runtime_error("sumsq: result pointer is required");
        *host_out = k_sumsq_to_host(vec(g, n, PK_F32));
    });
}
int pk_set_gemm_backend(int hand_written) {
    const int before = gemm_backend();
    set_gemm_backend(hand_written <= 0 ? 0 : hand_written == 1 ? 1 : 2);
    gemm_mfma_force_tiles(hand_written == 3 ? 0 : hand_written == 4 ? 1 : hand_written >= 5 ? hand_written : -1);
    return before;
}
int pk_set_head_kernel(int in_product) {
    const int before = head_kernel();
    set_head_kernel(in_product);
    return before;
}
int pk_op_gemm(const void* a, int trans_a, const void* b, int trans_b, void* c, int64_t m, int64_t n, int64_t k,
               int dtype, int c_dtype, int accumulate, void* stream) {
    return op_guard(stream, [&] {
        if (!c) throw std::runtime_error("null device pointer");
        const Tensor A = trans_a ? mat(a, k, m, dtype) : mat(a, m, k, dtype);
        const Tensor B = trans_b ? mat(b, n, k, dtype) : mat(b, k, n, dtype);
        gemm(A, trans_a != 0, B, trans_b != 0, c, c_dtype, m, n, n, accumulate ? 1.0f : 0.0f);
    });
}

}  // extern "C"
