// Internal side of the device tensors: the kernel launchers used by the
// host-side tape. The types themselves (Tensor, Buffer, the allocator, the
// tape context) are public and live in include/paperkiln_amd.hpp.
#pragma once
#include <memory>
#include <vector>
#include <hip/hip_runtime.h>

#include "paperkiln_amd.hpp"

namespace pk {

void hip_check(hipError_t e, const char* what);  // throws Error(PK_ERR_HIP), as cuda_check throws (cuda_ops.cu:34-38)

// ---- kernel launchers (elementwise.hip) -----------------------------------
// All take row-major contiguous tensors; T = fp32 or bf16 storage, fp32 math.
void k_fill(const Tensor& y, float v);
void k_cast(const Tensor& src, const Tensor& dst);                      // dtype conversion / copy
void k_cast_cols(const Tensor& src, const Tensor& dst, int64_t col_off);
// many such casts (fp32 -> a column block of a bf16 matrix) as one launch; false = not applicable, nothing done
struct CastJob {
    Tensor src, dst;
    int64_t col_off;
};
bool k_cast_many(const std::vector<CastJob>& list);  // dst[:, off:off+src.cols] = src
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
// ops.cpp:447-478; with an addend (dx's shape and type) dx = addend + the gradient through the norm
void k_rmsnorm_bwd(const Tensor& dy, const Tensor& x, const float* rinv, const Tensor& w, const Tensor* dw_f32,
                   const Tensor* dx, const Tensor* addend = nullptr);
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
void k_mean_f32(const float* x, int64_t n, const Tensor& out);         // the same sum / n into a [1,1] float, no host round trip
double k_sumsq_to_host(const Tensor& g);                               // clip_grad_norm's sum, ops.cpp:1046-1052
// The same in two halves, so that many gradients cost one host round trip: per-block partial sums (at most
// SUMSQ_MAX_PARTS doubles) into device memory, then one copy and a host sum over all of them.
constexpr int SUMSQ_MAX_PARTS = 1024;
int k_sumsq_parts(const Tensor& g, double* part_dev);
double k_sum_f64_to_host(const double* part_dev, int64_t n);
// grad_scale != 1: g is scaled in place first (the clip of ops::clip_grad_norm), in the same pass
void k_adamw(const Tensor& p, const Tensor& g, const Tensor& m, const Tensor& v, float lr, float b1, float b2,
             float eps, float wd, float c1, float c2, float grad_scale = 1.0f);                 // nn.cpp:301-321

// C[M,N] (+)= op(A) . op(B), row-major, bf16 or fp32 operands, fp32 accumulate
// (device::gemm, src/device.cpp:91-125). C may be a column slice of a wider
// matrix (ldc). beta is 0 or 1.
void gemm(const Tensor& A, bool tA, const Tensor& B, bool tB, void* C, int c_dtype, int64_t M, int64_t N, int64_t ldc,
          float beta, int64_t lda = 0);
// gemm_mfma.hip: the hand-written bf16 matrix-core GEMM. Returns false (nothing done) for operands it does not take.
// With an addend (C's type and row pitch; beta must be 1) C = addend + op(A) op(B), the sum rounded once.
bool gemm_mfma_bf16(const void* a, bool tA, int64_t lda, const void* b, bool tB, int64_t ldb, void* c, int c_dtype,
                    int64_t M, int64_t N, int64_t K, int64_t ldc, float beta, hipStream_t st, const void* addend = nullptr);
// The same product left as fp32 partial products part[s][M][N], s < nparts (the contraction cut into slices where the
// output alone would leave the chip idle), for a caller that adds them on the way to where the result goes.
bool gemm_mfma_bf16_parts(const void* a, bool tA, int64_t lda, const void* b, bool tB, int64_t ldb, int64_t M, int64_t N,
                          int64_t K, hipStream_t st, std::unique_ptr<Buffer>& part, int& nparts);
// The tied head's cross-entropy inside its logits product A B^T (bf16 [M, K] and [N, K]): the logits are formed tile
// by tile, twice, and never stored. gemm_head_rows: per row the maximum, 1 / sum exp(z - maximum) and the loss
// (stats: scratch of gemm_head_spans(N) * M float pairs, zt: of M floats); gemm_head_dlogits: bf16 dlogits.
// Both return false, having done nothing, for operands the kernel does not take.
// Several weight-gradient products C_p += A_p^T B_p (A_p [K, M_p], B_p [K, N_p] bf16; C_p [M_p, N_p] fp32) that share
// the contraction length, as one launch of the hand-written kernel. False, with nothing done, where that does not
// apply (operands it does not take, too few tiles): the caller multiplies them one by one.
struct GroupedProduct {
    const void* a;
    int64_t lda;
    const void* b;
    int64_t ldb;
    float* c;
    int64_t ldc;
    int64_t M, N;
};
bool gemm_mfma_grouped_tn(const GroupedProduct* ps, int count, int64_t K, hipStream_t st);
int64_t gemm_head_spans(int64_t N);
bool gemm_head_takes(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K);
bool gemm_head_rows(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K, const int* target,
                    void* stats, float* zt, float* row_max, float* row_inv, float* nll, hipStream_t st);
bool gemm_head_dlogits(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                       const int* target, const float* row_max, const float* row_inv, float gscale, void* dl, int64_t ldc,
                       hipStream_t st);
// Which GEMM serves bf16 operands: 1 (default) and 2 = the hand-written kernel for everything it takes (1 also
// groups a backward pass's weight-gradient products into shared launches), 0 = the library only. Set from the environment
// (PK_GEMM=library) or by a caller that wants to compare them.
void set_gemm_backend(int hand_written);
void gemm_mfma_force_tiles(int which);  // -1: by shape (default); 0, 1, 5 .. 11: one kernel form always (measurement)
int gemm_backend();
// How the chunked tied head forms its cross-entropy from bf16 operands: 1 (default) = inside the logits product
// (gemm_head_rows / gemm_head_dlogits: no logits in memory), 0 = a logits product into fp32 and a row kernel over it.
void set_head_kernel(int in_product);
int head_kernel();
// dst[k] ([A.cols, B.cols/nsplit] fp32, contiguous) = beta * dst[k] + A^T B[:, k-th column block], k < nsplit <= 4
void gemm_tn_split(const Tensor& A, const Tensor& B, float* const* dst, int nsplit, float beta);

}  // namespace pk
