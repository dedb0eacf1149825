/* TEST INFRASTRUCTURE ONLY -- the CPU oracle.
 *
 * A plain-C, single-threaded fp32 restatement of the reference's attention
 * path (paperkiln src/ops.cpp:863-1027) extended with the two things the
 * reference computes implicitly but never returns: the per-row logsumexp and
 * the GQA head map. Only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg may load this library, and only as the checker. The
 * product library (libpaperkiln_amd.so) never links it and has no CPU path.
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   pko_attn_head_fwd / _bwd : pinned against the compiled reference
 *       (oracle/_ref) and the committed fixtures, plus closed forms (T=1,
 *       Q=0), fp64 brute force and finite differences.
 *   pko_attn_fwd / _bwd (batched GQA) : pinned through the head functions and
 *       the "GQA == MHA with repeated KV heads, dK/dV summed" equivalence.
 *   LSE : the reference never materialises it; pinned by
 *       LSE_i = scale*s_ij - log A_ij on the reference's own A, and by the
 *       row-sum-to-one invariant.
 */
#ifndef PK_ORACLE_H
#define PK_ORACLE_H
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Return codes: 0 ok; 1 shape mismatch; 2 rows not a multiple of seq_len;
 * 3 window given without causal; 4 allocation failure. These are the
 * conditions the reference throws on (src/ops.cpp:866-870, 951-956). */

/* One head, the reference's unit of work. q,k: [rows,dk]; v,y: [rows,dv];
 * A: [rows,rows] receives the attention weights (masked entries hard 0);
 * lse: [rows] = mx + log z in scaled natural-log units.
 * seq_len 0 = one sequence; otherwise rows are stacked blocks of seq_len.
 * window 0 = fused_attention semantics (causal flag honoured);
 * window >= 1 = swa_attention semantics (causal band + `sinks` sink keys). */
int pko_attn_head_fwd(const float* q, const float* k, const float* v, size_t rows, size_t dk,
                      size_t dv, float scale, size_t seq_len, int causal, size_t window,
                      size_t sinks, float* y, float* lse, float* A);

/* Backward closure of the same node (src/ops.cpp:902-933, 997-1026): consumes
 * the A written by the forward. Outputs are overwritten, not accumulated. */
int pko_attn_head_bwd(const float* q, const float* k, const float* v, const float* A,
                      const float* dy, size_t rows, size_t dk, size_t dv, float scale,
                      size_t seq_len, int causal, size_t window, size_t sinks, float* dq,
                      float* dk_out, float* dv_out);

/* Batched GQA form over contiguous [B,T,H,dk] tensors (the reference's
 * [N, H*dk] activation layout, src/llama.cpp:48-50). Query head h reads KV
 * head h / (Hq/Hkv). lse: [B,Hq,T]. dk/dv: [B,T,Hkv,dk], summed over each
 * group the way Variable::accumulate would (src/autograd.cpp:16-24). */
int pko_attn_fwd(const float* q, const float* k, const float* v, size_t B, size_t T, size_t Hq,
                 size_t Hkv, size_t dk, float scale, int causal, size_t window, size_t sinks,
                 float* o, float* lse);
int pko_attn_bwd(const float* q, const float* k, const float* v, const float* d_o, size_t B,
                 size_t T, size_t Hq, size_t Hkv, size_t dk, float scale, int causal,
                 size_t window, size_t sinks, float* dq, float* dk_out, float* dv_out);

/* ops::attention_mask (src/ops.cpp:1029-1044): additive 0 / -1e9 mask. */
int pko_attention_mask(size_t rows, size_t seq_len, int causal, float* out);

/* Visible (query,key) pairs per head for the work model: causal T(T+1)/2 or
 * the band count of src/ops.cpp:960-965. */
unsigned long long pko_visible_pairs(size_t T, int causal, size_t window, size_t sinks);

/* ---- Llama block ops (fp32, the reference's loop order) ------------------
 * Pinned by tests/test_oracle_blockops.py: against vectors written by the
 * compiled reference (tests/golden/blockops_fp32.npz), against the compiled
 * reference itself where it is present, and against fp64 finite differences
 * and closed forms. AdamW and clip_grad_norm are pinned by the parameters the
 * reference's own optimiser produced (tests/golden/llama_*.npz). */

/* ops::rmsnorm forward (src/ops.cpp:437-445): y = x * rms_inv * w, rms_inv = 1/sqrt(mean(x^2)+eps). */
void pko_rmsnorm_fwd(const float* x, const float* w, size_t R, size_t C, float eps, float* y, float* rms_inv);
/* its backward (src/ops.cpp:447-478); dw and dx are overwritten. */
void pko_rmsnorm_bwd(const float* dy, const float* x, const float* rms_inv, const float* w, size_t R, size_t C,
                     float* dw, float* dx);
/* ops::silu (src/ops.cpp:404-424). */
void pko_silu_fwd(const float* x, size_t n, float* y);
void pko_silu_bwd(const float* x, const float* dy, size_t n, float* dx);
/* ops::apply_rope (src/ops.cpp:481-537) on a fused [T, 3d] matrix: adjacent pairs of the FIRST head_dim
 * columns of the q third and of the k third are rotated (the reference's loop never reaches the other
 * heads); inverse != 0 is the backward. Returns -1 on the reference's argument errors. */
int pko_rope(const float* x, const int* pos, size_t T, size_t d3, float theta, size_t head_dim, int inverse,
             float* y);
/* ops::embedding (src/ops.cpp:329-348): gather; backward scatter-adds into a zeroed table. -1 = id out of range. */
int pko_embedding_fwd(const float* table, size_t V, size_t d, const int* ids, size_t n, float* y);
int pko_embedding_bwd(const float* dy, const int* ids, size_t n, size_t V, size_t d, float* dtable);
/* ops::cross_entropy (src/ops.cpp:350-376) with Matrix::apply_softmax (components.cpp:229-251): mean NLL with
 * the max(p, 1e-12) clamp, double accumulation; dlogits = (P - onehot) / R. -1 = target out of range. */
int pko_cross_entropy(const float* logits, const int* targets, size_t R, size_t C, float* loss, float* dlogits);
/* nn::AdamW::step for one parameter at step t >= 1 (src/nn.cpp:301-321). */
void pko_adamw(float* p, const float* g, float* m, float* v, size_t n, float lr, float b1, float b2, float eps,
               float wd, int t);
/* ops::clip_grad_norm over a list of gradients (src/ops.cpp:1046-1064); returns the norm before clipping. */
float pko_clip_grad_norm(float* const* grads, const size_t* sizes, size_t nparams, float max_norm);

#ifdef __cplusplus
}
#endif
#endif
