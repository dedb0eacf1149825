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

#ifdef __cplusplus
}
#endif
#endif
