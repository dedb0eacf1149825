/* paperkiln_amd -- C ABI of the MI355X (gfx950) attention hot path.
 *
 * Plain pointers and sizes only; every pointer is DEVICE memory unless it is
 * named host_*. A call enqueues work on `stream` (a hipStream_t passed as
 * void*; NULL = the default stream) and returns without synchronising; work
 * on one stream is ordered. Every entry returns PK_OK or an error code and
 * leaves a message for pk_last_error() (thread-local).
 *
 * The reference (paperkiln, C++ namespace microtorch) has no FFI registry:
 * its seam is a set of C++ free functions that return "handled?" plus the tape
 * ops themselves. Each entry below names the reference function it stands
 * behind (paths relative to the paperkiln tree).
 */
#ifndef PAPERKILN_AMD_H
#define PAPERKILN_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    PK_OK = 0,
    PK_ERR_SHAPE = 1,       /* the reference's "shape mismatch" throws, src/ops.cpp:866-870 */
    PK_ERR_ARGUMENT = 2,    /* bad flag / null pointer / unsupported dtype */
    PK_ERR_WORKSPACE = 3,   /* workspace too small */
    PK_ERR_HIP = 4,         /* a HIP runtime call failed (cuda_check's role, src/cuda_ops.cu:34-38) */
    PK_ERR_OOM = 5
};

enum { PK_F32 = 0, PK_BF16 = 1 };

/* A [B, T, H, dk] tensor view: element strides for batch, token and head; the
 * head_dim axis is contiguous. The reference's activation layout, a row-major
 * [B*T, H*dk] Matrix whose heads are column slices (src/llama.cpp:48-50,
 * src/nn.cpp:146-148), is {stride_b = T*H*dk, stride_t = H*dk, stride_h = dk};
 * a fused [N, 3d] qkv projection is read in place with stride_t = 3*H*dk. */
typedef struct pk_tensor4 {
    void* ptr;
    int64_t stride_b, stride_t, stride_h;
} pk_tensor4;

typedef struct pk_attn_shape {
    int32_t B;          /* sequences; the reference's rows / seq_len blocks (src/ops.cpp:869-879) */
    int32_t T;          /* tokens per sequence (seq_len) */
    int32_t Hq, Hkv;    /* query heads, KV heads; Hq % Hkv == 0; query head h reads KV head h/(Hq/Hkv) */
    int32_t dk;         /* head_dim */
    int32_t causal;     /* fused_attention's `causal` flag */
    int32_t window;     /* 0 = no band (fused_attention); >=1 = swa_attention's window (causal only) */
    int32_t sinks;      /* swa_attention's always-visible leading keys */
    float scale;        /* the op's `scale` argument (1/sqrt(dk) at every reference call site) */
    int32_t dtype;      /* PK_F32 | PK_BF16: element type of q, k, v, o, dO */
    int32_t grad_dtype; /* PK_F32 | PK_BF16: element type of dq, dk, dv */
} pk_attn_shape;

const char* pk_last_error(void);

/* Library / device bring-up. Returns the gfx architecture name through
 * arch[0..arch_len) when non-NULL. Fails loudly when no gfx950 device is
 * visible: there is no CPU path behind this ABI.
 * Stands where device::set(Device::CUDA) / cuda_compiled() do (src/device.cpp:32-46). */
int pk_init(int device, char* arch, size_t arch_len);

/* Forward of ops::fused_attention (src/ops.cpp:863-902) and, with window>=1,
 * ops::swa_attention (src/ops.cpp:948-995), for all B*Hq heads in one launch.
 * Writes O and the per-row logsumexp lse[B,Hq,T] (fp32, natural log of the
 * sum of exp(scale*s_ij) over the visible set) and nothing else: the [T,T]
 * weight matrix the reference keeps for its closure (src/ops.cpp:876,902) is
 * never materialised. */
int pk_attn_fwd(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k,
                const pk_tensor4* v, const pk_tensor4* o, float* lse, void* stream);

/* Bytes of scratch pk_attn_bwd needs for this shape AND mask: the row sums
 * D_i [B,Hq,T] fp32; for a band mask with 1..32 sink keys, room for the
 * partial dK/dV rows of the sink keys (the queries past the band of the first
 * key block may be handed to extra workgroups whose partial sums are added in
 * a fixed order); and, without a band, where query heads share KV heads
 * (Hq > Hkv) on a shape too small to fill the GPU, room for the fp32 partial
 * dK/dV of the workgroups that the heads of a group are dealt to (added in a
 * fixed order as well). Ask with the window and sinks the backward will run
 * with. */
size_t pk_attn_bwd_workspace_bytes(const pk_attn_shape* s);

/* Backward closure of the same node (src/ops.cpp:902-933, 997-1026),
 * recomputed from Q, K and LSE: dV = P^T dO, dP = dO V^T,
 * dS = scale * P .* (dP - rowsum(dO .* O)), dQ = dS K, dK = dS^T Q.
 * dK/dV are summed over the Hq/Hkv query heads of each KV head, which is what
 * Variable::accumulate does when one K/V Variable parents several head nodes
 * (src/autograd.cpp:16-24). Outputs are overwritten (not accumulated). */
int pk_attn_bwd(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k,
                const pk_tensor4* v, const pk_tensor4* o, const float* lse,
                const pk_tensor4* d_o, const pk_tensor4* dq, const pk_tensor4* dk,
                const pk_tensor4* dv, void* workspace, size_t workspace_bytes, void* stream);

/* The same backward by parts, so that a caller can bracket kernels with
 * events: PK_BWD_DELTA (row sums D_i = sum_d O*dO into the workspace),
 * PK_BWD_DKDV (needs DELTA done), PK_BWD_DQ (needs DELTA done). On the
 * matrix-core paths DELTA | DQ in one call is a single kernel (dQ forms D_i for its own
 * rows and writes them), and pk_attn_bwd == that kernel followed by DKDV.
 * The reference has no counterpart: its closure is a single host function
 * (src/ops.cpp:902-933). */
enum { PK_BWD_DELTA = 1, PK_BWD_DKDV = 2, PK_BWD_DQ = 4, PK_BWD_ALL = 7 };
int pk_attn_bwd_stages(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k,
                       const pk_tensor4* v, const pk_tensor4* o, const float* lse,
                       const pk_tensor4* d_o, const pk_tensor4* dq, const pk_tensor4* dk,
                       const pk_tensor4* dv, void* workspace, size_t workspace_bytes, int stages,
                       void* stream);

/* pk_attn_bwd without a workspace argument and without any allocation: the scratch is a device array inside
 * the library (PK_ATTN_BWD_STATIC_MAX_WORKSPACE bytes on every GPU the library runs on, held until the process
 * ends). It has no counterpart in the reference; it is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. Same kernels as pk_attn_bwd, and the same
 * results bit for bit wherever the array also holds the partial sums of a GQA head split (see
 * pk_attn_bwd_workspace_bytes); where only those do not fit, the heads of a group are walked by one workgroup,
 * which changes the order of summation of dK/dV and nothing else. A shape whose row sums and sink rows alone
 * exceed the array is refused with PK_ERR_WORKSPACE. All calls on
 * one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race; calls
 * on one stream are ordered and safe. pk_init looks the array up for its device; otherwise the first call does. */
#define PK_ATTN_BWD_STATIC_MAX_WORKSPACE ((size_t)32 << 20)
int pk_attn_bwd_static(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k,
                       const pk_tensor4* v, const pk_tensor4* o, const float* lse,
                       const pk_tensor4* d_o, const pk_tensor4* dq, const pk_tensor4* dk,
                       const pk_tensor4* dv, void* stream);

/* ---- device memory ------------------------------------------------------
 * Caching allocator with a byte-level high-water mark: the HIP counterpart of
 * the per-call cudaMalloc/cudaFree in src/cuda_resident.cu:226-263 and
 * src/cuda_ops.cu:63-72, and the byte receipt that the reference's
 * live_variables() (include/microtorch/autograd.hpp:61-64) cannot give.
 * A freed block is handed out again at once, without waiting for the GPU, to
 * a request made for the stream that used the block last (the stream it was
 * allocated for, or the `stream` argument of the last pk_* call it was passed
 * to): later work on that stream runs after the earlier work that used the
 * block. A request for another stream takes the block over only once that
 * stream has nothing queued any more. A block that several streams use at the
 * same time is the caller's to keep alive until all of them are done. */
int pk_alloc(size_t bytes, void** out);
int pk_free(void* p);   /* PK_ERR_ARGUMENT for a pointer pk_alloc did not return or that was freed before */
/* Host <-> device copies on `stream`; both return after the copy has completed. They stand where the
 * reference's h2d / d2h helpers and its RAII upload buffer do (src/cuda_ops.cu:45-72), for host code that
 * keeps the reference's host-in / host-out convention and has no HIP header of its own. */
int pk_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes, void* stream);
int pk_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream);
size_t pk_live_bytes(void);
size_t pk_peak_bytes(void);
void pk_reset_peak(void);
void pk_trim(void);

/* ---- activation-checkpointed Llama step ---------------------------------
 * nn::Llama (include/microtorch/llama.hpp:14-51, src/llama.cpp) on the
 * device-resident tape. Parameters are fp32 master copies named exactly as the
 * reference names them ("layers.N.self_attn.q_proj.weight", ...; Linear
 * weights are [in, out], y = x W). compute_dtype PK_BF16 runs activations and
 * GEMM operands in bf16 with fp32 accumulation. */
typedef struct pk_llama_config {
    int32_t vocab, d, n_layers, n_heads, d_ff;
    float rope_theta;
    int32_t tie_embeddings;  /* must be 1: the tied head of llama.cpp:88 */
    int32_t compute_dtype;   /* PK_F32 | PK_BF16 */
    int32_t rope_all_heads;  /* 0 = the reference as written: apply_rope(concat, pos, theta, dk) rotates only
                                the first head of q and of k (src/ops.cpp:498-499, called at llama.cpp:36) */
    int32_t window, sinks;   /* 0,0 = causal fused_attention; window>=1 = swa_attention in every block */
} pk_llama_config;

typedef struct pk_llama_stats {
    int64_t live_vars_after_forward;        /* the reference's receipt (tests/test_checkpointing.cpp:46-60) */
    int64_t activation_bytes_after_forward; /* allocator bytes held by the tape between forward and backward */
    int64_t peak_activation_bytes;          /* high-water mark over forward + backward, parameters, gradients,
                                               optimizer state and bf16 parameter shadows excluded */
} pk_llama_stats;

/* Llama::Llama(cfg, seed): N(0, 0.02) Linear / Embedding weights, unit norm gains.
 * A model owns its tape state (element type, stream, parameter shadows): models of different compute_dtype
 * may live side by side, and each may be driven from a host thread of its own on a stream of its own; calls
 * on ONE model are serialised by a lock inside it. pk_llama_adamw_step and the parameter accessors run on
 * the stream of the model's last pk_llama_loss_backward. The byte counters (pk_live_bytes, pk_peak_bytes,
 * pk_llama_stats) are process-wide, so they are only meaningful while one model steps at a time. */
int pk_llama_create(const pk_llama_config* cfg, unsigned seed, void** handle);
int pk_llama_destroy(void* handle);
int pk_llama_num_params(void* handle);
int pk_llama_param_info(void* handle, int i, char* name, size_t name_len, int64_t* rows, int64_t* cols);
int pk_llama_set_param(void* handle, int i, const float* host);
int pk_llama_get_param(void* handle, int i, float* host);
int pk_llama_get_grad(void* handle, int i, float* host);
/* zero_grad -> forward -> mean cross-entropy -> backward: the step of tools/mtstudio.cpp:456-471.
 * ids/targets are host arrays of n tokens, B = n/seq_len stacked sequences (seq_len 0 = one).
 * checkpoint_blocks: Llama::checkpoint_blocks (llama.hpp:45). fused_head 1 evaluates the tied head
 * and the loss in row chunks (no [n, vocab] matrix); 0 materialises the logits as the reference does. */
int pk_llama_loss_backward(void* handle, const int* host_ids, const int* host_targets, int64_t n, int64_t seq_len,
                           int checkpoint_blocks, int do_backward, int fused_head, float* loss,
                           pk_llama_stats* stats, void* stream);
/* ops::clip_grad_norm (src/ops.cpp:1046-1064; skipped when max_norm <= 0) then nn::AdamW::step (src/nn.cpp:301-321). */
int pk_llama_adamw_step(void* handle, float lr, float b1, float b2, float eps, float wd, float max_norm,
                        float* total_norm);
/* Rows of the tied head (llama.cpp:88 + ops::cross_entropy, src/ops.cpp:350-376) evaluated at a time when
 * fused_head = 1: the [n, vocab] logits the reference materialises exist here one [rows, vocab] chunk at a
 * time. Default: 4096 rows where the cross-entropy runs inside the logits product (bf16 operands; the chunk's scratch is
 * its bf16 dlogits), 2048 where fp32 logits are stored -- 262 MB at a vocabulary of 32000 either way; smaller chunks lower
 * the activation peak, larger ones run fewer, larger GEMMs. */
int pk_llama_set_head_chunk(void* handle, int64_t rows);

/* ---- block operators -------------------------------------------------------
 * The operators of one Llama block as single calls on device memory: row-major
 * contiguous matrices, dtype PK_F32 or PK_BF16 storage, fp32 arithmetic. They
 * stand where the reference's devops entry points do
 * (include/microtorch/device_cache.hpp:97-127: add, mul, scale, axpy, fill,
 * rmsnorm_fwd, rmsnorm_bwd) and add the ones the reference still runs as host
 * loops. Calls only enqueue on `stream` unless a host result is named. */
int pk_op_add(const void* a, const void* b, void* y, int64_t n, int dtype, void* stream);   /* ops::add, src/ops.cpp:60-65 */
int pk_op_mul(const void* a, const void* b, void* y, int64_t n, int dtype, void* stream);   /* ops::mul, src/ops.cpp:76-83 */
int pk_op_scale(const void* a, float s, void* y, int64_t n, int dtype, void* stream);       /* devops::scale */
int pk_op_axpy(void* y, float a, const void* x, int64_t n, int dtype, void* stream);        /* Variable::accumulate, src/autograd.cpp:16-24 */
int pk_op_fill(void* y, float v, int64_t n, int dtype, void* stream);                       /* devops::fill */
/* ops::silu and its closure (src/ops.cpp:404-424). */
int pk_op_silu_fwd(const void* x, void* y, int64_t n, int dtype, void* stream);
int pk_op_silu_bwd(const void* x, const void* dy, void* dx, int64_t n, int dtype, void* stream);
/* mul(silu(gate), up), LlamaBlock's SwiGLU (src/llama.cpp:55-58), as one pass each way instead of the two tape nodes
 * ops::silu and ops::mul (src/ops.cpp:404-424, 76-83). */
int pk_op_silu_mul_fwd(const void* gate, const void* up, void* y, int64_t n, int dtype, void* stream);
int pk_op_silu_mul_bwd(const void* gate, const void* up, const void* dy, void* dgate, void* dup, int64_t n, int dtype,
                       void* stream);
/* ops::rmsnorm (src/ops.cpp:426-479; devops::rmsnorm_fwd / rmsnorm_bwd). w, rms_inv[rows] and dw are fp32;
 * dw and dx may be NULL (the reference's want_dw / want_dx) and are overwritten, not accumulated. */
int pk_op_rmsnorm_fwd(const void* x, const float* w, float eps, void* y, float* rms_inv, int64_t rows, int64_t cols,
                      int dtype, void* stream);
int pk_op_rmsnorm_bwd(const void* dy, const void* x, const float* rms_inv, const float* w, float* dw, void* dx,
                      int64_t rows, int64_t cols, int dtype, void* stream);
/* ops::apply_rope (src/ops.cpp:481-537) on a fused [rows, 3d] projection; pos[rows] on the device. all_heads = 0
 * rotates only the first head of the q and k thirds, as the reference's loop does; 1 rotates every head.
 * inverse = 1 is the backward closure. y may alias qkv. */
int pk_op_rope(const void* qkv, const int* pos, float theta, int64_t rows, int64_t d, int head_dim, int all_heads,
               int inverse, void* y, int dtype, void* stream);
/* ops::embedding (src/ops.cpp:329-348): gather from an fp32 table; the backward scatter-ADDS into dtable (fp32),
 * which the caller zeroes. ids[n] on the device; an id outside the table is the caller's to reject (the reference
 * throws, src/ops.cpp:333). */
int pk_op_embedding_fwd(const float* table, const int* ids, void* y, int64_t n, int64_t vocab, int64_t d, int dtype,
                        void* stream);
int pk_op_embedding_bwd(const void* dy, const int* ids, float* dtable, int64_t n, int64_t vocab, int64_t d, int dtype,
                        void* stream);
/* ops::cross_entropy (src/ops.cpp:350-376), fused: logits[rows, vocab] are REPLACED by dlogits =
 * (P - onehot) * upstream / rows; nll_rows[rows] (device, fp32) receives -log(max(p_target, 1e-12)). When loss is
 * non-NULL the call waits for the stream and returns the mean there (double accumulation, as the reference). */
int pk_op_cross_entropy(void* logits, const int* targets, int64_t rows, int64_t vocab, float upstream, float* nll_rows,
                        float* loss, int dtype, void* stream);
/* nn::AdamW::step for one fp32 parameter at step t >= 1 (src/nn.cpp:301-321). */
int pk_op_adamw(float* p, const float* g, float* m, float* v, int64_t n, float lr, float b1, float b2, float eps,
                float wd, int t, void* stream);
/* The sum of squares ops::clip_grad_norm accumulates in double (src/ops.cpp:1047-1053); waits for the stream. */
int pk_op_sumsq(const float* g, int64_t n, double* host_out, void* stream);
/* device::gemm (src/device.cpp:91-125; include/microtorch/device_cache.hpp:63-71): C[m,n] (+)= op(A) op(B), row-major,
 * op = transpose when the flag is set (A is [k,m] then, B is [n,k]); operands dtype, output c_dtype, fp32 accumulate. */
int pk_op_gemm(const void* a, int trans_a, const void* b, int trans_b, void* c, int64_t m, int64_t n, int64_t k,
               int dtype, int c_dtype, int accumulate, void* stream);
/* Which kernel multiplies bf16 operands. 1 (default): this library's own matrix-core GEMM (the counterpart of the
 * reference's tiled kernel, src/cuda_resident.cu:141-171) for everything it takes (16-byte aligned rows, sizes that
 * are multiples of 8) -- measured on the MI355X it is ahead of rocBLAS or level with it on every Linear product of a
 * d = 512 block and of a 32000-word tied head -- in the form it picks per shape, rocBLAS for the rest; and the
 * weight-gradient products X^T dY of a backward pass over 2048 tokens or more are held back and multiplied several
 * at a time as one grouped launch. 2: the same kernel, every product on its own. 0: rocBLAS for everything, as for
 * fp32 operands. Measurement settings, all like 2 but with one form forced: 3 / 4 the register-staged
 * kernel with 128 x 128 / 256 x 256 tiles; 5, 6, 7 the LDS-ring kernel with 128 x 128 tiles and 4, 2, 3 ring slots;
 * 8 the ring kernel with 256 x 256 tiles; 9, 10, 11 the ring kernel with 128 x 128 tiles shared by two wavefront sets
 * and 2, 3, 4 slots. Process-wide; returns the previous setting (0, 1 or 2). The environment variable
 * PK_GEMM=library selects 0 at load time. */
int pk_set_gemm_backend(int mode);
/* How the chunked tied head (llama.cpp:88 followed by ops::cross_entropy, src/ops.cpp:350-376) forms the loss and
 * dlogits from bf16 operands. 1 (default): inside the logits product -- the library's own GEMM forms every tile of
 * logits twice, first for the rows' maxima and sums of exponentials (and the loss), then to emit bf16 dlogits, and the
 * [rows, vocab] logits never reach memory. 0: one logits product into an fp32 matrix and a row kernel over it (also
 * what fp32 operands, rocBLAS-only mode and shapes the own GEMM does not take get). Process-wide; returns the previous
 * setting. */
int pk_set_head_kernel(int in_product);

#ifdef __cplusplus
}
#endif
#endif /* PAPERKILN_AMD_H */
