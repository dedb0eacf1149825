// Internal declarations shared by the HIP translation units of
// libpaperkiln_amd.so. Nothing here is part of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "paperkiln_amd.h"

namespace pk {

// Thread-local message behind pk_last_error().
void set_error(const std::string& msg);
int fail(int code, const std::string& msg);
int hip_fail(hipError_t e, const char* what);

#define PK_HIP(expr)                                            \
    do {                                                        \
        hipError_t _e = (expr);                                 \
        if (_e != hipSuccess) return ::pk::hip_fail(_e, #expr); \
    } while (0)

// elementwise.hip: tells the caching allocator that one of its blocks is about to be used on `stream`, so that the
// block, once freed, is only recycled behind that use (no-op for pointers that are not its blocks)
void dev_touch(const void* p, void* stream);

// Kernel-side view of one attention problem. Strides are in elements.
struct AttnArgs {
    const void* q;
    const void* k;
    const void* v;
    void* o;         // fwd: written; bwd: read
    float* lse;      // fwd: written; bwd: read   [B,Hq,T]
    const void* d_o; // bwd only
    void* dq;
    void* dk;
    void* dv;
    float* delta;    // bwd scratch: rowsum(dO .* O)   [B,Hq,T]
    float* tail;     // bwd scratch: partial dK/dV rows of the sink keys (see sink_tail), or null
    float* part;     // bwd scratch: per-split partial dK/dV of a GQA group (see gqa_head_split), or null
    int head_split;  // number of workgroups that share the query heads of one KV head in the dK/dV launch (1 = no split)
    int64_t q_sb, q_st, q_sh;
    int64_t k_sb, k_st, k_sh;
    int64_t v_sb, v_st, v_sh;
    int64_t o_sb, o_st, o_sh;
    int64_t do_sb, do_st, do_sh;
    int64_t dq_sb, dq_st, dq_sh;
    int64_t dk_sb, dk_st, dk_sh;
    int64_t dv_sb, dv_st, dv_sh;
    int B, T, Hq, Hkv, dk_dim;
    int causal, window, sinks;
    int grad_f32; // dq/dk/dv element type: 1 = fp32, 0 = bf16
    float scale;
};

// Visible-set test shared by every kernel: the reference's two ranges
// [b0, sink_hi) u [win_lo, i] (paperkiln src/ops.cpp:879-880, 960-965) in
// per-sequence coordinates. `window == 0` means no band.
__host__ __device__ inline bool pk_visible(int qi, int kj, int T, int causal, int window,
                                           int sinks) {
    if (kj >= T) return false;
    if (causal && kj > qi) return false;
    if (window > 0 && kj + window <= qi && kj >= sinks) return false;
    return true;
}

// Sink tail. With a band mask and a few sink keys (window > 0, 0 < sinks <= 32) the queries past the
// band of key block 0 see nothing of that block but the sink keys, yet the workgroup that owns the
// block would walk every one of them alone: the longest chain of the dK/dV launch by far. The
// matrix-core dK/dV kernels cut that tail into chunks of TAIL_CHUNK queries, each taken by a
// workgroup of its own. Every piece -- the block's own band part and each chunk -- writes its fp32
// partial dK and dV rows of the sink keys into the workspace,
//   tail[((unit * (nch + 1) + piece) * 2 + {0: dK, 1: dV}) * 32 + key][head_dim],   piece nch = band part,
// and a small kernel adds the pieces in a fixed order into the output rows (no atomics, repeatable).
constexpr int TAIL_CHUNK = 512;
struct SinkTail {
    int q0;   // first query of the tail, a multiple of 64
    int nch;  // number of chunks; 0 = the tail is not split
};
__host__ __device__ inline SinkTail sink_tail(int T, int window, int sinks) {
    SinkTail t = {0, 0};
    if (window <= 0 || sinks <= 0 || sinks > 32) return t;
    const long long q0 = ((127LL + window - 1) / 64 + 1) * 64;  // first 64-query tile wholly past block 0's band
    if (q0 >= T) return t;
    t.q0 = static_cast<int>(q0);
    t.nch = (T - t.q0 + TAIL_CHUNK - 1) / TAIL_CHUNK;
    return t;
}
__host__ __device__ inline size_t sink_tail_bytes(int kv_units, int nch, int dk) {
    return nch > 0 ? sizeof(float) * static_cast<size_t>(kv_units) * (nch + 1) * 2 * 32 * dk : 0;
}
__host__ __device__ inline float* sink_tail_rows(float* tail, int unit, int nch, int piece, int which, int dk) {
    return tail + ((static_cast<size_t>(unit) * (nch + 1) + piece) * 2 + which) * 32 * dk;
}
// Whether splitting pays: the tail is one chain of (T - q0) / step query steps (at `speedup` times the
// pace of a full step), the rest of the launch is about
// ceil(workgroups / 256 CUs) workgroups in turn of (128 + window) / step + `prologue` steps each; the
// chunks cost a prologue apiece, so the tail is only split where it would outlast the rest.
__host__ inline bool sink_tail_pays(const SinkTail& t, int T, int window, int kv_units, int step, int prologue,
                                    float speedup) {
    if (t.nch == 0) return false;
    const float chain = static_cast<float>(T - t.q0) / step / speedup;
    const int nkb = (T + 127) / 128;
    const float rest = static_cast<float>((static_cast<int64_t>(nkb) * kv_units + 255) / 256) *
                       ((128 + window) / step + prologue);
    return chain > rest;
}
// GQA head split. One dK/dV workgroup owns 128 keys of one (batch, KV head) and walks the query tiles of every
// query head of the group in turn, so a launch has ceil(T/128) * B * Hkv workgroups (half that when causal
// blocks are paired) however many query heads there are: 14 query heads on 2 KV heads at B = 4, T = 2048
// fill 64 of 256 CUs. Where the launch would leave CUs idle, the heads of a group are dealt to `hs`
// workgroups; split r takes heads [r rep / hs, (r + 1) rep / hs), writes its fp32 partial dK and dV to
//   part[((unit * hs + r) * 2 + {0: dK, 1: dV}) * T + key][head_dim]
// and a second kernel adds the splits in order (no atomics, repeatable). Band-free bf16 kernels only.
__host__ __device__ inline int gqa_head_split(int B, int T, int Hq, int Hkv, int dk, int causal, int window, int bf16) {
    const int rep = Hq / Hkv;
    if (!bf16 || rep <= 1 || window != 0 || (dk != 64 && dk != 128)) return 1;
    const int nkb = (T + 127) / 128;
    const long long wgs = static_cast<long long>(causal ? (nkb + 1) / 2 : nkb) * B * Hkv;
    if (wgs >= 384) return 1;  // at least one and a half workgroups per CU already
    const int hs = static_cast<int>((512 + wgs - 1) / wgs);
    return hs < rep ? hs : rep;
}
__host__ __device__ inline size_t gqa_part_bytes(int kv_units, int hs, int T, int dk) {
    return hs > 1 ? sizeof(float) * 2 * static_cast<size_t>(kv_units) * hs * T * dk : 0;
}
// adds the splits into dK / dV; attn_bwd_dkdv3.hip
int launch_gqa_reduce(const AttnArgs& a, hipStream_t st);

// adds the pieces into dK/dV rows [0, sinks) of every (batch, KV head); attn_bwd_dkdv2.hip
int launch_sink_tail_reduce(const AttnArgs& a, hipStream_t st);

// attn_generic.hip: fp32-math kernels for any head_dim <= 256 and either
// element type. The fp32 contract (max-abs 1e-5 vs the CPU reference) lives here.
int launch_generic_fwd(const AttnArgs& a, bool bf16_in, hipStream_t st);
int launch_generic_bwd(const AttnArgs& a, bool bf16_in, int stages, hipStream_t st);

// attn_f32_mfma.hip: fp32 tensors on the fp32 matrix instruction, head_dim 32 / 64 / 128.
bool f32_mfma_supported(const AttnArgs& a);
int launch_f32_mfma_fwd(const AttnArgs& a, hipStream_t st);
int launch_f32_mfma_bwd(const AttnArgs& a, int stages, hipStream_t st);

// attn_fwd_mfma.hip / attn_bwd_mfma.hip: bf16 MFMA kernels, head_dim 64 or 128.
bool mfma_supported(const AttnArgs& a);
int launch_mfma_fwd(const AttnArgs& a, hipStream_t st);
int launch_mfma_bwd(const AttnArgs& a, int stages, hipStream_t st);
int launch_mfma_dkdv2(const AttnArgs& a, hipStream_t st);
// attn_bwd_dkdv3.hip: dK / dV with 64 keys per wavefront and hand-fixed register classes (head_dim 64 or 128, no band)
bool mfma_dkdv3_takes(const AttnArgs& a);
int launch_mfma_dkdv3(const AttnArgs& a, hipStream_t st);
// attn_bwd_dq3.hip: dQ with 64 queries per wavefront, same construction (head_dim 64 or 128, no band)
bool mfma_dq3_takes(const AttnArgs& a);
int launch_mfma_dq3(const AttnArgs& a, bool fuse_delta, hipStream_t st);

}  // namespace pk
