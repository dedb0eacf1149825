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

}  // namespace pk
