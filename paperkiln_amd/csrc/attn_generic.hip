// Generic flash-attention kernels: fp32 arithmetic on plain VALU FMAs, any
// head_dim <= 256, any T, fp32 or bf16 storage. This is the path that carries
// the fp32 contract (max-abs 1e-5 against the reference's CPU attention,
// paperkiln src/ops.cpp:863-1027) and the shapes the MFMA kernels do not take.
//
// Tiling: 32 queries x 32 keys per step, 256 threads as 8 x 32. Thread
// (ty, tx) owns score entries (rows 4ty..4ty+3, key tx) and output entries
// (rows 4ty..4ty+3, columns tx + 32c). All tiles sit in LDS with a +1 float
// pad so that column-strided reads hit distinct banks.
#include "pk_internal.h"

namespace pk {
namespace {

constexpr int TM = 32;   // query rows per tile
constexpr int TN = 32;   // keys per tile
constexpr int RPT = 4;   // rows per thread
constexpr int MAXC = 8;  // ceil(256 / 32) column slots per thread

struct F32 {
    typedef float type;
    __device__ static float ld(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
    __device__ static void st(void* p, int64_t i, float x) { static_cast<float*>(p)[i] = x; }
};
struct BF16 {
    typedef uint16_t type;
    __device__ static float ld(const void* p, int64_t i) {
        return __uint_as_float(static_cast<uint32_t>(static_cast<const uint16_t*>(p)[i]) << 16);
    }
    __device__ static void st(void* p, int64_t i, float x) {
        uint32_t u = __float_as_uint(x);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u)
            u |= 0x00400000u;  // NaN stays NaN: no rounding carry into the exponent
        else
            u += 0x7FFFu + ((u >> 16) & 1u);  // round to nearest even
        static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(u >> 16);
    }
};

// Sum / max over the 32 lanes that share one ty (half a wavefront).
__device__ inline float half_wave_max(float x) {
#pragma unroll
    for (int o = 16; o >= 1; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
    return x;
}
__device__ inline float half_wave_sum(float x) {
#pragma unroll
    for (int o = 16; o >= 1; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// Copy rows [r0, r0+32) of one head into LDS as fp32, zero-filling rows >= T.
template <typename IO>
__device__ inline void load_tile(float* dst, int ld, const void* src, int64_t base, int64_t st_t,
                                 int r0, int T, int D) {
    for (int idx = threadIdx.x; idx < TM * D; idx += blockDim.x) {
        const int r = idx / D, c = idx - r * D;
        const int t = r0 + r;
        dst[r * ld + c] = t < T ? IO::ld(src, base + t * st_t + c) : 0.0f;
    }
}

// A key tile is worth visiting for a query tile iff some pair is visible.
__device__ inline bool tile_live(int q0, int k0, int T, int causal, int window, int sinks) {
    const int qhi = min(q0 + TM, T) - 1, khi = min(k0 + TN, T) - 1;
    if (q0 >= T || k0 >= T) return false;
    if (causal && k0 > qhi) return false;
    if (window > 0 && !(khi + window > q0 || k0 < sinks)) return false;
    return true;
}

template <typename IO>
__global__ __launch_bounds__(256) void generic_fwd(AttnArgs a) {
    extern __shared__ float smem[];
    const int D = a.dk_dim, ld = D + 1;
    float* Qs = smem;
    float* Ks = Qs + TM * ld;
    float* Vs = Ks + TN * ld;
    float* Ps = Vs + TN * ld;  // [TM][TN+1]
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int q0 = blockIdx.x * TM, h = blockIdx.y, b = blockIdx.z;
    const int hk = h / (a.Hq / a.Hkv);
    const int64_t qb = b * a.q_sb + h * a.q_sh, kb = b * a.k_sb + hk * a.k_sh,
                  vb = b * a.v_sb + hk * a.v_sh, ob = b * a.o_sb + h * a.o_sh;

    load_tile<IO>(Qs, ld, a.q, qb, a.q_st, q0, a.T, D);
    float m[RPT], l[RPT], acc[RPT][MAXC];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        m[r] = -1e30f;  // the reference's running-max seed, src/ops.cpp:881
        l[r] = 0.0f;
#pragma unroll
        for (int c = 0; c < MAXC; ++c) acc[r][c] = 0.0f;
    }
    const int ncol = (D + 31) / 32;

    for (int k0 = 0; k0 < a.T; k0 += TN) {
        if (!tile_live(q0, k0, a.T, a.causal, a.window, a.sinks)) continue;  // block-uniform
        __syncthreads();
        load_tile<IO>(Ks, ld, a.k, kb, a.k_st, k0, a.T, D);
        load_tile<IO>(Vs, ld, a.v, vb, a.v_st, k0, a.T, D);
        __syncthreads();
        float s[RPT] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int d = 0; d < D; ++d) {
            const float kv = Ks[tx * ld + d];
#pragma unroll
            for (int r = 0; r < RPT; ++r) s[r] = fmaf(Qs[(ty * RPT + r) * ld + d], kv, s[r]);
        }
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
            const int qi = q0 + ty * RPT + r;
            const bool vis = pk_visible(qi, k0 + tx, a.T, a.causal, a.window, a.sinks);
            const float sc = vis ? s[r] * a.scale : -INFINITY;
            const float mn = fmaxf(m[r], half_wave_max(sc));
            const float p = vis ? expf(sc - mn) : 0.0f;
            const float alpha = expf(m[r] - mn);
            l[r] = l[r] * alpha + half_wave_sum(p);
            m[r] = mn;
            Ps[(ty * RPT + r) * (TN + 1) + tx] = p;
#pragma unroll
            for (int c = 0; c < MAXC; ++c) acc[r][c] *= alpha;
        }
        __syncthreads();
        for (int j = 0; j < TN; ++j) {
            float pj[RPT];
#pragma unroll
            for (int r = 0; r < RPT; ++r) pj[r] = Ps[(ty * RPT + r) * (TN + 1) + j];
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                if (c < ncol) {
                    const int col = tx + 32 * c;
                    const float vv = col < D ? Vs[j * ld + col] : 0.0f;
#pragma unroll
                    for (int r = 0; r < RPT; ++r) acc[r][c] = fmaf(pj[r], vv, acc[r][c]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int qi = q0 + ty * RPT + r;
        if (qi >= a.T) continue;
        const float inv = 1.0f / l[r];
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int col = tx + 32 * c;
            if (c < ncol && col < D) IO::st(a.o, ob + qi * a.o_st + col, acc[r][c] * inv);
        }
        if (tx == 0) a.lse[(static_cast<int64_t>(b) * a.Hq + h) * a.T + qi] = m[r] + logf(l[r]);
    }
}

// delta[b,h,t] = sum_d O * dO : the reference's `dot` (src/ops.cpp:920-921),
// which equals rowsum(dP .* P) without needing P. One wavefront per row.
template <typename IO>
__global__ __launch_bounds__(256) void generic_delta(AttnArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    const int64_t rows = static_cast<int64_t>(a.B) * a.Hq * a.T;
    if (row >= rows) return;
    const int t = row % a.T;
    const int h = (row / a.T) % a.Hq;
    const int b = row / (static_cast<int64_t>(a.T) * a.Hq);
    const int64_t ob = b * a.o_sb + h * a.o_sh + t * a.o_st;
    const int64_t gb = b * a.do_sb + h * a.do_sh + t * a.do_st;
    float s = 0.0f;
    for (int d = lane; d < a.dk_dim; d += 64) s = fmaf(IO::ld(a.o, ob + d), IO::ld(a.d_o, gb + d), s);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
    if (lane == 0) a.delta[row] = s;
}

// Shared by both backward kernels: rebuild P and dS for (rows 4ty.., key tx)
// from Q, K, LSE (src/ops.cpp:917-926 with A replaced by exp(scale*s - lse)).
__device__ inline void recompute_p_ds(const AttnArgs& a, const float* Qs, const float* dOs,
                                      const float* Ks, const float* Vs, const float* lse_s,
                                      const float* dl_s, int ld, int D, int q0, int k0, int tx,
                                      int ty, float* Ps, float* dSs) {
    float s[RPT] = {0.0f, 0.0f, 0.0f, 0.0f}, dp[RPT] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int d = 0; d < D; ++d) {
        const float kv = Ks[tx * ld + d], vv = Vs[tx * ld + d];
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
            s[r] = fmaf(Qs[(ty * RPT + r) * ld + d], kv, s[r]);
            dp[r] = fmaf(dOs[(ty * RPT + r) * ld + d], vv, dp[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = ty * RPT + r;
        const bool vis = pk_visible(q0 + row, k0 + tx, a.T, a.causal, a.window, a.sinks) &&
                         (q0 + row) < a.T;
        const float p = vis ? expf(s[r] * a.scale - lse_s[row]) : 0.0f;
        Ps[row * (TN + 1) + tx] = p;
        dSs[row * (TN + 1) + tx] = a.scale * p * (dp[r] - dl_s[row]);
    }
}

template <typename IO, typename GO>
__global__ __launch_bounds__(256) void generic_bwd_dkdv(AttnArgs a) {
    extern __shared__ float smem[];
    const int D = a.dk_dim, ld = D + 1;
    float* Qs = smem;
    float* dOs = Qs + TM * ld;
    float* Ks = dOs + TM * ld;
    float* Vs = Ks + TN * ld;
    float* Ps = Vs + TN * ld;
    float* dSs = Ps + TM * (TN + 1);
    float* lse_s = dSs + TM * (TN + 1);
    float* dl_s = lse_s + TM;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int k0 = blockIdx.x * TN, hk = blockIdx.y, b = blockIdx.z;
    const int rep = a.Hq / a.Hkv, ncol = (D + 31) / 32;
    load_tile<IO>(Ks, ld, a.k, b * a.k_sb + hk * a.k_sh, a.k_st, k0, a.T, D);
    load_tile<IO>(Vs, ld, a.v, b * a.v_sb + hk * a.v_sh, a.v_st, k0, a.T, D);
    float dka[RPT][MAXC], dva[RPT][MAXC];
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
        for (int c = 0; c < MAXC; ++c) dka[r][c] = dva[r][c] = 0.0f;

    for (int h = hk * rep; h < (hk + 1) * rep; ++h) {  // the GQA group of this KV head
        const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T;
        for (int q0 = 0; q0 < a.T; q0 += TM) {
            if (!tile_live(q0, k0, a.T, a.causal, a.window, a.sinks)) continue;
            __syncthreads();
            load_tile<IO>(Qs, ld, a.q, b * a.q_sb + h * a.q_sh, a.q_st, q0, a.T, D);
            load_tile<IO>(dOs, ld, a.d_o, b * a.do_sb + h * a.do_sh, a.do_st, q0, a.T, D);
            if (threadIdx.x < TM) {
                const int t = q0 + threadIdx.x;
                lse_s[threadIdx.x] = t < a.T ? a.lse[lrow + t] : 0.0f;
                dl_s[threadIdx.x] = t < a.T ? a.delta[lrow + t] : 0.0f;
            }
            __syncthreads();
            recompute_p_ds(a, Qs, dOs, Ks, Vs, lse_s, dl_s, ld, D, q0, k0, tx, ty, Ps, dSs);
            __syncthreads();
            // dV = P^T dO (src/ops.cpp:907-910), dK = dS^T Q (:930-932):
            // thread owns keys 4ty..4ty+3, columns tx + 32c.
            for (int i = 0; i < TM; ++i) {
                float pi[RPT], di[RPT];
#pragma unroll
                for (int r = 0; r < RPT; ++r) {
                    pi[r] = Ps[i * (TN + 1) + ty * RPT + r];
                    di[r] = dSs[i * (TN + 1) + ty * RPT + r];
                }
#pragma unroll
                for (int c = 0; c < MAXC; ++c) {
                    if (c < ncol) {
                        const int col = tx + 32 * c;
                        const float go = col < D ? dOs[i * ld + col] : 0.0f;
                        const float qv = col < D ? Qs[i * ld + col] : 0.0f;
#pragma unroll
                        for (int r = 0; r < RPT; ++r) {
                            dva[r][c] = fmaf(pi[r], go, dva[r][c]);
                            dka[r][c] = fmaf(di[r], qv, dka[r][c]);
                        }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int kj = k0 + ty * RPT + r;
        if (kj >= a.T) continue;
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int col = tx + 32 * c;
            if (c < ncol && col < D) {
                GO::st(a.dk, b * a.dk_sb + hk * a.dk_sh + kj * a.dk_st + col, dka[r][c]);
                GO::st(a.dv, b * a.dv_sb + hk * a.dv_sh + kj * a.dv_st + col, dva[r][c]);
            }
        }
    }
}

template <typename IO, typename GO>
__global__ __launch_bounds__(256) void generic_bwd_dq(AttnArgs a) {
    extern __shared__ float smem[];
    const int D = a.dk_dim, ld = D + 1;
    float* Qs = smem;
    float* dOs = Qs + TM * ld;
    float* Ks = dOs + TM * ld;
    float* Vs = Ks + TN * ld;
    float* Ps = Vs + TN * ld;
    float* dSs = Ps + TM * (TN + 1);
    float* lse_s = dSs + TM * (TN + 1);
    float* dl_s = lse_s + TM;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int q0 = blockIdx.x * TM, h = blockIdx.y, b = blockIdx.z;
    const int hk = h / (a.Hq / a.Hkv), ncol = (D + 31) / 32;
    const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T;
    load_tile<IO>(Qs, ld, a.q, b * a.q_sb + h * a.q_sh, a.q_st, q0, a.T, D);
    load_tile<IO>(dOs, ld, a.d_o, b * a.do_sb + h * a.do_sh, a.do_st, q0, a.T, D);
    if (threadIdx.x < TM) {
        const int t = q0 + threadIdx.x;
        lse_s[threadIdx.x] = t < a.T ? a.lse[lrow + t] : 0.0f;
        dl_s[threadIdx.x] = t < a.T ? a.delta[lrow + t] : 0.0f;
    }
    float dqa[RPT][MAXC];
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
        for (int c = 0; c < MAXC; ++c) dqa[r][c] = 0.0f;

    for (int k0 = 0; k0 < a.T; k0 += TN) {
        if (!tile_live(q0, k0, a.T, a.causal, a.window, a.sinks)) continue;
        __syncthreads();
        load_tile<IO>(Ks, ld, a.k, b * a.k_sb + hk * a.k_sh, a.k_st, k0, a.T, D);
        load_tile<IO>(Vs, ld, a.v, b * a.v_sb + hk * a.v_sh, a.v_st, k0, a.T, D);
        __syncthreads();
        recompute_p_ds(a, Qs, dOs, Ks, Vs, lse_s, dl_s, ld, D, q0, k0, tx, ty, Ps, dSs);
        __syncthreads();
        // dQ = dS K (src/ops.cpp:927-929)
        for (int j = 0; j < TN; ++j) {
            float dj[RPT];
#pragma unroll
            for (int r = 0; r < RPT; ++r) dj[r] = dSs[(ty * RPT + r) * (TN + 1) + j];
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                if (c < ncol) {
                    const int col = tx + 32 * c;
                    const float kv = col < D ? Ks[j * ld + col] : 0.0f;
#pragma unroll
                    for (int r = 0; r < RPT; ++r) dqa[r][c] = fmaf(dj[r], kv, dqa[r][c]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int qi = q0 + ty * RPT + r;
        if (qi >= a.T) continue;
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int col = tx + 32 * c;
            if (c < ncol && col < D) GO::st(a.dq, b * a.dq_sb + h * a.dq_sh + qi * a.dq_st + col, dqa[r][c]);
        }
    }
}

template <typename K>
int set_lds(K kernel, size_t bytes) {
    PK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    return PK_OK;
}

template <typename IO>
int fwd_impl(const AttnArgs& a, hipStream_t st) {
    const int ld = a.dk_dim + 1;
    const size_t lds = sizeof(float) * (3 * TM * ld + TM * (TN + 1));
    if (int rc = set_lds(generic_fwd<IO>, lds)) return rc;
    dim3 grid((a.T + TM - 1) / TM, a.Hq, a.B);
    hipLaunchKernelGGL(generic_fwd<IO>, grid, dim3(256), lds, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

template <typename IO, typename GO>
int bwd_impl(const AttnArgs& a, int stages, hipStream_t st) {
    const int ld = a.dk_dim + 1;
    const size_t lds = sizeof(float) * (4 * TM * ld + 2 * TM * (TN + 1) + 2 * TM);
    if (int rc = set_lds(generic_bwd_dkdv<IO, GO>, lds)) return rc;
    if (int rc = set_lds(generic_bwd_dq<IO, GO>, lds)) return rc;
    const int64_t rows = static_cast<int64_t>(a.B) * a.Hq * a.T;
    if (stages & PK_BWD_DELTA) {
        hipLaunchKernelGGL(generic_delta<IO>, dim3((rows + 3) / 4), dim3(256), 0, st, a);
        PK_HIP(hipGetLastError());
    }
    if (stages & PK_BWD_DKDV) {
        hipLaunchKernelGGL((generic_bwd_dkdv<IO, GO>), dim3((a.T + TN - 1) / TN, a.Hkv, a.B), dim3(256),
                           lds, st, a);
        PK_HIP(hipGetLastError());
    }
    if (stages & PK_BWD_DQ) {
        hipLaunchKernelGGL((generic_bwd_dq<IO, GO>), dim3((a.T + TM - 1) / TM, a.Hq, a.B), dim3(256),
                           lds, st, a);
        PK_HIP(hipGetLastError());
    }
    return PK_OK;
}

}  // namespace

int launch_generic_fwd(const AttnArgs& a, bool bf16_in, hipStream_t st) {
    return bf16_in ? fwd_impl<BF16>(a, st) : fwd_impl<F32>(a, st);
}

int launch_generic_bwd(const AttnArgs& a, bool bf16_in, int stages, hipStream_t st) {
    if (bf16_in) return a.grad_f32 ? bwd_impl<BF16, F32>(a, stages, st) : bwd_impl<BF16, BF16>(a, stages, st);
    return a.grad_f32 ? bwd_impl<F32, F32>(a, stages, st) : bwd_impl<F32, BF16>(a, stages, st);
}

}  // namespace pk
