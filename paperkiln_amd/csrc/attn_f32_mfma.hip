// fp32 flash attention (forward, dQ, dK/dV) on the fp32 matrix instruction of
// gfx950, v_mfma_f32_32x32x2_f32: the full-precision path of the reference's
// ops::fused_attention / ops::swa_attention (paperkiln src/ops.cpp:863-934,
// 948-995) for fp32 tensors with head_dim 32, 64 or 128. Products and sums are
// fp32 throughout, so the result stays inside the fp32 contract (max-abs 1e-5
// against the CPU reference); the scalar kernels of attn_generic.hip remain the
// path for every other head size and for unaligned rows.
//
// v_mfma_f32_32x32x2_f32 operands (g = lane / 32, c = lane % 32):
//   A (32 x 2): lane holds A[row c][k = g]          (one float)
//   B (2 x 32): lane holds B[k = g][column c]
//   C (32 x 32): lane holds column c, element r is row m(r, g) = (r/4)*8 + 4g + r%4
// The contraction index may be permuted freely as long as A and B agree, which
// gives two fragment shapes that are both plain 16-byte LDS reads:
//   * contraction over head_dim (S = Q K^T, dP = dO V^T): a lane reads four
//     consecutive floats d = 8j + 4g .. +3 of its row; element i of chunk j
//     is the operand of MFMA step 4j + i on both sides;
//   * contraction over the rows of a C tile (O^T += V^T P^T and the like):
//     register r of the C tile IS the B operand of step r (its row is
//     m(r, g)), and the A operand is row m(r, g) of the other matrix, of which
//     lane c reads the NI = head_dim/32 consecutive columns NI*c .. NI*c+NI-1,
//     one per output block. Block i of the product then holds columns
//     NI*m + i, i.e. the NI blocks of register r are NI consecutive floats of
//     the output row: one vector store.
// As in the bf16 kernels the forward and dQ kernels work on S^T (lane = query,
// so the softmax row statistics are in-lane), dK/dV on S (lane = key).
#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr int BN = 64;   // keys per tile (forward, dQ)
constexpr int BQ = 32;   // queries per step (dK/dV)
constexpr float LOG2E = 1.4426950408889634f;

__device__ inline f32x16 mfma2(float a, float b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

template <int NI> struct FVec;
template <> struct FVec<1> { typedef float type; };
template <> struct FVec<2> { typedef f32x2 type; };
template <> struct FVec<4> { typedef f32x4 type; };
template <int NI> __device__ inline float fv_get(const typename FVec<NI>::type& v, int i) { return v[i]; }
template <> __device__ inline float fv_get<1>(const float& v, int) { return v; }
template <int NI> __device__ inline void fv_set(typename FVec<NI>::type& v, int i, float x) { v[i] = x; }
template <> __device__ inline void fv_set<1>(float& v, int, float x) { v = x; }

__device__ inline int crow(int r, int g) { return (r >> 2) * 8 + 4 * g + (r & 3); }

// ROWS rows of a [T, D] fp32 matrix, from row r0 on, into an LDS tile of pitch D + 4 (16-byte row
// reads of 32 different rows then fall on 64 different banks). Rows past the end repeat the last
// row: every use of them is masked.
template <int D, int ROWS>
__device__ inline void stage_tile(float* dst, const float* src, int64_t st, int r0, int T) {
    constexpr int NCH = D / 4, P = D + 4;
#pragma unroll
    for (int i = 0; i < ROWS * NCH / 256; ++i) {
        const int c = threadIdx.x + 256 * i;
        const int row = c / NCH, ch = c % NCH;
        const int t = min(r0 + row, T - 1);
        *reinterpret_cast<f32x4*>(dst + row * P + ch * 4) = *reinterpret_cast<const f32x4*>(src + t * st + ch * 4);
    }
}

// ---------------------------------------------------------------- forward
// One workgroup = 4 wavefronts = 128 queries of one (batch, head); each wavefront owns 32 queries and
// walks the visible 64-key tiles. S^T = K Q^T with Q in registers, online softmax in base 2 on the
// C registers, O^T += V^T P^T with P^T taken from those registers as they are.
template <int D>
__global__ __launch_bounds__(256, 2) void f32_fwd(AttnArgs a) {
    constexpr int NI = D / 32, NJ = D / 8, P = D + 4, BM = 128;
    typedef typename FVec<NI>::type FV;
    __shared__ __attribute__((aligned(16))) float Ks[BN * P];
    __shared__ __attribute__((aligned(16))) float Vs[BN * P];

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, c32 = lane & 31;
    const int nqb = (a.T + BM - 1) / BM, rep = a.Hq / a.Hkv;
    // Full-causal work per query block grows with its index: a workgroup takes blocks i and
    // nqb-1-i back to back where the halved grid still fills the chip (pair_causal_blocks), else the
    // blocks are dispatched singly, heaviest first.
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    int blk, rr, kvu;
    if (!xcd_map(paired ? (nqb + 1) / 2 : nqb, rep, a.Hkv * a.B, blk, rr, kvu)) return;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv, h = hk * rep + rr;
    const int npass = (paired && blk != nqb - 1 - blk) ? 2 : 1;
  for (int pass = 0; pass < npass; ++pass) {
    const int q0 = (pass == 0 ? nqb - 1 - blk : blk) * BM;
    const int qlo = q0 + w * 32, qhi = qlo + 31, qi = qlo + c32;
    const float* kbase = static_cast<const float*>(a.k) + b * a.k_sb + hk * a.k_sh;
    const float* vbase = static_cast<const float*>(a.v) + b * a.v_sb + hk * a.v_sh;
    const float cexp = a.scale * LOG2E;

    // Q as the B operand of S^T: lane = query, chunk j = d 8j + 4g .. +3
    f32x4 qreg[NJ];
    {
        const float* qrow = static_cast<const float*>(a.q) + b * a.q_sb + h * a.q_sh + min(qi, a.T - 1) * a.q_st;
#pragma unroll
        for (int j = 0; j < NJ; ++j) qreg[j] = *reinterpret_cast<const f32x4*>(qrow + 8 * j + 4 * g);
    }
    f32x16 acc[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    float m = -1e30f, l = 0.0f;  // the reference's running-max seed, src/ops.cpp:881

    // Key tiles this query block can see: the sink tiles [0, ns) and the band / causal tiles [lo, hi].
    const int qmax = min(q0 + BM, a.T) - 1;
    const int hi = (a.causal ? qmax : a.T - 1) / BN;
    const int lo = a.window > 0 ? max(0, q0 + 1 - a.window) / BN : 0;
    const int ns = a.window > 0 ? min((a.sinks + BN - 1) / BN, lo) : 0;
    const QueryVis vis(qi, a.T, a.causal, a.window, a.sinks);

    for (int t = ns > 0 ? 0 : lo; t <= hi; t = (t + 1 == ns) ? lo : t + 1) {
        const int n0 = t * BN;
        __syncthreads();  // the previous tile has been read
        stage_tile<D, BN>(Ks, kbase, a.k_st, n0, a.T);
        stage_tile<D, BN>(Vs, vbase, a.v_st, n0, a.T);
        __syncthreads();
        // wavefront-uniform: nothing of this 32 x 64 block is visible
        if (qlo >= a.T) continue;
        if (a.causal && n0 > qhi) continue;
        if (a.window > 0 && n0 + BN - 1 + a.window <= qlo && n0 >= a.sinks) continue;

        f32x16 s[2];
#pragma unroll
        for (int r = 0; r < 16; ++r) s[0][r] = s[1][r] = 0.0f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const f32x4 k0 = *reinterpret_cast<const f32x4*>(Ks + c32 * P + 8 * j + 4 * g);
            const f32x4 k1 = *reinterpret_cast<const f32x4*>(Ks + (32 + c32) * P + 8 * j + 4 * g);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s[0] = mfma2(k0[i], qreg[j][i], s[0]);
                s[1] = mfma2(k1[i], qreg[j][i], s[1]);
            }
        }
        const bool full = (n0 + BN - 1 < a.T) && (!a.causal || n0 + BN - 1 <= qlo) &&
                          (a.window == 0 || n0 + a.window > qhi || n0 + BN - 1 < a.sinks);
        if (!full) {
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[nb][r] = vis(n0 + nb * 32 + crow(r, g)) ? s[nb][r] : -INFINITY;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[nb][r]);
        mx = xhalf_max(mx);
        const float mn = fmaxf(m, mx);
        if (__any(mn > m)) {  // wavefront-uniform
            const float alpha = __builtin_amdgcn_exp2f((m - mn) * cexp);
            l *= alpha;
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][r] *= alpha;
            m = mn;
        }
        const float mc = m * cexp;
        float psum = 0.0f;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s[nb][r], cexp, -mc));
                s[nb][r] = p;
                psum += p;
            }
        l += psum;  // per-lane partial; the two halves meet in the epilogue
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const FV vf = *reinterpret_cast<const FV*>(Vs + (nb * 32 + crow(r, g)) * P + NI * c32);
#pragma unroll
                for (int i = 0; i < NI; ++i) acc[i] = mfma2(fv_get<NI>(vf, i), s[nb][r], acc[i]);
            }
    }

    const float lt = xhalf_sum(l);
    if (qi < a.T) {
        const float inv = 1.0f / lt;
        float* orow = static_cast<float*>(a.o) + b * a.o_sb + h * a.o_sh + qi * a.o_st;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            FV out;
#pragma unroll
            for (int i = 0; i < NI; ++i) fv_set<NI>(out, i, acc[i][r] * inv);
            *reinterpret_cast<FV*>(orow + NI * crow(r, g)) = out;
        }
        if (g == 0) a.lse[(static_cast<int64_t>(b) * a.Hq + h) * a.T + qi] = m * a.scale + logf(lt);
    }
  }
}

// ---------------------------------------------------------------- dQ
// Same tiling as the forward. Per 32-key block: S^T = K Q^T and dP^T = V dO^T (two independent
// accumulator chains), P = exp(S*scale - LSE), dS = P .* (dP - delta), dQ^T += K^T dS^T with dS^T
// taken from the C registers. With FUSE_DELTA the prologue forms delta = rowsum(O .* dO) for the
// workgroup's own rows (src/ops.cpp:920-921) and publishes it for the dK/dV kernel.
template <int D, bool FUSE_DELTA>
__global__ __launch_bounds__(256, 1) void f32_dq(AttnArgs a) {
    constexpr int NI = D / 32, NJ = D / 8, P = D + 4, BM = 128;
    typedef typename FVec<NI>::type FV;
    constexpr int CPT = BN * (D / 4) / 256;  // 16-byte chunks per thread, tensor and tile
    // two K/V tile buffers: tile t+1 is fetched into registers before the matrix work on tile t and
    // stored behind it, one barrier per tile
    __shared__ __attribute__((aligned(16))) float Kbuf[2][BN * P];
    __shared__ __attribute__((aligned(16))) float Vbuf[2][BN * P];

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, c32 = lane & 31;
    const int nqb = (a.T + BM - 1) / BM, rep = a.Hq / a.Hkv;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);  // as in the forward
    int blk, rr, kvu;
    if (!xcd_map(paired ? (nqb + 1) / 2 : nqb, rep, a.Hkv * a.B, blk, rr, kvu)) return;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv, h = hk * rep + rr;
    const int npass = (paired && blk != nqb - 1 - blk) ? 2 : 1;
  for (int pass = 0; pass < npass; ++pass) {
    const int q0 = (pass == 0 ? nqb - 1 - blk : blk) * BM;
    const int qlo = q0 + w * 32, qhi = qlo + 31, qi = qlo + c32;
    const int qc = min(qi, a.T - 1);
    const float* kbase = static_cast<const float*>(a.k) + b * a.k_sb + hk * a.k_sh;
    const float* vbase = static_cast<const float*>(a.v) + b * a.v_sb + hk * a.v_sh;
    const float cexp = a.scale * LOG2E;
    const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T + qc;

    f32x4 qreg[NJ], greg[NJ];
    float delta;
    {
        const float* qrow = static_cast<const float*>(a.q) + b * a.q_sb + h * a.q_sh + qc * a.q_st;
        const float* grow = static_cast<const float*>(a.d_o) + b * a.do_sb + h * a.do_sh + qc * a.do_st;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            qreg[j] = *reinterpret_cast<const f32x4*>(qrow + 8 * j + 4 * g);
            greg[j] = *reinterpret_cast<const f32x4*>(grow + 8 * j + 4 * g);
        }
        if (FUSE_DELTA) {
            const float* orow = static_cast<const float*>(a.o) + b * a.o_sb + h * a.o_sh + qc * a.o_st;
            float d = 0.0f;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const f32x4 o4 = *reinterpret_cast<const f32x4*>(orow + 8 * j + 4 * g);
#pragma unroll
                for (int i = 0; i < 4; ++i) d = fmaf(o4[i], greg[j][i], d);
            }
            delta = xhalf_sum(d);
            if (g == 0 && qi < a.T) a.delta[lrow] = delta;
        } else {
            delta = a.delta[lrow];
        }
    }
    const float nlse = -a.lse[lrow] * LOG2E;
    f32x16 acc[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;

    const int qmax = min(q0 + BM, a.T) - 1;
    const int hi = (a.causal ? qmax : a.T - 1) / BN;
    const int lo = a.window > 0 ? max(0, q0 + 1 - a.window) / BN : 0;
    const int ns = a.window > 0 ? min((a.sinks + BN - 1) / BN, lo) : 0;
    const QueryVis vis(qi, a.T, a.causal, a.window, a.sinks);

    f32x4 kr[CPT], vr[CPT];
    auto fetch = [&](int n0) {  // rows past the end repeat the last row: every use of them is masked
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 256 * i;
            const int tt = min(n0 + c / (D / 4), a.T - 1), ch = c % (D / 4);
            kr[i] = *reinterpret_cast<const f32x4*>(kbase + tt * a.k_st + ch * 4);
            vr[i] = *reinterpret_cast<const f32x4*>(vbase + tt * a.v_st + ch * 4);
        }
    };
    auto commit = [&](int slot) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 256 * i;
            const int row = c / (D / 4), ch = c % (D / 4);
            *reinterpret_cast<f32x4*>(Kbuf[slot] + row * P + ch * 4) = kr[i];
            *reinterpret_cast<f32x4*>(Vbuf[slot] + row * P + ch * 4) = vr[i];
        }
    };
    int t = ns > 0 ? 0 : lo, cur = 0;
    fetch(t * BN);
    commit(0);
    __syncthreads();
    for (; t <= hi; cur ^= 1) {
        const int n0 = t * BN;
        const int tn = (t + 1 == ns) ? lo : t + 1;
        t = tn;
        if (tn <= hi) fetch(tn * BN);  // in flight during the matrix work
        const float* Ks = Kbuf[cur];
        const float* Vs = Vbuf[cur];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            if (qlo >= a.T) continue;
            const int nn = n0 + nb * 32;
            // wavefront-uniform: nothing of this 32 x 32 block is visible
            if (nn >= a.T) continue;
            if (a.causal && nn > qhi) continue;
            if (a.window > 0 && nn + 31 + a.window <= qlo && nn >= a.sinks) continue;
            f32x16 s, dp;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.0f;
            // One wavefront per SIMD: nothing else covers the LDS latency, so every fragment is read one
            // group of MFMAs ahead of its use and the order is pinned (reads of the next group, then
            // the MFMAs of this one).
            {
                f32x4 kf = *reinterpret_cast<const f32x4*>(Ks + (nb * 32 + c32) * P + 4 * g);
                f32x4 vf = *reinterpret_cast<const f32x4*>(Vs + (nb * 32 + c32) * P + 4 * g);
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    f32x4 nk = kf, nv = vf;
                    if (j + 1 < NJ) {
                        nk = *reinterpret_cast<const f32x4*>(Ks + (nb * 32 + c32) * P + 8 * (j + 1) + 4 * g);
                        nv = *reinterpret_cast<const f32x4*>(Vs + (nb * 32 + c32) * P + 8 * (j + 1) + 4 * g);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s = mfma2(kf[i], qreg[j][i], s);
                        dp = mfma2(vf[i], greg[j][i], dp);
                    }
                    kf = nk;
                    vf = nv;
                }
#pragma unroll
                for (int j = 0; j + 1 < NJ; ++j) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
                }
            }
            const bool full = (nn + 31 < a.T) && (!a.causal || nn + 31 <= qlo) &&
                              (a.window == 0 || nn + a.window > qhi || nn + 31 < a.sinks);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s[r], cexp, nlse));
                s[r] = p * (dp[r] - delta);
            }
            if (!full) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = vis(nn + crow(r, g)) ? s[r] : 0.0f;
            }
            {
                FV kc = *reinterpret_cast<const FV*>(Ks + (nb * 32 + crow(0, g)) * P + NI * c32);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    FV nc = kc;
                    if (r + 1 < 16) nc = *reinterpret_cast<const FV*>(Ks + (nb * 32 + crow(r + 1, g)) * P + NI * c32);
#pragma unroll
                    for (int i = 0; i < NI; ++i) acc[i] = mfma2(fv_get<NI>(kc, i), s[r], acc[i]);
                    kc = nc;
                }
#pragma unroll
                for (int r = 0; r + 1 < 16; ++r) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, NI, 0);
                }
            }
        }
        // the other buffer was last read one tile ago, before the previous barrier
        if (tn <= hi) commit(cur ^ 1);
        __syncthreads();
    }

    if (qi < a.T) {
        float* drow = static_cast<float*>(a.dq) + b * a.dq_sb + h * a.dq_sh + qi * a.dq_st;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            FV out;
#pragma unroll
            for (int i = 0; i < NI; ++i) fv_set<NI>(out, i, acc[i][r] * a.scale);
            *reinterpret_cast<FV*>(drow + NI * crow(r, g)) = out;
        }
    }
  }
}

// ---------------------------------------------------------------- dK, dV
// One workgroup = 8 wavefronts = 128 keys of one (batch, KV head), walking the query tiles that can see
// the block, 32 queries per step, for every query head of the group. The work of a step is split
// between two sets of wavefronts, as in the bf16 kernel; wavefront kbw of each role owns keys
// 32 kbw .. +31 of the block:
//   role 0 (wavefronts 0-3): S = Q K^T -> P = exp(S*scale - LSE) -> dV^T += dO^T P     (K rows resident)
//   role 1 (wavefronts 4-7): dP = dO V^T -> dS = P .* (dP - delta) -> dK^T += Q^T dS   (V rows resident)
// Each role holds one resident operand and one accumulator set, which fits 256 registers: two
// wavefronts per SIMD, all MFMAs in the plain-register form. P goes from role 0 to role 1 through
// LDS as it lies in the C registers (both roles have lane = key, element r = query m(r, g)), and
// role 1 runs one step behind role 0, so one barrier per step orders the hand-over and the
// three-slot Q / dO ring (role 0 reads step s, role 1 step s-1, step s+1 is being stored).
template <int D>
__global__ __launch_bounds__(512, 1) void f32_dkdv(AttnArgs a) {
    constexpr int NI = D / 32, NJ = D / 8, P = D + 4, BNK = 128, NCH = D / 4;
    constexpr int CPT = (BQ * NCH + 511) / 512;  // 16-byte chunks per thread, tensor and step
    typedef typename FVec<NI>::type FV;
    __shared__ __attribute__((aligned(16))) float Qs[3][BQ * P];
    __shared__ __attribute__((aligned(16))) float Gs[3][BQ * P];
    __shared__ __attribute__((aligned(16))) float Pbuf[2][4][4 * 64 * 4];  // [step parity][kbw][r/4][lane][4]
    __shared__ __attribute__((aligned(16))) float nlse_s[3][BQ];
    __shared__ __attribute__((aligned(16))) float dl_s[3][BQ];

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int role = w >> 2, kbw = w & 3;
    const int g = lane >> 5, c32 = lane & 31;
    const int nkb = (a.T + BNK - 1) / BNK, rep = a.Hq / a.Hkv;
    const SinkTail tl = a.tail ? sink_tail(a.T, a.window, a.sinks) : SinkTail{0, 0};
    const bool paired = a.causal && a.window == 0;
    int blk0, rr, kvu;
    if (!xcd_map(paired ? (nkb + 1) / 2 : nkb + tl.nch, 1, a.Hkv * a.B, blk0, rr, kvu)) return;
    const int chunk = blk0 >= nkb ? blk0 - nkb : -1;
    if (chunk >= 0) blk0 = 0;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv;
    const float cexp = a.scale * LOG2E;
    const int npass = (paired && blk0 != nkb - 1 - blk0) ? 2 : 1;

  for (int pass = 0; pass < npass; ++pass) {
    const int kblk = pass == 0 ? blk0 : nkb - 1 - blk0;  // heavy block first
    const int k0 = kblk * BNK, kw0 = k0 + kbw * 32, kj = kw0 + c32;

    // the resident operand: K rows for role 0, V rows for role 1 (lane = key, chunk j = d 8j + 4g .. +3)
    f32x4 kv[NJ];
    {
        const float* src = role == 0 ? static_cast<const float*>(a.k) + b * a.k_sb + hk * a.k_sh
                                     : static_cast<const float*>(a.v) + b * a.v_sb + hk * a.v_sh;
        const float* row = src + min(kj, a.T - 1) * (role == 0 ? a.k_st : a.v_st);
#pragma unroll
        for (int j = 0; j < NJ; ++j) kv[j] = *reinterpret_cast<const f32x4*>(row + 8 * j + 4 * g);
    }
    f32x16 acc[NI];  // dV^T (role 0) or dK^T (role 1)
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;

    const int khi = min(k0 + BNK, a.T) - 1;
    int qt_lo = a.causal ? k0 / BQ : 0;
    int qt_hi = (a.window > 0 && (k0 >= a.sinks || tl.nch > 0)) ? min(a.T - 1, khi + a.window - 1) / BQ : (a.T - 1) / BQ;
    if (chunk >= 0) {
        qt_lo = (tl.q0 + chunk * TAIL_CHUNK) / BQ;
        qt_hi = min(a.T - 1, tl.q0 + (chunk + 1) * TAIL_CHUNK - 1) / BQ;
    } else if (tl.nch > 0 && kblk == 0) {
        qt_hi = tl.q0 / BQ - 1;  // the band part ends where the first chunk starts
    }
    const int nqt = qt_hi - qt_lo + 1;
    const int steps = nqt * rep;
    const KeyVis vis(kj, a.T, a.causal, a.window, a.sinks);

    f32x4 qr[CPT], gr[CPT];
    float lse_r = 0.0f, dl_r = 0.0f;
    auto fetch = [&](int step) {
        const int h = hk * rep + step / nqt, q0 = (qt_lo + step % nqt) * BQ;
        const float* qb = static_cast<const float*>(a.q) + b * a.q_sb + h * a.q_sh;
        const float* gb = static_cast<const float*>(a.d_o) + b * a.do_sb + h * a.do_sh;
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 512 * i;
            if (c < BQ * NCH) {
                const int t = min(q0 + c / NCH, a.T - 1), ch = c % NCH;
                qr[i] = *reinterpret_cast<const f32x4*>(qb + t * a.q_st + ch * 4);
                gr[i] = *reinterpret_cast<const f32x4*>(gb + t * a.do_st + ch * 4);
            }
        }
        if (threadIdx.x < BQ) {
            const int t = min(q0 + static_cast<int>(threadIdx.x), a.T - 1);
            const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T + t;
            lse_r = a.lse[lrow];  // scaled when it is stored: arithmetic on it here would wait for every load just issued
            dl_r = a.delta[lrow];
        }
    };
    auto commit = [&](int slot) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 512 * i;
            if (c < BQ * NCH) {
                const int row = c / NCH, ch = c % NCH;
                *reinterpret_cast<f32x4*>(Qs[slot] + row * P + ch * 4) = qr[i];
                *reinterpret_cast<f32x4*>(Gs[slot] + row * P + ch * 4) = gr[i];
            }
        }
        if (threadIdx.x < BQ) {
            nlse_s[slot][threadIdx.x] = -lse_r * LOG2E;
            dl_s[slot][threadIdx.x] = dl_r;
        }
    };
    // wavefront-uniform: is anything of (query tile of step `step`) x (this wavefront's 32 keys) visible?
    auto tile_live = [&](int step, int& qlo) {
        qlo = (qt_lo + step % nqt) * BQ;
        const int qhi = qlo + 31;
        if (qlo >= a.T || kw0 >= a.T) return false;
        if (a.causal && kw0 > qhi) return false;
        if (a.window > 0 && kw0 + 31 + a.window <= qlo && kw0 >= a.sinks) return false;
        return true;
    };

    if (steps > 0) {
        fetch(0);
        commit(0);
        if (steps > 1) fetch(1);
    }
    __syncthreads();
    // iteration s: role 0 works on step s, role 1 on step s-1
    for (int s = 0; s <= steps; ++s) {
        if (s + 1 < steps) {
            commit((s + 1) % 3);  // slot last read (by role 1) before the previous barrier
            if (s + 2 < steps) fetch(s + 2);
        }
        const int st = role == 0 ? s : s - 1;
        int qlo;
        if (st >= 0 && st < steps && tile_live(st, qlo)) {
            const float* Qt = Qs[st % 3];
            const float* Gt = Gs[st % 3];
            const float* At = role == 0 ? Qt : Gt;  // rows contracted over head_dim: Q for S, dO for dP
            const float* Ct = role == 0 ? Gt : Qt;  // rows that multiply the C tile: dO for dV, Q for dK
            float* pb = &Pbuf[st & 1][kbw][lane * 4];
            f32x16 t;
#pragma unroll
            for (int r = 0; r < 16; ++r) t[r] = 0.0f;
            {
                f32x4 af = *reinterpret_cast<const f32x4*>(At + c32 * P + 4 * g);
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    f32x4 nf = af;
                    if (j + 1 < NJ) nf = *reinterpret_cast<const f32x4*>(At + c32 * P + 8 * (j + 1) + 4 * g);
#pragma unroll
                    for (int i = 0; i < 4; ++i) t = mfma2(af[i], kv[j][i], t);
                    af = nf;
                }
            }
            if (role == 0) {
                const int qhi = qlo + 31;
                const bool full = qhi < a.T && kw0 + 31 < a.T && (!a.causal || kw0 + 31 <= qlo) &&
                                  (a.window == 0 || kw0 + a.window > qhi || kw0 + 31 < a.sinks);
                // lane = key kj; element r = query qlo + crow(r, g): four consecutive queries per r/4
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const f32x4 nl = *reinterpret_cast<const f32x4*>(&nlse_s[st % 3][qd * 8 + 4 * g]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) t[qd * 4 + e] = __builtin_amdgcn_exp2f(fmaf(t[qd * 4 + e], cexp, nl[e]));
                }
                if (!full) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) t[r] = vis(qlo + crow(r, g)) ? t[r] : 0.0f;
                }
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const f32x4 pv = {t[qd * 4], t[qd * 4 + 1], t[qd * 4 + 2], t[qd * 4 + 3]};
                    *reinterpret_cast<f32x4*>(pb + qd * 256) = pv;
                }
            } else {
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const f32x4 pv = *reinterpret_cast<const f32x4*>(pb + qd * 256);
                    const f32x4 dl = *reinterpret_cast<const f32x4*>(&dl_s[st % 3][qd * 8 + 4 * g]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) t[qd * 4 + e] = pv[e] * (t[qd * 4 + e] - dl[e]);
                }
            }
            {
                FV cf = *reinterpret_cast<const FV*>(Ct + crow(0, g) * P + NI * c32);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    FV nf = cf;
                    if (r + 1 < 16) nf = *reinterpret_cast<const FV*>(Ct + crow(r + 1, g) * P + NI * c32);
#pragma unroll
                    for (int i = 0; i < NI; ++i) acc[i] = mfma2(fv_get<NI>(cf, i), t[r], acc[i]);
                    cf = nf;
                }
            }
        }
        __syncthreads();
    }

    bool store = kj < a.T;
    float* orow = role == 0 ? static_cast<float*>(a.dv) + b * a.dv_sb + hk * a.dv_sh + kj * a.dv_st
                            : static_cast<float*>(a.dk) + b * a.dk_sb + hk * a.dk_sh + kj * a.dk_st;
    if (tl.nch > 0 && kblk == 0) {
        // a piece of a split sink tail: the sink keys' rows go to the workspace as partial sums
        // (a chunk writes nothing else; the band part writes its other rows as usual)
        if (kbw == 0 && kj < a.sinks)
            orow = sink_tail_rows(a.tail, kvu, tl.nch, chunk >= 0 ? chunk : tl.nch, role == 0 ? 1 : 0, D) + kj * D;
        else if (chunk >= 0)
            store = false;
    }
    if (store) {
        const float sc = role == 0 ? 1.0f : a.scale;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            FV out;
#pragma unroll
            for (int i = 0; i < NI; ++i) fv_set<NI>(out, i, acc[i][r] * sc);
            *reinterpret_cast<FV*>(orow + NI * crow(r, g)) = out;
        }
    }
    __syncthreads();  // the next pass refills the ring
  }
}

bool aligned_f32(const void* p, int64_t sb, int64_t st, int64_t sh) {
    return (reinterpret_cast<uintptr_t>(p) % 16 == 0) && sb % 4 == 0 && st % 4 == 0 && sh % 4 == 0;
}

template <int D>
int launch_fwd(const AttnArgs& a, hipStream_t st) {
    const int nqb = (a.T + 127) / 128;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    const dim3 grid(xcd_grid(paired ? (nqb + 1) / 2 : nqb, a.Hq / a.Hkv, a.Hkv * a.B));
    hipLaunchKernelGGL(f32_fwd<D>, grid, dim3(256), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

template <int D>
int launch_bwd(const AttnArgs& a_in, int stages, hipStream_t st) {
    AttnArgs a = a_in;
    // a tail step is one wavefront's matrix work, as long as a full step's
    if (!sink_tail_pays(a.tail ? sink_tail(a.T, a.window, a.sinks) : SinkTail{0, 0}, a.T, a.window, a.Hkv * a.B, 32, 1, 1.0f))
        a.tail = nullptr;
    const int nqb = (a.T + 127) / 128;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    const dim3 dq_grid(xcd_grid(paired ? (nqb + 1) / 2 : nqb, a.Hq / a.Hkv, a.Hkv * a.B));
    const bool fused = (stages & PK_BWD_DELTA) && (stages & PK_BWD_DQ);
    if (fused) {  // dQ forms delta itself and runs first; dK/dV reads what it wrote
        hipLaunchKernelGGL((f32_dq<D, true>), dq_grid, dim3(256), 0, st, a);
        PK_HIP(hipGetLastError());
    } else if (stages & PK_BWD_DELTA) {
        if (int rc = launch_generic_bwd(a, false, PK_BWD_DELTA, st)) return rc;
    }
    if (stages & PK_BWD_DKDV) {
        const int nch = a.tail ? sink_tail(a.T, a.window, a.sinks).nch : 0;
        const int nkb = (a.T + 127) / 128;
        const bool paired = a.causal && a.window == 0;
        const dim3 grid(xcd_grid(paired ? (nkb + 1) / 2 : nkb + nch, 1, a.Hkv * a.B));
        hipLaunchKernelGGL(f32_dkdv<D>, grid, dim3(512), 0, st, a);
        PK_HIP(hipGetLastError());
        if (nch > 0)
            if (int rc = launch_sink_tail_reduce(a, st)) return rc;
    }
    if (!fused && (stages & PK_BWD_DQ)) {
        hipLaunchKernelGGL((f32_dq<D, false>), dq_grid, dim3(256), 0, st, a);
        PK_HIP(hipGetLastError());
    }
    return PK_OK;
}

}  // namespace

// fp32 tensors (gradients fp32 as well), head_dim 32 / 64 / 128, a positive scale (the running
// max is tracked on raw scores) and 16-byte-aligned rows.
bool f32_mfma_supported(const AttnArgs& a) {
    if (a.dk_dim != 32 && a.dk_dim != 64 && a.dk_dim != 128) return false;
    if (!(a.scale > 0.0f)) return false;
    if (!aligned_f32(a.q, a.q_sb, a.q_st, a.q_sh) || !aligned_f32(a.k, a.k_sb, a.k_st, a.k_sh) ||
        !aligned_f32(a.v, a.v_sb, a.v_st, a.v_sh) || !aligned_f32(a.o, a.o_sb, a.o_st, a.o_sh))
        return false;
    if (a.d_o) {
        if (!a.grad_f32) return false;
        if (!aligned_f32(a.d_o, a.do_sb, a.do_st, a.do_sh) || !aligned_f32(a.dq, a.dq_sb, a.dq_st, a.dq_sh) ||
            !aligned_f32(a.dk, a.dk_sb, a.dk_st, a.dk_sh) || !aligned_f32(a.dv, a.dv_sb, a.dv_st, a.dv_sh))
            return false;
    }
    return true;
}

int launch_f32_mfma_fwd(const AttnArgs& a, hipStream_t st) {
    switch (a.dk_dim) {
        case 32: return launch_fwd<32>(a, st);
        case 64: return launch_fwd<64>(a, st);
        default: return launch_fwd<128>(a, st);
    }
}

int launch_f32_mfma_bwd(const AttnArgs& a, int stages, hipStream_t st) {
    switch (a.dk_dim) {
        case 32: return launch_bwd<32>(a, stages, st);
        case 64: return launch_bwd<64>(a, stages, st);
        default: return launch_bwd<128>(a, stages, st);
    }
}

}  // namespace pk
