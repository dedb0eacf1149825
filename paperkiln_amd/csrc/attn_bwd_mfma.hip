// bf16 flash-attention recompute backward for gfx950. Replaces the backward
// closure of ops::fused_attention / ops::swa_attention (paperkiln
// src/ops.cpp:902-933, 997-1026), which reads the saved [T,T] matrix A: here P
// is rebuilt from Q, K and the forward's logsumexp, so the tape node keeps
// only O and LSE.
//
//   delta_i = sum_d O_id dO_id            (= the reference's `dot`, :920-921)
//   P_ij    = exp(scale*s_ij - LSE_i)     (0 where masked)
//   dV = P^T dO          dP = dO V^T      dS = P .* (dP - delta)
//   dQ = scale * dS K    dK = scale * dS^T Q
//
// Three launches, no atomics, deterministic:
//   mfma_delta    one pass over O and dO.
//   mfma_dkdv     a workgroup owns 128 keys of one KV head (32 per wavefront,
//                 K and V held in registers), loops over the query heads of
//                 its GQA group and over the query tiles that can see it.
//                 S = Q K^T and dP = dO V^T come out with lane = key, so
//                 P and dS feed dV^T += dO^T P and dK^T += Q^T dS straight
//                 from registers; Q^T / dO^T are transposing LDS reads of the
//                 same row-major tiles.
//   mfma_dq       a workgroup owns 128 queries of one head (32 per
//                 wavefront, Q and dO in registers), loops over the visible
//                 key tiles: S^T = K Q^T, dP^T = V dO^T (lane = query, so LSE
//                 and delta are per-lane scalars), dQ^T += K^T dS^T.
#include <cstdlib>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
#ifndef PK_DKDV_OCC
#define PK_DKDV_OCC 1
#endif

// ---- delta --------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void mfma_delta(AttnArgs a) {
    constexpr int LPR = D / 8;        // lanes per row, 16 bytes each
    constexpr int RPB = 256 / LPR;    // rows per block
    const int sub = threadIdx.x % LPR;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * RPB + threadIdx.x / LPR;
    const int64_t rows = static_cast<int64_t>(a.B) * a.Hq * a.T;
    float s = 0.0f;
    if (row < rows) {
        const int t = row % a.T;
        const int h = (row / a.T) % a.Hq;
        const int b = row / (static_cast<int64_t>(a.T) * a.Hq);
        const u32x4 ov = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.o) + b * a.o_sb +
                                                         h * a.o_sh + t * a.o_st + sub * 8);
        const u32x4 gv = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.d_o) +
                                                         b * a.do_sb + h * a.do_sh + t * a.do_st + sub * 8);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            s = fmaf(__uint_as_float(ov[i] << 16), __uint_as_float(gv[i] << 16), s);
            s = fmaf(__uint_as_float(ov[i] & 0xFFFF0000u), __uint_as_float(gv[i] & 0xFFFF0000u), s);
        }
    }
#pragma unroll
    for (int o = LPR / 2; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
    if (row < rows && sub == 0) a.delta[row] = s;
}

// ---- shared tile movers ---------------------------------------------------
template <int D, int ROWS>
struct Tile {
    static constexpr int S = D + 8;             // row pitch (elements)
    static constexpr int NCH = D / 8;           // 16-byte chunks per row
    static constexpr int CPT = ROWS * NCH / 256;
    __device__ static void load(const void* base, int64_t off, int64_t st_t, int r0, int T, u32x4* r) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 256 * i;
            const int row = c / NCH, ch = c % NCH;
            u32x4 z = {0, 0, 0, 0};
            if (r0 + row < T)
                z = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + off +
                                                    (r0 + row) * st_t + ch * 8);
            r[i] = z;
        }
    }
    __device__ static void store(uint16_t* lds, const u32x4* r) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 256 * i;
            const int row = c / NCH, ch = c % NCH;
            *reinterpret_cast<u32x4*>(lds + row * S + ch * 8) = r[i];
        }
    }
};

// Row `row` of a head as an MFMA operand held in registers:
// element chunk kk covers d = 16kk + 8g .. +7.
template <int D>
__device__ inline void load_row_operand(const void* base, int64_t off, int64_t st_t, int row, int T,
                                        int g, bf16x8* out) {
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
        u32x4 z = {0, 0, 0, 0};
        if (row < T)
            z = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + off + row * st_t +
                                                kk * 16 + g * 8);
        out[kk] = *reinterpret_cast<bf16x8*>(&z);
    }
}

template <bool F32>
__device__ inline void store4(void* base, int64_t idx, float x0, float x1, float x2, float x3) {
    if (F32) {
        f32x4 v = {x0, x1, x2, x3};
        *reinterpret_cast<f32x4*>(static_cast<float*>(base) + idx) = v;
    } else {
        u32x2 v = {pack_bf16(x0, x1), pack_bf16(x2, x3)};
        *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(base) + idx) = v;
    }
}

// ---- dK, dV ---------------------------------------------------------------
template <int D, bool GF32>
__global__ __launch_bounds__(256, PK_DKDV_OCC) void mfma_dkdv(AttnArgs a) {
    constexpr int BMQ = 64;   // queries per step
    constexpr int BNK = 128;  // keys per workgroup
    constexpr int KK = D / 16, DB = D / 32;
    using QT = Tile<D, BMQ>;
    __shared__ __attribute__((aligned(16))) uint16_t Qs[BMQ * QT::S];
    __shared__ __attribute__((aligned(16))) uint16_t dOs[BMQ * QT::S];
    __shared__ __attribute__((aligned(16))) float nlse_s[BMQ];  // -LSE * log2(e)
    __shared__ __attribute__((aligned(16))) float dl_s[BMQ];

    const int lane = threadIdx.x & 63;
    // the wavefront index as a scalar: every test on it becomes a scalar branch
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, c32 = lane & 31;
    const int nkb = (a.T + BNK - 1) / BNK, rep = a.Hq / a.Hkv;
    // Full-causal: key block i is seen by T - 128i queries; blocks i and nkb-1-i
    // are taken back to back so that every workgroup carries the same work.
    const bool paired = a.causal && a.window == 0;
    int blk, rr, kvu;
    if (!xcd_map(paired ? (nkb + 1) / 2 : nkb, 1, a.Hkv * a.B, blk, rr, kvu)) return;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv;
    const int npass = (paired && blk != nkb - 1 - blk) ? 2 : 1;
  for (int pass = 0; pass < npass; ++pass) {
    const int kblk = pass == 0 ? blk : nkb - 1 - blk;  // heavy block first
    const int k0 = kblk * BNK;
    const int kw0 = k0 + w * 32;  // this wavefront's keys
    const float cexp = a.scale * LOG2E;

    bf16x8 kreg[KK], vreg[KK];
    load_row_operand<D>(a.k, b * a.k_sb + hk * a.k_sh, a.k_st, kw0 + c32, a.T, g, kreg);
    load_row_operand<D>(a.v, b * a.v_sb + hk * a.v_sh, a.v_st, kw0 + c32, a.T, g, vreg);

    f32x16 dk_acc[DB], dv_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dk_acc[db][r] = dv_acc[db][r] = 0.0f;

    // Query tiles that can see keys [k0, k0+127] (src/ops.cpp:960-965 inverted).
    const int khi = min(k0 + BNK, a.T) - 1;
    const int qt_lo = a.causal ? k0 / BMQ : 0;
    const int qt_hi = (a.window > 0 && k0 >= a.sinks) ? min(a.T - 1, khi + a.window - 1) / BMQ
                                                       : (a.T - 1) / BMQ;
    const int nqt = qt_hi - qt_lo + 1;
    const int steps = nqt * rep;

    u32x4 qr[QT::CPT], gr[QT::CPT];
    float lse_r = 0.0f, dl_r = 0.0f;
    auto fetch = [&](int step) {
        const int h = hk * rep + step / nqt, q0 = (qt_lo + step % nqt) * BMQ;
        QT::load(a.q, b * a.q_sb + h * a.q_sh, a.q_st, q0, a.T, qr);
        QT::load(a.d_o, b * a.do_sb + h * a.do_sh, a.do_st, q0, a.T, gr);
        if (threadIdx.x < BMQ) {
            const int t = q0 + threadIdx.x;
            const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T + t;
            lse_r = t < a.T ? -a.lse[lrow] * LOG2E : 0.0f;
            dl_r = t < a.T ? a.delta[lrow] : 0.0f;
        }
    };
    auto commit = [&]() {
        QT::store(Qs, qr);
        QT::store(dOs, gr);
        if (threadIdx.x < BMQ) {
            nlse_s[threadIdx.x] = lse_r;
            dl_s[threadIdx.x] = dl_r;
        }
    };
    if (steps > 0) {
        fetch(0);
        commit();
    }
    __syncthreads();

    for (int step = 0; step < steps; ++step) {
        const int q0 = (qt_lo + step % nqt) * BMQ;
        if (step + 1 < steps) fetch(step + 1);

#pragma unroll
        for (int qb = 0; qb < BMQ / 32; ++qb) {
            const int qlo = q0 + qb * 32, qhi = qlo + 31;
            if (qlo >= a.T || kw0 >= a.T) continue;
            if (a.causal && kw0 > qhi) continue;
            if (a.window > 0 && kw0 + 31 + a.window <= qlo && kw0 >= a.sinks) continue;

            f32x16 s, dp;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.0f;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const bf16x8 qf = lds_read8(Qs + (qb * 32 + c32) * QT::S + kk * 16 + g * 8);
                s = mfma32(qf, kreg[kk], s);
                const bf16x8 gf = lds_read8(dOs + (qb * 32 + c32) * QT::S + kk * 16 + g * 8);
                dp = mfma32(gf, vreg[kk], dp);
            }
            const bool full = qhi < a.T && kw0 + 31 < a.T && (!a.causal || kw0 + 31 <= qlo) &&
                              (a.window == 0 || kw0 + a.window > qhi || kw0 + 31 < a.sinks);
            const KeyVis kvis(kw0 + c32, a.T, a.causal, a.window, a.sinks);
            // lane = key kw0+c32; element r = query qlo + (r/4)*8 + 4g + r%4
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const f32x4 nl = *reinterpret_cast<const f32x4*>(nlse_s + qb * 32 + qd * 8 + g * 4);
                const f32x4 dl = *reinterpret_cast<const f32x4*>(dl_s + qb * 32 + qd * 8 + g * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = qd * 4 + e;
                    const float p = __builtin_amdgcn_exp2f(fmaf(s[r], cexp, nl[e]));
                    s[r] = p;
                    dp[r] = p * (dp[r] - dl[e]);
                }
            }
            if (!full) {  // off the common path: interior tiles carry no mask arithmetic at all
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const bool vis = kvis(qlo + (r >> 2) * 8 + g * 4 + (r & 3));
                    s[r] = vis ? s[r] : 0.0f;
                    dp[r] = vis ? dp[r] : 0.0f;
                }
            }
            const bf16x8 p0 = c_to_operand<0>(s), p1 = c_to_operand<1>(s);
            const bf16x8 d0 = c_to_operand<0>(dp), d1 = c_to_operand<1>(dp);
            // dV^T += dO^T P ; dK^T += Q^T dS (A = transposed LDS tiles). Consecutive
            // MFMAs go to different accumulators (a dependent pair costs 52 cycles, not 32).
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                dv_acc[db] = mfma32(lds_read_tr_operand_perm<D>(dOs, QT::S, qb * 32, db, lane), p0, dv_acc[db]);
                dk_acc[db] = mfma32(lds_read_tr_operand_perm<D>(Qs, QT::S, qb * 32, db, lane), d0, dk_acc[db]);
            }
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                dv_acc[db] = mfma32(lds_read_tr_operand_perm<D>(dOs, QT::S, qb * 32 + 16, db, lane), p1, dv_acc[db]);
                dk_acc[db] = mfma32(lds_read_tr_operand_perm<D>(Qs, QT::S, qb * 32 + 16, db, lane), d1, dk_acc[db]);
            }
        }
        __syncthreads();
        if (step + 1 < steps) commit();
        __syncthreads();
    }

    const int kj = kw0 + c32;
    if (kj < a.T) {
        const int64_t kb = b * a.dk_sb + hk * a.dk_sh + kj * a.dk_st;
        const int64_t vb = b * a.dv_sb + hk * a.dv_sh + kj * a.dv_st;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int d0 = TrMap<D>::col0(db, qd, g);
                store4<GF32>(a.dk, kb + d0, dk_acc[db][qd * 4] * a.scale, dk_acc[db][qd * 4 + 1] * a.scale,
                             dk_acc[db][qd * 4 + 2] * a.scale, dk_acc[db][qd * 4 + 3] * a.scale);
                store4<GF32>(a.dv, vb + d0, dv_acc[db][qd * 4], dv_acc[db][qd * 4 + 1],
                             dv_acc[db][qd * 4 + 2], dv_acc[db][qd * 4 + 3]);
            }
    }
    __syncthreads();  // the next pass refills the tile buffers
  }
}

// ---- dQ -------------------------------------------------------------------
template <int D, bool GF32>
__global__ __launch_bounds__(256, 2) void mfma_dq(AttnArgs a) {
    constexpr int BM = 128, BN = 64;
    constexpr int KK = D / 16, DB = D / 32;
    using KT = Tile<D, BN>;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[BN * KT::S];
    __shared__ __attribute__((aligned(16))) uint16_t Vs[BN * KT::S];

    const int lane = threadIdx.x & 63;
    // the wavefront index as a scalar: every test on it becomes a scalar branch
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, c32 = lane & 31;
    const int nqb = (a.T + BM - 1) / BM, rep = a.Hq / a.Hkv;
    const bool paired = a.causal && a.window == 0;  // as in the forward kernel
    int blk, rr, kvu;
    if (!xcd_map(paired ? (nqb + 1) / 2 : nqb, rep, a.Hkv * a.B, blk, rr, kvu)) return;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv, h = hk * rep + rr;
    const int npass = (paired && blk != nqb - 1 - blk) ? 2 : 1;
  for (int pass = 0; pass < npass; ++pass) {
    const int qblk = pass == 0 ? nqb - 1 - blk : blk;
    const int q0 = qblk * BM;
    const int qlo = q0 + w * 32, qhi = qlo + 31, qi = qlo + c32;
    const int64_t kb = b * a.k_sb + hk * a.k_sh, vb = b * a.v_sb + hk * a.v_sh;
    const float cexp = a.scale * LOG2E;

    bf16x8 qreg[KK], greg[KK];
    load_row_operand<D>(a.q, b * a.q_sb + h * a.q_sh, a.q_st, qi, a.T, g, qreg);
    load_row_operand<D>(a.d_o, b * a.do_sb + h * a.do_sh, a.do_st, qi, a.T, g, greg);
    float nlse = 0.0f, dl = 0.0f;
    if (qi < a.T) {
        const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T + qi;
        nlse = -a.lse[lrow] * LOG2E;
        dl = a.delta[lrow];
    }
    const QueryVis qvis(qi, a.T, a.causal, a.window, a.sinks);
    f32x16 dq_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_acc[db][r] = 0.0f;

    const int qmax = min(q0 + BM, a.T) - 1;
    const int hi = (a.causal ? qmax : a.T - 1) / BN;
    const int lo = a.window > 0 ? max(0, q0 + 1 - a.window) / BN : 0;
    const int ns = a.window > 0 ? min((a.sinks + BN - 1) / BN, lo) : 0;
    int t = ns > 0 ? 0 : lo;

    u32x4 kr[KT::CPT], vr[KT::CPT];
    KT::load(a.k, kb, a.k_st, t * BN, a.T, kr);
    KT::load(a.v, vb, a.v_st, t * BN, a.T, vr);
    KT::store(Ks, kr);
    KT::store(Vs, vr);
    __syncthreads();

    while (t <= hi) {
        const int n0 = t * BN;
        const int tn = (t + 1 == ns) ? lo : t + 1;
        if (tn <= hi) {
            KT::load(a.k, kb, a.k_st, tn * BN, a.T, kr);
            KT::load(a.v, vb, a.v_st, tn * BN, a.T, vr);
        }
        const bool skip = qlo >= a.T || (a.causal && n0 > qhi) ||
                          (a.window > 0 && n0 + BN - 1 + a.window <= qlo && n0 >= a.sinks);
        if (!skip) {
            const bool full = (n0 + BN - 1 < a.T) && (!a.causal || n0 + BN - 1 <= qlo) &&
                              (a.window == 0 || n0 + a.window > qhi || n0 + BN - 1 < a.sinks);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                f32x16 s, dp;
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.0f;
                // matrix phases issue ahead of co-resident waves' exponent phases
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) {
                    const bf16x8 kf = lds_read8(Ks + (nb * 32 + c32) * KT::S + kk * 16 + g * 8);
                    s = mfma32(kf, qreg[kk], s);
                    const bf16x8 vf = lds_read8(Vs + (nb * 32 + c32) * KT::S + kk * 16 + g * 8);
                    dp = mfma32(vf, greg[kk], dp);
                }
                __builtin_amdgcn_s_setprio(0);
                // lane = query qi; element r = key n0 + nb*32 + (r/4)*8 + 4g + r%4
#pragma unroll
                for (int r = 0; r < 16; ++r) dp[r] = __builtin_amdgcn_exp2f(fmaf(s[r], cexp, nlse)) * (dp[r] - dl);
                if (!full) {  // off the common path: interior tiles carry no mask arithmetic at all
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        dp[r] = qvis(n0 + nb * 32 + (r >> 2) * 8 + g * 4 + (r & 3)) ? dp[r] : 0.0f;
                }
                const bf16x8 d0 = c_to_operand<0>(dp), d1 = c_to_operand<1>(dp);
                __builtin_amdgcn_s_setprio(1);
                // dQ^T += K^T dS^T, DB independent chains per k-chunk
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    dq_acc[db] = mfma32(lds_read_tr_operand_perm<D>(Ks, KT::S, nb * 32, db, lane), d0, dq_acc[db]);
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    dq_acc[db] = mfma32(lds_read_tr_operand_perm<D>(Ks, KT::S, nb * 32 + 16, db, lane), d1, dq_acc[db]);
                __builtin_amdgcn_s_setprio(0);
            }
        }
        __syncthreads();
        if (tn <= hi) {
            KT::store(Ks, kr);
            KT::store(Vs, vr);
        }
        __syncthreads();
        t = tn;
    }

    if (qi < a.T) {
        const int64_t ob = b * a.dq_sb + h * a.dq_sh + qi * a.dq_st;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd)
                store4<GF32>(a.dq, ob + TrMap<D>::col0(db, qd, g), dq_acc[db][qd * 4] * a.scale,
                             dq_acc[db][qd * 4 + 1] * a.scale, dq_acc[db][qd * 4 + 2] * a.scale,
                             dq_acc[db][qd * 4 + 3] * a.scale);
    }
    __syncthreads();  // the next pass refills the tile buffers
  }
}

template <int D, bool GF32>
int launch(const AttnArgs& a, int stages, hipStream_t st) {
    const int64_t rows = static_cast<int64_t>(a.B) * a.Hq * a.T;
    constexpr int RPB = 256 / (D / 8);
    const int nb128 = (a.T + 127) / 128;
    const bool paired = a.causal && a.window == 0;
    if (stages & PK_BWD_DELTA) {
        hipLaunchKernelGGL((mfma_delta<D>), dim3((rows + RPB - 1) / RPB), dim3(256), 0, st, a);
        PK_HIP(hipGetLastError());
    }
    static const bool old_dkdv = getenv("PK_DKDV_OLD") != nullptr;
    if ((stages & PK_BWD_DKDV) && !old_dkdv) {
        if (int rc = launch_mfma_dkdv2(a, st)) return rc;
    } else if (stages & PK_BWD_DKDV) {
        hipLaunchKernelGGL((mfma_dkdv<D, GF32>), dim3(xcd_grid(paired ? (nb128 + 1) / 2 : nb128, 1, a.Hkv * a.B)), dim3(256),
                           0, st, a);
        PK_HIP(hipGetLastError());
    }
    if (stages & PK_BWD_DQ) {
        hipLaunchKernelGGL((mfma_dq<D, GF32>), dim3(xcd_grid(paired ? (nb128 + 1) / 2 : nb128, a.Hq / a.Hkv, a.Hkv * a.B)),
                           dim3(256), 0, st, a);
        PK_HIP(hipGetLastError());
    }
    return PK_OK;
}

}  // namespace

int launch_mfma_bwd(const AttnArgs& a, int stages, hipStream_t st) {
    if (a.dk_dim == 128) return a.grad_f32 ? launch<128, true>(a, stages, st) : launch<128, false>(a, stages, st);
    return a.grad_f32 ? launch<64, true>(a, stages, st) : launch<64, false>(a, stages, st);
}

}  // namespace pk
