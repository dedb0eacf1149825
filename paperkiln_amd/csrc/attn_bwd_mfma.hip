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
// No atomics, deterministic. The full backward is two launches, mfma_dq (which
// also forms delta) then mfma_dkdv2; asked for by parts it is three:
//   mfma_delta    one pass over O and dO (only when delta is wanted without dQ).
//   mfma_dkdv2    (attn_bwd_dkdv2.hip) a workgroup owns 128 keys of one KV
//                 head and loops over the query heads of its GQA group and
//                 over the query tiles that can see it.
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
template <int D, int ROWS, int NW = 4>
struct Tile {
    static constexpr int S = D + 8;             // row pitch (elements)
    static constexpr int NCH = D / 8;           // 16-byte chunks per row
    static constexpr int CPT = ROWS * NCH / (64 * NW);
    // this thread's byte offsets inside a tile whose rows are st_t elements apart
    __device__ static void offsets(int64_t st_t, int* boff) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 64 * NW * i;
            boff[i] = static_cast<int>((c / NCH) * st_t + (c % NCH) * 8) * 2;
        }
    }
    // rows r0 .. r0+ROWS-1 of the matrix at base + off; rows past T read as zero
    __device__ static void load(const void* base, int64_t off, int64_t st_t, int r0, int T, const int* boff, u32x4* r) {
        const __amdgpu_buffer_rsrc_t rs = tile_rsrc(base, off, st_t, r0, T, D);
#pragma unroll
        for (int i = 0; i < CPT; ++i) r[i] = tile_load16(rs, boff[i]);
    }
    __device__ static void store(uint16_t* lds, const u32x4* r) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = threadIdx.x + 64 * NW * i;
            const int row = c / NCH, ch = c % NCH;
            *reinterpret_cast<u32x4*>(lds + lds_row<D>(row) * S + ch * 8) = r[i];
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

// ---- dQ -------------------------------------------------------------------
// FUSE_DELTA: the workgroup also forms delta for its own 128 rows (it holds their dO
// already; O costs one more row read), uses it and writes it for the dK/dV kernel,
// which then has to run after this one. Saves the separate pass over O and dO.
template <int D, bool GF32, bool FUSE_DELTA, int NW>
__global__ __launch_bounds__(64 * NW, 2) void mfma_dq(AttnArgs a) {
    constexpr int BM = 32 * NW, BN = 64;
    constexpr int KK = D / 16, DB = D / 32;
    using KT = Tile<D, BN, NW>;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[BN * KT::S];
    __shared__ __attribute__((aligned(16))) uint16_t Vs[BN * KT::S];

    const int lane = threadIdx.x & 63;
    // the wavefront index as a scalar: every test on it becomes a scalar branch
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, c32 = lane & 31;
    const int nqb = (a.T + BM - 1) / BM, rep = a.Hq / a.Hkv;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    int blk, rr, kvu;
    // unpaired causal blocks without a band: heaviest blocks of every unit first
    if (!paired && a.causal && a.window == 0 ? !xcd_map_block_major(nqb, rep, a.Hkv * a.B, blk, rr, kvu)
                                             : !xcd_map(paired ? (nqb + 1) / 2 : nqb, rep, a.Hkv * a.B, blk, rr, kvu))
        return;
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
    const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T + qi;
    if (qi < a.T) nlse = -a.lse[lrow] * LOG2E;
    if (FUSE_DELTA) {
        bf16x8 oreg[KK];  // zero rows past the end, as dO
        load_row_operand<D>(a.o, b * a.o_sb + h * a.o_sh, a.o_st, qi, a.T, g, oreg);
        float part = 0.0f;  // this lane's half of the row: d = 16kk + 8g .. +7
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const u32x4 ov = *reinterpret_cast<const u32x4*>(&oreg[kk]);
            const u32x4 gv = *reinterpret_cast<const u32x4*>(&greg[kk]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                part = fmaf(__uint_as_float(ov[i] << 16), __uint_as_float(gv[i] << 16), part);
                part = fmaf(__uint_as_float(ov[i] & 0xFFFF0000u), __uint_as_float(gv[i] & 0xFFFF0000u), part);
            }
        }
        dl = xhalf_sum(part);
        if (qi < a.T && g == 0) a.delta[lrow] = dl;
    } else if (qi < a.T) {
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
    int koff[KT::CPT], voff[KT::CPT];
    KT::offsets(a.k_st, koff);
    KT::offsets(a.v_st, voff);
    KT::load(a.k, kb, a.k_st, t * BN, a.T, koff, kr);
    KT::load(a.v, vb, a.v_st, t * BN, a.T, voff, vr);
    KT::store(Ks, kr);
    KT::store(Vs, vr);
    __syncthreads();

    while (t <= hi) {
        const int n0 = t * BN;
        const int tn = (t + 1 == ns) ? lo : t + 1;
        if (tn <= hi) {
            KT::load(a.k, kb, a.k_st, tn * BN, a.T, koff, kr);
            KT::load(a.v, vb, a.v_st, tn * BN, a.T, voff, vr);
        }
        const bool skip = qlo >= a.T || (a.causal && n0 > qhi) ||
                          (a.window > 0 && n0 + BN - 1 + a.window <= qlo && n0 >= a.sinks);
        if (!skip) {
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                // a 32-key half no query of this wavefront can see (past the diagonal, or before the band and without
                // a sink key) costs nothing; which of the mask's tests the half can fail decides its masking loop
                const int k0 = n0 + nb * 32, k1 = k0 + 31;
                if ((a.causal && k0 > qhi) || (a.window > 0 && k1 + a.window <= qlo && k0 >= a.sinks)) continue;
                const MaskKind kind = mask_kind(k0, k1, qlo, qhi, a.T, a.causal, a.window, a.sinks);
                f32x16 s, dp;
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.0f;
                // matrix phases issue ahead of co-resident waves' exponent phases
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) {
                    const bf16x8 kf = lds_read8(Ks + (nb * 32 + lds_row<D>(c32)) * KT::S + kk * 16 + g * 8);
                    s = mfma32(kf, qreg[kk], s);
                    const bf16x8 vf = lds_read8(Vs + (nb * 32 + lds_row<D>(c32)) * KT::S + kk * 16 + g * 8);
                    dp = mfma32(vf, greg[kk], dp);
                }
                __builtin_amdgcn_s_setprio(0);
                // lane = query qi; element r = key n0 + nb*32 + (r/4)*8 + 4g + r%4
#pragma unroll
                for (int r = 0; r < 16; ++r) dp[r] = __builtin_amdgcn_exp2f(fmaf(s[r], cexp, nlse)) * (dp[r] - dl);
                // off the common path: interior blocks carry no mask arithmetic at all
                if (kind != MaskKind::NONE) mask_block(dp, kind, qvis, k0 + g * 4, 0.0f);
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
        for (int db = 0; db < DB; ++db) {
            if (!GF32) {
                store_acc_bf16<D>(static_cast<uint16_t*>(a.dq) + ob, db, g, dq_acc[db], a.scale);
                continue;
            }
#pragma unroll
            for (int qd = 0; qd < 4; ++qd)
                store4<GF32>(a.dq, ob + TrMap<D>::col0(db, qd, g), dq_acc[db][qd * 4] * a.scale,
                             dq_acc[db][qd * 4 + 1] * a.scale, dq_acc[db][qd * 4 + 2] * a.scale,
                             dq_acc[db][qd * 4 + 3] * a.scale);
        }
    }
    __syncthreads();  // the next pass refills the tile buffers
  }
}

template <int D, bool GF32>
int launch(const AttnArgs& a, int stages, hipStream_t st) {
    const int64_t rows = static_cast<int64_t>(a.B) * a.Hq * a.T;
    constexpr int RPB = 256 / (D / 8);
    // dQ with 8 wavefronts (256 queries) per K/V tile where the paired causal grid still gives every CU two
    // workgroups in turn, as in the forward kernel; 4 wavefronts otherwise.
    const int nb256 = (a.T + 255) / 256;
    const bool wide = D == 128 && a.causal && a.window == 0 && static_cast<int64_t>((nb256 + 1) / 2) * a.Hq * a.B >= 512;
    const int nbq = wide ? nb256 : (a.T + 127) / 128;
    const bool paired = pair_causal_blocks(nbq, a.Hq * a.B, a.causal, a.window);
    const dim3 dq_grid(xcd_grid(paired ? (nbq + 1) / 2 : nbq, a.Hq / a.Hkv, a.Hkv * a.B));
    // delta and dQ asked for together: dQ forms delta itself and runs first, dK/dV reads what it wrote
    const bool fused = (stages & PK_BWD_DELTA) && (stages & PK_BWD_DQ);
    const bool dq3 = mfma_dq3_takes(a);  // 64 queries per wavefront, one wavefront per SIMD
    if (fused) {
        if (dq3) {
            if (int rc = launch_mfma_dq3(a, true, st)) return rc;
        } else if (wide)
            hipLaunchKernelGGL((mfma_dq<D, GF32, true, 8>), dq_grid, dim3(512), 0, st, a);
        else
            hipLaunchKernelGGL((mfma_dq<D, GF32, true, 4>), dq_grid, dim3(256), 0, st, a);
        PK_HIP(hipGetLastError());
    } else if (stages & PK_BWD_DELTA) {
        hipLaunchKernelGGL((mfma_delta<D>), dim3((rows + RPB - 1) / RPB), dim3(256), 0, st, a);
        PK_HIP(hipGetLastError());
    }
    if (stages & PK_BWD_DKDV) {
        // without a band: 64 keys per wavefront, one wavefront per SIMD; with one: 32 keys, two per SIMD
        if (int rc = mfma_dkdv3_takes(a) ? launch_mfma_dkdv3(a, st) : launch_mfma_dkdv2(a, st)) return rc;
    }
    if (!fused && (stages & PK_BWD_DQ)) {
        if (dq3) {
            if (int rc = launch_mfma_dq3(a, false, st)) return rc;
        } else if (wide)
            hipLaunchKernelGGL((mfma_dq<D, GF32, false, 8>), dq_grid, dim3(512), 0, st, a);
        else
            hipLaunchKernelGGL((mfma_dq<D, GF32, false, 4>), dq_grid, dim3(256), 0, st, a);
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
