// bf16 flash-attention forward for gfx950: O and per-row logsumexp only.
// Replaces the forward half of the reference's per-head
// ops::fused_attention / ops::swa_attention (paperkiln src/ops.cpp:863-902,
// 948-995), which materialise a [T,T] fp32 weight matrix per head.
//
// One workgroup = NW wavefronts (4 or 8) = one (batch, head, 32*NW*NQ-query
// block). Each wavefront owns NQ blocks of 32 queries and walks the visible key tiles
// (64 keys per step). The work is phrased TRANSPOSED so that every softmax
// row lives in one lane pair:
//   S^T[key, query] = K . Q^T      A = K tile from LDS (ds_read_b128),
//                                  B = Q, held in registers for the whole loop
//   C layout => lane c holds query c: row max / row sum are in-lane loops plus
//   one v_permlane32_swap with lane c^32.
//   O^T[d, query]  += V^T . P^T    B = exp2(S^T) straight from the C registers
//                                  (no LDS round trip), A = V^T fetched from
//                                  the row-major V tile with transposing LDS
//                                  reads (ds_read_b64_tr_b16).
// Softmax runs in base 2 with the scale folded into one FMA per element:
// p = exp2(s*c - m*c), c = scale*log2(e). Fully masked 32x64 blocks are
// skipped per wavefront, fully masked key tiles are never loaded.
#include <cstdlib>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr int BN = 64;  // keys per step

template <int D, int NW>
struct FwdCfg {
    static constexpr int KS = D + 8;    // K tile row pitch: 4 banks past a multiple of 64 -> b128 row reads conflict-free
    static constexpr int VS = D + 32;   // V tile row pitch: 16 banks past -> the 4-row transposing reads conflict-free
    static constexpr int NCH = D / 8;   // 16-byte chunks per row
    static constexpr int CPT = BN * NCH / (64 * NW);  // chunks per thread per tile
};

// koff / voff: this thread's byte offsets inside a tile (fixed for the whole kernel); keys past the end read as zero
template <int D, int NW>
__device__ inline void load_kv_regs(const AttnArgs& a, int64_t kb, int64_t vb, int n0, const int* koff, const int* voff,
                                    u32x4* kr, u32x4* vr) {
    using C = FwdCfg<D, NW>;
    const __amdgpu_buffer_rsrc_t krs = tile_rsrc(a.k, kb, a.k_st, n0, a.T, D);
    const __amdgpu_buffer_rsrc_t vrs = tile_rsrc(a.v, vb, a.v_st, n0, a.T, D);
#pragma unroll
    for (int i = 0; i < C::CPT; ++i) {
        kr[i] = tile_load16(krs, koff[i]);
        vr[i] = tile_load16(vrs, voff[i]);
    }
}

template <int D, int NW>
__device__ inline void store_kv_lds(uint16_t* Ks, uint16_t* Vs, const u32x4* kr, const u32x4* vr) {
    using C = FwdCfg<D, NW>;
#pragma unroll
    for (int i = 0; i < C::CPT; ++i) {
        const int c = threadIdx.x + 64 * NW * i;
        const int row = c / C::NCH, ch = c % C::NCH;
        *reinterpret_cast<u32x4*>(Ks + row * C::KS + ch * 8) = kr[i];
        *reinterpret_cast<u32x4*>(Vs + row * C::VS + ch * 8) = vr[i];
    }
}

// Rescaling the O accumulators costs three VALU ops per element on this
// machine (they live in accumulation registers), so it is done lazily: the
// running reference max only moves when some row's new max exceeds it by more
// than LAZY_T in log2 units. Between moves P = exp2(s*c - m*c) may reach
// 2^LAZY_T, which bf16 P and the fp32 accumulators hold without loss; the
// final O = acc / l and LSE = m*scale + ln(l) are exact for any reference m.
constexpr float LAZY_T = 6.0f;

// A K or V tile's position as a scalar buffer resource that is ADVANCED from tile to tile instead of rebuilt: base
// pointer plus the bytes left up to the end of the last row (the resource's num_records, so rows past the end read
// as zero). For matrices below 2 GiB from the first row of the (batch, head) to the last, which the launcher checks.
struct TileCursor {
    const uint16_t* p;
    int left;        // bytes from p to the end of row T - 1 (below 2^31)
    int step;        // bytes per tile of BN rows
    __device__ TileCursor(const void* base, int64_t elem_off, int64_t st, int r0, int T, int D) {
        const uint32_t st32 = static_cast<uint32_t>(st), first = static_cast<uint32_t>(min(r0, T));
        const uint32_t rows = static_cast<uint32_t>(T) - first;
        p = static_cast<const uint16_t*>(base) + elem_off + static_cast<uint64_t>(first) * st32;
        left = rows ? static_cast<int>(((rows - 1) * st32 + D) * 2u) : 0;
        step = static_cast<int>(static_cast<uint32_t>(BN) * st32 * 2u);
    }
    __device__ __amdgpu_buffer_rsrc_t rsrc() const {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p), 0, left, 0x00020000);
    }
    __device__ void next() {
        p = reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(p) + step);
        left = max(left - step, 0);  // signed on purpose: the unsigned form becomes a saturating subtraction, a vector instruction
    }
};

// WIN = false: no band (plain causal or full attention). Key tiles are then walked in order from 0, so the tile
// positions are cursors that advance, and which tiles a wavefront skips or masks is decided by comparing the tile
// index with two numbers formed once per pass -- a lone scalar instruction costs a wavefront as much issue time as a
// vector one, and the general form of these tests was 70 scalar instructions per tile.
template <int D, int NQ, int OCC, int NW, bool WIN>
__global__ __launch_bounds__(64 * NW, OCC) void mfma_fwd(AttnArgs a) {
    using C = FwdCfg<D, NW>;
    constexpr int BM = 32 * NW * NQ;
    constexpr int KK = D / 16;  // k-chunks of the QK^T contraction
    constexpr int DB = D / 32;  // 32-row blocks of O^T
    // two K/V tile buffers: tile t+1 is stored while tile t is being read, one barrier per tile
    __shared__ __attribute__((aligned(16))) uint16_t Kbuf[2][BN * C::KS];
    __shared__ __attribute__((aligned(16))) uint16_t Vbuf[2][BN * C::VS];

    const int lane = threadIdx.x & 63;
    // the wavefront index as a scalar: every test on it becomes a scalar branch
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, c32 = lane & 31;
    const int nqb = (a.T + BM - 1) / BM, rep = a.Hq / a.Hkv;
    // Full-causal work per query block grows linearly with its index, so a
    // workgroup takes blocks i and nqb-1-i back to back: every workgroup then
    // carries the same number of key tiles and the last wave of workgroups
    // does not idle three quarters of the chip.
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
    const int64_t qb_off = b * a.q_sb + h * a.q_sh;
    const int64_t kb = b * a.k_sb + hk * a.k_sh, vb = b * a.v_sb + hk * a.v_sh;
    const float cexp = a.scale * 1.4426950408889634f;

    // Q as the B operand: lane c holds query c, d = 16kk + 8g .. +7.
    bf16x8 qreg[NQ][KK];
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
        const int row = q0 + (w * NQ + qb) * 32 + c32;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            u32x4 z = {0, 0, 0, 0};
            if (row < a.T)
                z = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.q) + qb_off +
                                                    row * a.q_st + kk * 16 + g * 8);
            qreg[qb][kk] = *reinterpret_cast<bf16x8*>(&z);
        }
    }

    f32x16 acc_o[NQ][DB];
    float m[NQ], l[NQ];
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
        m[qb] = -1e30f;  // the reference's running-max seed, src/ops.cpp:881
        l[qb] = 0.0f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc_o[qb][db][r] = 0.0f;
    }

    // Key tiles this query block can see: the sink tiles [0, ns) and the
    // band / causal tiles [lo, hi] (src/ops.cpp:960-965 in tile units).
    const int qmax = min(q0 + BM, a.T) - 1;
    const int hi = (a.causal ? qmax : a.T - 1) / BN;
    const int lo = a.window > 0 ? max(0, q0 + 1 - a.window) / BN : 0;
    const int ns = a.window > 0 ? min((a.sinks + BN - 1) / BN, lo) : 0;
    int t = ns > 0 ? 0 : lo;

    u32x4 kr[C::CPT], vr[C::CPT];
    int koff[C::CPT], voff[C::CPT];
#pragma unroll
    for (int i = 0; i < C::CPT; ++i) {
        const int c = threadIdx.x + 64 * NW * i;
        koff[i] = static_cast<int>((c / C::NCH) * a.k_st + (c % C::NCH) * 8) * 2;
        voff[i] = static_cast<int>((c / C::NCH) * a.v_st + (c % C::NCH) * 8) * 2;
    }
    TileCursor kc(a.k, kb, a.k_st, t * BN, a.T, D), vc(a.v, vb, a.v_st, t * BN, a.T, D);
    auto load_next = [&](int tn) {
        if (WIN) {
            load_kv_regs<D, NW>(a, kb, vb, tn * BN, koff, voff, kr, vr);
        } else {
            kc.next();
            vc.next();
            const __amdgpu_buffer_rsrc_t krs = kc.rsrc(), vrs = vc.rsrc();
#pragma unroll
            for (int i = 0; i < C::CPT; ++i) {
                kr[i] = tile_load16(krs, koff[i]);
                vr[i] = tile_load16(vrs, voff[i]);
            }
        }
    };
    load_kv_regs<D, NW>(a, kb, vb, t * BN, koff, voff, kr, vr);
    store_kv_lds<D, NW>(Kbuf[0], Vbuf[0], kr, vr);
    __syncthreads();
    int cur = 0;
    // no band, one 32-query block per wavefront: tiles [0, t_last] are visible to this wavefront's block, tiles
    // [0, t_full) need no mask (wholly inside the sequence and, when causal, wholly at or before its first query)
    const int qlo_w = q0 + w * NQ * 32;
    const int t_last = qlo_w >= a.T ? -1 : (a.causal ? min(hi, (qlo_w + 32 * NQ - 1) / BN) : hi);
    const int t_full = min(a.T / BN, a.causal ? (qlo_w + 1) / BN : 0x7fffffff);

    while (t <= hi) {
        const int n0 = t * BN;
        const int tn = (t + 1 == ns) ? lo : t + 1;
        if (tn <= hi) load_next(tn);  // in flight during the math
        const uint16_t* Ks = Kbuf[cur];
        const uint16_t* Vs = Vbuf[cur];

#pragma unroll
        for (int qb = 0; qb < NQ; ++qb) {
            const int qlo = q0 + (w * NQ + qb) * 32, qhi = qlo + 31;
            // wavefront-uniform: nothing of this 32x64 block is visible
            if (!WIN && NQ == 1) {
                if (t > t_last) continue;
            } else {
                if (qlo >= a.T) continue;
                if (a.causal && n0 > qhi) continue;
                if (a.window > 0 && n0 + BN - 1 + a.window <= qlo && n0 >= a.sinks) continue;
            }

            // Two independent accumulator chains, issued alternately: a dependent
            // v_mfma_32x32x16 pair costs 52 cycles, an independent one 32.
            f32x16 s[2];
            // With a band, a 32-key half of the tile that no query of this wavefront can see (past the diagonal, or
            // before the band and without a sink key) is neither multiplied nor exponentiated: at window 256 that is
            // one half in four (the band's two edges and most of the sink tile).
            bool half_live[2] = {true, true};
            if (WIN) {
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const int k0 = n0 + nb * 32, k1 = k0 + 31;
                    half_live[nb] = !(a.causal && k0 > qhi) && !(a.window > 0 && k1 + a.window <= qlo && k0 >= a.sinks);
                }
            }
            // Waves in a matrix phase issue ahead of co-resident waves in the
            // exponent phase: the matrix pipe is the scarcer resource.
            __builtin_amdgcn_s_setprio(1);
            if (!WIN || (half_live[0] && half_live[1])) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[0][r] = s[1][r] = 0.0f;
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) {
                    const bf16x8 k0f = lds_read8(Ks + c32 * C::KS + kk * 16 + g * 8);
                    const bf16x8 k1f = lds_read8(Ks + (32 + c32) * C::KS + kk * 16 + g * 8);
                    s[0] = mfma32(k0f, qreg[qb][kk], s[0]);
                    s[1] = mfma32(k1f, qreg[qb][kk], s[1]);
                }
            } else {  // one half only (the other reads as -inf: its exponentials are zeros and its PV is skipped)
                const int nl = half_live[0] ? 0 : 1;
                f32x16 sl;
#pragma unroll
                for (int r = 0; r < 16; ++r) sl[r] = 0.0f;
#pragma unroll
                for (int kk = 0; kk < KK; ++kk)
                    sl = mfma32(lds_read8(Ks + (nl * 32 + c32) * C::KS + kk * 16 + g * 8), qreg[qb][kk], sl);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    s[0][r] = nl == 0 ? sl[r] : -INFINITY;
                    s[1][r] = nl == 1 ? sl[r] : -INFINITY;
                }
            }
            __builtin_amdgcn_s_setprio(0);
            // Which of the mask's tests a half can fail is wavefront-uniform: none on interior tiles (no mask
            // arithmetic at all), one on the diagonal or on the band's far edge (one compare and one select an element)
            if (!WIN && NQ == 1) {
                if (!(t < t_full)) {
                    const QueryVis vis(qlo + c32, a.T, a.causal, a.window, a.sinks);
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb) {
                        const MaskKind kind = mask_kind(n0 + nb * 32, n0 + nb * 32 + 31, qlo, qhi, a.T, a.causal, 0, 0);
                        if (kind != MaskKind::NONE) mask_block(s[nb], kind, vis, n0 + nb * 32 + g * 4, -INFINITY);
                    }
                }
            } else {
                const QueryVis vis(qlo + c32, a.T, a.causal, a.window, a.sinks);
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const MaskKind kind = mask_kind(n0 + nb * 32, n0 + nb * 32 + 31, qlo, qhi, a.T, a.causal, a.window, a.sinks);
                    if (half_live[nb] && kind != MaskKind::NONE) mask_block(s[nb], kind, vis, n0 + nb * 32 + g * 4, -INFINITY);
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[nb][r]);
            mx = xhalf_max(mx);
            if (__any((mx - m[qb]) * cexp > LAZY_T)) {  // wavefront-uniform, rare after the first tiles
                const float mn = fmaxf(m[qb], mx);
                const float alpha = __builtin_amdgcn_exp2f((m[qb] - mn) * cexp);
                l[qb] *= alpha;
                m[qb] = mn;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc_o[qb][db][r] *= alpha;
            }
            const float mc = m[qb] * cexp;
            // four independent chains: an addition that waits for the one before it takes half as long again to issue
            float psum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(s[nb][r], cexp, -mc));
                    s[nb][r] = p;
                    psum[r & 3] += p;
                }
            l[qb] += (psum[0] + psum[1]) + (psum[2] + psum[3]);  // per-lane partial; the two halves meet in the epilogue

            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                if (WIN && !half_live[nb]) continue;  // P of this half is all zeros
                const bf16x8 p0 = c_to_operand<0>(s[nb]);
                const bf16x8 p1 = c_to_operand<1>(s[nb]);
#pragma unroll
                for (int db = 0; db < DB; ++db)  // DB independent chains per k-chunk
                    acc_o[qb][db] = mfma32(lds_read_tr_operand(Vs, C::VS, nb * 32, db * 32, lane), p0, acc_o[qb][db]);
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    acc_o[qb][db] = mfma32(lds_read_tr_operand(Vs, C::VS, nb * 32 + 16, db * 32, lane), p1, acc_o[qb][db]);
            }
            __builtin_amdgcn_s_setprio(0);
        }

        // The other buffer was last read one iteration ago, before the previous barrier.
        if (tn <= hi) store_kv_lds<D, NW>(Kbuf[cur ^ 1], Vbuf[cur ^ 1], kr, vr);
        __syncthreads();
        cur ^= 1;
        t = tn;
    }

    // Epilogue: O = acc / l, LSE = m*scale + ln(l) (natural log, scaled units).
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
        const int qi = q0 + (w * NQ + qb) * 32 + c32;
        const float lt = xhalf_sum(l[qb]);
        if (qi >= a.T) continue;
        const float inv = 1.0f / lt;
        uint16_t* orow = static_cast<uint16_t*>(a.o) + b * a.o_sb + h * a.o_sh + qi * a.o_st;
#pragma unroll
        for (int db = 0; db < DB; ++db) store_acc_bf16_natural(orow, db, g, acc_o[qb][db], inv);
        if (g == 0)
            a.lse[(static_cast<int64_t>(b) * a.Hq + h) * a.T + qi] = m[qb] * a.scale + logf(lt);
    }
    __syncthreads();  // the next pass refills the tile buffers
  }
}

template <int D, int NQ, int OCC, int NW, bool WIN>
int launch_win(const AttnArgs& a, hipStream_t st) {
    constexpr int BM = 32 * NW * NQ;
    const int nqb = (a.T + BM - 1) / BM;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    dim3 grid(xcd_grid(paired ? (nqb + 1) / 2 : nqb, a.Hq / a.Hkv, a.Hkv * a.B));
    hipLaunchKernelGGL((mfma_fwd<D, NQ, OCC, NW, WIN>), grid, dim3(64 * NW), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}
template <int D, int NQ, int OCC, int NW>
int launch(const AttnArgs& a, hipStream_t st) {
    // the cursor form keeps byte counts in 32 bits: K and V of one (batch, head) must span less than 2 GiB
    const int64_t span = static_cast<int64_t>(a.T) * (a.k_st > a.v_st ? a.k_st : a.v_st) * 2;
    if (a.window == 0 && span < (int64_t{1} << 31)) return launch_win<D, NQ, OCC, NW, false>(a, st);
    return launch_win<D, NQ, OCC, NW, true>(a, st);
}

// 16-byte-aligned rows, and a row stride that keeps a tile's per-thread byte offsets
// (up to 256 rows of a buffer-loaded tile) positive and inside 31 bits.
bool aligned16(const void* p, int64_t sb, int64_t st, int64_t sh) {
    return (reinterpret_cast<uintptr_t>(p) % 16 == 0) && sb % 8 == 0 && st % 8 == 0 && sh % 8 == 0 && st > 0 &&
           st < (int64_t{1} << 22);
}

}  // namespace

// The MFMA kernels take bf16 storage, head_dim 64 or 128, a positive scale
// (the running max is tracked on raw scores) and 16-byte-aligned rows.
bool mfma_supported(const AttnArgs& a) {
    if (a.dk_dim != 64 && a.dk_dim != 128) return false;
    if (!(a.scale > 0.0f)) return false;
    if (!aligned16(a.q, a.q_sb, a.q_st, a.q_sh) || !aligned16(a.k, a.k_sb, a.k_st, a.k_sh) ||
        !aligned16(a.v, a.v_sb, a.v_st, a.v_sh) || !aligned16(a.o, a.o_sb, a.o_st, a.o_sh))
        return false;
    if (a.d_o) {
        if (!aligned16(a.d_o, a.do_sb, a.do_st, a.do_sh)) return false;
        if (!aligned16(a.dq, a.dq_sb, a.dq_st, a.dq_sh) || !aligned16(a.dk, a.dk_sb, a.dk_st, a.dk_sh) ||
            !aligned16(a.dv, a.dv_sb, a.dv_st, a.dv_sh))
            return false;
    }
    return true;
}

int launch_mfma_fwd(const AttnArgs& a, hipStream_t st) {
    // One 32-query block per wavefront, two workgroups per CU.
    // Eight wavefronts (256 queries) per K/V tile halve the tile traffic per MFMA (2.7 % faster at T = 4096, 6 % at
    // T = 16384; slower at head_dim 64 and with a window). One such workgroup fills a CU, so it is only used where the
    // paired causal grid still gives every CU at least two of them in turn.
    const int nqb256 = (a.T + 255) / 256;
    const bool wide = a.dk_dim == 128 && a.causal && a.window == 0 &&
                      static_cast<int64_t>((nqb256 + 1) / 2) * a.Hq * a.B >= 512;
    if (a.dk_dim == 128) return wide ? launch<128, 1, 2, 8>(a, st) : launch<128, 1, 2, 4>(a, st);
    return launch<64, 1, 2, 4>(a, st);
}

}  // namespace pk
