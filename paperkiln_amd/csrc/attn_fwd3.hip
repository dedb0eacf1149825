// Forward with 64 queries per wavefront (see attn_fwd_mfma.hip for the mathematics, attn_bwd_dq3.hip for the
// construction this kernel shares: one wavefront per SIMD, matrix instructions in inline assembly with fixed register
// classes, K / V tiles through a ring of LDS slots filled by loads that write the LDS themselves).
//
// A wavefront owns two blocks of 32 queries. Q of both blocks stays in accumulation registers as the B operand of
// S^T = K Q^T (lane = query), the O^T accumulators (head_dim x 64 queries) likewise, and every K row fragment and every
// transposed V fragment read from the LDS feeds TWO matrix instructions. A K / V tile is 64 keys, worked on as two units
// of 32 keys. Per unit and wavefront at head_dim 128:
//   G1   S^T = K Q^T                 16 matrix instructions (8 fragments, two blocks each)
//   E    P = exp2(S c - m c), row sums, packed to bf16                   (lane = query: all in-lane)
//   G2   O^T += V^T P^T              16 matrix instructions (8 transposed fragments)
//   per tile t:   G1(t, 1) || E(t, 0)  .  G2(t, 0)  .  G1(t+1, 0) || E(t, 1)  .  G2(t, 1)
//
// The running maximum. With the accumulators in accumulation registers, rescaling O^T by exp2(m_old - m_new) costs a
// register move each way per element, so it is not done per tile: m only moves when a unit's maximum exceeds it by more
// than 2^8 (TAU), which after the first unit of a row practically never happens; until then P is formed against the
// stale m (P <= 2^8: no harm in fp32 sums or in bf16's exponent range, and numerator and denominator carry the same
// factor). The rare rescale is a branch around the common path.
//
// Matrix instructions issued from asm statements get no hazard handling from the compiler: a score tile is first read
// a whole phase after the instruction that wrote it, the packed P operand is formed at least two issue slots before the
// instruction that reads it, and the places that touch the accumulators outside matrix instructions wait first
// (tests/test_asm_hazards.py checks the first two on the compiled assembly).
#include <type_traits>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr float TAU = 8.0f;  // log2 of the largest P formed against a stale maximum
constexpr int BN = 64;       // keys per tile
constexpr int BMW = 64;      // queries per wavefront
constexpr int BM = 256;      // queries per workgroup
#define LDSP(T, addr) (reinterpret_cast<PK_LDS T*>(static_cast<uintptr_t>(addr)))

// t = a . b   /   t += a . b      score tile in ordinary registers, B operand (Q) in accumulation registers
__device__ __forceinline__ void mma_s0(f32x16& t, bf16x8 a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(t) : "v"(a), "a"(b));
}
__device__ __forceinline__ void mma_s(f32x16& t, bf16x8 a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(t) : "v"(a), "a"(b));
}
// acc += a . b                    O^T accumulator in accumulation registers, B operand (packed P) in ordinary ones
__device__ __forceinline__ void mma_o(f32x16& acc, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// the same for the first use of a packed P operand: two idle states so that the instruction never reads a register
// written by the vector instruction just before it
__device__ __forceinline__ void mma_o_fresh(f32x16& acc, bf16x8 a, bf16x8 b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
template <int D>
__global__ __launch_bounds__(256, 1) void mfma_fwd3(AttnArgs a) {
    constexpr int KK = D / 16, DB = D / 32;
    constexpr int S = D + 8;      // tile row pitch (elements): 16-byte row reads conflict-free
    constexpr int NCH = D / 8;    // 16-byte chunks per row
    // a tile row in LDS is NCH + 1 units of 16 bytes (the last one padding); one load instruction fills 64 units
    constexpr int UPR = NCH + 1, UNITS = BN * UPR, NI = UNITS / 256;
    static_assert(UNITS - NI * 256 == 64, "the remainder is 16 lanes of each wavefront");
    static_assert(UNITS % 64 == 0, "whole load instructions per wavefront");
    constexpr uint32_t SLOTB = BN * S * 2;
    constexpr int RING = 4;  // tile slots: t, t+1 (read), t+2 (landed or landing), t+3 (asked for)
    __shared__ __attribute__((aligned(16))) uint16_t Kt[RING][BN * S];
    __shared__ __attribute__((aligned(16))) uint16_t Vt[RING][BN * S];

    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, c32 = lane & 31;
    const int nqb = (a.T + BM - 1) / BM, rep = a.Hq / a.Hkv;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    int blk, rr, kvu;
    if (!xcd_map(paired ? (nqb + 1) / 2 : nqb, rep, a.Hkv * a.B, blk, rr, kvu)) return;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv, h = hk * rep + rr;
    const int npass = (paired && blk != nqb - 1 - blk) ? 2 : 1;
    const float cexp = a.scale * LOG2E;

    auto lds32 = [](const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); };
    const uint32_t k_lds = lds32(Kt[0]), v_lds = lds32(Vt[0]);
    // lane parts of the LDS read addresses: a 16-byte row read at (row c32, 8 elements from 8g), and the
    // transposing read of V^T as lds_read_tr_operand_perm lays it out
    const uint32_t x_lane = static_cast<uint32_t>(lds_row<D>(c32) * S + g * 8) * 2u;
    const int tj = lane & 15, tu = (lane >> 4) & 1;
    const uint32_t y_lane = static_cast<uint32_t>(lds_row<D>(4 * g + (tj >> 2)) * S + TrMap<D>::src_col(0, tu, tj & 3)) * 2u;
    auto mem_row = [](int R) {  // which memory row a load puts into LDS row R of a tile: the inverse of lds_row
        const int r = R & 15, bq = r & 3, aq = ((r - 9 * bq) & 15) >> 2;
        return D == 64 ? (R & ~15) | (4 * bq + aq) : R;
    };

    // Tile staging: which 16 bytes of a tile this lane fetches with its i-th load (the LDS side is lane after lane).
    const uint32_t k_st2 = static_cast<uint32_t>(a.k_st) * 2u, v_st2 = static_cast<uint32_t>(a.v_st) * 2u;
    uint32_t offk[NI + 1], offv[NI + 1];
#pragma unroll
    for (int i = 0; i <= NI; ++i) {
        const int u = i < NI ? 256 * i + static_cast<int>(threadIdx.x) : 256 * NI + 16 * w + (lane & 15);
        const uint32_t row = mem_row(u / UPR), ch = min(u % UPR, NCH - 1);  // the padding unit repeats the last chunk
        offk[i] = row * k_st2 + ch * 16u;
        offv[i] = row * v_st2 + ch * 16u;
    }
    auto unit_base = [&](int i) { return static_cast<uint32_t>(i < NI ? 256 * i + 64 * w : 256 * NI + 16 * w) * 16u; };
    auto dma16 = [](uint32_t lds, uint32_t voff, const char* base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory");
    };

    for (int pass = 0; pass < npass; ++pass) {
        const int qblk = pass == 0 ? nqb - 1 - blk : blk;
        const int q0 = qblk * BM, qw = q0 + w * BMW;  // the workgroup's and this wavefront's first query
        const char* kbase = reinterpret_cast<const char*>(a.k) + (b * a.k_sb + hk * a.k_sh) * 2;
        const char* vbase = reinterpret_cast<const char*>(a.v) + (b * a.v_sb + hk * a.v_sh) * 2;
        // key tiles: all the workgroup can see, and the last one this wavefront can see
        const int qmax = min(q0 + BM, a.T) - 1;
        const int hi = (a.causal ? qmax : a.T - 1) / BN;
        const int hi_w = qw >= a.T ? -1 : (a.causal ? min(qw + BMW, a.T) - 1 : a.T - 1) / BN;

        // piece k of tile t into ring slot: k = 2i (K) or 2i + 1 (V), i-th load of this lane
        const char *f_kb = kbase, *f_vb = vbase;
        uint32_t f_limk = 0, f_limv = 0, f_slot = 0;
        auto fetch_setup = [&](int t) {
            const int f_t = min(t, hi);  // a fetch past the end re-reads the last tile
            const int n0 = f_t * BN;
            const int last = min(BN - 1, a.T - 1 - n0);  // rows past the end re-read the last row (those keys are masked)
            f_limk = static_cast<uint32_t>(last) * k_st2 + (NCH - 1) * 16u;
            f_limv = static_cast<uint32_t>(last) * v_st2 + (NCH - 1) * 16u;
            f_kb = kbase + static_cast<int64_t>(n0) * a.k_st * 2;
            f_vb = vbase + static_cast<int64_t>(n0) * a.v_st * 2;
            f_slot = static_cast<uint32_t>(t % RING) * SLOTB;
        };
        auto dma_piece = [&](int k) {
            const int i = k >> 1;
            if (i < NI || lane < 16) {
                if ((k & 1) == 0)
                    dma16(k_lds + f_slot + unit_base(i), min(offk[i], f_limk), f_kb);
                else
                    dma16(v_lds + f_slot + unit_base(i), min(offv[i], f_limv), f_vb);
            }
        };
        constexpr int NPIECE = 2 * (NI + 1);
        auto dma_tile = [&](int t) {
            fetch_setup(t);
#pragma unroll
            for (int k = 0; k < NPIECE; ++k) dma_piece(k);
        };

        // Resident operands. Q of the two 32-query blocks (B operand, lane = query) goes through LDS: a lane's operand
        // chunks are 16 bytes out of every 32 of its own row, so loading them straight from memory touches a cache
        // line per lane and instruction. The wavefront fills the K half of ring slot w with the same row-filling loads
        // as the tiles and reads its operands from there.
        bf16x8 qreg[2][KK];
        f32x16 acc[2][DB];  // O^T of the two query blocks
        {
            const int last_row = max(min(BMW - 1, a.T - 1 - qw), 0);  // rows past the end repeat the last one (never stored)
            const uint32_t region_q = k_lds + static_cast<uint32_t>(w) * SLOTB;
            const char* src = reinterpret_cast<const char*>(a.q) +
                              (b * a.q_sb + h * a.q_sh + static_cast<int64_t>(min(qw, a.T - 1)) * a.q_st) * 2;
            const uint32_t st2 = static_cast<uint32_t>(a.q_st) * 2u;
            int row = lane / UPR, ch = lane % UPR;  // unit 64 i + lane of the padded tile
#pragma unroll
            for (int i = 0; i < UNITS / 64; ++i) {
                dma16(region_q + static_cast<uint32_t>(i) * 1024u,
                      static_cast<uint32_t>(min(mem_row(row), last_row)) * st2 + static_cast<uint32_t>(min(ch, NCH - 1)) * 16u, src);
                row += 64 / UPR, ch += 64 % UPR;
                if (ch >= UPR) ch -= UPR, ++row;
            }
            // the accumulators are cleared while the rows are on their way
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int db = 0; db < DB; ++db) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[qb][db][r] = 0.0f;
                    asm volatile("" : "+a"(acc[qb][db]));
                }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int kk = 0; kk < KK; ++kk)
                    qreg[qb][kk] = *LDSP(const bf16x8, region_q + x_lane + (qb * 32 * S + kk * 16) * 2);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        __syncthreads();  // every wavefront has read its region: the slots may take their tiles
        dma_tile(0);
        dma_tile(1);
        dma_tile(2);  // waited for at the end of the first iteration
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) asm volatile("" : "+a"(qreg[qb][kk]));
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NPIECE) : "memory");  // tiles 0 and 1 are in
        __syncthreads();

        const QueryVis qvis[2] = {QueryVis(qw + c32, a.T, a.causal, a.window, a.sinks),
                                  QueryVis(qw + 32 + c32, a.T, a.causal, a.window, a.sinks)};
        // per query (both lanes of a pair hold the same value): the maximum P is formed against, in log2 units
        float mc[2] = {-1e30f, -1e30f};
        // per lane: the sum of its half of the row, in two parts so that the additions do not wait for one another
        float l0[2] = {0.0f, 0.0f}, l1[2] = {0.0f, 0.0f};

        constexpr int PF = 3;              // fragments in flight
        constexpr int N1 = 2 * KK;         // matrix instructions of a G1 phase: kk x two query blocks
        constexpr int N2 = 4 * DB;         // of a G2 phase: two k-chunks x DB column blocks x two query blocks
        constexpr int EPS = 32 / N1;       // elements per slot
        static_assert(EPS == 2 || EPS == 4, "head_dim 128 or 64");
        f32x16 sc[2][2];                   // [unit parity][query block]: S^T as the matrix pipe leaves it
        bf16x8 dsp[2][2];                  // packed P^T of the unit in hand, [query block][16-key half]
        uint32_t pk[4];                    // packed pairs of the half block in hand

        // G1 fragment kk of unit (slot address ka, 32-key half nb): K rows
        auto g1frag = [&](uint32_t ka, int nb, int kk) { return *LDSP(const bf16x8, ka + (nb * 32 * S + kk * 16) * 2); };
        // G2 fragment fi of a unit: V^T, 16-key half kc = fi / DB, column block db = fi % DB
        auto g2frag = [&](uint32_t ya, int nb, int fi) {
            const uint32_t at = ya + ((nb * 32 + (fi / DB) * 16) * S + TrMap<D>::src_col(fi % DB, 0, 0) - TrMap<D>::src_col(0, 0, 0)) * 2;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, at));
            const s16x4 hi2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, at + TR_HI_ROWS<D> * S * 2));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi2[0], hi2[1], hi2[2], hi2[3]};
            return *reinterpret_cast<const bf16x8*>(&v);
        };
        // `have`: the first PF fragments were asked for in the last slots of the phase before (nx); `next(j)` asks for
        // fragment j of the phase that follows, in this phase's last slots, so that no phase opens with an LDS round trip
        bf16x8 nx[PF];
        auto g1 = [&](uint32_t ka, int nb, f32x16(&s_)[2], auto shadow, auto have, auto next) {
            bf16x8 f[KK];
#pragma unroll
            for (int j = 0; j < PF; ++j) f[j] = decltype(have)::value ? nx[j] : g1frag(ka, nb, j);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sl = 0; sl < N1; ++sl) {
                const int kk = sl >> 1, qb = sl & 1;
                if (kk == 0)
                    mma_s0(s_[qb], f[kk], qreg[qb][kk]);
                else
                    mma_s(s_[qb], f[kk], qreg[qb][kk]);
                if (qb == 0) {
                    if (kk + PF < KK)
                        f[kk + PF] = g1frag(ka, nb, kk + PF);
                    else
                        nx[kk + PF - KK] = next(kk + PF - KK);
                }
                shadow(sl);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto g2 = [&](uint32_t ya, int nb, auto shadow, auto next) {
            bf16x8 f[N2 / 2];
#pragma unroll
            for (int j = 0; j < PF; ++j) f[j] = nx[j];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sl = 0; sl < N2; ++sl) {
                const int fi = sl >> 1, qb = sl & 1;
                if (fi % DB == 0)
                    mma_o_fresh(acc[qb][0], f[fi], dsp[qb][fi / DB]);
                else
                    mma_o(acc[qb][fi % DB], f[fi], dsp[qb][fi / DB]);
                if (qb == 0) {
                    if (fi + PF < N2 / 2)
                        f[fi + PF] = g2frag(ya, nb, fi + PF);
                    else
                        nx[fi + PF - N2 / 2] = next(fi + PF - N2 / 2);
                }
                shadow(sl);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // Elementwise work of a unit, EPS elements per slot (element e: query block e / 16, register e % 16), staggered
        // over three slots because each instruction is the input of the next: slot sl forms x = S c - m c of its
        // elements, p = exp2(x) of the elements of slot sl - 1, and adds the elements of slot sl - 2 to the row sum and packs
        // them; the last two slots' worth finishes in the first two slots of the G2 phase that follows.
        float xq[EPS] = {}, pq[EPS] = {};
        auto elem = [&](const f32x16(&s_)[2], int sl) {
            if (sl >= 2 && sl < N1 + 2) {
#pragma unroll
                for (int i = 0; i < EPS; i += 2) {
                    const int e = (sl - 2) * EPS + i, qb = e >> 4, r = e & 15;
                    const uint32_t p2 = pack_bf16(pq[i], pq[i + 1]);
                    pk[(r & 7) >> 1] = p2;
                    l0[qb] += pq[i];  // the sums take P before it is rounded: LSE is held to 1e-3
                    l1[qb] += pq[i + 1];
                    if ((r & 7) == 6) {
                        u32x4 u = {pk[0], pk[1], pk[2], pk[3]};
                        dsp[qb][r >> 3] = *reinterpret_cast<bf16x8*>(&u);
                        // formed here, in this slot (the compiler may otherwise sink the chain to just before its reader)
                        asm volatile("" : "+v"(dsp[qb][r >> 3]));
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < EPS; ++i)
                if (sl >= 1 && sl < N1 + 1) pq[i] = __builtin_amdgcn_exp2f(xq[i]);
#pragma unroll
            for (int i = 0; i < EPS; ++i) {
                const int e = sl * EPS + i;
                if (sl < N1) xq[i] = fmaf(s_[e >> 4][e & 15], cexp, -mc[e >> 4]);
            }
        };
        // A unit on the diagonal or past the end of the keys: what the mask hides becomes -inf before anything reads it
        auto mask_unit = [&](f32x16(&s_)[2], int n0u) {
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    s_[qb][r] = qvis[qb](n0u + (r >> 2) * 8 + g * 4 + (r & 3)) ? s_[qb][r] : -INFINITY;
        };
        auto unit_full = [&](int n0u) {  // every key of the unit visible to every query of the wavefront
            return n0u + 31 < a.T && (!a.causal || n0u + 31 <= qw);
        };
        // Before a unit's elementwise work: does its maximum exceed the one in use by more than TAU for any query of
        // the wavefront? Then (rarely: at the first unit, and where the scores grow by a factor of 2^8 along a row)
        // the maximum moves and what has been accumulated is rescaled -- through ordinary registers, after the matrix
        // instructions in flight have written their results.
        auto track_max = [&](const f32x16(&s_)[2]) {
            float um[2];
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                float m4[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    m4[j] = fmaxf(fmaxf(s_[qb][4 * j], s_[qb][4 * j + 1]), fmaxf(s_[qb][4 * j + 2], s_[qb][4 * j + 3]));
                um[qb] = xhalf_max(fmaxf(fmaxf(m4[0], m4[1]), fmaxf(m4[2], m4[3]))) * cexp;
            }
            const bool need = (um[0] > mc[0] + TAU) | (um[1] > mc[1] + TAU);
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(need) != 0, 0)) {
                asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    const float mnew = fmaxf(mc[qb], um[qb]);
                    const float al = __builtin_amdgcn_exp2f(mc[qb] - mnew);
                    mc[qb] = mnew;
                    l0[qb] *= al;
                    l1[qb] *= al;
#pragma unroll
                    for (int db = 0; db < DB; ++db) {
                        asm volatile("" : "+a"(acc[qb][db]));
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[qb][db][r] *= al;
                        asm volatile("" : "+a"(acc[qb][db]));
                    }
                }
                asm volatile("s_nop 3" ::: "memory");
            }
        };

        if (hi_w >= 0)
            g1(k_lds + x_lane, 0, sc[0], [](int) {}, std::false_type{}, [&](int j) { return g1frag(k_lds + x_lane, 1, j); });
        // the first reads of these scores follow at once here (in the loop a whole G2 phase lies between): let the last
        // matrix instructions of this prologue write their results first
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
        for (int t = 0; t <= hi; ++t) {
            const uint32_t slot = static_cast<uint32_t>(t % RING) * SLOTB, slot1 = static_cast<uint32_t>((t + 1) % RING) * SLOTB;
            fetch_setup(t + 3);
            auto stage = [&](int first, int sl) {  // the arriving tile, half of its loads in each G2 phase
                if (sl % 3 == 1 && sl / 3 < NPIECE / 2) dma_piece(first + sl / 3);
            };
            if (t <= hi_w) {
                const int n0 = t * BN;
                const uint32_t ka = k_lds + slot + x_lane, ka1 = k_lds + slot1 + x_lane, ya = v_lds + slot + y_lane;
                // ---- G1(t, 1) || E(t, 0)
                if (__builtin_expect(!unit_full(n0), 0)) mask_unit(sc[0], n0);
                track_max(sc[0]);
                g1(ka, 1, sc[1], [&](int sl) { elem(sc[0], sl); }, std::true_type{}, [&](int j) { return g2frag(ya, 0, j); });
                // ---- G2(t, 0)
                g2(ya, 0,
                   [&](int sl) {
                       if (sl < 2) elem(sc[0], N1 + sl);
                       stage(0, sl);
                   },
                   [&](int j) { return g1frag(ka1, 0, j); });
                // ---- G1(t+1, 0) || E(t, 1)
                if (__builtin_expect(!unit_full(n0 + 32), 0)) mask_unit(sc[1], n0 + 32);
                track_max(sc[1]);
                g1(ka1, 0, sc[0], [&](int sl) { elem(sc[1], sl); }, std::true_type{}, [&](int j) { return g2frag(ya, 1, j); });
                // ---- G2(t, 1); its last slots ask for the first fragments of the next iteration's G1(t+1, 1): that tile
                // has been readable since the barrier before this iteration
                g2(ya, 1,
                   [&](int sl) {
                       if (sl < 2) elem(sc[1], N1 + sl);
                       stage(NPIECE / 2, sl);
                   },
                   [&](int j) { return g1frag(ka1, 1, j); });
            }
            if (t > hi_w) {  // past this wavefront's diagonal: only the staging (a second skip, not an else)
#pragma unroll
                for (int k = 0; k < NPIECE; ++k) dma_piece(k);
            }
            // Tile t+2 (asked for one iteration ago) has landed; the NPIECE loads of tile t+3 issued in this iteration
            // may stay in flight (loads complete in order). Every wavefront issues exactly NPIECE load instructions
            // per iteration, on either path.
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NPIECE) : "memory");
            __syncthreads();
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may land in the ring after the pass

        // the last matrix instructions may still be writing the accumulators
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int db = 0; db < DB; ++db) asm volatile("" : "+a"(acc[qb][db]));
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const int qi = qw + qb * 32 + c32;
            const float lt = xhalf_sum(l0[qb] + l1[qb]);
            if (qi >= a.T) continue;
            const float inv = 1.0f / lt;
            uint16_t* orow = static_cast<uint16_t*>(a.o) + b * a.o_sb + h * a.o_sh + qi * a.o_st;
#pragma unroll
            for (int db = 0; db < DB; ++db) store_acc_bf16<D>(orow, db, g, acc[qb][db], inv);
            if (g == 0) a.lse[(static_cast<int64_t>(b) * a.Hq + h) * a.T + qi] = mc[qb] * (1.0f / LOG2E) + logf(lt);
        }
        // no barrier: every wavefront passed the barrier of the last iteration after its last read of the ring
    }
}

template <int D>
int launch(const AttnArgs& a, hipStream_t st) {
    const int nqb = (a.T + BM - 1) / BM;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    const dim3 grid(xcd_grid(paired ? (nqb + 1) / 2 : nqb, a.Hq / a.Hkv, a.Hkv * a.B));
    hipLaunchKernelGGL((mfma_fwd3<D>), grid, dim3(256), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

}  // namespace

bool mfma_fwd3_takes(const AttnArgs& a) {
    // a lane's byte offset inside a 64-row tile of K / V is kept in 32 bits
    const int64_t reach = 2 * BN * (a.k_st > a.v_st ? a.k_st : a.v_st);
    return a.dk_dim == 128 && a.window == 0 && reach < (int64_t{1} << 31) && 2 * BMW * a.q_st < (int64_t{1} << 31);
}

int launch_mfma_fwd3(const AttnArgs& a, hipStream_t st) { return launch<128>(a, st); }

}  // namespace pk
