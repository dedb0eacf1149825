// Software-pipelined bf16 flash-attention forward for gfx950, head_dim 128.
// Same mathematics and operand layouts as attn_fwd_mfma.hip (S^T = K Q^T,
// O^T += V^T P^T, lazy rescale); what changes is the schedule.
//
// Measured on the machine: one wavefront can retire a 32x32x16 MFMA every 32
// cycles, but every LDS fragment read it issues also occupies ~27 (b128) or
// ~32 (transposing b64) cycles of its own in-order memory queue. With one LDS
// fragment per MFMA the loop is bound by LDS issue, not by the matrix pipe.
// So here a wavefront owns 64 queries (two 32-query blocks): every K and V^T
// fragment read from LDS feeds TWO MFMAs. That takes all 512 registers, hence
// one wavefront per SIMD, and the overlap of MFMA, LDS and VALU work that two
// wavefronts would give is recovered by pipelining across key tiles inside
// the wavefront:
//
//   iteration i:   S(i+1) = K(i+1) Q^T      (MFMA)   ||  P(i) = exp2(S(i) - m)   (VALU)
//                  O^T   += V(i)^T P(i)^T   (MFMA)   ||  mask / row max of S(i+1) (VALU)
//
// K tiles run two ahead of the loop (three-deep LDS ring) and V tiles one ahead
// (two-deep ring), so one barrier per key tile suffices.
#include <type_traits>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr int BN = 64;
constexpr int NQ = 2;
constexpr int BM = 128 * NQ;

// LDS tiles are dense [64 rows][D] (no padding) because they are filled by
// global_load_lds_dwordx4: the 64 lanes of one instruction write 64
// consecutive 16-byte chunks = four full rows. Bank conflicts are avoided by
// an XOR swizzle of the 16-byte chunk index instead: chunk c of row r is
// stored at chunk c ^ swz(r). swz maps the 16 rows of a b128 fragment read to
// 16 different chunks, and the 4 consecutive rows of a transposing read to 4
// different groups of four chunks, so both access kinds touch every bank once.
__device__ inline int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

// Issue the direct-to-LDS loads of one [64][128] bf16 tile (16 KB): 16
// wave-level instructions, 4 per wavefront. Rows past the end re-read the
// last row: finite values whose scores are masked, so they meet P == 0 exactly.
__device__ inline void tile_to_lds(const void* base, int64_t off, int64_t st_t, int n0, int T, uint16_t* lds,
                                   int w, int lane) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int inst = w * 4 + j;
        const int row = inst * 4 + (lane >> 4);
        const int ch = (lane & 15) ^ swz(row);
        const int t = min(n0 + row, T - 1);
        const uint16_t* g = static_cast<const uint16_t*>(base) + off + t * st_t + ch * 8;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                         (__attribute__((address_space(3))) void*)(lds + inst * 512), 16, 0, 0);
    }
}
__device__ inline void wait_tiles() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <int D>
__global__ __launch_bounds__(256, 1) void mfma_fwd_pipe(AttnArgs a) {
    static_assert(D == 128, "the swizzle and the loaders are written for 256-byte rows");
    constexpr int KK = D / 16, DB = D / 32;
    __shared__ __attribute__((aligned(1024))) uint16_t Kbuf[3][BN * D];
    __shared__ __attribute__((aligned(1024))) uint16_t Vbuf[2][BN * D];

    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int g = lane >> 5, c32 = lane & 31;
    const int nqb = (a.T + BM - 1) / BM, rep = a.Hq / a.Hkv;
    const bool paired = a.causal && a.window == 0;
    int blk, rr, kvu;
    if (!xcd_map(paired ? (nqb + 1) / 2 : nqb, rep, a.Hkv * a.B, blk, rr, kvu)) return;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv, h = hk * rep + rr;
    const int64_t kb = b * a.k_sb + hk * a.k_sh, vb = b * a.v_sb + hk * a.v_sh;
    const float cexp = a.scale * 1.4426950408889634f;
    const int npass = (paired && blk != nqb - 1 - blk) ? 2 : 1;

    for (int pass = 0; pass < npass; ++pass) {
        const int qblk = pass == 0 ? nqb - 1 - blk : blk;
        const int q0 = qblk * BM;
        const int qlo0 = q0 + w * 64;  // this wavefront's 64 queries

        bf16x8 qreg[NQ][KK];
#pragma unroll
        for (int qb = 0; qb < NQ; ++qb) {
            const int row = qlo0 + qb * 32 + c32;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                u32x4 z = {0, 0, 0, 0};
                if (row < a.T)
                    z = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.q) + b * a.q_sb + h * a.q_sh +
                                                        row * a.q_st + kk * 16 + g * 8);
                qreg[qb][kk] = *reinterpret_cast<bf16x8*>(&z);
            }
        }
        f32x16 acc_o[NQ][DB];
        float m[NQ], l[NQ];
#pragma unroll
        for (int qb = 0; qb < NQ; ++qb) {
            m[qb] = -1e30f;
            l[qb] = 0.0f;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc_o[qb][db][r] = 0.0f;
        }
        const QueryVis vis0(qlo0 + c32, a.T, a.causal, a.window, a.sinks);
        const QueryVis vis1(qlo0 + 32 + c32, a.T, a.causal, a.window, a.sinks);

        // key tiles: sink tiles [0, ns) then band / causal tiles [lo, hi]
        const int qmax = min(q0 + BM, a.T) - 1;
        const int hi = (a.causal ? qmax : a.T - 1) / BN;
        const int lo = a.window > 0 ? max(0, q0 + 1 - a.window) / BN : 0;
        const int ns = a.window > 0 ? min((a.sinks + BN - 1) / BN, lo) : 0;
        auto next = [&](int t) { return (t + 1 == ns) ? lo : t + 1; };

        // swizzled LDS addressing, per lane: K fragments are 16-byte reads of row c32,
        // chunk 2kk+g; V^T operands are two transposing 8-byte reads (see mfma_common.h).
        const int kx = g ^ swz(c32);
        const int vj = lane & 15, vu = (lane >> 4) & 1;
        const int v_fh = ((vj >> 2) & 3) << 2;              // swz(row) & 12, row & 3 == vj >> 2
        const int v_c0 = 2 * vu + ((vj & 3) >> 1);          // chunk inside the 32-column block
        const int v_lo = (4 * g + (vj >> 2)) * D + (((v_c0 ^ g)) << 3) + ((vj & 1) << 2);
        const int v_hi = (4 * g + (vj >> 2) + 8) * D + (((v_c0 ^ (g + 2))) << 3) + ((vj & 1) << 2);
        auto v_operand = [&](const uint16_t* Vt, int row0, int db) {
            const int cg = ((4 * db) ^ v_fh) << 3;           // swizzled group of four chunks
            const s16x4 lo4 = lds_read_tr4(Vt + row0 * D + v_lo + cg);
            const s16x4 hi4 = lds_read_tr4(Vt + row0 * D + v_hi + cg);
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            s16x8 v = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
            return *reinterpret_cast<bf16x8*>(&v);
        };

        // The pipeline advances in 32-key half tiles (register budget): S for one
        // half tile is 2 x 16 accumulator registers.
        f32x16 s_a[NQ], s_b[NQ];
        auto needs_mask = [&](int n0) {  // wavefront-uniform: some (query, key) of the 64 x 32 block is hidden
            const int qlo = qlo0, qhi = qlo0 + 63;
            const bool full = (n0 + 31 < a.T) && qhi < a.T && (!a.causal || n0 + 31 <= qlo) &&
                              (a.window == 0 || n0 + a.window > qhi || n0 + 31 < a.sinks);
            return !full;
        };
        // One half step, a single basic block so that the scheduler can interleave:
        //   S_next = K_next Q^T (16 MFMA, 8 LDS reads)  ||  P = exp2(S_cur*c - m*c), row sums (VALU)
        //   O^T += V^T P^T      (16 MFMA, 16 LDS reads) ||  mask + row max of S_next (VALU)
        // Returns the per-block row maxima of S_next for the rescale test that follows.
        auto half_step = [&](auto masked, const uint16_t* Kn, int nbn, int n0n, f32x16 (&sn)[NQ],
                             f32x16 (&sc)[NQ], const uint16_t* Vc, int nbc, float (&mx)[NQ]) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sn[0][r] = sn[1][r] = 0.0f;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const bf16x8 kf = lds_read8(Kn + (nbn * 32 + c32) * D + (((2 * kk) ^ kx) << 3));
                sn[0] = mfma32(kf, qreg[0][kk], sn[0]);
                sn[1] = mfma32(kf, qreg[1][kk], sn[1]);
            }
            bf16x8 pop[NQ][2];
#pragma unroll
            for (int qb = 0; qb < NQ; ++qb) {
                const float mc = m[qb] * cexp;
                float psum = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(sc[qb][r], cexp, -mc));
                    sc[qb][r] = p;
                    psum += p;
                }
                l[qb] += psum;
                pop[qb][0] = c_to_operand<0>(sc[qb]);
                pop[qb][1] = c_to_operand<1>(sc[qb]);
            }
#ifdef PK_SB
            __builtin_amdgcn_sched_barrier(0);
#endif
#ifndef NO_SGB1
#pragma unroll
            for (int i = 0; i < 16; ++i) {  // one S MFMA, then its share of the softmax VALU work
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x402, 7, 0);
            }
#endif
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const bf16x8 vf = v_operand(Vc, nbc * 32 + hf * 16, db);
                    acc_o[0][db] = mfma32(vf, pop[0][hf], acc_o[0][db]);
                    acc_o[1][db] = mfma32(vf, pop[1][hf], acc_o[1][db]);
                }
#pragma unroll
            for (int qb = 0; qb < NQ; ++qb) {
                if (decltype(masked)::value) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int kj = n0n + (r >> 2) * 8 + g * 4 + (r & 3);
                        const bool v = qb == 0 ? vis0(kj) : vis1(kj);
                        sn[qb][r] = v ? sn[qb][r] : -INFINITY;
                    }
                }
                float x = -INFINITY;
#pragma unroll
                for (int r = 0; r < 16; ++r) x = fmaxf(x, sn[qb][r]);
                mx[qb] = xhalf_max(x);
            }
#ifndef NO_SGB2
#pragma unroll
            for (int i = 0; i < 16; ++i) {  // one PV MFMA, its LDS reads, a few row-max ops
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x402, 2, 0);
            }
#endif
        };
        // The same half step for fully visible half tiles, scheduled by hand: every MFMA
        // is followed in program order by its share of independent VALU work, and a
        // scheduling fence keeps the compiler from regrouping them. The matrix pipe runs an
        // MFMA for 32 cycles while the wavefront issues the exp2 / fma / add that follow it.
        auto half_step_interior = [&](const uint16_t* Kn, int nbn, f32x16 (&sn)[NQ], f32x16 (&sc)[NQ],
                                      const uint16_t* Vc, int nbc, float (&mx)[NQ]) {
            const float mc0 = m[0] * cexp, mc1 = m[1] * cexp;
            float ps0 = 0.0f, ps1 = 0.0f;
            bf16x8 kf[KK];
            kf[0] = lds_read8(Kn + (nbn * 32 + c32) * D + (((0) ^ kx) << 3));
            kf[1] = lds_read8(Kn + (nbn * 32 + c32) * D + (((2) ^ kx) << 3));
#pragma unroll
            for (int r = 0; r < 16; ++r) sn[0][r] = sn[1][r] = 0.0f;
            bf16x8 vf[2 * DB];  // V^T operands, fetched two MFMA pairs ahead
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                if (kk + 2 < KK) kf[kk + 2] = lds_read8(Kn + (nbn * 32 + c32) * D + (((2 * (kk + 2)) ^ kx) << 3));
                if (kk == KK - 2) vf[0] = v_operand(Vc, nbc * 32, 0);
                if (kk == KK - 1) vf[1] = v_operand(Vc, nbc * 32, 1);
                sn[0] = mfma32(kf[kk], qreg[0][kk], sn[0]);
                {
                    const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[0][2 * kk], cexp, -mc0));
                    const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[0][2 * kk + 1], cexp, -mc0));
                    sc[0][2 * kk] = p0;
                    sc[0][2 * kk + 1] = p1;
                    ps0 += p0 + p1;
                }
                __builtin_amdgcn_sched_barrier(0);
                sn[1] = mfma32(kf[kk], qreg[1][kk], sn[1]);
                {
                    const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[1][2 * kk], cexp, -mc1));
                    const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[1][2 * kk + 1], cexp, -mc1));
                    sc[1][2 * kk] = p0;
                    sc[1][2 * kk + 1] = p1;
                    ps1 += p0 + p1;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            l[0] += ps0;
            l[1] += ps1;
            bf16x8 pop[NQ][2];
            pop[0][0] = c_to_operand<0>(sc[0]);
            pop[1][0] = c_to_operand<0>(sc[1]);
            float x0 = -INFINITY, x1 = -INFINITY;
#pragma unroll
            for (int j = 0; j < 2 * DB; ++j) {  // j = hf * DB + db
                const int hf = j / DB, db = j % DB;
                if (j + 2 < 2 * DB) vf[j + 2] = v_operand(Vc, nbc * 32 + ((j + 2) / DB) * 16, (j + 2) % DB);
                if (j == DB - 1) {
                    pop[0][1] = c_to_operand<1>(sc[0]);
                    pop[1][1] = c_to_operand<1>(sc[1]);
                }
                acc_o[0][db] = mfma32(vf[j], pop[0][hf], acc_o[0][db]);
                x0 = fmaxf(x0, fmaxf(sn[0][2 * j], sn[0][2 * j + 1]));
                __builtin_amdgcn_sched_barrier(0);
                acc_o[1][db] = mfma32(vf[j], pop[1][hf], acc_o[1][db]);
                x1 = fmaxf(x1, fmaxf(sn[1][2 * j], sn[1][2 * j + 1]));
                __builtin_amdgcn_sched_barrier(0);
            }
            mx[0] = xhalf_max(x0);
            mx[1] = xhalf_max(x1);
        };
        auto rescale = [&](float (&mx)[NQ]) {  // lazy: taken only when some row max moved by > 2^lazy_t
#pragma unroll
            for (int qb = 0; qb < NQ; ++qb) {
                if (__any((mx[qb] - m[qb]) * cexp > a.lazy_t)) {
                    const float mn = fmaxf(m[qb], mx[qb]);
                    const float alpha = __builtin_amdgcn_exp2f((m[qb] - mn) * cexp);
                    l[qb] *= alpha;
                    m[qb] = mn;
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc_o[qb][db][r] *= alpha;
                }
            }
        };

        // ---- prologue: K(t0), K(t1), V(t0) resident; S(t0, first half) computed ----
        int t = ns > 0 ? 0 : lo;
        int tn = next(t), tnn = next(tn);
        tile_to_lds(a.k, kb, a.k_st, t * BN, a.T, Kbuf[0], w, lane);
        tile_to_lds(a.v, vb, a.v_st, t * BN, a.T, Vbuf[0], w, lane);
        tile_to_lds(a.k, kb, a.k_st, min(tn, hi) * BN, a.T, Kbuf[1], w, lane);
        wait_tiles();
        __syncthreads();
        {
            float mx[NQ];
#pragma unroll
            for (int r = 0; r < 16; ++r) s_a[0][r] = s_a[1][r] = 0.0f;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const bf16x8 kf = lds_read8(Kbuf[0] + c32 * D + (((2 * kk) ^ kx) << 3));
                s_a[0] = mfma32(kf, qreg[0][kk], s_a[0]);
                s_a[1] = mfma32(kf, qreg[1][kk], s_a[1]);
            }
#pragma unroll
            for (int qb = 0; qb < NQ; ++qb) {
                float x = -INFINITY;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int kj = t * BN + (r >> 2) * 8 + g * 4 + (r & 3);
                    const bool v = qb == 0 ? vis0(kj) : vis1(kj);
                    s_a[qb][r] = v ? s_a[qb][r] : -INFINITY;
                    x = fmaxf(x, s_a[qb][r]);
                }
                mx[qb] = xhalf_max(x);
            }
            rescale(mx);
        }

        int i = 0, ki = 0;
#ifdef PK_TIMING
        long long tacc[6] = {0, 0, 0, 0, 0, 0};
        long long tprev = __builtin_readcyclecounter();
#define PK_TICK(i) { long long now = __builtin_readcyclecounter(); tacc[i] += now - tprev; tprev = now; }
#else
#define PK_TICK(i)
#endif
        // One key tile = two half steps + the loads of the tiles ahead + one barrier.
        auto iteration = [&](auto masked) {
            const bool has_n = tn <= hi;
            // K runs two tiles ahead, V one tile ahead; past the end the last tile is re-read and ignored.
            // K(t-1) (three-deep ring) and V(t-1) were last read before the previous barrier.
            tile_to_lds(a.k, kb, a.k_st, min(tnn, hi) * BN, a.T, Kbuf[ki == 0 ? 2 : ki - 1], w, lane);
            tile_to_lds(a.v, vb, a.v_st, min(tn, hi) * BN, a.T, Vbuf[(i + 1) & 1], w, lane);
            const uint16_t* Kc = Kbuf[ki];
            const uint16_t* Kn = Kbuf[ki == 2 ? 0 : ki + 1];
            const uint16_t* Vc = Vbuf[i & 1];
            float mx[NQ];
            PK_TICK(0)
            // half step A:  S(t, keys 32..63)  ||  softmax + PV of keys 0..31
            if (decltype(masked)::value)
                half_step(masked, Kc, 1, t * BN + 32, s_b, s_a, Vc, 0, mx);
            else
                half_step_interior(Kc, 1, s_b, s_a, Vc, 0, mx);
            PK_TICK(1)
            rescale(mx);
            PK_TICK(2)
            // half step B:  S(t+1, keys 0..31)  ||  softmax + PV of keys 32..63
            if (decltype(masked)::value)
                half_step(masked, Kn, 0, has_n ? tn * BN : a.T, s_a, s_b, Vc, 1, mx);
            else
                half_step_interior(Kn, 0, s_a, s_b, Vc, 1, mx);
            PK_TICK(1)
            rescale(mx);
            PK_TICK(2)
            wait_tiles();
            PK_TICK(3)
            __syncthreads();
            PK_TICK(4)
            t = tn;
            tn = tnn;
            tnn = next(tnn);
            ++i;
            ki = ki == 2 ? 0 : ki + 1;
        };
        // Does iteration t touch a half tile that is partly hidden from this wavefront?
        auto tile_masked = [&]() { return needs_mask(t * BN + 32) || tn > hi || needs_mask(tn * BN); };
        // Three loops with ONE body variant each (masked prefix: sinks / band start; unmasked
        // interior; masked suffix: diagonal / ragged end), so that no iteration carries the
        // accumulators across a merge of differently allocated variants.
        while (t <= hi && tile_masked()) iteration(std::true_type{});
        while (t <= hi && !tile_masked()) iteration(std::false_type{});
        while (t <= hi) iteration(std::true_type{});

#ifdef PK_TIMING
        if (a.delta && lane == 0) {
            long long* dbg = reinterpret_cast<long long*>(a.delta) + (static_cast<long long>(blockIdx.x) * 4 + w) * 8;
            for (int q = 0; q < 5; ++q) dbg[q] += tacc[q];
            dbg[5] += i;
        }
#endif
        // epilogue
#pragma unroll
        for (int qb = 0; qb < NQ; ++qb) {
            const int qi = qlo0 + qb * 32 + c32;
            const float lt = xhalf_sum(l[qb]);
            if (qi < a.T) {
                const float inv = 1.0f / lt;
                uint16_t* orow = static_cast<uint16_t*>(a.o) + b * a.o_sb + h * a.o_sh + qi * a.o_st;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int qd = 0; qd < 4; ++qd) {
                        u32x2 pk2 = {pack_bf16(acc_o[qb][db][qd * 4 + 0] * inv, acc_o[qb][db][qd * 4 + 1] * inv),
                                     pack_bf16(acc_o[qb][db][qd * 4 + 2] * inv, acc_o[qb][db][qd * 4 + 3] * inv)};
                        *reinterpret_cast<u32x2*>(orow + db * 32 + qd * 8 + g * 4) = pk2;
                    }
                if (g == 0) a.lse[(static_cast<int64_t>(b) * a.Hq + h) * a.T + qi] = m[qb] * a.scale + logf(lt);
            }
        }
        __syncthreads();
    }
}

}  // namespace

int launch_mfma_fwd_pipe(const AttnArgs& a, hipStream_t st) {
    const int nqb = (a.T + BM - 1) / BM;
    const bool paired = a.causal && a.window == 0;
    dim3 grid(xcd_grid(paired ? (nqb + 1) / 2 : nqb, a.Hq / a.Hkv, a.Hkv * a.B));
    hipLaunchKernelGGL((mfma_fwd_pipe<128>), grid, dim3(256), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

}  // namespace pk
