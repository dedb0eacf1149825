// dK / dV of the recompute backward, third generation (see attn_bwd_mfma.hip for
// the mathematics and the operand layouts, attn_bwd_dkdv2.hip for the role split).
//
// The LDS hands a CU 128 bytes per clock: one 1 KB operand fragment per 32 clocks
// per SIMD, the issue rate of the 32x32x16 MFMA. A wavefront that owns 32 keys
// feeds every fragment it reads to ONE matrix instruction, so the LDS is as busy
// as the matrix pipe and neither passes half. Here a wavefront owns 64 keys: two
// resident operand sets (K or V of two 32-key blocks), two accumulator sets, and
// every Q / dO fragment read from the LDS feeds TWO matrix instructions. That is
// 192 persistent registers, so one wavefront per SIMD, four per workgroup:
//
//   role 0 (wavefronts 0-1, keys 0-63 / 64-127):  S -> P = exp2(S*c - LSE) -> dV^T += dO^T P
//   role 1 (wavefronts 2-3, keys 0-63 / 64-127):  dP -> dS = P .* (dP - delta) -> dK^T += Q^T dS
//
// P goes from role 0 to role 1 through LDS one step behind, as in the second
// generation.
//
// Register classes are fixed by hand. Every matrix instruction is written as inline
// assembly: the dV^T / dK^T accumulators (128 registers) are pinned in the accumulation
// register file ("a" constraint) and never leave it until the epilogue; the score tiles
// S / dP, which the VALU works on, are produced straight into ordinary registers ("v").
// Left to the compiler, a function that needs more than 256 registers gets the
// accumulation-register form for ALL its matrix instructions and pays a register move
// per score, plus moves of the accumulators at every loop edge. The price of the
// assembly is that the compiler no longer knows these are matrix instructions: the wait
// states between a matrix instruction writing ordinary registers and the first VALU
// read of them (passes + 3 = 11 issue slots for the 8-pass 32x32x16) are the program's to
// provide -- by the software pipeline's own distances on the fast path, by s_nop on the
// edge path and before the epilogue.
#include <type_traits>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr int BMQ = 64;   // queries per step
constexpr int BNK = 128;  // keys per workgroup (4 blocks of 32)
typedef __fp16 h16x2 __attribute__((ext_vector_type(2)));

// t = a . b            (fresh score tile in ordinary registers)
__device__ __forceinline__ void mma_v0(f32x16& t, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(t) : "v"(a), "v"(b));
}
// t += a . b           (score tile, ordinary registers)
__device__ __forceinline__ void mma_v(f32x16& t, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(t) : "v"(a), "v"(b));
}
// acc += a . b         (dV^T / dK^T accumulator, accumulation registers)
__device__ __forceinline__ void mma_a(f32x16& acc, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// wait states for a matrix result in ordinary registers before the VALU may read it
__device__ __forceinline__ void mma_settle() { asm volatile("s_nop 7\n\ts_nop 7" ::: "memory"); }

template <bool F32>
__device__ inline void store4g(void* base, int64_t idx, float x0, float x1, float x2, float x3) {
    if (F32) {
        f32x4 v = {x0, x1, x2, x3};
        *reinterpret_cast<f32x4*>(static_cast<float*>(base) + idx) = v;
    } else {
        u32x2 v = {pack_bf16(x0, x1), pack_bf16(x2, x3)};
        *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(base) + idx) = v;
    }
}

template <int D, bool GF32>
__global__ __launch_bounds__(256, 1) void mfma_dkdv3(AttnArgs a) {
    constexpr int KK = D / 16, DB = D / 32;
    constexpr int S = D + 8;            // tile row pitch (elements): 16-byte row reads conflict-free
    constexpr int NCH = D / 8;          // 16-byte chunks per row
    constexpr int CPT = BMQ * NCH / 256;  // chunks per thread per tensor per step
    __shared__ __attribute__((aligned(16))) uint16_t Qs[3][BMQ * S];
    __shared__ __attribute__((aligned(16))) uint16_t dOs[3][BMQ * S];
    __shared__ __attribute__((aligned(16))) uint16_t Pbuf[2][2][4][64 * 16];  // [step parity][query block][key block][lane][16]
    __shared__ __attribute__((aligned(16))) float nlse_s[3][BMQ];            // -LSE * log2(e)
    __shared__ __attribute__((aligned(16))) float dl_s[3][BMQ];

    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int role = w >> 1, khalf = w & 1;
    const int g = lane >> 5, c32 = lane & 31;
    const int nkb = (a.T + BNK - 1) / BNK, rep = a.Hq / a.Hkv;
    // Full-causal: key block i is seen by T - 128i queries; blocks i and nkb-1-i
    // are taken back to back so that every workgroup carries the same work.
    const bool paired = a.causal && a.window == 0;
    int blk, rr, kvu;
    if (a.window > 0 && a.sinks > 0 && nkb > 1) {
        if (!xcd_map_block0_first(nkb, a.Hkv * a.B, blk, kvu)) return;
    } else if (!xcd_map(paired ? (nkb + 1) / 2 : nkb, 1, a.Hkv * a.B, blk, rr, kvu)) {
        return;
    }
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv;
    const float cexp = a.scale * LOG2E;
    const int npass = (paired && blk != nkb - 1 - blk) ? 2 : 1;

    for (int pass = 0; pass < npass; ++pass) {
        const int kblk = pass == 0 ? blk : nkb - 1 - blk;  // heavy block first
        const int k0 = kblk * BNK;
        const int kw0 = k0 + khalf * 64;  // this wavefront's 64 keys: sub-blocks kw0 + 32*kb
        const int kj0 = kw0 + c32;

        // The wavefront's resident operands: K for role 0, V for role 1 (B operand,
        // lane = key, chunk kk covers d = 16kk + 8g .. +7), one set per 32-key sub-block.
        // Keys past the end re-read the last row; their P is masked to zero and nothing is stored.
        bf16x8 kv[2][KK];
        {
            const void* src = role == 0 ? a.k : a.v;
            const int64_t off = role == 0 ? b * a.k_sb + hk * a.k_sh : b * a.v_sb + hk * a.v_sh;
            const int64_t st = role == 0 ? a.k_st : a.v_st;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const int t = min(kj0 + 32 * kb, a.T - 1);
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) {
                    const u32x4 z = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(src) + off + t * st +
                                                                    kk * 16 + g * 8);
                    kv[kb][kk] = *reinterpret_cast<const bf16x8*>(&z);
                }
            }
        }
        const KeyVis kvis[2] = {KeyVis(kj0, a.T, a.causal, a.window, a.sinks),
                                KeyVis(kj0 + 32, a.T, a.causal, a.window, a.sinks)};

        // Query tiles that can see keys [k0, k0+127] (paperkiln src/ops.cpp:960-965 inverted).
        const int khi = min(k0 + BNK, a.T) - 1;
        const int qt_lo = a.causal ? k0 / BMQ : 0;
        const int qt_hi = (a.window > 0 && k0 >= a.sinks) ? min(a.T - 1, khi + a.window - 1) / BMQ : (a.T - 1) / BMQ;
        const int nqt = qt_hi - qt_lo + 1;
        const int steps = nqt * rep;

        u32x4 qr[CPT], gr[CPT];
        // Staging is all this wavefront's own time (nobody shares its SIMD), so it is kept to the loads and stores
        // themselves: a thread's position inside a tile is fixed (row tid / 16 + 16 i, chunk tid % 16), its byte
        // offsets are formed once, the tile's position is a scalar base, and the (head, query tile) of the next
        // fetch is counted up instead of divided out.
        const int frow = static_cast<int>(threadIdx.x) / NCH, fch = static_cast<int>(threadIdx.x) % NCH;
        const uint32_t q_st2 = static_cast<uint32_t>(a.q_st) * 2u, do_st2 = static_cast<uint32_t>(a.do_st) * 2u;
        const uint32_t fch16 = static_cast<uint32_t>(fch) * 16u;
        const int lds_off = frow * S + fch * 8;
        constexpr int RPI = 256 / NCH;  // tile rows between a thread's consecutive chunks
        // byte offsets of this thread's chunks inside a tile; a row past the end of the sequence is clamped to
        // the last one by clamping the offset (offsets grow with the row: the chunk offset is below the pitch)
        uint32_t offq[CPT], offg[CPT];
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            offq[i] = static_cast<uint32_t>(frow + RPI * i) * q_st2 + fch16;
            offg[i] = static_cast<uint32_t>(frow + RPI * i) * do_st2 + fch16;
        }
        int f_h = 0, f_qt = 0;  // head inside the group and query tile of the next fetch
        // A tile is fetched and committed in CPT pieces (one 16-byte chunk of Q and one of dO per thread each), so
        // that the step loop can drop one piece into the shadow of a matrix instruction. The pieces have no
        // branch: rows past the end of the sequence re-read the last row (their P is masked to zero), a fetch
        // past the last step re-reads the last tile, and a commit past it fills a slot nobody reads.
        const char *f_qb = nullptr, *f_gb = nullptr;  // scalar bases of the tile being fetched
        uint32_t f_limq = 0, f_limg = 0;              // offsets of this thread's chunk in the last row that exists
        // per-row scalars: wavefronts 0 and 1 carry LSE of rows 32w + lane (lanes 0-31), wavefronts 2 and 3 delta
        const float* const r_arr = w < 2 ? a.lse : a.delta;
        const float r_mul = w < 2 ? -LOG2E : 1.0f;
        const int rrow = (w & 1) * 32 + (lane & 31);
        const float* f_rb = nullptr;  // row 0 of the tile in that array
        uint32_t f_roff = 0;
        float row_r = 0.0f;
        auto fetch_setup = [&]() {  // steps are fetched in order
            const int h = hk * rep + f_h, q0 = (qt_lo + f_qt) * BMQ;
            if (f_qt + 1 < nqt)
                ++f_qt;
            else if (f_h + 1 < rep)
                f_qt = 0, ++f_h;
            const int last = min(BMQ - 1, a.T - 1 - q0);
            f_limq = static_cast<uint32_t>(last) * q_st2 + fch16;
            f_limg = static_cast<uint32_t>(last) * do_st2 + fch16;
            f_roff = static_cast<uint32_t>(min(rrow, last)) * 4u;
            f_qb = reinterpret_cast<const char*>(a.q) + (b * a.q_sb + h * a.q_sh + q0 * a.q_st) * 2;
            f_gb = reinterpret_cast<const char*>(a.d_o) + (b * a.do_sb + h * a.do_sh + q0 * a.do_st) * 2;
            f_rb = r_arr + ((static_cast<int64_t>(b) * a.Hq + h) * a.T + q0);
        };
        auto fetch_q = [&](int i) {  // global -> registers
            qr[i] = *reinterpret_cast<const u32x4*>(f_qb + min(offq[i], f_limq));
            // scaled when it is stored: arithmetic on it here would wait for every load just issued
            if (i == 0 && lane < 32) row_r = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(f_rb) + f_roff);
        };
        auto fetch_g = [&](int i) {
            gr[i] = *reinterpret_cast<const u32x4*>(f_gb + min(offg[i], f_limg));
        };
        auto fetch_piece = [&](int i) {
            fetch_q(i);
            fetch_g(i);
        };
        auto commit_piece = [&](int slot, int i) {  // registers -> LDS ring slot
            *reinterpret_cast<u32x4*>(Qs[slot] + lds_off + i * RPI * S) = qr[i];
            *reinterpret_cast<u32x4*>(dOs[slot] + lds_off + i * RPI * S) = gr[i];
            if (i == 0 && lane < 32) (w < 2 ? nlse_s[slot] : dl_s[slot])[rrow] = row_r * r_mul;
        };
        auto fetch = [&]() {
            fetch_setup();
#pragma unroll
            for (int i = 0; i < CPT; ++i) fetch_piece(i);
        };
        auto commit = [&](int slot) {
#pragma unroll
            for (int i = 0; i < CPT; ++i) commit_piece(slot, i);
        };
        fetch();
        commit(0);
        fetch();
        // every load issued so far (the resident K / V rows above all) has landed: otherwise the wait-count
        // bookkeeping carries "kv may be in flight" around the loop and makes each step wait for its own prefetch
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();

        // Everything from here to the stores is instantiated once per role and entered through ONE branch on the
        // role: inside the step loop no instruction depends on which role a wavefront plays, so the loop has no
        // branch but the rare ones (a step to skip, a block on the diagonal). A taken branch costs a wavefront that
        // has its SIMD to itself the whole instruction-fetch bubble; two per slot were a quarter of the run time.
        // The accumulators are defined, used and stored inside one instantiation, so they never meet at a join.
        auto run_role = [&](auto role_tag) {
        constexpr int rl = decltype(role_tag)::value;
        f32x16 acc[2][DB];  // dV^T (role 0) or dK^T (role 1) of the two sub-blocks
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[kb][db][r] = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int db = 0; db < DB; ++db) asm volatile("" : "+a"(acc[kb][db]));
        // iteration s: role 0 works on step s, role 1 on step s-1.
        //
        // Every kind of step (interior, diagonal, ragged) runs the same sequence of matrix instructions: masked
        // positions are computed and then zeroed, and a 32 x 64 block that is wholly invisible inside a live
        // step costs its matrix instructions (about 3 % of a causal pass). With two different sequences on
        // the two sides of a branch the register allocator gives each side its own copy of all 128
        // accumulators and moves them back at the join, every iteration; a branch that merely skips the one
        // sequence is harmless.
        //
        // One wavefront per SIMD has nobody to hide its elementwise work behind, so the two 32-query blocks of a
        // step are software-pipelined against each other, one slice of VALU work in the shadow of each matrix
        // instruction:
        //   phase 1  GEMM1(block 0)
        //   phase 2  GEMM1(block 1)  ||  elementwise(block 0)
        //   phase 3  GEMM2(block 0)  ||  elementwise(block 1)
        //   phase 4  GEMM2(block 1)
        //
        // Staging for the coming steps rides in phase 4: in iteration s the tile of step s+1 goes from registers to
        // its ring slot (last read, by role 1, before the previous barrier) and the tile of step s+2 from memory to
        // registers. Role 1 idles in iteration 0 and does that staging in one go; role 0 idles in the last
        // iteration, where nothing is left to stage. Both roles meet the same number of barriers.
        if (rl == 1) {
            commit(1);
            fetch();
            __syncthreads();
        }
        for (int stp = 0; stp < steps; ++stp) {
            const int cslot = (stp + rl + 1) % 3;
            {
  // role 1 runs one step behind
                const int qbase = (qt_lo + stp % nqt) * BMQ;
                bool full[2];
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    const int qlo = qbase + qb * 32, qhi = qlo + 31;
                    full[qb] = qhi < a.T && kw0 + 63 < a.T && (!a.causal || kw0 + 63 <= qlo);
                }
                constexpr int PF = 3, NS = 2 * KK;  // fragments in flight; slots (= MFMAs) per GEMM
                const int slot3 = stp % 3;
                const uint16_t* X = (rl == 0 ? Qs[slot3] : dOs[slot3]) + c32 * S + g * 8;  // GEMM1 rows
                const uint16_t* Y = rl == 0 ? dOs[slot3] : Qs[slot3];                       // GEMM2, transposed
                const float* rowc = (rl == 0 ? nlse_s[slot3] : dl_s[slot3]) + g * 4;
                auto xfrag = [&](int qb, int j) { return lds_read8(X + qb * 32 * S + j * 16); };
                auto yfrag = [&](int qb, int j) {
                    return lds_read_tr_operand_perm<D>(Y, S, qb * 32 + (j / DB) * 16, j % DB, lane);
                };
                f32x16 t0[2], t1[2];          // S or dP of query block 0 / 1, [sub-block], as the matrix pipe leaves them
                // The elementwise results live in scalars of their own: written back into the 16-register tuples
                // under the role branch they would make every slot copy whole tuples at the join.
                float e0[2][16], e1[2][16];   // P or dS of query block 0 / 1
                bf16x8 op0[2][2], op1[2][2];  // packed P or dS, [sub-block][16-query half]
                f32x4 rc[4];                  // per-row constants of the block being worked on
                u32x4 pr[2][2];               // role 1: P handed over, [sub-block][half]
                bf16x8 fr[NS / 2 + PF];       // fragment window of the running GEMM
                // elementwise work on elements [lo, hi) of a query block: sub-block e/16, register e%16
                auto elems = [&](const f32x16(&t)[2], float(&y)[2][16], int lo, int hi) {
                    if (rl == 0) {
#pragma unroll
                        for (int e = lo; e < hi; ++e) {
                            const int kb = e >> 4, r = e & 15;
                            y[kb][r] = __builtin_amdgcn_exp2f(fmaf(t[kb][r], cexp, rc[r >> 2][r & 3]));
                        }
                    } else {
#pragma unroll
                        for (int e = lo; e < hi; ++e) {
                            const int kb = e >> 4, r = e & 15;
                            const h16x2* ph = reinterpret_cast<const h16x2*>(&pr[kb][0]);
                            y[kb][r] = static_cast<float>(ph[r >> 1][r & 1]) * (t[kb][r] - rc[r >> 2][r & 3]);
                        }
                    }
                };
                auto side_loads = [&](int qb) {
#pragma unroll
                    for (int qd = 0; qd < 4; ++qd) rc[qd] = *reinterpret_cast<const f32x4*>(rowc + qb * 32 + qd * 8);
                    if (rl == 1) {
#pragma unroll
                        for (int kb = 0; kb < 2; ++kb) {
                            const uint16_t* pb = Pbuf[stp & 1][qb][khalf * 2 + kb] + lane * 16;
                            pr[kb][0] = *reinterpret_cast<const u32x4*>(pb);
                            pr[kb][1] = *reinterpret_cast<const u32x4*>(pb + 8);
                        }
                    }
                };
                auto pack8 = [&](const float(&y)[16], int h) {
                    u32x4 u = {pack_bf16(y[8 * h + 0], y[8 * h + 1]), pack_bf16(y[8 * h + 2], y[8 * h + 3]),
                               pack_bf16(y[8 * h + 4], y[8 * h + 5]), pack_bf16(y[8 * h + 6], y[8 * h + 7])};
                    return *reinterpret_cast<bf16x8*>(&u);
                };
                auto finish = [&](int qb, float(&y)[2][16], bf16x8(&op)[2][2]) {
                    if (rl == 0 && !full[qb]) {  // diagonal / ragged block: zero what the mask hides (role 1 inherits the zeros)
                        const int qlo = qbase + qb * 32;
#pragma unroll
                        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                y[kb][r] = kvis[kb](qlo + (r >> 2) * 8 + g * 4 + (r & 3)) ? y[kb][r] : 0.0f;
                    }
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) {
                        op[kb][0] = pack8(y[kb], 0);
                        op[kb][1] = pack8(y[kb], 1);
                    }
                    if (rl == 0) {  // hand P over in fp16 (11 significant bits in [0, 1])
#pragma unroll
                        for (int kb = 0; kb < 2; ++kb) {
                            uint16_t* pb = Pbuf[stp & 1][qb][khalf * 2 + kb] + lane * 16;
                            h16x2 ph[8];
#pragma unroll
                            for (int i = 0; i < 8; ++i) {
                                const f32x2 p2 = {y[kb][2 * i], y[kb][2 * i + 1]};
                                ph[i] = __builtin_convertvector(p2, h16x2);
                            }
                            *reinterpret_cast<u32x4*>(pb) = *reinterpret_cast<u32x4*>(&ph[0]);
                            *reinterpret_cast<u32x4*>(pb + 8) = *reinterpret_cast<u32x4*>(&ph[4]);
                        }
                    }
                };
                // staging piece p rides in phase p+1, the two roles in different slots: a wavefront whose load finds
                // the address unit's queue full stalls, matrix instructions and all, so the loads are spread thin
                static_assert(CPT == 4 && NS >= 14, "one staging piece per phase");
                auto stage = [&](int piece, int sl) {
                    constexpr int first = rl * 8;
                    if (sl == first + 1) commit_piece(cslot, piece);
                    if (sl == first + 3) fetch_q(piece);
                    if (sl == first + 5) fetch_g(piece);
                };
                fetch_setup();
                // ---- phase 1: GEMM1(block 0)
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = xfrag(0, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    if (j == 0)
                        mma_v0(t0[kb], fr[j], kv[kb][j]);
                    else
                        mma_v(t0[kb], fr[j], kv[kb][j]);
                    if (kb == 0 && j + PF < KK) fr[j + PF] = xfrag(0, j + PF);
                    stage(0, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // ---- phase 2: GEMM1(block 1) || elementwise(block 0)
                side_loads(0);
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = xfrag(1, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    if (j == 0)
                        mma_v0(t1[kb], fr[j], kv[kb][j]);
                    else
                        mma_v(t1[kb], fr[j], kv[kb][j]);
                    if (kb == 0 && j + PF < KK) fr[j + PF] = xfrag(1, j + PF);
                    // t0[0] was finished two matrix instructions before the first slot, t0[1] one before: the
                    // first half of the slots works on t0[0] only
                    elems(t0, e0, sl * 32 / NS, (sl + 1) * 32 / NS);
                    stage(1, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
                finish(0, e0, op0);
                // ---- phase 3: GEMM2(block 0) || elementwise(block 1)
                side_loads(1);
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = yfrag(0, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    mma_a(acc[kb][j % DB], fr[j], op0[kb][j / DB]);
                    if (kb == 0 && j + PF < 2 * DB) fr[j + PF] = yfrag(0, j + PF);
                    elems(t1, e1, sl * 32 / NS, (sl + 1) * 32 / NS);
                    stage(2, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
                finish(1, e1, op1);
                // ---- phase 4: GEMM2(block 1) || staging, one piece per matrix instruction
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = yfrag(1, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    mma_a(acc[kb][j % DB], fr[j], op1[kb][j / DB]);
                    if (kb == 0 && j + PF < 2 * DB) fr[j + PF] = yfrag(1, j + PF);
                    stage(3, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __syncthreads();
        }
        if (rl == 0) __syncthreads();

        // the last matrix instructions may still be writing the accumulators
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int db = 0; db < DB; ++db) asm volatile("" : "+a"(acc[kb][db]));
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const int kj = kj0 + 32 * kb;
            if (kj >= a.T) continue;
            void* dst = rl == 0 ? a.dv : a.dk;
            const int64_t ob = rl == 0 ? b * a.dv_sb + hk * a.dv_sh + kj * a.dv_st
                                       : b * a.dk_sb + hk * a.dk_sh + kj * a.dk_st;
            const float sc = rl == 0 ? 1.0f : a.scale;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int qd = 0; qd < 4; ++qd)
                    store4g<GF32>(dst, ob + TrMap<D>::col0(db, qd, g), acc[kb][db][qd * 4] * sc, acc[kb][db][qd * 4 + 1] * sc,
                                  acc[kb][db][qd * 4 + 2] * sc, acc[kb][db][qd * 4 + 3] * sc);
        }
        };  // run_role
        if (role == 0)
            run_role(std::integral_constant<int, 0>{});
        else
            run_role(std::integral_constant<int, 1>{});
        __syncthreads();  // the next pass refills the ring
    }
}

template <int D, bool GF32>
int launch(const AttnArgs& a, hipStream_t st) {
    const int nb128 = (a.T + 127) / 128;
    const bool paired = a.causal && a.window == 0;
    hipLaunchKernelGGL((mfma_dkdv3<D, GF32>), dim3(xcd_grid(paired ? (nb128 + 1) / 2 : nb128, 1, a.Hkv * a.B)),
                       dim3(256), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

}  // namespace

bool mfma_dkdv3_takes(const AttnArgs& a) {
    // a thread's byte offset inside a 64-row tile of Q / dO is kept in 32 bits
    const int64_t reach = 2 * BMQ * (a.q_st > a.do_st ? a.q_st : a.do_st);
    return a.dk_dim == 128 && a.window == 0 && reach < (int64_t{1} << 31);
}

int launch_mfma_dkdv3(const AttnArgs& a, hipStream_t st) {
    return a.grad_f32 ? launch<128, true>(a, st) : launch<128, false>(a, st);
}

}  // namespace pk
