// dK / dV of the recompute backward, third generation (see attn_bwd_mfma.hip for
// the mathematics and the operand layouts, attn_bwd_dkdv2.hip for the role split).
//
// The LDS hands a CU 128 bytes per clock: one 1 KB operand fragment per 32 clocks
// per SIMD, the issue rate of the 32x32x16 MFMA. A wavefront that owns 32 keys
// feeds every fragment it reads to ONE matrix instruction, so the LDS is as busy
// as the matrix pipe and neither passes half. Here a wavefront owns 64 keys: two
// resident operand sets (K or V of two 32-key blocks), two accumulator sets, and
// every Q / dO fragment read from the LDS feeds TWO matrix instructions. That is
// 192 persistent registers at head_dim 128 (96 at 64), so one wavefront per SIMD, four per workgroup:
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
// provide -- by the software pipeline's own distances inside the loop (a phase of matrix
// instructions lies between a score tile and its first reader) and by s_nop before the
// epilogue. Likewise a matrix instruction must not read, as A or B, a register that the
// vector instruction just before it wrote: it would see the old contents. Both distances
// are checked on the compiled assembly by tests/test_asm_hazards.py.
//
// What a wavefront that has its SIMD to itself pays for (measured with a stream of
// independent matrix instructions and N other instructions between each pair): the matrix
// instruction occupies the pipe for 32 clocks and the issue port for about 8; an ordinary
// vector instruction takes about 5 clocks of issue (8 when it reads the result of the one
// before, 8.6 for v_exp_f32), a scalar one about the same. So a matrix instruction hides
// five vector instructions and not one more, and nothing here is free: the loop below is
// written to issue as few instructions as possible. LDS addresses are a per-lane register
// plus an immediate, positions in memory are pointers that are advanced rather than
// recomputed, -delta enters the dP tile as the matrix instruction's own C operand, and
// what must run between two phases is kept to the eight pack instructions the next phase
// needs at once. LDS reads, LDS writes and global loads cost their issue slot and no more
// when the matrix pipe is the bound (one per four matrix instructions measured free).
#include <cstdlib>
#include <type_traits>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr int BMQ = 64;   // queries per step
constexpr int BNK = 128;  // keys per workgroup (4 blocks of 32)
typedef __fp16 h16x2 __attribute__((ext_vector_type(2)));
// typed LDS pointer from a 32-bit LDS byte address
#define LDSP(T, addr) (reinterpret_cast<PK_LDS T*>(static_cast<uintptr_t>(addr)))

// t = a . b            (fresh score tile in ordinary registers)
__device__ __forceinline__ void mma_v0(f32x16& t, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(t) : "v"(a), "v"(b));
}
// t = a . b + c        (fresh score tile started from a tile of constants)
__device__ __forceinline__ void mma_vc(f32x16& t, bf16x8 a, bf16x8 b, const f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(t) : "v"(a), "v"(b), "v"(c));
}
// t += a . b           (score tile, ordinary registers)
__device__ __forceinline__ void mma_v(f32x16& t, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(t) : "v"(a), "v"(b));
}
// acc += a . b         (dV^T / dK^T accumulator, accumulation registers)
__device__ __forceinline__ void mma_a(f32x16& acc, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

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
    // Threads that stage tiles: the two wavefronts of role 1. Role 0 carries the exponentials and is the longer
    // of the two; with all four wavefronts staging (NSTG = 256) the step is 4 % slower.
    constexpr int NSTG = 128;
    constexpr int CPT = BMQ * NCH / NSTG;  // chunks per staging thread per tensor per step
    __shared__ __attribute__((aligned(16))) uint16_t Qs[3][BMQ * S];
    __shared__ __attribute__((aligned(16))) uint16_t dOs[3][BMQ * S];
    __shared__ __attribute__((aligned(16))) uint16_t Pbuf[2][2][4][64 * 16];  // [step parity][query block][key block][half][lane][8]
    __shared__ __attribute__((aligned(16))) float nlse_s[3][BMQ];            // -LSE * log2(e)
    __shared__ __attribute__((aligned(16))) float dl_s[3][BMQ];

    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int role = w >> 1, khalf = w & 1;
    const int g = lane >> 5, c32 = lane & 31;
    const int nkb = (a.T + BNK - 1) / BNK, rep = a.Hq / a.Hkv;
    // Full-causal: key block i is seen by T - 128i queries; blocks i and nkb-1-i
    // are taken back to back so that every workgroup carries the same work.
    const bool paired = a.causal && a.window == 0;
    // hs > 1: the query heads of the group are dealt to hs workgroups (gqa_head_split); this one takes heads
    // [hfirst, hfirst + nh) of the group and leaves fp32 partial sums for launch_gqa_reduce
    const int hs = a.head_split;
    int blk, rr = 0, kvu;
    if (a.window > 0 && a.sinks > 0 && nkb > 1) {
        if (!xcd_map_block0_first(nkb, a.Hkv * a.B, blk, kvu)) return;
    } else if (!xcd_map(paired ? (nkb + 1) / 2 : nkb, hs, a.Hkv * a.B, blk, rr, kvu)) {
        return;
    }
    const int hfirst = rr * rep / hs, nh = (rr + 1) * rep / hs - hfirst;
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
        const int steps = nqt * nh;

        u32x4 qr[CPT], gr[CPT];
        // Staging is all this wavefront's own time (nobody shares its SIMD), so it is kept to the loads and stores
        // themselves: a thread's position inside a tile is fixed (row tid / 16 + 16 i, chunk tid % 16), its byte
        // offsets are formed once, the tile's position is a scalar base, and the (head, query tile) of the next
        // fetch is counted up instead of divided out.
        const int stid = static_cast<int>(threadIdx.x) - (256 - NSTG);  // negative: this thread stages nothing
        const int frow = stid / NCH, fch = stid % NCH;
        const uint32_t q_st2 = static_cast<uint32_t>(a.q_st) * 2u, do_st2 = static_cast<uint32_t>(a.do_st) * 2u;
        const uint32_t fch16 = static_cast<uint32_t>(fch) * 16u;
        const int lds_off = lds_row<D>(frow) * S + fch * 8;  // rows frow + RPI i: RPI is 8 (head_dim 128, natural order) or 16 (a whole row group)
        constexpr int RPI = NSTG / NCH;  // tile rows between a thread's consecutive chunks
        // byte offsets of this thread's chunks inside a tile; a row past the end of the sequence is clamped to
        // the last one by clamping the offset (offsets grow with the row: the chunk offset is below the pitch)
        uint32_t offq[CPT], offg[CPT];
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            offq[i] = static_cast<uint32_t>(frow + RPI * i) * q_st2 + fch16;
            offg[i] = static_cast<uint32_t>(frow + RPI * i) * do_st2 + fch16;
        }
        // A tile is fetched and committed in CPT pieces (one 16-byte chunk of Q and one of dO per thread each), so
        // that the step loop can drop one piece into the shadow of a matrix instruction. The pieces have no
        // branch: rows past the end of the sequence re-read the last row (their P is masked to zero), a fetch
        // past the last step re-reads the last tile, and a commit past it fills a slot nobody reads.
        //
        // The position of the next fetch is kept as pointers that are advanced, not recomputed: one wavefront
        // per SIMD issues every instruction of its own, scalar ones included, at about five clocks each.
        int f_h = 0, f_qt = 0;       // head inside the group and query tile of the next fetch
        int f_q0 = qt_lo * BMQ;      // first query row of that tile
        const int h0 = hk * rep + hfirst;
        const char* f_qb = reinterpret_cast<const char*>(a.q) + (b * a.q_sb + h0 * a.q_sh + f_q0 * a.q_st) * 2;
        const char* f_gb = reinterpret_cast<const char*>(a.d_o) + (b * a.do_sb + h0 * a.do_sh + f_q0 * a.do_st) * 2;
        // per-row scalars: wavefronts 0 and 1 carry LSE of rows 32w + lane (lanes 0-31), wavefronts 2 and 3 delta
        // (with role 1 alone staging: wavefront 2 all of LSE, wavefront 3 all of delta)
        const bool r_lse = NSTG == 256 ? w < 2 : w == 2;
        const int r_lanes = NSTG == 256 ? 32 : 64;
        const float* const r_arr = r_lse ? a.lse : a.delta;
        const float r_mul = r_lse ? -LOG2E : -1.0f;  // what the LDS holds: -LSE log2(e) and -delta
        const int rrow = NSTG == 256 ? (w & 1) * 32 + (lane & 31) : lane;
        const char* f_rb = reinterpret_cast<const char*>(r_arr + ((static_cast<int64_t>(b) * a.Hq + h0) * a.T + f_q0));
        // steps from one tile to the next: inside a head, and from the last tile of a head to the first of the next
        const int64_t qd_tile = BMQ * a.q_st * 2, qd_head = a.q_sh * 2 - (nqt - 1) * qd_tile;
        const int64_t gd_tile = BMQ * a.do_st * 2, gd_head = a.do_sh * 2 - (nqt - 1) * gd_tile;
        const int64_t rd_tile = BMQ * 4, rd_head = static_cast<int64_t>(a.T) * 4 - (nqt - 1) * rd_tile;
        uint32_t f_limq = 0, f_limg = 0;  // offsets of this thread's chunk in the last row that exists
        uint32_t f_roff = 0;
        float row_r = 0.0f;
        const char *c_qb = f_qb, *c_gb = f_gb, *c_rb = f_rb;  // the tile being fetched
        auto fetch_setup = [&]() {  // steps are fetched in order
            c_qb = f_qb, c_gb = f_gb, c_rb = f_rb;
            const int last = min(BMQ - 1, a.T - 1 - f_q0);
            f_limq = static_cast<uint32_t>(last) * q_st2 + fch16;
            f_limg = static_cast<uint32_t>(last) * do_st2 + fch16;
            f_roff = static_cast<uint32_t>(min(rrow, last)) * 4u;
            // masks instead of selects: a nested select becomes a branch, and a taken branch costs the most of all
            const int64_t in_head = -static_cast<int64_t>(f_qt + 1 < nqt);
            const int64_t next_head = ~in_head & -static_cast<int64_t>(f_h + 1 < nh);
            f_qb += (qd_tile & in_head) | (qd_head & next_head);
            f_gb += (gd_tile & in_head) | (gd_head & next_head);
            f_rb += (rd_tile & in_head) | (rd_head & next_head);
            f_q0 += (BMQ & static_cast<int>(in_head)) | (-(nqt - 1) * BMQ & static_cast<int>(next_head));
            f_qt = (f_qt + 1) & static_cast<int>(in_head) | f_qt & static_cast<int>(~(in_head | next_head));
            f_h -= static_cast<int>(next_head);
        };
        auto fetch_q = [&](int i) {  // global -> registers
            qr[i] = *reinterpret_cast<const u32x4*>(c_qb + min(offq[i], f_limq));
            // scaled when it is stored: arithmetic on it here would wait for every load just issued
            if (i == 0 && lane < r_lanes) row_r = *reinterpret_cast<const float*>(c_rb + f_roff);
        };
        auto fetch_g = [&](int i) {
            gr[i] = *reinterpret_cast<const u32x4*>(c_gb + min(offg[i], f_limg));
        };
        auto fetch_piece = [&](int i) {
            fetch_q(i);
            fetch_g(i);
        };
        auto commit_piece = [&](int slot, int i) {  // registers -> LDS ring slot
            *reinterpret_cast<u32x4*>(Qs[slot] + lds_off + i * RPI * S) = qr[i];
            *reinterpret_cast<u32x4*>(dOs[slot] + lds_off + i * RPI * S) = gr[i];
            if (i == 0 && lane < r_lanes) (r_lse ? nlse_s[slot] : dl_s[slot])[rrow] = row_r * r_mul;
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
        if (NSTG == 256 || role == 1) {
            fetch();
            commit(0);
            fetch();
        }
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
        // LDS positions as 32-bit byte addresses: a lane's own part is formed once, the ring slot is added once a
        // step, and every read below is that register plus a constant the instruction carries.
        auto lds32 = [](const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); };
        constexpr uint32_t SLOTB = BMQ * S * 2;
        const uint32_t x_slot0 = lds32(rl == 0 ? Qs[0] : dOs[0]), y_slot0 = lds32(rl == 0 ? dOs[0] : Qs[0]);
        const uint32_t x_lane = static_cast<uint32_t>(lds_row<D>(c32) * S + g * 8) * 2u;  // GEMM1: row c32, 8 elements from 8g
        const int tj = lane & 15, tu = (lane >> 4) & 1;
        const uint32_t y_lane = static_cast<uint32_t>(lds_row<D>(4 * g + (tj >> 2)) * S + TrMap<D>::src_col(0, tu, tj & 3)) * 2u;
        const uint32_t rc_lane = lds32(rl == 0 ? nlse_s[0] : dl_s[0]) + g * 16u;
        const uint32_t p_lane = lds32(Pbuf) + khalf * 2u * 2048u + lane * 16u;  // [parity][qb][khalf*2+kb][half][lane][8]
        int c_qt = 0, slot3 = 0, cslot = (rl + 1) % 3;  // query tile of this step, its ring slot, the slot staged into
        for (int stp = 0; stp < steps; ++stp) {
            {
                const int qbase = (qt_lo + c_qt) * BMQ;
                bool full[2];
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    const int qlo = qbase + qb * 32, qhi = qlo + 31;
                    full[qb] = qhi < a.T && kw0 + 63 < a.T && (!a.causal || kw0 + 63 <= qlo) &&
                               (a.window == 0 || qhi < kw0 + a.window);  // the band's far edge is tightest for key kw0
                }
                constexpr int PF = 3, NS = 2 * KK;  // fragments in flight; slots (= MFMAs) per GEMM
                const uint32_t xa = x_slot0 + slot3 * SLOTB + x_lane;
                const uint32_t ya = y_slot0 + slot3 * SLOTB + y_lane;
                const uint32_t rca = rc_lane + slot3 * (BMQ * 4u);
                const uint32_t pa = p_lane + (stp & 1) * (2u * 4u * 2048u);
                auto xfrag = [&](int qb, int j) { return *LDSP(const bf16x8, xa + (qb * 32 * S + j * 16) * 2); };
                auto yfrag = [&](int qb, int j) {
                    const uint32_t at = ya + ((qb * 32 + (j / DB) * 16) * S + TrMap<D>::src_col(j % DB, 0, 0) - TrMap<D>::src_col(0, 0, 0)) * 2;
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, at));
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, at + TR_HI_ROWS<D> * S * 2));
                    typedef short s16x8 __attribute__((ext_vector_type(8)));
                    const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    return *reinterpret_cast<const bf16x8*>(&v);
                };
                f32x16 t0[2], t1[2];          // S or dP of query block 0 / 1, [sub-block], as the matrix pipe leaves them
                // The elementwise results live in scalars of their own: written back into the 16-register tuples
                // under the role branch they would make every slot copy whole tuples at the join.
                float e0[2][16], e1[2][16];   // P or dS of query block 0 / 1
                bf16x8 op0[2][2], op1[2][2];  // packed P or dS, [sub-block][16-query half]
                f32x4 rc[2][4];               // role 0: -LSE log2(e) of the rows of query block 0 / 1
                f32x16 nd0, nd1;              // role 1: -delta of the rows of query block 0 / 1, laid out like a score tile
                u32x4 pr[2][2][2];            // role 1: P handed over, [query block][sub-block][half]
                bf16x8 fr[NS / 2 + PF];       // fragment window of the running GEMM
                // elementwise work on elements [lo, hi) of a query block: sub-block e/16, register e%16
                auto elems = [&](int qb, const f32x16(&t)[2], float(&y)[2][16], int lo, int hi) {
                    if (rl == 0) {
#pragma unroll
                        for (int e = lo; e < hi; ++e) {
                            const int kb = e >> 4, r = e & 15;
                            y[kb][r] = __builtin_amdgcn_exp2f(fmaf(t[kb][r], cexp, rc[qb][r >> 2][r & 3]));
                        }
                    } else {
#pragma unroll
                        for (int e = lo; e < hi; ++e) {
                            const int kb = e >> 4, r = e & 15;
                            // dS = P (dP - delta): t holds dP - delta already, P is one half of a packed fp16 pair and
                            // is widened by the instruction itself
                            const uint32_t pw = pr[qb][kb][r >> 3][(r >> 1) & 3];
                            if (r & 1)
                                asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(y[kb][r]) : "v"(pw), "v"(t[kb][r]));
                            else
                                asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(y[kb][r]) : "v"(pw), "v"(t[kb][r]));
                        }
                    }
                };
                auto row_consts = [&](int qb, int qd) { return *LDSP(const f32x4, rca + (qb * 32 + qd * 8) * 4); };
                auto minus_delta = [&](int qb) {  // role 1, before GEMM1 of the block: its accumulators start from -delta
                    const f32x4 c0 = row_consts(qb, 0), c1 = row_consts(qb, 1), c2 = row_consts(qb, 2), c3 = row_consts(qb, 3);
                    const f32x16 v = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3],
                                      c2[0], c2[1], c2[2], c2[3], c3[0], c3[1], c3[2], c3[3]};
                    return v;
                };
                // Row constants (role 0) and the P handed over (role 1) of a block are asked for half a phase before the
                // first slot that uses them: asked for at the phase's start, the lone wavefront sits out the LDS latency.
                auto side_loads = [&](int qb) {
                    if (rl == 0) {
#pragma unroll
                        for (int qd = 0; qd < 4; ++qd) rc[qb][qd] = row_consts(qb, qd);
                    } else {
#pragma unroll
                        for (int kb = 0; kb < 2; ++kb) {
                            pr[qb][kb][0] = *LDSP(const u32x4, pa + qb * 8192 + kb * 2048);
                            pr[qb][kb][1] = *LDSP(const u32x4, pa + qb * 8192 + kb * 2048 + 1024);
                        }
                    }
                };
                auto pack8 = [&](const float(&y)[16], int h) {
                    u32x4 u = {pack_bf16(y[8 * h + 0], y[8 * h + 1]), pack_bf16(y[8 * h + 2], y[8 * h + 3]),
                               pack_bf16(y[8 * h + 4], y[8 * h + 5]), pack_bf16(y[8 * h + 6], y[8 * h + 7])};
                    return *reinterpret_cast<bf16x8*>(&u);
                };
                // What follows the elementwise work of a block -- masking on the diagonal, packing to bf16, handing P
                // over -- would leave the matrix pipe idle if it ran between two phases. Only what the next phase
                // needs at once stays there (finish_head: the first k-half of the packed operand); the rest rides in
                // the first slots of that phase (finish_slot).
                auto finish_head = [&](int qb, float(&y)[2][16], bf16x8(&op)[2][2]) {
                    // diagonal / ragged block: zero what the mask hides (role 1 inherits the zeros). Marked unlikely so
                    // that the common case falls through: jumping over the masking code is a taken branch
                    if (__builtin_expect(rl == 0 && !full[qb], 0)) {
                        const int qlo = qbase + qb * 32;
#pragma unroll
                        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                y[kb][r] = kvis[kb](qlo + (r >> 2) * 8 + g * 4 + (r & 3)) ? y[kb][r] : 0.0f;
                    }
                    op[0][0] = pack8(y[0], 0);
                    op[1][0] = pack8(y[1], 0);
                };
                auto finish_slot = [&](int qb, float(&y)[2][16], bf16x8(&op)[2][2], int sl) {
                    if (sl < 2) op[sl][1] = pack8(y[sl], 1);  // first used in slot 8 + sl
                };
                // P goes to role 1 in fp16 (11 significant bits in [0, 1]), a quarter of a block per slot. Both blocks
                // are handed over in phase 4, the phase with the least other work for role 0 (phase 3 carries the
                // exponentials of block 1).
                auto hand_over = [&](int qb, const float(&y)[2][16], int quarter) {
                    const int kb = quarter >> 1, hf = quarter & 1;
                    h16x2 ph[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const f32x2 p2 = {y[kb][8 * hf + 2 * i], y[kb][8 * hf + 2 * i + 1]};
                        ph[i] = __builtin_convertvector(p2, h16x2);
                    }
                    *LDSP(u32x4, pa + qb * 8192 + kb * 2048 + hf * 1024) = *reinterpret_cast<u32x4*>(&ph[0]);
                };
                // staging piece p rides in phase p+1, the two roles in different slots: a wavefront whose load finds
                // the address unit's queue full stalls, matrix instructions and all, so the loads are spread thin
                auto stage = [&](int phase, int sl) {
                    if (NSTG == 256) {
                        constexpr int first = rl * 8;
                        if (sl == first + 1) commit_piece(cslot, phase);
                        if (sl == first + 3) fetch_q(phase);
                        if (sl == first + 5) fetch_g(phase);
                    } else if (rl == 1) {  // two pieces a phase
                        static_assert(CPT == 4 || (CPT == 8 && NS >= 14), "one or two pieces a phase");
                        constexpr int PPP = CPT / 4;  // pieces per phase
                        if (sl == 1) commit_piece(cslot, PPP * phase);
                        if (sl == 3) fetch_q(PPP * phase);
                        if (sl == 5) fetch_g(PPP * phase);
                        if (PPP == 2 && sl == 9) commit_piece(cslot, 2 * phase + 1);
                        if (PPP == 2 && sl == 11) fetch_q(2 * phase + 1);
                        if (PPP == 2 && sl == 13) fetch_g(2 * phase + 1);
                    }
                };
                if (NSTG == 256 || rl == 1) fetch_setup();
                // ---- phase 1: GEMM1(block 0)
                if (rl == 1) nd0 = minus_delta(0);
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = xfrag(0, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    if (j == 0 && rl == 1)
                        mma_vc(t0[kb], fr[j], kv[kb][j], nd0);
                    else if (j == 0)
                        mma_v0(t0[kb], fr[j], kv[kb][j]);
                    else
                        mma_v(t0[kb], fr[j], kv[kb][j]);
                    // The matrix instruction reads its C operand over its passes and nothing interlocks a vector write
                    // to those registers: -delta stays allocated until a further matrix instruction has been issued.
                    if (sl == 2 && rl == 1) asm volatile("" ::"v"(nd0));
                    if (kb == 0 && j + PF < KK) fr[j + PF] = xfrag(0, j + PF);
                    if (sl == NS / 2) side_loads(0);
                    if (sl == NS / 2 + 2 && rl == 1) nd1 = minus_delta(1);
                    stage(0, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // ---- phase 2: GEMM1(block 1) || elementwise(block 0)
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = xfrag(1, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    if (j == 0 && rl == 1)
                        mma_vc(t1[kb], fr[j], kv[kb][j], nd1);
                    else if (j == 0)
                        mma_v0(t1[kb], fr[j], kv[kb][j]);
                    else
                        mma_v(t1[kb], fr[j], kv[kb][j]);
                    if (sl == 2 && rl == 1) asm volatile("" ::"v"(nd1));
                    if (kb == 0 && j + PF < KK) fr[j + PF] = xfrag(1, j + PF);
                    // t0[0] was finished two matrix instructions before the first slot, t0[1] one before: the
                    // first half of the slots works on t0[0] only
                    elems(0, t0, e0, sl * 32 / NS, (sl + 1) * 32 / NS);
                    if (sl == NS / 2) side_loads(1);
                    stage(1, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
                finish_head(0, e0, op0);
                // the packs stay ahead of the fragment reads: a matrix instruction must not directly follow the
                // vector instruction that writes one of its operands
                __builtin_amdgcn_sched_barrier(0);
                // ---- phase 3: GEMM2(block 0) || elementwise(block 1)
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = yfrag(0, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    mma_a(acc[kb][j % DB], fr[j], op0[kb][j / DB]);
                    if (kb == 0 && j + PF < 2 * DB) fr[j + PF] = yfrag(0, j + PF);
                    elems(1, t1, e1, sl * 32 / NS, (sl + 1) * 32 / NS);
                    finish_slot(0, e0, op0, sl);
                    if (rl == 0 && NS < 12 && sl >= 2 && sl < 6) hand_over(0, e0, sl - 2);  // phase 4 is too short to take both
                    stage(2, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
                finish_head(1, e1, op1);
                // the packs stay ahead of the fragment reads: a matrix instruction must not directly follow the
                // vector instruction that writes one of its operands
                __builtin_amdgcn_sched_barrier(0);
                // ---- phase 4: GEMM2(block 1) || staging, one piece per matrix instruction
#pragma unroll
                for (int j = 0; j < PF; ++j) fr[j] = yfrag(1, j);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sl = 0; sl < NS; ++sl) {
                    const int j = sl >> 1, kb = sl & 1;
                    mma_a(acc[kb][j % DB], fr[j], op1[kb][j / DB]);
                    if (kb == 0 && j + PF < 2 * DB) fr[j + PF] = yfrag(1, j + PF);
                    finish_slot(1, e1, op1, sl);
                    if (rl == 0 && sl >= 2 && sl < 6) hand_over(1, e1, sl - 2);
                    if (rl == 0 && NS >= 12 && sl >= 8 && sl < 12) hand_over(0, e0, sl - 8);
                    stage(3, sl);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            c_qt = c_qt + 1 == nqt ? 0 : c_qt + 1;
            slot3 = slot3 == 2 ? 0 : slot3 + 1;
            cslot = cslot == 2 ? 0 : cslot + 1;
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
            const float sc = rl == 0 ? 1.0f : a.scale;
            if (hs > 1) {  // fp32 partial sums of this split, rows of pitch D
                float* prow = a.part + ((static_cast<size_t>(kvu) * hs + rr) * 2 + (rl == 0 ? 1 : 0)) * a.T * D +
                              static_cast<size_t>(kj) * D;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int qd = 0; qd < 4; ++qd)
                        store4g<true>(prow, TrMap<D>::col0(db, qd, g), acc[kb][db][qd * 4] * sc, acc[kb][db][qd * 4 + 1] * sc,
                                      acc[kb][db][qd * 4 + 2] * sc, acc[kb][db][qd * 4 + 3] * sc);
                continue;
            }
            void* dst = rl == 0 ? a.dv : a.dk;
            const int64_t ob = rl == 0 ? b * a.dv_sb + hk * a.dv_sh + kj * a.dv_st
                                       : b * a.dk_sb + hk * a.dk_sh + kj * a.dk_st;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (!GF32) {
                    store_acc_bf16<D>(static_cast<uint16_t*>(dst) + ob, db, g, acc[kb][db], sc);
                    continue;
                }
#pragma unroll
                for (int qd = 0; qd < 4; ++qd)
                    store4g<GF32>(dst, ob + TrMap<D>::col0(db, qd, g), acc[kb][db][qd * 4] * sc, acc[kb][db][qd * 4 + 1] * sc,
                                  acc[kb][db][qd * 4 + 2] * sc, acc[kb][db][qd * 4 + 3] * sc);
            }
        }
        };  // run_role
        if (role == 0)
            run_role(std::integral_constant<int, 0>{});
        else
            run_role(std::integral_constant<int, 1>{});
        // No barrier here: after the last barrier of the step loop nobody reads the rings any more, the stores above
        // touch no LDS, and a barrier would make every wavefront wait for its stores to be acknowledged before the
        // next pass may ask for its rows.
    }
}

// dK / dV = the splits' partial sums added in split order; four consecutive head_dim elements per thread
template <bool GF32>
__global__ __launch_bounds__(256) void gqa_reduce(AttnArgs a) {
    const int D = a.dk_dim, hs = a.head_split;
    const int64_t per_unit = static_cast<int64_t>(a.T) * D / 4;  // quads per (unit, tensor)
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= per_unit * 2 * a.Hkv * a.B) return;
    const int64_t quad = idx % per_unit;
    const int which = static_cast<int>((idx / per_unit) & 1), kvu = static_cast<int>(idx / (2 * per_unit));
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv;
    const int t = static_cast<int>(quad / (D / 4)), d = static_cast<int>(quad % (D / 4)) * 4;
    const size_t split_stride = static_cast<size_t>(2) * a.T * D;
    const float* src = a.part + (static_cast<size_t>(kvu) * hs * 2 + which) * a.T * D + static_cast<size_t>(t) * D + d;
    f32x4 sum = *reinterpret_cast<const f32x4*>(src);
    for (int r = 1; r < hs; ++r) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(src + r * split_stride);
        sum[0] += x[0], sum[1] += x[1], sum[2] += x[2], sum[3] += x[3];
    }
    void* dst = which == 0 ? a.dk : a.dv;
    const int64_t at = which == 0 ? b * a.dk_sb + hk * a.dk_sh + t * a.dk_st + d : b * a.dv_sb + hk * a.dv_sh + t * a.dv_st + d;
    store4g<GF32>(dst, at, sum[0], sum[1], sum[2], sum[3]);
}

template <int D, bool GF32>
int launch(const AttnArgs& a, hipStream_t st) {
    const int nb128 = (a.T + 127) / 128;
    const bool paired = a.causal && a.window == 0;
    const int hs = a.part ? a.head_split : 1;
    AttnArgs b = a;
    b.head_split = hs;
    hipLaunchKernelGGL((mfma_dkdv3<D, GF32>), dim3(xcd_grid(paired ? (nb128 + 1) / 2 : nb128, hs, a.Hkv * a.B)),
                       dim3(256), 0, st, b);
    PK_HIP(hipGetLastError());
    return hs > 1 ? launch_gqa_reduce(b, st) : PK_OK;
}

}  // namespace

bool mfma_dkdv3_takes(const AttnArgs& a) {
    // a thread's byte offset inside a 64-row tile of Q / dO is kept in 32 bits
    const int64_t reach = 2 * BMQ * (a.q_st > a.do_st ? a.q_st : a.do_st);
    // head_dim 64 (phases of 8 matrix instructions instead of 16) or 128; with a band the 32-key kernel is ahead
    // (0.22 against 0.24 ms at head_dim 128, window 256 + 4 sinks, T 4096): the steps are
    // few, most of them masked, and the workgroup that owns the sink keys alone walks every query tile
    // Short sequences (a workgroup meets a handful of query steps) are left to the 32-key kernel, which is ahead
    // below T = 512 at head_dim 128 and below T = 1024 at head_dim 64 (measured, B x H = 16 .. 256) -- unless query
    // heads share KV heads: only this kernel deals the heads of a group to several workgroups.
    const int t_min = a.dk_dim == 128 ? 512 : 1024;
    return (a.dk_dim == 128 || a.dk_dim == 64) && a.window == 0 && (a.T >= t_min || a.Hq > a.Hkv) &&
           reach < (int64_t{1} << 31);
}

int launch_gqa_reduce(const AttnArgs& a, hipStream_t st) {
    const int64_t quads = static_cast<int64_t>(a.T) * a.dk_dim / 4 * 2 * a.Hkv * a.B;
    const dim3 grid(static_cast<unsigned>((quads + 255) / 256));
    if (a.grad_f32)
        hipLaunchKernelGGL(gqa_reduce<true>, grid, dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL(gqa_reduce<false>, grid, dim3(256), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

int launch_mfma_dkdv3(const AttnArgs& a, hipStream_t st) {
    if (a.dk_dim == 64) return a.grad_f32 ? launch<64, true>(a, st) : launch<64, false>(a, st);
    return a.grad_f32 ? launch<128, true>(a, st) : launch<128, false>(a, st);
}

}  // namespace pk
