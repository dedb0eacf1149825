// dQ of the recompute backward with 64 queries per wavefront (see attn_bwd_mfma.hip for the
// mathematics and the transposed formulation, attn_bwd_dkdv3.hip for the measured issue costs
// that shape this kernel).
//
// A wavefront that owns 32 queries feeds every K / V fragment it reads from the LDS to ONE
// matrix instruction. Here a wavefront owns 64 queries (two blocks of 32): Q and dO of both
// blocks stay in registers for the whole pass (as B operands, lane = query), the two dQ^T
// accumulator sets likewise, and every fragment read from the LDS feeds TWO matrix
// instructions. That is 256 persistent registers -- all of them accumulation registers, which
// the matrix instruction accepts for its B operand as well as for C / D -- so one wavefront per
// SIMD, four per workgroup (256 queries per K / V tile).
//
// A K / V tile is 64 keys, worked on as two units of 32 keys. Per unit and wavefront:
//   G1   S^T = K Q^T and dP^T = V dO^T   32 matrix instructions (16 fragments, two blocks each)
//   E    dS = exp2(S c - LSE) (dP - delta), packed to bf16         (lane = query: all in-lane)
//   G2   dQ^T += K^T dS^T                16 matrix instructions (8 transposed fragments)
// at head_dim 128, half as many matrix instructions (and the same E) at head_dim 64.
// With nobody else on its SIMD the wavefront overlaps these by hand: E of a unit rides in the
// shadows of G1 of the next one, one element per matrix instruction,
//   per tile t:   G1(t, 1) || E(t, 0)  .  G2(t, 0)  .  G1(t+1, 0) || E(t, 1)  .  G2(t, 1)
// and the tiles come through a ring of four LDS slots (t for both G2 phases and the first G1, t+1
// for the second G1, t+2 landed or landing, t+3 asked for), one barrier per tile. Tiles are fetched with loads that write the
// LDS themselves (global_load_lds_dwordx4): the ordinary registers are taken by the four score
// tiles of two units (128), and a tile has a whole iteration to arrive.
//
// All matrix instructions are inline assembly with fixed register classes, as in the dK / dV
// kernel; the wait states between a matrix instruction and the first VALU read of its result
// are provided by the pipeline's own distances (a whole phase) and by s_nop before the epilogue,
// and a packed dS operand is formed at least two issue slots before the matrix instruction that
// reads it (tests/test_asm_hazards.py checks both on the compiled assembly).
#include <type_traits>

#include <cstdlib>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr int BN = 64;    // keys per tile
constexpr int BMW = 64;   // queries per wavefront
constexpr int BM = 256;   // queries per workgroup
// typed LDS pointer from a 32-bit LDS byte address
#define LDSP(T, addr) (reinterpret_cast<PK_LDS T*>(static_cast<uintptr_t>(addr)))

// t = a . b   /   t += a . b      score tile in ordinary registers, B operand (Q or dO) in accumulation registers
__device__ __forceinline__ void mma_s0(f32x16& t, bf16x8 a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(t) : "v"(a), "a"(b));
}
__device__ __forceinline__ void mma_s(f32x16& t, bf16x8 a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(t) : "v"(a), "a"(b));
}
// t = a . b + c                  score tile started from a tile of constants
__device__ __forceinline__ void mma_sc(f32x16& t, bf16x8 a, const bf16x8& b, const f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(t) : "v"(a), "a"(b), "v"(c));
}
// acc += a . b                    dQ^T accumulator in accumulation registers, B operand (packed dS) in ordinary ones
__device__ __forceinline__ void mma_q(f32x16& acc, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// The same for the first use of a packed dS operand: a matrix instruction that reads a register written by the vector
// instruction just before it gets the old contents (the compiler spaces the two apart only for matrix instructions it
// emits itself), so two idle states go first.
__device__ __forceinline__ void mma_q_fresh(f32x16& acc, bf16x8 a, bf16x8 b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

template <bool F32>
__device__ inline void store4q(void* base, int64_t idx, float x0, float x1, float x2, float x3) {
    if (F32) {
        f32x4 v = {x0, x1, x2, x3};
        *reinterpret_cast<f32x4*>(static_cast<float*>(base) + idx) = v;
    } else {
        u32x2 v = {pack_bf16(x0, x1), pack_bf16(x2, x3)};
        *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(base) + idx) = v;
    }
}

// Row `row` of a head as an MFMA operand: chunk kk covers d = 16kk + 8g .. +7; rows past the end are zero.
template <int D>
__device__ inline void row_operand(const void* base, int64_t off, int64_t st_t, int row, int T, int g, bf16x8* out) {
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
        u32x4 z = {0, 0, 0, 0};
        if (row < T)
            z = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + off + row * st_t + kk * 16 + g * 8);
        out[kk] = *reinterpret_cast<bf16x8*>(&z);
    }
}

// FUSE_DELTA: the workgroup also forms delta = rowsum(dO .* O) for its own rows (it holds their dO already),
// uses it and writes it for the dK / dV kernel, which then has to run after this one.
template <int D, bool GF32, bool FUSE_DELTA>
__global__ __launch_bounds__(256, 1) void mfma_dq3(AttnArgs a) {
    constexpr int KK = D / 16, DB = D / 32;
    constexpr int S = D + 8;      // tile row pitch (elements): 16-byte row reads conflict-free
    constexpr int NCH = D / 8;    // 16-byte chunks per row
    // a tile row in LDS is NCH + 1 units of 16 bytes (the last one padding); one load instruction fills 64 units
    constexpr int UPR = NCH + 1, UNITS = BN * UPR, NI = UNITS / 256;
    static_assert(UNITS - NI * 256 == 64, "the remainder is 16 lanes of each wavefront");
    constexpr uint32_t SLOTB = BN * S * 2;
    constexpr int RING = 4;  // tile slots: t (both G2 phases, the first G1), t+1 (the second G1), t+2 (landed or landing), t+3 (asked for)
    __shared__ __attribute__((aligned(16))) uint16_t Kt[RING][BN * S];
    __shared__ __attribute__((aligned(16))) uint16_t Vt[RING][BN * S];

    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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
    const float cexp = a.scale * LOG2E;

    auto lds32 = [](const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); };
    const uint32_t k_lds = lds32(Kt[0]), v_lds = lds32(Vt[0]);
    // lane parts of the LDS read addresses: a 16-byte row read at (row c32, 8 elements from 8g), and the
    // transposing read of K^T as lds_read_tr_operand_perm lays it out
    const uint32_t x_lane = static_cast<uint32_t>(lds_row<D>(c32) * S + g * 8) * 2u;
    const int tj = lane & 15, tu = (lane >> 4) & 1;
    const uint32_t y_lane = static_cast<uint32_t>(lds_row<D>(4 * g + (tj >> 2)) * S + TrMap<D>::src_col(0, tu, tj & 3)) * 2u;
    // Which memory row a load puts into LDS row R of a tile: the inverse of lds_row (R = 4a + 9b mod 16 inside a group
    // of 16 with b = R % 4 at head_dim 64; the identity at 128).
    auto mem_row = [](int R) {
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
    // m0 is set and used inside the one statement. It is not on the clobber list: the compiler treats m0 as a reserved
    // register (it rejects the clobber with a warning), never keeps a value in it across other code and writes it
    // directly before each instruction of its own that reads it, so nothing of the compiler's can be live in m0 here.
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
        int f_t = 0;                   // tile being fetched (clamped to the last one: a fetch past the end re-reads it)
        const char *f_kb = kbase, *f_vb = vbase;
        uint32_t f_limk = 0, f_limv = 0, f_slot = 0;
        auto fetch_setup = [&](int t) {
            f_t = min(t, hi);
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
        // Resident operands: Q and dO of the two 32-query blocks (B operands, lane = query), the per-query scalars.
        // A lane's operand chunks are 16 bytes out of every 32 of its own row, so loading them straight from memory
        // touches a cache line per lane and instruction (18 000 cycles per pass, measured). The rows therefore go
        // through LDS: a wavefront fills tile-sized regions of its own in the still empty ring with the same
        // row-filling loads as the tiles and reads its operands from there. Nobody else reads these rows, so each
        // round trip goes to memory (about 5000 cycles): Q and dO together in the first, O (for delta) together with
        // the first two K / V tiles in the second.
        bf16x8 qreg[2][KK], greg[2][KK];
        float nlse[2], dl[2];
        f32x16 acc[2][DB];  // dQ^T of the two query blocks
        {
            // asked for first, used after the second round trip
            float lse_raw[2];
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                const int qi = qw + qb * 32 + c32;
                const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + h) * a.T + qi;
                lse_raw[qb] = qi < a.T ? a.lse[lrow] : 0.0f;
                if (!FUSE_DELTA) dl[qb] = qi < a.T ? a.delta[lrow] : 0.0f;
            }
            const int last_row = max(min(BMW - 1, a.T - 1 - qw), 0);  // rows past the end repeat the last one (never stored)
            auto stage_rows = [&](uint32_t region, const void* base, int64_t off, int64_t st_t) {
                const char* src = reinterpret_cast<const char*>(base) + (off + static_cast<int64_t>(min(qw, a.T - 1)) * st_t) * 2;
                const uint32_t st2 = static_cast<uint32_t>(st_t) * 2u;
                int row = lane / UPR, ch = lane % UPR;  // unit 64 i + lane of the padded tile
#pragma unroll
                for (int i = 0; i < UNITS / 64; ++i) {
                    dma16(region + static_cast<uint32_t>(i) * 1024u,
                          static_cast<uint32_t>(min(mem_row(row), last_row)) * st2 + static_cast<uint32_t>(min(ch, NCH - 1)) * 16u, src);
                    row += 64 / UPR, ch += 64 % UPR;
                    if (ch >= UPR) ch -= UPR, ++row;
                }
            };
            static_assert(UNITS % 64 == 0, "whole load instructions per wavefront");
            auto staged = [&](uint32_t region, int qb, int kk) {
                return *LDSP(const bf16x8, region + x_lane + (qb * 32 * S + kk * 16) * 2);
            };
            // first round trip: Q into the K half of ring slot w, dO into its V half
            const uint32_t region_q = k_lds + static_cast<uint32_t>(w) * SLOTB, region_g = v_lds + static_cast<uint32_t>(w) * SLOTB;
            stage_rows(region_q, a.q, b * a.q_sb + h * a.q_sh, a.q_st);
            stage_rows(region_g, a.d_o, b * a.do_sb + h * a.do_sh, a.do_st);
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
                for (int kk = 0; kk < KK; ++kk) {
                    qreg[qb][kk] = staged(region_q, qb, kk);
                    greg[qb][kk] = staged(region_g, qb, kk);
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __syncthreads();  // every wavefront has read its regions: slots 0 and 1 may take their tiles
            // second round trip: the first two tiles, and O into a region of slots 2 / 3
            const uint32_t region_o = ((w & 1) ? v_lds : k_lds) + static_cast<uint32_t>(2 + (w >> 1)) * SLOTB;
            if (FUSE_DELTA) stage_rows(region_o, a.o, b * a.o_sb + h * a.o_sh, a.o_st);
            dma_tile(0);
            dma_tile(1);
            // loads complete in order: O is in when only the 2 NPIECE tile loads are left, and delta is formed while
            // those are on their way
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NPIECE) : "memory");
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                const int qi = qw + qb * 32 + c32;
                // a query past the end: p = exp2(-huge) = 0, so nothing it holds matters
                nlse[qb] = -1e30f;
                if (FUSE_DELTA) dl[qb] = 0.0f;
                if (qi < a.T) nlse[qb] = -lse_raw[qb] * LOG2E;
                if (FUSE_DELTA) {
                    // this lane's half of the row (d = 16kk + 8g .. +7), in four sums so that the additions do not
                    // wait for one another
                    float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk) {
                        const bf16x8 o8 = staged(region_o, qb, kk);
                        const u32x4 ov = *reinterpret_cast<const u32x4*>(&o8);
                        const u32x4 gv = *reinterpret_cast<const u32x4*>(&greg[qb][kk]);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            part[i] = fmaf(__uint_as_float(ov[i] << 16), __uint_as_float(gv[i] << 16), part[i]);
                            part[i] = fmaf(__uint_as_float(ov[i] & 0xFFFF0000u), __uint_as_float(gv[i] & 0xFFFF0000u), part[i]);
                        }
                    }
                    dl[qb] = xhalf_sum((part[0] + part[1]) + (part[2] + part[3]));
                }
            }
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        }
        __syncthreads();  // every wavefront has read its O region: the third tile may land there; tiles 0 and 1 are in
        dma_tile(2);      // waited for at the end of the first iteration
        if (FUSE_DELTA) {  // written after the barrier, which would otherwise wait for the store to be acknowledged
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                const int qi = qw + qb * 32 + c32;
                if (qi < a.T && g == 0) a.delta[(static_cast<int64_t>(b) * a.Hq + h) * a.T + qi] = dl[qb];
            }
        }
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                asm volatile("" : "+a"(qreg[qb][kk]));
                asm volatile("" : "+a"(greg[qb][kk]));
            }
        // -delta of a lane's query in every element of a score-tile-shaped register set
        f32x16 ndl[2];
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int r = 0; r < 16; ++r) ndl[qb][r] = -dl[qb];
        const QueryVis qvis[2] = {QueryVis(qw + c32, a.T, a.causal, a.window, a.sinks),
                                  QueryVis(qw + 32 + c32, a.T, a.causal, a.window, a.sinks)};


        constexpr int PF = 3;              // fragments in flight
        constexpr int N1 = 4 * KK;         // matrix instructions of a G1 phase: (K, V) x kk x two query blocks
        constexpr int N2 = 4 * DB;         // of a G2 phase: two k-chunks x DB column blocks x two query blocks
        f32x16 sc[2][2], dp[2][2];         // [unit parity][query block]: S^T and dP^T as the matrix pipe leaves them
        bf16x8 dsp[2][2];                  // packed dS^T of the unit in hand, [query block][16-key half]
        float y[8];                        // dS of the half block in hand (scalars: see the dK / dV kernel)

        // G1 fragment fi of unit (slot base kb / vb, 32-key half nb): even = K rows, odd = V rows, chunk kk = fi / 2
        auto g1frag = [&](uint32_t ka, uint32_t va, int nb, int fi) {
            return *LDSP(const bf16x8, ((fi & 1) ? va : ka) + (nb * 32 * S + (fi >> 1) * 16) * 2);
        };
        // G2 fragment fi of a unit: K^T, 16-key half kc = fi / DB, column block db = fi % DB
        auto g2frag = [&](uint32_t ya, int nb, int fi) {
            const uint32_t at = ya + ((nb * 32 + (fi / DB) * 16) * S + TrMap<D>::src_col(fi % DB, 0, 0) - TrMap<D>::src_col(0, 0, 0)) * 2;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, at));
            const s16x4 hi2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, at + TR_HI_ROWS<D> * S * 2));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi2[0], hi2[1], hi2[2], hi2[3]};
            return *reinterpret_cast<const bf16x8*>(&v);
        };
        // one G1 phase: unit (tile slot addresses ka / va, half nb) into score set `into`; `shadow(sl)` is the
        // other work of slot sl
        // `have`: the first PF fragments were asked for in the last slots of the phase before (nx); `next(j)` asks for
        // fragment j of the phase that follows, in this phase's last slots, so that no phase opens with an LDS round trip
        bf16x8 nx[PF];
        auto g1 = [&](uint32_t ka, uint32_t va, int nb, f32x16(&s_)[2], f32x16(&d_)[2], auto shadow, auto have, auto next) {
            bf16x8 f[N1 / 2];
#pragma unroll
            for (int j = 0; j < PF; ++j) f[j] = decltype(have)::value ? nx[j] : g1frag(ka, va, nb, j);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sl = 0; sl < N1; ++sl) {
                const int fi = sl >> 1, qb = sl & 1, kk = fi >> 1;
                if (fi & 1) {
                    if (kk == 0)
                        mma_sc(d_[qb], f[fi], greg[qb][kk], ndl[qb]);  // dP - delta: delta enters as the C operand
                    else
                        mma_s(d_[qb], f[fi], greg[qb][kk]);
                } else {
                    if (kk == 0)
                        mma_s0(s_[qb], f[fi], qreg[qb][kk]);
                    else
                        mma_s(s_[qb], f[fi], qreg[qb][kk]);
                }
                if (qb == 0) {
                    if (fi + PF < N1 / 2)
                        f[fi + PF] = g1frag(ka, va, nb, fi + PF);
                    else
                        nx[fi + PF - N1 / 2] = next(fi + PF - N1 / 2);
                }
                shadow(sl);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // one G2 phase: dQ^T += K^T dS^T of the unit in hand
        auto g2 = [&](uint32_t ya, int nb, auto shadow, auto next) {
            bf16x8 f[N2 / 2];
#pragma unroll
            for (int j = 0; j < PF; ++j) f[j] = nx[j];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sl = 0; sl < N2; ++sl) {
                const int fi = sl >> 1, qb = sl & 1;
                if (fi % DB == 0)
                    mma_q_fresh(acc[qb][0], f[fi], dsp[qb][fi / DB]);
                else
                    mma_q(acc[qb][fi % DB], f[fi], dsp[qb][fi / DB]);
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
        // Elementwise work of one element e (query block e / 16, register e % 16) of the unit whose scores are in
        // (s_, d_); after the 8th and 16th element of a block its packed half is formed.
        // Three instructions per element -- x = S c - LSE, p = exp2(x), dS = p (dP - delta) -- each the input of the next:
        // issued back to back they wait for one another (a dependent vector instruction issues after 8 clocks, an
        // independent one after 5), so they are staggered over three slots. Slot sl forms x of element sl (of the pair 2 sl, 2 sl + 1
        // at head_dim 64, where a phase has half the slots), p of element sl - 1 and dS of element sl - 2; the last two elements finish in the first two slots of the G2 phase
        // that follows. After the 8th and 16th element of a block its packed half is formed.
        constexpr int EPS = 32 / N1;  // elements per slot: 1 at head_dim 128, 2 at 64
        float xq[EPS] = {}, pq[EPS] = {};
        auto elem = [&](const f32x16(&s_)[2], const f32x16(&d_)[2], int sl) {
#pragma unroll
            for (int i = 0; i < EPS; ++i) {
                if (sl >= 2 && sl < N1 + 2) {
                    const int e = (sl - 2) * EPS + i, qb = e >> 4, r = e & 15;
                    y[r & 7] = pq[i] * d_[qb][r];  // d_ holds dP - delta
                    if ((r & 7) == 7) {
                        u32x4 u = {pack_bf16(y[0], y[1]), pack_bf16(y[2], y[3]), pack_bf16(y[4], y[5]), pack_bf16(y[6], y[7])};
                        dsp[qb][r >> 3] = *reinterpret_cast<bf16x8*>(&u);
                        // formed here, in this slot: without the pin the compiler may sink the whole chain of the half
                        // to just before the matrix instruction that reads it, which then reads a register written one
                        // instruction earlier -- inside an asm statement the compiler keeps no distance for that
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
                if (sl < N1) xq[i] = fmaf(s_[e >> 4][e & 15], cexp, nlse[e >> 4]);
            }
        };
        // A unit on the diagonal or past the end of the keys: what the mask hides becomes -inf before the exponentials
        // (p = 0, dS = 0). Off the common path; tiles away from the diagonal carry no mask arithmetic at all.
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

        if (hi_w >= 0)
            g1(k_lds + x_lane, v_lds + x_lane, 0, sc[0], dp[0], [](int) {}, std::false_type{},
               [&](int j) { return g1frag(k_lds + x_lane, v_lds + x_lane, 1, j); });
        // the first elementwise slots follow at once here (in the loop a whole G2 phase lies between): let the last
        // matrix instructions of this prologue write their results first
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
        for (int t = 0; t <= hi; ++t) {
            const uint32_t slot = static_cast<uint32_t>(t % RING) * SLOTB, slot1 = static_cast<uint32_t>((t + 1) % RING) * SLOTB;
            fetch_setup(t + 3);
            auto stage = [&](int first, int sl) {  // the arriving tile, five loads in each G2 phase
                if (sl % 3 == 1 && sl / 3 < NPIECE / 2) dma_piece(first + sl / 3);
            };
            if (t <= hi_w) {
                const int n0 = t * BN;
                const uint32_t ka = k_lds + slot + x_lane, va = v_lds + slot + x_lane, ya = k_lds + slot + y_lane;
                // ---- G1(t, 1) || E(t, 0)
                if (__builtin_expect(!unit_full(n0), 0)) mask_unit(sc[0], n0);
                const uint32_t ka1 = k_lds + slot1 + x_lane, va1 = v_lds + slot1 + x_lane;
                g1(ka, va, 1, sc[1], dp[1], [&](int sl) { elem(sc[0], dp[0], sl); }, std::true_type{},
                   [&](int j) { return g2frag(ya, 0, j); });
                // ---- G2(t, 0)
                g2(ya, 0,
                   [&](int sl) {
                       if (sl < 2) elem(sc[0], dp[0], N1 + sl);
                       stage(0, sl);
                   },
                   [&](int j) { return g1frag(ka1, va1, 0, j); });
                // ---- G1(t+1, 0) || E(t, 1)
                if (__builtin_expect(!unit_full(n0 + 32), 0)) mask_unit(sc[1], n0 + 32);
                g1(ka1, va1, 0, sc[0], dp[0], [&](int sl) { elem(sc[1], dp[1], sl); }, std::true_type{},
                   [&](int j) { return g2frag(ya, 1, j); });
                // ---- G2(t, 1); its last slots ask for the first fragments of the next iteration's G1(t+1, 1): that tile
                // has been readable since the barrier before this iteration
                g2(ya, 1,
                   [&](int sl) {
                       if (sl < 2) elem(sc[1], dp[1], N1 + sl);
                       stage(NPIECE / 2, sl);
                   },
                   [&](int j) { return g1frag(ka1, va1, 1, j); });
            }
            if (t > hi_w) {  // past this wavefront's diagonal: only the staging (a second skip, not an else: see dK / dV)
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
            if (qi >= a.T) continue;
            const int64_t ob = b * a.dq_sb + h * a.dq_sh + qi * a.dq_st;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (!GF32) {
                    store_acc_bf16<D>(static_cast<uint16_t*>(a.dq) + ob, db, g, acc[qb][db], a.scale);
                    continue;
                }
#pragma unroll
                for (int qd = 0; qd < 4; ++qd)
                    store4q<GF32>(a.dq, ob + TrMap<D>::col0(db, qd, g), acc[qb][db][qd * 4] * a.scale,
                                  acc[qb][db][qd * 4 + 1] * a.scale, acc[qb][db][qd * 4 + 2] * a.scale,
                                  acc[qb][db][qd * 4 + 3] * a.scale);
            }
        }
        // No barrier here: every wavefront passed the barrier of the last iteration after its last read of the ring,
        // the stores above touch no LDS, and the next pass meets its own barriers before anybody reads what another
        // wavefront wrote. A barrier would also make each wavefront wait for its dQ stores to be acknowledged before
        // the next pass may ask for its rows.
    }
}

template <int D, bool GF32>
int launch(const AttnArgs& a, bool fuse_delta, hipStream_t st) {
    const int nqb = (a.T + BM - 1) / BM;
    const bool paired = pair_causal_blocks(nqb, a.Hq * a.B, a.causal, a.window);
    const dim3 grid(xcd_grid(paired ? (nqb + 1) / 2 : nqb, a.Hq / a.Hkv, a.Hkv * a.B));
    if (fuse_delta)
        hipLaunchKernelGGL((mfma_dq3<D, GF32, true>), grid, dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((mfma_dq3<D, GF32, false>), grid, dim3(256), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

}  // namespace

bool mfma_dq3_takes(const AttnArgs& a) {
    // a lane's byte offset inside a 64-row tile of K / V is kept in 32 bits
    const int64_t reach = 2 * BN * (a.k_st > a.v_st ? a.k_st : a.v_st);
    // One workgroup of 256 queries fills a CU, so nothing hides its prologue and epilogue (two memory round trips and a
    // pipeline fill, the cost of about six key tiles): it is ahead of the 128-query kernel, two workgroups per CU,
    // only where a workgroup walks many tiles. Measured over B x H = 16 .. 256, full causal: ahead from T = 2048 at
    // head_dim 128 (4 .. 26 %) and from T = 4096 at head_dim 64 (2 .. 13 %), behind below that (3 .. 35 %).
    const int t_min = a.dk_dim == 128 ? 2048 : 4096;
    return (a.dk_dim == 128 || a.dk_dim == 64) && a.window == 0 && a.T >= t_min && reach < (int64_t{1} << 31);
}

int launch_mfma_dq3(const AttnArgs& a, bool fuse_delta, hipStream_t st) {
    if (a.dk_dim == 64) return a.grad_f32 ? launch<64, true>(a, fuse_delta, st) : launch<64, false>(a, fuse_delta, st);
    return a.grad_f32 ? launch<128, true>(a, fuse_delta, st) : launch<128, false>(a, fuse_delta, st);
}

}  // namespace pk
