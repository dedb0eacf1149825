// dK / dV of the recompute backward, second generation (see attn_bwd_mfma.hip
// for the mathematics and the operand layouts).
//
// Measured: the one-wavefront-per-SIMD kernel that keeps K, V, dK^T and dV^T
// of 32 keys in one wavefront's registers leaves the matrix pipe idle while
// that wavefront does its exp2 / LDS work, and cannot be run two per SIMD
// (it needs > 256 registers). Here the work of one 32-key block is split
// between TWO wavefronts that share a SIMD:
//
//   role 0 (wavefronts 0-3):  S = Q K^T -> P = exp2(S*c - LSE) -> dV^T += dO^T P
//   role 1 (wavefronts 4-7):  dP = dO V^T -> dS = P .* (dP - delta) -> dK^T += Q^T dS
//
// Each holds one operand (K or V) and one accumulator (dV^T or dK^T): ~180
// registers, two wavefronts per SIMD, 16 MFMAs each per 32 x 32 block, no
// recomputation. P goes from role 0 to role 1 through LDS as packed fp16 pairs in
// the accumulator's own element order (lane-private 32 bytes, conflict-free). Role 1
// runs ONE STEP BEHIND role 0, so the hand-over needs no extra barrier: the
// step barrier that publishes the next Q / dO tile also publishes P.
//
// Step = 64 queries of one query head. Q / dO tiles sit in a three-deep LDS
// ring (role 0 reads step s, role 1 step s-1, step s+1 is being stored).
#include <cstdlib>
#include <type_traits>

#include "mfma_common.h"
#include "pk_internal.h"

namespace pk {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
// Two geometries. 128 keys per workgroup (8 wavefronts, 64-query steps, one workgroup per CU) is the general one.
// With a narrow band a key block meets only a handful of query steps, and the fixed costs of a workgroup -- resident
// rows, first tiles, pipeline fill, epilogue -- weigh as much as its steps; there a workgroup takes 64 keys with 4
// wavefronts and 32-query steps, so that TWO workgroups fit a CU (registers: still two wavefronts per SIMD; LDS: 61 KB
// each) and one's fixed costs run beside the other's steps. Finer tiles also waste less on the band's edges.
typedef __fp16 h16x2 __attribute__((ext_vector_type(2)));

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

// TAIL: the launch carries the extra workgroups of a split sink tail (a separate instantiation, so
// that the plain causal kernel keeps its register budget)
template <int D, bool GF32, bool TAIL, int BNK, int BMQ>
__global__ __launch_bounds__(4 * BNK, 2) void mfma_dkdv2(AttnArgs a) {
    constexpr int KK = D / 16, DB = D / 32;
    constexpr int NTHR = 4 * BNK, NKB = BNK / 32, NQB = BMQ / 32;  // threads; 32-key blocks; 32-query blocks per step
    constexpr int S = D + 8;            // tile row pitch (elements): 16-byte row reads conflict-free
    constexpr int NCH = D / 8;          // 16-byte chunks per row
    constexpr int CPT = BMQ * NCH / NTHR;  // chunks per thread per tensor per step
    static_assert(CPT >= 1 && BMQ * NCH % NTHR == 0, "every thread stages the same number of chunks");
    __shared__ __attribute__((aligned(16))) uint16_t tiles[2][3][BMQ * S];  // [Q | dO][ring slot]
    uint16_t (*const Qs)[BMQ * S] = tiles[0];
    uint16_t (*const dOs)[BMQ * S] = tiles[1];
    __shared__ __attribute__((aligned(16))) uint16_t Pbuf[2][NQB][NKB][2 * 64 * 8];  // [step parity][query block][key block][half][lane][8]
    __shared__ __attribute__((aligned(16))) float nlse_s[3][BMQ];            // -LSE * log2(e)
    __shared__ __attribute__((aligned(16))) float dl_s[3][BMQ];

    const int lane = threadIdx.x & 63;
    // the wavefront index as a scalar: every test on it becomes a scalar branch
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int role = w / NKB, kbw = w % NKB;
    const int g = lane >> 5, c32 = lane & 31;
    // Lane parts of the two LDS operand addresses (elements): a 16-byte row read at
    // (row c32, column 8g) and a transposing read as lds_read_tr_operand_perm lays it out.
    const int row_lane = lds_row<D>(c32) * S + g * 8;
    const int tr_lane = lds_row<D>(4 * g + ((lane & 15) >> 2)) * S + TrMap<D>::src_col(0, (lane >> 4) & 1, lane & 3);
    const int nkb = (a.T + BNK - 1) / BNK, rep = a.Hq / a.Hkv;
    // Full-causal: key block i is seen by T - 128i queries; blocks i and nkb-1-i
    // are taken back to back so that every workgroup carries the same work.
    const bool paired = a.causal && a.window == 0;
    int blk, rr, kvu;
    // Band mask with a few sink keys: the queries past block 0's band are cut into chunks that get
    // workgroups of their own (ids nkb .. nkb + nch - 1 of the unit), see sink_tail.
    const SinkTail tl = TAIL ? sink_tail(a.T, a.window, a.sinks) : SinkTail{0, 0};
    if (TAIL) {
        if (!xcd_map(nkb + tl.nch, 1, a.Hkv * a.B, blk, rr, kvu)) return;
    } else if (a.window > 0 && a.sinks > 0 && nkb > 1) {
        if (!xcd_map_block0_first(nkb, a.Hkv * a.B, blk, kvu)) return;
    } else if (!xcd_map(paired ? (nkb + 1) / 2 : nkb, 1, a.Hkv * a.B, blk, rr, kvu)) {
        return;
    }
    const int chunk = (TAIL && blk >= nkb) ? blk - nkb : -1;  // >= 0: this workgroup takes a chunk of the sink tail
    if (TAIL && chunk >= 0) blk = 0;
    const int hk = kvu % a.Hkv, b = kvu / a.Hkv;
    const float cexp = a.scale * LOG2E;
    const int npass = (paired && blk != nkb - 1 - blk) ? 2 : 1;

    for (int pass = 0; pass < npass; ++pass) {
        const int kblk = pass == 0 ? blk : nkb - 1 - blk;  // heavy block first
        const int k0 = kblk * BNK;
        const int kw0 = k0 + kbw * 32;  // this wavefront's 32 keys
        const int kj = kw0 + c32;

        // The wavefront's resident operand: K for role 0, V for role 1 (B operand,
        // lane = key, chunk kk covers d = 16kk + 8g .. +7). Keys past the end
        // re-read the last row; their P is masked to zero and nothing is stored.
        bf16x8 kv[KK];
        {
            const void* src = role == 0 ? a.k : a.v;
            const int64_t off = role == 0 ? b * a.k_sb + hk * a.k_sh : b * a.v_sb + hk * a.v_sh;
            const int64_t st = role == 0 ? a.k_st : a.v_st;
            const int t = min(kj, a.T - 1);
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const u32x4 z = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(src) + off + t * st +
                                                                kk * 16 + g * 8);
                kv[kk] = *reinterpret_cast<const bf16x8*>(&z);
            }
        }
        // Query tiles that can see keys [k0, k0+127] (paperkiln src/ops.cpp:960-965 inverted).
        const int khi = min(k0 + BNK, a.T) - 1;
        int qt_lo = a.causal ? k0 / BMQ : 0;
        int qt_hi = (a.window > 0 && (k0 >= a.sinks || TAIL)) ? min(a.T - 1, khi + a.window - 1) / BMQ
                                                              : (a.T - 1) / BMQ;
        if (TAIL && chunk >= 0) {
            qt_lo = (tl.q0 + chunk * TAIL_CHUNK) / BMQ;
            qt_hi = min(a.T - 1, tl.q0 + (chunk + 1) * TAIL_CHUNK - 1) / BMQ;
        } else if (TAIL && kblk == 0) {
            qt_hi = tl.q0 / BMQ - 1;  // the band part of block 0 ends where the chunks begin, whatever the block size
        }
        const int nqt = qt_hi - qt_lo + 1;
        const int steps = nqt * rep;

        u32x4 qr[CPT], gr[CPT];
        float lse_r = 0.0f, dl_r = 0.0f;
        // Steps are fetched in order, so the (head, query tile) of the next fetch is counted up, not divided out of
        // the step number, and a thread's position inside a tile (row tid / NCH + RPI i, chunk tid % NCH) is formed once.
        // (Tile positions as scalar bases plus per-thread 32-bit offsets, as the 64-key kernel keeps them, take a
        // third of the vector instructions out of the staging and measured no faster here, slower at head_dim 64.)
        int f_h = hk * rep, f_qt = 0;
        const int frow = static_cast<int>(threadIdx.x) / NCH, fch = static_cast<int>(threadIdx.x) % NCH;
        constexpr int RPI = NTHR / NCH;  // tile rows between a thread's consecutive chunks
        auto fetch = [&]() {  // global -> registers, rows past the end clamped
            const int q0 = (qt_lo + f_qt) * BMQ;
            const uint16_t* qb = static_cast<const uint16_t*>(a.q) + b * a.q_sb + f_h * a.q_sh + fch * 8;
            const uint16_t* gb = static_cast<const uint16_t*>(a.d_o) + b * a.do_sb + f_h * a.do_sh + fch * 8;
#pragma unroll
            for (int i = 0; i < CPT; ++i) {
                const int t = min(q0 + frow + RPI * i, a.T - 1);
                qr[i] = *reinterpret_cast<const u32x4*>(qb + t * a.q_st);
                gr[i] = *reinterpret_cast<const u32x4*>(gb + t * a.do_st);
            }
            if (threadIdx.x < BMQ) {
                const int t = min(q0 + static_cast<int>(threadIdx.x), a.T - 1);
                const int64_t lrow = (static_cast<int64_t>(b) * a.Hq + f_h) * a.T + t;
                lse_r = a.lse[lrow];  // scaled when it is stored: arithmetic on it here would wait for every load just issued
                dl_r = a.delta[lrow];
            }
            const bool wrap = f_qt + 1 == nqt;
            f_qt = wrap ? 0 : f_qt + 1;
            f_h += wrap;
        };
        auto commit = [&](int slot) {  // registers -> LDS ring slot
            // The store addresses are rebuilt from the thread index at every call (the
            // empty statement hides its value): a handful of shifts, where addresses
            // kept live across the step were the ones the allocator sent to scratch.
            int tid = threadIdx.x;
            asm volatile("" : "+v"(tid));
#pragma unroll
            for (int i = 0; i < CPT; ++i) {
                const int c = tid + NTHR * i;
                const int row = c / NCH, ch = c % NCH;
                *reinterpret_cast<u32x4*>(Qs[slot] + lds_row<D>(row) * S + ch * 8) = qr[i];
                *reinterpret_cast<u32x4*>(dOs[slot] + lds_row<D>(row) * S + ch * 8) = gr[i];
            }
            if (tid < BMQ) {
                nlse_s[slot][tid] = -lse_r * LOG2E;
                dl_s[slot][tid] = dl_r;
            }
        };
        // wavefront-uniform: is anything of (query block qb of the step at query tile `qt`) x (this key block) visible?
        auto block_live = [&](int qt, int qb, int& qlo) {
            qlo = (qt_lo + qt) * BMQ + qb * 32;
            const int qhi = qlo + 31;
            if (qlo >= a.T || kw0 >= a.T) return false;
            if (a.causal && kw0 > qhi) return false;
            if (a.window > 0 && kw0 + 31 + a.window <= qlo && kw0 >= a.sinks) return false;
            return true;
        };

        if (steps > 0) {
            fetch();
            commit(0);
            if (steps > 1) fetch();
        }
        // Every load issued so far -- the resident K / V rows above all -- has landed before the step loop is
        // entered. Without this the wait-count bookkeeping carries "kv may still be in flight" around the loop
        // and puts a vmcnt wait in front of each MFMA that reads kv, which in every later step waits for the
        // NEXT tile's prefetch instead (a full memory latency per step).
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();

        // transposed operand (k-chunk = rows row0 + {4g..4g+3} u {8+4g..}) of column block db, from a
        // pointer that already carries the lane part
        auto tr_operand = [&](const uint16_t* p, int row0, int db) {
            p += row0 * S + TrMap<D>::src_col(db, 0, 0);
            const s16x4 lo = lds_read_tr4(p), hi = lds_read_tr4(p + TR_HI_ROWS<D> * S);
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            return *reinterpret_cast<const bf16x8*>(&v);
        };
        // The step loop and the stores are instantiated once per role and entered through one branch on the role: with
        // the role tested inside the loop the two sides of the branch each get their own copy of the accumulators,
        // which are moved back at the join in every step (64 register moves a step, found in the compiled loop).
        auto run_role = [&](auto role_tag) {
        constexpr int rl = decltype(role_tag)::value;
        f32x16 acc[DB];  // dV^T (role 0) or dK^T (role 1)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[db][r] = 0.0f;
        // iteration s: role 0 works on step s, role 1 on step s-1; the query tile of either is counted, not divided out
        int c_qt = 0, slot = 0;  // query tile and ring slot of the step this role works on
        for (int s = 0; s <= steps; ++s) {
            if (s + 1 < steps) {
                commit((s + 1) % 3);  // slot last read (by role 1) before the previous barrier
                if (s + 2 < steps) fetch();
            }
            if (rl == 0) {
                if (s < steps) {
                    // One register each for the row-read and the transposing-read address of
                        // this step; every fragment is then an immediate offset away. Left to
                        // itself the compiler keeps a dozen pre-offset copies and spills.
                    int xrow = slot * (BMQ * S) + row_lane;                     // Q rows
                    int ytr = (3 + slot) * (BMQ * S) + tr_lane;                 // dO transposed
                    asm volatile("" : "+v"(xrow), "+v"(ytr));
                    const uint16_t* flat = &tiles[0][0][0];
#pragma unroll
                    for (int qb = 0; qb < NQB; ++qb) {
                        int qlo;
                        if (!block_live(c_qt, qb, qlo)) continue;
                        // One accumulator chain: the other role's wavefront on this SIMD issues
                        // into the gaps a dependent MFMA pair leaves, and the registers of a
                        // second chain would push the kernel into scratch.
                        f32x16 sc;
#pragma unroll
                        for (int r = 0; r < 16; ++r) sc[r] = 0.0f;
#pragma unroll
                        for (int kk = 0; kk < KK; ++kk)
                            sc = mfma32(lds_read8(flat + xrow + qb * 32 * S + kk * 16), kv[kk], sc);
                        const int qhi = qlo + 31;
                        const bool full = qhi < a.T && kw0 + 31 < a.T && (!a.causal || kw0 + 31 <= qlo) &&
                                          (a.window == 0 || kw0 + a.window > qhi || kw0 + 31 < a.sinks);
                        // lane = key kj; element r = query qlo + (r/4)*8 + 4g + r%4
#pragma unroll
                        for (int qd = 0; qd < 4; ++qd) {
                            const f32x4 nl = *reinterpret_cast<const f32x4*>(&nlse_s[slot][qb * 32 + qd * 8 + g * 4]);
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                sc[qd * 4 + e] = __builtin_amdgcn_exp2f(fmaf(sc[qd * 4 + e], cexp, nl[e]));
                        }
                        if (!full) {  // off the common path: interior tiles carry no mask arithmetic at all
                            const KeyVis kvis(kj, a.T, a.causal, a.window, a.sinks);
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                sc[r] = kvis(qlo + (r >> 2) * 8 + g * 4 + (r & 3)) ? sc[r] : 0.0f;
                        }
                        const bf16x8 p0 = c_to_operand<0>(sc), p1 = c_to_operand<1>(sc);
                        // hand-over copy in fp16: P is in [0, 1], where fp16 carries 11 significant
                        // bits against bf16's 8, so dS is built from a P as good as the old fp32 one
                        // the two 16-byte halves of a lane sit 1 KB apart: consecutive lanes then
                        // write consecutive 16-byte chunks and no two lanes share a bank
                        uint16_t* pb = Pbuf[s & 1][qb][kbw] + lane * 8;
                        h16x2 ph[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const f32x2 pr = {sc[2 * i], sc[2 * i + 1]};
                            ph[i] = __builtin_convertvector(pr, h16x2);  // round to nearest even
                        }
                        *reinterpret_cast<u32x4*>(pb) = *reinterpret_cast<u32x4*>(&ph[0]);
                        *reinterpret_cast<u32x4*>(pb + 512) = *reinterpret_cast<u32x4*>(&ph[4]);
                        // dV^T += dO^T P
#pragma unroll
                        for (int db = 0; db < DB; ++db)
                            acc[db] = mfma32(tr_operand(flat + ytr, qb * 32, db), p0, acc[db]);
#pragma unroll
                        for (int db = 0; db < DB; ++db)
                            acc[db] = mfma32(tr_operand(flat + ytr, qb * 32 + 16, db), p1, acc[db]);
                    }
                    c_qt = c_qt + 1 == nqt ? 0 : c_qt + 1;
                    slot = slot == 2 ? 0 : slot + 1;
                }
            } else {
                if (s >= 1) {
                    const int sp = s - 1;
                    int xrow = (3 + slot) * (BMQ * S) + row_lane;               // dO rows
                    int ytr = slot * (BMQ * S) + tr_lane;                       // Q transposed
                    asm volatile("" : "+v"(xrow), "+v"(ytr));
                    const uint16_t* flat = &tiles[0][0][0];
#pragma unroll
                    for (int qb = 0; qb < NQB; ++qb) {
                        int qlo;
                        if (!block_live(c_qt, qb, qlo)) continue;
                        f32x16 dp;
#pragma unroll
                        for (int r = 0; r < 16; ++r) dp[r] = 0.0f;
#pragma unroll
                        for (int kk = 0; kk < KK; ++kk)
                            dp = mfma32(lds_read8(flat + xrow + qb * 32 * S + kk * 16), kv[kk], dp);
                        const uint16_t* pb = Pbuf[sp & 1][qb][kbw] + lane * 8;
                        u32x4 praw[2];
                        praw[0] = *reinterpret_cast<const u32x4*>(pb);
                        praw[1] = *reinterpret_cast<const u32x4*>(pb + 512);
                        const h16x2* ph = reinterpret_cast<const h16x2*>(praw);
                        // dS = P .* (dP - delta); P arrives as fp16 pairs of elements (2i, 2i+1)
#pragma unroll
                        for (int qd = 0; qd < 4; ++qd) {
                            const f32x4 dl = *reinterpret_cast<const f32x4*>(&dl_s[slot][qb * 32 + qd * 8 + g * 4]);
                            dp[qd * 4 + 0] = static_cast<float>(ph[2 * qd][0]) * (dp[qd * 4 + 0] - dl[0]);
                            dp[qd * 4 + 1] = static_cast<float>(ph[2 * qd][1]) * (dp[qd * 4 + 1] - dl[1]);
                            dp[qd * 4 + 2] = static_cast<float>(ph[2 * qd + 1][0]) * (dp[qd * 4 + 2] - dl[2]);
                            dp[qd * 4 + 3] = static_cast<float>(ph[2 * qd + 1][1]) * (dp[qd * 4 + 3] - dl[3]);
                        }
                        const bf16x8 d0 = c_to_operand<0>(dp), d1 = c_to_operand<1>(dp);
                        // dK^T += Q^T dS
#pragma unroll
                        for (int db = 0; db < DB; ++db)
                            acc[db] = mfma32(tr_operand(flat + ytr, qb * 32, db), d0, acc[db]);
#pragma unroll
                        for (int db = 0; db < DB; ++db)
                            acc[db] = mfma32(tr_operand(flat + ytr, qb * 32 + 16, db), d1, acc[db]);
                    }
                    c_qt = c_qt + 1 == nqt ? 0 : c_qt + 1;
                    slot = slot == 2 ? 0 : slot + 1;
                }
            }
            __syncthreads();
        }

        // Pieces of a split sink tail: the sink keys' rows go to the workspace as fp32 partial sums
        // (a chunk writes nothing else; the band part of block 0 writes its other rows as usual).
        const bool piece = TAIL && kblk == 0;
        if (piece && kbw == 0 && kj < a.sinks) {
            float* rows = sink_tail_rows(a.tail, kvu, tl.nch, chunk >= 0 ? chunk : tl.nch, rl == 0 ? 1 : 0, D) + kj * D;
            const float sc = rl == 0 ? 1.0f : a.scale;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int qd = 0; qd < 4; ++qd)
                    store4g<true>(rows, TrMap<D>::col0(db, qd, g), acc[db][qd * 4] * sc, acc[db][qd * 4 + 1] * sc,
                                  acc[db][qd * 4 + 2] * sc, acc[db][qd * 4 + 3] * sc);
        }
        if (kj < a.T && chunk < 0 && !(piece && kj < a.sinks)) {
            void* dst = rl == 0 ? a.dv : a.dk;
            const int64_t ob = rl == 0 ? b * a.dv_sb + hk * a.dv_sh + kj * a.dv_st
                                         : b * a.dk_sb + hk * a.dk_sh + kj * a.dk_st;
            const float sc = rl == 0 ? 1.0f : a.scale;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (!GF32) {
                    store_acc_bf16<D>(static_cast<uint16_t*>(dst) + ob, db, g, acc[db], sc);
                    continue;
                }
#pragma unroll
                for (int qd = 0; qd < 4; ++qd)
                    store4g<GF32>(dst, ob + TrMap<D>::col0(db, qd, g), acc[db][qd * 4] * sc, acc[db][qd * 4 + 1] * sc,
                                  acc[db][qd * 4 + 2] * sc, acc[db][qd * 4 + 3] * sc);
            }
        }
        };  // run_role
        if (role == 0)
            run_role(std::integral_constant<int, 0>{});
        else
            run_role(std::integral_constant<int, 1>{});
        __syncthreads();  // the next pass refills the ring
    }
}

// dK / dV rows [0, sinks) of every (batch, KV head) = the band part plus the chunks, in that order.
template <bool GF32>
__global__ __launch_bounds__(256) void sink_tail_reduce(AttnArgs a, int nch) {
    const int kvu = blockIdx.x, hk = kvu % a.Hkv, b = kvu / a.Hkv, D = a.dk_dim;
    for (int idx = threadIdx.x; idx < 2 * a.sinks * D; idx += 256) {
        const int which = idx / (a.sinks * D), j = (idx / D) % a.sinks, d = idx % D;
        float sum = sink_tail_rows(a.tail, kvu, nch, nch, which, D)[j * D + d];
        for (int c = 0; c < nch; ++c) sum += sink_tail_rows(a.tail, kvu, nch, c, which, D)[j * D + d];
        void* dst = which == 0 ? a.dk : a.dv;
        const int64_t at = which == 0 ? b * a.dk_sb + hk * a.dk_sh + j * a.dk_st + d
                                      : b * a.dv_sb + hk * a.dv_sh + j * a.dv_st + d;
        if (GF32) {
            static_cast<float*>(dst)[at] = sum;
        } else {
            const uint32_t two = pack_bf16(sum, 0.0f);
            static_cast<uint16_t*>(dst)[at] = static_cast<uint16_t>(two & 0xffffu);
        }
    }
}

template <int D, bool GF32, int BNK, int BMQ>
int launch_geo(const AttnArgs& a_in, hipStream_t st) {
    AttnArgs a = a_in;
    const int nkb = (a.T + BNK - 1) / BNK;
    const bool paired = a.causal && a.window == 0;
    SinkTail tl = a.tail ? sink_tail(a.T, a.window, a.sinks) : SinkTail{0, 0};
    // a tail step keeps two of the eight wavefronts busy but takes as long as a full one (measured)
    if (!sink_tail_pays(tl, a.T, a.window, a.Hkv * a.B, 64, 3, 1.0f)) {
        a.tail = nullptr;
        tl.nch = 0;
    }
    if (tl.nch > 0) {
        hipLaunchKernelGGL((mfma_dkdv2<D, GF32, true, BNK, BMQ>), dim3(xcd_grid(nkb + tl.nch, 1, a.Hkv * a.B)), dim3(4 * BNK), 0,
                           st, a);
        PK_HIP(hipGetLastError());
        return launch_sink_tail_reduce(a, st);
    }
    hipLaunchKernelGGL((mfma_dkdv2<D, GF32, false, BNK, BMQ>), dim3(xcd_grid(paired ? (nkb + 1) / 2 : nkb, 1, a.Hkv * a.B)),
                       dim3(4 * BNK), 0, st, a);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

template <int D, bool GF32>
int launch(const AttnArgs& a, hipStream_t st) {
    // A band of a few key blocks: the small geometry, two workgroups per CU. Measured at B=4 H=16 T=4096, head_dim 128,
    // small against large: window 128 0.190 / 0.229 ms, 256 0.190 / 0.223, 512 0.264 / 0.276, 1024 0.404 / 0.387,
    // 2048 0.623 / 0.565; at head_dim 64 (window 256) 0.142 / 0.134, so only head_dim 128 takes it.
    if (D == 128 && a.window > 0 && a.window <= 512) return launch_geo<D, GF32, 64, 32>(a, st);
    return launch_geo<D, GF32, 128, 64>(a, st);
}

}  // namespace

int launch_sink_tail_reduce(const AttnArgs& a, hipStream_t st) {
    const int nch = sink_tail(a.T, a.window, a.sinks).nch;
    if (a.grad_f32)
        hipLaunchKernelGGL(sink_tail_reduce<true>, dim3(a.Hkv * a.B), dim3(256), 0, st, a, nch);
    else
        hipLaunchKernelGGL(sink_tail_reduce<false>, dim3(a.Hkv * a.B), dim3(256), 0, st, a, nch);
    PK_HIP(hipGetLastError());
    return PK_OK;
}

int launch_mfma_dkdv2(const AttnArgs& a, hipStream_t st) {
    if (a.dk_dim == 128) return a.grad_f32 ? launch<128, true>(a, st) : launch<128, false>(a, st);
    return a.grad_f32 ? launch<64, true>(a, st) : launch<64, false>(a, st);
}

}  // namespace pk
