// bf16 GEMM on the gfx950 matrix cores for the Linear layers of the Llama block: the MI355X counterpart of the
// reference's tiled GEMM with transpose flags (paperkiln src/cuda_resident.cu:141-171, entry step_resident_gemm
// :226-263, reached through device::gemm, src/device.cpp:91-125).
//
//   C[M, N] (+)= op(A) op(B),   row-major, bf16 operands, fp32 accumulation, C in bf16 or fp32
//
// One workgroup of four wavefronts owns a 128 x 128 tile of C and walks the contraction in slices of 64; each
// wavefront owns 64 x 64 of it as 2 x 2 accumulators of v_mfma_f32_32x32x16_bf16. Operand tiles are staged in LDS,
// double-buffered, one barrier per slice, the next slice's global loads in flight while the current one is
// multiplied. An operand whose contraction index is contiguous in memory (A of "N", B of "T") is kept as
// [row][k] with a pitch of 72 elements and read with 16-byte row reads; one whose contraction index is the row
// index in memory (A of "T", B of "N") is kept as [k][column] with a pitch of 160 and read with
// ds_read_b64_tr_b16, so no operand is ever transposed in memory. Both pitches are conflict-free for their read.
// The product is formed as C^T (the B fragment in the MFMA's A slot), which leaves each lane with runs of four
// consecutive columns of one row of C; the tile then goes through LDS once so that the global stores are whole
// 16-byte chunks of consecutive columns.
//
// Long contractions with a small result (weight gradients over all tokens) are cut along the contraction axis
// into slices that separate workgroups multiply into fp32 partial tiles; the partial tiles are added in slice
// order by a second kernel -- no atomics, the same bits on every run.
#include <algorithm>
#include <memory>
#include <type_traits>

#include "mfma_common.h"
#include "tensor.h"

namespace pk {
namespace {

constexpr int BK = 64;
constexpr int PITCH_ROW = BK + 8;  // [rows][64 k]: 16-byte row reads conflict-free

// Tile geometry: WGM x WGN wavefronts, each owning FM x FN accumulators of 32 x 32.
//   Small: 2 x 2 wavefronts of 2 x 2 -> 128 x 128, 256 threads, two workgroups per CU. For outputs of a few
//          hundred tiles, where more and smaller workgroups fill the chip better.
//   Large: 2 x 4 wavefronts of 4 x 2 -> 256 x 256, 512 threads, one workgroup per CU: half the operand bytes per
//          MFMA, which is what the vector memory path (64 bytes per clock and CU) asks for on long runs.
//   KS > 1 (ring kernel only): KS sets of WGM x WGN wavefronts share the tile, set q multiplying the q-th part of every
//          64-deep slice; their accumulators are added through LDS at the end. Two wavefronts per SIMD from one
//          workgroup, for outputs of so few tiles that a CU gets no second workgroup.
template <int WGM_, int WGN_, int FM_, int FN_, int KS_ = 1>
struct Geo {
    static constexpr int WGM = WGM_, WGN = WGN_, FM = FM_, FN = FN_, KS = KS_;
    static constexpr int BM = WGM * FM * 32, BN = WGN * FN * 32, NTHR = WGM * WGN * KS * 64;
    // [64 k][columns] tiles: a pitch of 32 past a multiple of 128 keeps the transposing reads conflict-free
    static constexpr int PITCH_TR_A = BM + 32, PITCH_TR_B = BN + 32;
    static constexpr int A_EL = BM * PITCH_ROW > BK * PITCH_TR_A ? BM * PITCH_ROW : BK * PITCH_TR_A;
    static constexpr int B_EL = BN * PITCH_ROW > BK * PITCH_TR_B ? BN * PITCH_ROW : BK * PITCH_TR_B;
    static constexpr int CH_A = BM * BK / 8 / NTHR, CH_B = BN * BK / 8 / NTHR;  // 16-byte chunks per thread and slice
};
using GeoSmall = Geo<2, 2, 2, 2>;
using GeoLarge = Geo<2, 4, 4, 2>;
using GeoSmallK2 = Geo<2, 2, 2, 2, 2>;

struct GemmArgs {
    const uint16_t* a;
    const uint16_t* b;
    void* c;
    int M, N, K;
    int64_t lda, ldb, ldc;
    int beta;         // 0: C = product, 1: C = D + product
    const void* d;    // D of beta 1: C's type and row pitch; null = C itself (C += product)
    int k_per_split;  // contraction elements per blockIdx.z (a multiple of BK); K when not split
    int64_t part_stride;  // elements between the fp32 partial results of two slices (split only)
    int tiles_m, tiles_n;
    int splits;  // slices of the contraction (gemm_ring walks them itself; gemm_bf16 takes them from blockIdx.z)
};

// What the two passes of the tied head's cross-entropy do with a tile of logits instead of storing it (gemm_ring's
// EPI parameter). Pass 1: per row and per 64-column span of a wavefront, the span's maximum and its sum of
// exp(z - maximum), to stats[span][row], and the target column's logit to zt[row]. Pass 2: the same tile formed
// again, turned into dlogits = (exp(z - row_max) row_inv - [column == target]) gscale and stored as bf16.
struct HeadArgs {
    const int* target;     // [M]
    float2* stats;         // pass 1: [spans][M]
    float* zt;             // pass 1: [M]
    const float* row_max;  // pass 2: [M]
    const float* row_inv;  // pass 2: [M], 1 / sum_j exp(z_j - row_max)
    float gscale;          // pass 2
};
constexpr float LOG2E = 1.4426950408889634f;

// Several products of one launch (gemm_ring's EPI 3): C_p (+)= op(A_p) op(B_p), p < count, all with the contraction
// length, transposition flags and result type of the launch; the workgroups walk the tiles of all of them as one
// sequence (problem after problem, each row by row). For products that are each too small to fill the chip and would
// otherwise each cut their contraction into slices and add partial results afterwards.
constexpr int GROUP_MAX = 8;
struct GroupArgs {
    int count;
    int tile_end[GROUP_MAX];  // tiles of problems 0 .. p
    const uint16_t* a[GROUP_MAX];
    const uint16_t* b[GROUP_MAX];
    void* c[GROUP_MAX];
    int M[GROUP_MAX], N[GROUP_MAX], tiles_n[GROUP_MAX];
    int lda[GROUP_MAX], ldb[GROUP_MAX], ldc[GROUP_MAX];
};

// Transposing operand read in natural k order: lane (c32, g) receives rows row0 + 8g .. 8g + 7 of column
// col0 + c32 of a [k][column] tile.
__device__ inline bf16x8 read_tr_nat(const uint16_t* tile, int pitch, int row0, int col0, int lane) {
    const int g = lane >> 5, u = (lane >> 4) & 1, j = lane & 15;
    const uint16_t* p = tile + (row0 + 8 * g + (j >> 2)) * pitch + col0 + 16 * u + 4 * (j & 3);
    const s16x4 lo = lds_read_tr4(p), hi = lds_read_tr4(p + 4 * pitch);
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return *reinterpret_cast<const bf16x8*>(&v);
}

// One operand tile of the slice starting at k0: global -> registers (NCH 16-byte chunks per thread).
// TR = false: memory is [row][k] (rows = the SPAN rows / columns of C this tile covers);
// TR = true:  memory is [k][column].
template <bool TR, int SPAN, int NTHR, int NCH>
__device__ inline void fetch_tile(const uint16_t* base, int64_t ld, int rc0, int rc_count, int k0, int k_end, u32x4 (&r)[NCH]) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = static_cast<int>(threadIdx.x) + NTHR * i;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        if (!TR) {
            const int row = c >> 3, ch = c & 7;
            const bool ok = rc0 + row < rc_count && k0 + ch * 8 < k_end;
            r[i] = ok ? *reinterpret_cast<const u32x4*>(base + static_cast<int64_t>(rc0 + row) * ld + k0 + ch * 8) : zero;
        } else {
            constexpr int CPR = SPAN / 8;
            const int row = c / CPR, ch = c % CPR;
            const bool ok = k0 + row < k_end && rc0 + ch * 8 < rc_count;
            r[i] = ok ? *reinterpret_cast<const u32x4*>(base + static_cast<int64_t>(k0 + row) * ld + rc0 + ch * 8) : zero;
        }
    }
}
template <bool TR, int SPAN, int NTHR, int NCH>
__device__ inline void commit_tile(uint16_t* tile, const u32x4 (&r)[NCH]) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = static_cast<int>(threadIdx.x) + NTHR * i;
        if (!TR) {
            *reinterpret_cast<u32x4*>(tile + (c >> 3) * PITCH_ROW + (c & 7) * 8) = r[i];
        } else {
            constexpr int CPR = SPAN / 8;
            *reinterpret_cast<u32x4*>(tile + (c / CPR) * (SPAN + 32) + (c % CPR) * 8) = r[i];
        }
    }
}

// Epilogue through LDS, one strip of 32 rows per wavefront row at a time: the strip as [WGM * 32][BN + pad]
// in the output's element type, then 16-byte chunks of consecutive columns to global memory (read-add-write
// when accumulating). `lds` is the kernel's whole LDS allocation, free to overwrite when this is called.
template <typename G, bool CF32>
__device__ inline void store_tile(const f32x16 (&acc)[G::FM][G::FN], void* lds, const GemmArgs& g, int m0, int n0, int wm, int wn,
                                  int c32, int gh, bool writer = true) {
    constexpr int BN = G::BN, NTHR = G::NTHR, FM = G::FM, FN = G::FN;
    typedef typename std::conditional<CF32, float, uint16_t>::type CT;
    constexpr int CP = BN + (CF32 ? 4 : 8);  // pitch in elements: rows stay 16-byte aligned
    constexpr int EPC = CF32 ? 4 : 8;        // elements per 16-byte chunk
    constexpr int CPR = BN / EPC;            // chunks per strip row
    CT* cs = reinterpret_cast<CT*>(lds);
    CT* cout = static_cast<CT*>(g.c) + (g.part_stride ? static_cast<int64_t>(blockIdx.z) * g.part_stride : 0);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                if (!writer) continue;  // wavefront-uniform: the wavefronts that hold the tile's sums
                const int row = wm * 32 + c32, col = (wn * FN + j) * 32 + qd * 8 + gh * 4;
                if (CF32) {
                    const f32x4 v = {acc[i][j][qd * 4], acc[i][j][qd * 4 + 1], acc[i][j][qd * 4 + 2], acc[i][j][qd * 4 + 3]};
                    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(cs) + row * CP + col) = v;
                } else {
                    const u32x2 v = {pack_bf16(acc[i][j][qd * 4], acc[i][j][qd * 4 + 1]),
                                     pack_bf16(acc[i][j][qd * 4 + 2], acc[i][j][qd * 4 + 3])};
                    *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(cs) + row * CP + col) = v;
                }
            }
        __syncthreads();
        for (int c = threadIdx.x; c < G::WGM * 32 * CPR; c += NTHR) {
            const int srow = c / CPR, ch = c % CPR;
            // strip row srow belongs to wavefront row srow / 32, whose i-th block of 32 rows this is
            const int m = m0 + ((srow >> 5) * FM + i) * 32 + (srow & 31), n = n0 + ch * EPC;
            if (m >= g.M || n >= g.N) continue;
            u32x4 v = *reinterpret_cast<const u32x4*>(cs + srow * CP + ch * EPC);
            CT* dst = cout + static_cast<int64_t>(m) * g.ldc + n;
            if (g.beta) {
                const u32x4 old = *reinterpret_cast<const u32x4*>(dst);
                if (CF32) {
                    f32x4 s = *reinterpret_cast<const f32x4*>(&old) + *reinterpret_cast<const f32x4*>(&v);
                    v = *reinterpret_cast<const u32x4*>(&s);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float lo = __uint_as_float(old[e] << 16) + __uint_as_float(v[e] << 16);
                        const float hi = __uint_as_float(old[e] & 0xffff0000u) + __uint_as_float(v[e] & 0xffff0000u);
                        v[e] = pack_bf16(lo, hi);
                    }
                }
            }
            *reinterpret_cast<u32x4*>(dst) = v;
        }
        __syncthreads();
    }
}

template <typename G, bool TA, bool TB, bool CF32>
__global__ __launch_bounds__(G::NTHR, 2) void gemm_bf16(GemmArgs g) {
    constexpr int BM = G::BM, BN = G::BN, NTHR = G::NTHR, FM = G::FM, FN = G::FN;
    __shared__ __attribute__((aligned(16))) uint16_t lds[2 * (G::A_EL + G::B_EL)];  // [buffer][A | B]
    static_assert(G::WGM * 32 * (G::BN + 8) * (CF32 ? 4 : 2) <= sizeof(lds), "epilogue strip must fit the tile buffers");
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c32 = lane & 31, gh = lane >> 5, wm = w / G::WGN, wn = w % G::WGN;

    // XCD-aware tile order: workgroup ids go round-robin over the 8 XCDs, so XCD x takes the x-th eighth of the
    // tile list (columns fastest): the tiles that share rows of A meet in one L2.
    const int ntiles = g.tiles_m * g.tiles_n;
    const int per_xcd = (ntiles + 7) / 8;
    const int t = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (t >= ntiles) return;
    const int m0 = (t / g.tiles_n) * BM, n0 = (t % g.tiles_n) * BN;
    const int k_begin = blockIdx.z * g.k_per_split, k_end = min(g.K, k_begin + g.k_per_split);

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 ra[G::CH_A], rb[G::CH_B];
    // A: !TA [M][K] row form; TA [K][M] transposed form.  B: TB [N][K] row form; !TB [K][N] transposed form.
    fetch_tile<TA, BM, NTHR, G::CH_A>(g.a, g.lda, m0, g.M, k_begin, k_end, ra);
    fetch_tile<!TB, BN, NTHR, G::CH_B>(g.b, g.ldb, n0, g.N, k_begin, k_end, rb);
    commit_tile<TA, BM, NTHR, G::CH_A>(lds, ra);
    commit_tile<!TB, BN, NTHR, G::CH_B>(lds + G::A_EL, rb);
    __syncthreads();

    int buf = 0;
    for (int k0 = k_begin; k0 < k_end; k0 += BK) {
        const bool more = k0 + BK < k_end;
        if (more) {
            fetch_tile<TA, BM, NTHR, G::CH_A>(g.a, g.lda, m0, g.M, k0 + BK, k_end, ra);
            fetch_tile<!TB, BN, NTHR, G::CH_B>(g.b, g.ldb, n0, g.N, k0 + BK, k_end, rb);
        }
        const uint16_t* As = lds + buf * (G::A_EL + G::B_EL);
        const uint16_t* Bs = As + G::A_EL;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            bf16x8 fa[FM], fb[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i)
                fa[i] = TA ? read_tr_nat(As, G::PITCH_TR_A, kk * 16, (wm * FM + i) * 32, lane)
                           : lds_read8(As + ((wm * FM + i) * 32 + c32) * PITCH_ROW + kk * 16 + gh * 8);
#pragma unroll
            for (int j = 0; j < FN; ++j)
                fb[j] = !TB ? read_tr_nat(Bs, G::PITCH_TR_B, kk * 16, (wn * FN + j) * 32, lane)
                            : lds_read8(Bs + ((wn * FN + j) * 32 + c32) * PITCH_ROW + kk * 16 + gh * 8);
            // C^T blocks: rows = columns of C (from B), lane = row of C (from A)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = mfma32(fb[j], fa[i], acc[i][j]);
        }
        if (more) {
            uint16_t* nxt = lds + (buf ^ 1) * (G::A_EL + G::B_EL);
            commit_tile<TA, BM, NTHR, G::CH_A>(nxt, ra);
            commit_tile<!TB, BN, NTHR, G::CH_B>(nxt + G::A_EL, rb);
        }
        __syncthreads();
        buf ^= 1;
    }

    store_tile<G, CF32>(acc, lds, g, m0, n0, wm, wn, c32, gh);
}

// ---- the same tiles fed through a ring of LDS slots ---------------------------------------------------------------
// With one workgroup per CU (an output of 256 tiles or fewer, or tiles whose buffers fill the LDS) a slice's global
// loads have one slice of matrix work to hide behind, 512 clocks against a round trip of 1,500 - 2,000, and a loop
// that spends four scalar instructions per matrix instruction on addresses and branches is bound by instruction
// issue. Here the operand slices go from memory straight into LDS (buffer_load_dwordx4 ... lds: no staging
// registers, no LDS stores, a lane outside the buffer writes zeros), into a ring of NS slots; the loads of slice
// s + NS - 1 are issued before slice s is multiplied; a tile's buffer descriptors are formed once and the position
// in the contraction is the instruction's scalar offset (which the hardware counts in its range check); the slice
// loop is unrolled over the ring, so every LDS address is a register formed once plus an immediate.
//
// One load instruction fills 1 KB of LDS lane after lane, so a lane's place in LDS is fixed and what varies is which
// 16 bytes of memory it fetches. The tiles are therefore not padded but swizzled:
//   [row][64 k] operand (A of "N", B of "T"), rows of 128 bytes = 8 chunks: chunk c of row r lies at chunk
//     c ^ ((r & 7) ^ ((r >> 3) & 3)) of its row. The 16 rows a quarter-wavefront reads with one 16-byte row read
//     then cover all 64 banks once (and any 8 consecutive rows 32 banks once).
//   [64 k][columns] operand (A of "T", B of "N"), rows of 2 * SPAN bytes: the 64-byte segment s of row r lies at
//     segment s ^ (r & 3) within its group of four. The 4 rows x 64 bytes a half-wavefront reads with one
//     transposing read then cover all 64 banks once.
template <bool TR, int SPAN, int NW>
struct RingOp {
    static constexpr int CPR = TR ? SPAN / 8 : BK / 8;    // 16-byte chunks per LDS row
    static constexpr int ROWS = TR ? BK : SPAN;
    static constexpr int ROWB = CPR * 16;                 // bytes per LDS row
    static constexpr int NI = ROWS * CPR / 64;            // wavefront loads per slice
    static_assert(NI % NW == 0, "every wavefront issues the same number of loads");
    static constexpr int PER = NI / NW;                   // consecutive 1 KB pieces per wavefront
    static_assert(PER == 2 || PER == 4, "one m0 value and immediate offsets below 4096 per group");
    static constexpr int BYTES = NI * 1024;
    // the chunk of its LDS row that holds memory chunk c (and vice versa: the map is an involution)
    __device__ static int swz(int r, int c) { return TR ? c ^ ((r & 3) << 2) : c ^ ((r & 7) ^ ((r >> 3) & 3)); }
};
// Descriptor of an operand's tile: from BIAS bytes before the tile's first element of the contraction range to the
// operand's end (rows past the matrix, and rows past the contraction's end where the contraction index is the row,
// read as zeros); `step` bytes per slice.
struct TileDesc {
    u32x4 rsrc;
    int step;
};
template <bool TR>
__device__ inline TileDesc tile_desc(const uint16_t* base, int64_t ld, int rc0, int rc_count, int k_begin, int k_end) {
    const int64_t kspan = k_end - k_begin, rcs = rc_count - rc0;
    const char* p;
    int64_t left;
    TileDesc d;
    if (!TR) {  // [row][k]
        p = reinterpret_cast<const char*>(base + static_cast<int64_t>(rc0) * ld + k_begin);
        left = ((rcs - 1) * ld + kspan) * 2;
        d.step = BK * 2;
    } else {  // [k][column]
        p = reinterpret_cast<const char*>(base + static_cast<int64_t>(k_begin) * ld + rc0);
        left = ((kspan - 1) * ld + rcs) * 2;
        d.step = static_cast<int>(BK * ld * 2);
    }
    const uint64_t a = reinterpret_cast<uint64_t>(p) - BIAS;
    d.rsrc[0] = static_cast<uint32_t>(a);
    d.rsrc[1] = static_cast<uint32_t>(a >> 32) & 0xffffu;
    d.rsrc[2] = static_cast<uint32_t>(left + BIAS);
    d.rsrc[3] = 0x00020000u;
    return d;
}
template <int N>
__device__ inline void wait_loads_then_barrier() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}
// lane offsets of a wavefront's loads of one operand's slice, for a tile in the matrix's interior (every column there,
// every slice whole)
template <typename O>
__device__ inline void lane_offsets(uint32_t (&off)[O::PER], int w, int lane, int64_t ld) {
#pragma unroll
    for (int j = 0; j < O::PER; ++j) {
        const int u = (w * O::PER + j) * 64 + lane, r = u / O::CPR, c = O::swz(r, u % O::CPR);
        off[j] = static_cast<uint32_t>(r) * static_cast<uint32_t>(ld) * 2u + c * 16u + BIAS - j * 1024u;
    }
}
// ... and with the chunks that must not be read sent outside the buffer: columns past the matrix's edge of a
// [k][column] operand (every slice of an edge tile), chunks past the contraction's end in the last, partial slice of
// a [row][k] operand (they are the next row's)
template <typename O, bool TR>
__device__ inline void lane_offsets_masked(uint32_t (&off)[O::PER], const uint32_t (&whole)[O::PER], int w, int lane, int rc0,
                                           int rc_count, int ktail) {
#pragma unroll
    for (int j = 0; j < O::PER; ++j) {
        const int u = (w * O::PER + j) * 64 + lane, r = u / O::CPR, c = O::swz(r, u % O::CPR);
        const bool ok = TR ? rc0 + c * 8 < rc_count : (ktail == 0 || c * 8 < ktail);
        off[j] = ok ? whole[j] : OUTSIDE;
    }
}
__device__ inline void store16(u32x4 v, uint32_t off, u32x4 rsrc, uint32_t soff) {
    // invisible to the compiler's count of memory operations in flight, like the loads above; the data registers
    // may be overwritten by the very next instruction, which a 16-byte store does not allow: one idle state
    asm volatile("buffer_store_dwordx4 %0, %1, %2, %3 offen\n\ts_nop 0" ::"v"(v), "v"(off), "s"(rsrc), "s"(soff) : "memory");
}
// What a workgroup stores per tile, for the count of memory operations in flight: FM strips of all WGM * 32 rows
// (bf16) or FM * WGM strips of 32 rows (fp32, whose wider rows would not fit a ring slot otherwise), each
// rows * chunks-per-row / threads stores per thread.
template <typename G, bool CF32>
struct TileStore {
    static constexpr int EPC = CF32 ? 4 : 8;  // elements per 16-byte chunk
    static constexpr int CPR = G::BN / EPC;   // chunks per strip row
    static constexpr int SR = CF32 ? 32 : G::WGM * 32;
    static constexpr int PHASES = CF32 ? G::FM * G::WGM : G::FM;
    static_assert(SR * CPR % G::NTHR == 0 && G::NTHR % CPR == 0, "whole stores per thread, one chunk column per thread");
    static constexpr int PER_PHASE = SR * CPR / G::NTHR;
    static constexpr int NST = PHASES * PER_PHASE;
    static constexpr int CP = G::BN + EPC;  // strip pitch in elements: rows stay 16-byte aligned, writes conflict-free
    static constexpr int BYTES = SR * CP * (CF32 ? 4 : 2);
};

// C = op(A) op(B), persistent: gridDim.x workgroups walk the virtual blocks v = blockIdx.x, + gridDim.x, ...
// (virtual block -> (contraction slice, tile) as gemm_bf16 maps (blockIdx.z, blockIdx.x), XCD by XCD), and the ring
// runs on across tile boundaries: the first slices of the next tile are on their way while the last ones of this tile
// are multiplied and its result is stored, so a tile's first round trip to memory is paid once per workgroup.
template <typename G, bool TA, bool TB, bool CF32, int NS, bool SPREAD, int EPI = 0>
__global__ __launch_bounds__(G::NTHR, NS * (RingOp<TA, G::BM, G::NTHR / 64>::BYTES + RingOp<!TB, G::BN, G::NTHR / 64>::BYTES) <= 80 * 1024 ? 2 : 1)
void gemm_ring(GemmArgs g, HeadArgs hd, GroupArgs gr) {
    static_assert(EPI == 0 || EPI == 3 || (G::KS == 1 && !CF32), "the head's epilogues: one wavefront set, bf16 result");
    constexpr bool GROUPED = EPI == 3;
    constexpr int BM = G::BM, BN = G::BN, NTHR = G::NTHR, FM = G::FM, FN = G::FN, NW = NTHR / 64;
    using OA = RingOp<TA, BM, NW>;
    using OB = RingOp<!TB, BN, NW>;
    using ST = TileStore<G, CF32>;
    constexpr int SLOT = OA::BYTES + OB::BYTES, PERTOT = OA::PER + OB::PER;
    static_assert(NS >= 2 && NS * SLOT <= 160 * 1024, "the ring must fit the LDS");
    static_assert(ST::BYTES <= SLOT, "an epilogue strip must fit one ring slot");
    static_assert((NS - 2) * PERTOT + ST::NST < 64, "memory operations in flight must fit the counter");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[NS * SLOT];
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int KS = G::KS, NWQ = G::WGM * G::WGN, KPW = BK / 16 / KS;  // k-chunks of a slice per wavefront
    static_assert(KS == 1 || KS == 2, "one or two wavefront sets");
    static_assert(KS == 1 || (FM % 2 == 0 && NWQ * 64 * (FM / 2) * FN * 64 <= SLOT), "half of the second set's sums per slot");
    const int ks = KS == 1 ? 0 : w / NWQ, wq = w - ks * NWQ;
    const int c32 = lane & 31, gh = lane >> 5, wm = wq / G::WGN, wn = wq % G::WGN;

    // Virtual blocks: u = slice z of the contraction, then tile t row by row; XCD x (workgroups with blockIdx % 8 == x)
    // takes the x-th eighth of that sequence, so the workgroups that run on an XCD at one time work on one slice of
    // the contraction -- they stream the same rows of both operands through the XCD's L2 (the weight-gradient products
    // of a d = 512 block fetch 40 MB instead of 89 and run 6 - 10 % faster than with every slice spread over all XCDs)
    // -- and on whole rows of tiles. (Walking tiles in blocks of 4 or 8 rows instead halves what the L2s fetch for
    // [4096, 32000] x 512, 543 -> ~270 MB, and changes its time by nothing -- the last-level cache serves those misses
    // at 7 TB/s -- while [8192, 2752] x 512, whose weight matrix fits an L2 whole, loses 20 %.)
    const int ntiles = GROUPED ? gr.tile_end[gr.count - 1] : g.tiles_m * g.tiles_n;
    const int total = ntiles * g.splits, per_xcd = (total + 7) / 8, V = per_xcd * 8;
    const int stride = static_cast<int>(gridDim.x);
    struct Block {
        int m0, n0, k_begin, k_end, z, p;  // p: which problem of a grouped launch
    };
    auto next_block = [&](int v, Block& bl) {  // first virtual block at or after v (in steps of the grid) that is a tile
        for (; v < V; v += stride) {
            const int u = (v & 7) * per_xcd + (v >> 3);
            if (u >= total) continue;
            const int z = u / ntiles;
            int t = u - z * ntiles, p = 0, tiles_n = g.tiles_n;
            if (GROUPED) {
                while (t >= gr.tile_end[p]) ++p;
                if (p > 0) t -= gr.tile_end[p - 1];
                tiles_n = gr.tiles_n[p];
            }
            const int tm = t / tiles_n;
            bl.m0 = tm * BM;
            bl.n0 = (t - tm * tiles_n) * BN;
            bl.z = z;
            bl.p = p;
            bl.k_begin = z * g.k_per_split;
            bl.k_end = min(g.K, bl.k_begin + g.k_per_split);
            return v;
        }
        return V;
    };
    // the operands and sizes of the problem a block belongs to
    struct Prob {
        const uint16_t* a;
        const uint16_t* b;
        void* c;
        int M, N;
        int64_t lda, ldb, ldc;
    };
    auto prob = [&](const Block& bl) -> Prob {
        if (GROUPED) return Prob{gr.a[bl.p], gr.b[bl.p], gr.c[bl.p], gr.M[bl.p], gr.N[bl.p], gr.lda[bl.p], gr.ldb[bl.p], gr.ldc[bl.p]};
        return Prob{g.a, g.b, g.c, g.M, g.N, g.lda, g.ldb, g.ldc};
    };

    // ---- fetch side: a stream of slices, tile after tile ----
    uint32_t offa[OA::PER], offb[OB::PER], offa_c[OA::PER], offb_c[OB::PER];
    if (!GROUPED) {  // a grouped launch forms them per tile: the row pitches are the problem's
        lane_offsets<OA>(offa, w, lane, g.lda);
        lane_offsets<OB>(offb, w, lane, g.ldb);
    }
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
    const uint32_t dst_a = lds0 + w * OA::PER * 1024u, dst_b = lds0 + OA::BYTES + w * OB::PER * 1024u;
    Block fb;
    int fv = next_block(static_cast<int>(blockIdx.x), fb);
    if (fv >= V) return;  // nothing for this workgroup (before any barrier)
    TileDesc da, db;
    int f_slice = 0, f_nslices = 0, f_ktail = 0;
    uint32_t soff_a = 0, soff_b = 0;
    auto open = [&]() {  // the fetch stream enters virtual block fv
        f_slice = 0;
        soff_a = soff_b = 0;
        if (fv >= V) {  // past the last block: descriptors stay, every offset goes outside
            f_nslices = 0;
            return;
        }
        f_nslices = (fb.k_end - fb.k_begin + BK - 1) / BK;
        f_ktail = (fb.k_end - fb.k_begin) % BK;
        const Prob fp = prob(fb);
        if (GROUPED) {
            lane_offsets<OA>(offa, w, lane, fp.lda);
            lane_offsets<OB>(offb, w, lane, fp.ldb);
        }
        da = tile_desc<TA>(fp.a, fp.lda, fb.m0, fp.M, fb.k_begin, fb.k_end);
        db = tile_desc<!TB>(fp.b, fp.ldb, fb.n0, fp.N, fb.k_begin, fb.k_end);
        // the masked lane offsets: used by every slice of a [k][column] operand, by the last slice of a [row][k] one
        if (TA ? fb.m0 + BM > fp.M : f_ktail != 0)
            lane_offsets_masked<OA, TA>(offa_c, offa, w, lane, fb.m0, fp.M, f_ktail);
        else {
#pragma unroll
            for (int j = 0; j < OA::PER; ++j) offa_c[j] = offa[j];
        }
        if (!TB ? fb.n0 + BN > fp.N : f_ktail != 0)
            lane_offsets_masked<OB, !TB>(offb_c, offb, w, lane, fb.n0, fp.N, f_ktail);
        else {
#pragma unroll
            for (int j = 0; j < OB::PER; ++j) offb_c[j] = offb[j];
        }
    };
    // One call per slice of the stream, in order, also past the stream's end: a wavefront's count of loads in flight
    // stays the same, and the scalar offset is then outside every buffer, so nothing is fetched (the lanes write zeros
    // into a slot nobody reads).
    // A slice's loads are issued one by one between the matrix instructions of the slice in hand (all at once they
    // hold a wavefront for 500 clocks in which it issues nothing else, and every wavefront of the workgroup does so at
    // the same time): begin fixes where the slice goes and what it reads, piece<Q> issues its Q-th load, end moves
    // the stream on.
    uint32_t f_la = 0, f_lb = 0, f_sa = 0, f_sb = 0;
    bool f_ca = false, f_cb = false;  // this slice takes the masked lane offsets of A / of B
    auto fetch_begin = [&](int slot) {
        const bool none = f_nslices == 0, last = f_slice == f_nslices - 1;
        f_sa = none ? PAST_END : soff_a;
        f_sb = none ? PAST_END : soff_b;
        f_la = dst_a + static_cast<uint32_t>(slot) * SLOT;
        f_lb = dst_b + static_cast<uint32_t>(slot) * SLOT;
        f_ca = TA || last;
        f_cb = !TB || last;
    };
    auto fetch_piece = [&](auto qc) {
        constexpr int Q = decltype(qc)::value;
        if constexpr (Q < OA::PER) {
            dma_piece<Q>(f_la, f_ca ? offa_c[Q] : offa[Q], da.rsrc, f_sa);
        } else if constexpr (Q < PERTOT) {
            constexpr int J = Q - OA::PER;
            dma_piece<J>(f_lb, f_cb ? offb_c[J] : offb[J], db.rsrc, f_sb);
        }
    };
    auto fetch_end = [&]() {
        const bool none = f_nslices == 0;
        soff_a += da.step;
        soff_b += db.step;
        if (!none && ++f_slice == f_nslices) {
            fv = next_block(fv + stride, fb);
            open();
        }
    };
    auto fetch_pieces = [&](auto first, auto count) {  // pieces first .. first + count - 1
        constexpr int F = decltype(first)::value, N = decltype(count)::value;
        if constexpr (N > 0) {
            fetch_piece(std::integral_constant<int, F>{});
            if constexpr (N > 1) fetch_piece(std::integral_constant<int, F + 1>{});
            if constexpr (N > 2) fetch_piece(std::integral_constant<int, F + 2>{});
            if constexpr (N > 3) fetch_piece(std::integral_constant<int, F + 3>{});
            static_assert(N <= 4, "at most four pieces per k-chunk");
        }
    };
    auto fetch = [&](int slot) {  // the whole slice at once (before the first slice is multiplied)
        fetch_begin(slot);
        fetch_pieces(std::integral_constant<int, 0>{}, std::integral_constant<int, 4>{});
        if constexpr (PERTOT > 4) fetch_pieces(std::integral_constant<int, 4>{}, std::integral_constant<int, PERTOT - 4>{});
        fetch_end();
    };

    // ---- lane parts of the fragment reads ----
    // [row][k]: row c32 of a 32-row block, chunk 2 kk + gh, one address per kk (the swizzle is an exclusive-or with a
    // lane value, so kk cannot be an immediate); [k][column]: rows 8 gh + j / 4 (+ 4), columns 16 u + 4 (j % 4) of
    // 32-column block b, one address per block the wavefront reads.
    const int tj = lane & 15, tu = (lane >> 4) & 1;
    uint32_t r_row[KPW], ra_tr[FM], rb_tr[FN];  // r_row: for this wavefront's own k-chunks ks KPW .. ks KPW + KPW - 1
#pragma unroll
    for (int kq = 0; kq < KPW; ++kq)
        r_row[kq] = static_cast<uint32_t>(c32 * 128 + (RingOp<false, 128, 4>::swz(c32, 2 * (ks * KPW + kq) + gh)) * 16);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int blk = wm * FM + i, r = 8 * gh + (tj >> 2);
        ra_tr[i] = static_cast<uint32_t>(r * OA::ROWB + (((blk & ~3) | ((blk & 3) ^ (r & 3))) * 32 + 16 * tu + 4 * (tj & 3)) * 2);
    }
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int blk = wn * FN + j, r = 8 * gh + (tj >> 2);
        rb_tr[j] = static_cast<uint32_t>(r * OB::ROWB + (((blk & ~3) | ((blk & 3) ^ (r & 3))) * 32 + 16 * tu + 4 * (tj & 3)) * 2);
    }
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    auto read_tr = [](const uint8_t* p, int rowb) -> bf16x8 {
        const s16x4 lo = lds_read_tr4(reinterpret_cast<const uint16_t*>(p));
        const s16x4 hi = lds_read_tr4(reinterpret_cast<const uint16_t*>(p + 4 * rowb));
        const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return *reinterpret_cast<const bf16x8*>(&v);
    };
    auto read_a = [&](const uint8_t* As, int i, int kq, int kk) -> bf16x8 {
        if (!TA) return lds_read8(reinterpret_cast<const uint16_t*>(As + r_row[kq] + (wm * FM + i) * 32 * 128));
        return read_tr(As + ra_tr[i] + kk * 16 * OA::ROWB, OA::ROWB);
    };
    auto read_b = [&](const uint8_t* Bs, int j, int kq, int kk) -> bf16x8 {
        if (TB) return lds_read8(reinterpret_cast<const uint16_t*>(Bs + r_row[kq] + (wn * FN + j) * 32 * 128));
        return read_tr(Bs + rb_tr[j] + kk * 16 * OB::ROWB, OB::ROWB);
    };

    // ---- epilogue: lane parts of the stores (tile-relative), formed once ----
    typedef typename std::conditional<CF32, float, uint16_t>::type CT;
    constexpr int ES = CF32 ? 4 : 2;
    const int st_ch = static_cast<int>(threadIdx.x) % ST::CPR;  // the chunk column this thread stores in every strip
    uint32_t coff[ST::PER_PHASE];
#pragma unroll
    for (int k = 0; k < ST::PER_PHASE; ++k) {
        const int srow = (static_cast<int>(threadIdx.x) + k * NTHR) / ST::CPR;
        // bf16 strips hold the i-th 32-row block of every wavefront row: strip row -> tile row (srow / 32) FM 32 + srow % 32
        const int trow = CF32 ? srow : (srow >> 5) * FM * 32 + (srow & 31);
        coff[k] = (static_cast<uint32_t>(trow) * static_cast<uint32_t>(g.ldc) + st_ch * ST::EPC) * ES;  // (not grouped)
    }

    f32x16 acc[FM][FN];
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    };
    // lane (c32, gh) holds, of row (wm FM + i) 32 + c32 of the tile, columns (wn FN + j) 32 + 8 qd + 4 gh + e
    auto head_stats = [&](const Block& bl) {  // EPI 1
        const int span = (bl.n0 / BN) * G::WGN + wn, col0 = bl.n0 + wn * FN * 32 + gh * 4;
        if (bl.n0 + BN > g.N) {  // wavefront-uniform: columns past the matrix count for nothing
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (col0 + j * 32 + (r >> 2) * 8 + (r & 3) >= g.N) acc[i][j][r] = -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const int row = bl.m0 + (wm * FM + i) * 32 + c32;
            // the target's place among this lane's 16 FN sums of the row, if it is there: 16 j + r
            const int tt = (row < g.M ? hd.target[row] : -1) - (bl.n0 + wn * FN * 32);
            const bool has = tt >= 0 && tt < FN * 32 && ((tt >> 2) & 1) == gh && row < g.M;
            const int at = has ? (tt >> 5) * 16 + ((tt >> 3) & 3) * 4 + (tt & 3) : -1;
            float mx = -INFINITY, zt = 0.0f;
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    mx = fmaxf(mx, acc[i][j][r]);
                    zt = at == j * 16 + r ? acc[i][j][r] : zt;
                }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float ref = mx == -INFINITY ? 0.0f : mx * LOG2E;  // a span wholly past the last column sums to 0
            float sum = 0.0f;
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) sum += __builtin_amdgcn_exp2f(fmaf(acc[i][j][r], LOG2E, -ref));
            sum += __shfl_xor(sum, 32);
            if (row < g.M && gh == 0) hd.stats[static_cast<int64_t>(span) * g.M + row] = make_float2(mx, sum);
            if (has) hd.zt[row] = zt;
        }
    };
    auto head_dlogits = [&](const Block& bl) {  // EPI 2: the sums become dlogits where they lie
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const int row = bl.m0 + (wm * FM + i) * 32 + c32;
            const bool in = row < g.M;
            const int tt = (in ? hd.target[row] : -1) - (bl.n0 + wn * FN * 32);
            const bool has = tt >= 0 && tt < FN * 32 && ((tt >> 2) & 1) == gh && in;
            // P gscale = exp2(z log2e - (max log2e - log2(gscale / sum))): the scaling rides in the exponent
            const float ref = in ? fmaf(hd.row_max[row], LOG2E, -__builtin_amdgcn_logf(hd.row_inv[row] * hd.gscale)) : 0.0f;
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = __builtin_amdgcn_exp2f(fmaf(acc[i][j][r], LOG2E, -ref));
            if (__builtin_amdgcn_ballot_w64(has) != 0) {  // few wavefronts hold a target column of one of their rows
                const int at = has ? (tt >> 5) * 16 + ((tt >> 3) & 3) * 4 + (tt & 3) : -1;
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] -= at == j * 16 + r ? hd.gscale : 0.0f;
            }
        }
    };
    // the tile's result, through the ring slot `strip` (which every wavefront has finished reading)
    auto store_result = [&](uint8_t* strip, const Block& bl) {
        if (KS == 2) {  // set 1 hands its sums to set 0, half of them at a time: [wavefront][16-byte group][lane]
            f32x4* red = reinterpret_cast<f32x4*>(strip) + wq * ((FM / 2) * FN * 4) * 64 + lane;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                if (ks == 1) {
#pragma unroll
                    for (int i = 0; i < FM / 2; ++i)
#pragma unroll
                        for (int j = 0; j < FN; ++j)
#pragma unroll
                            for (int qd = 0; qd < 4; ++qd) {
                                const f32x16& a = acc[half * (FM / 2) + i][j];
                                const f32x4 v = {a[qd * 4], a[qd * 4 + 1], a[qd * 4 + 2], a[qd * 4 + 3]};
                                red[((i * FN + j) * 4 + qd) * 64] = v;
                            }
                }
                __syncthreads();
                if (ks == 0) {
#pragma unroll
                    for (int i = 0; i < FM / 2; ++i)
#pragma unroll
                        for (int j = 0; j < FN; ++j)
#pragma unroll
                            for (int qd = 0; qd < 4; ++qd) {
                                const f32x4 v = red[((i * FN + j) * 4 + qd) * 64];
#pragma unroll
                                for (int e = 0; e < 4; ++e) acc[half * (FM / 2) + i][j][qd * 4 + e] += v[e];
                            }
                }
                __syncthreads();
            }
        }
        // descriptor of C from the tile's first element on (rows past the matrix are dropped by the range check,
        // columns past it by the lane's offset)
        const Prob cp = prob(bl);
        CT* ctile = static_cast<CT*>(cp.c) + (g.part_stride ? static_cast<int64_t>(bl.z) * g.part_stride : 0) +
                    static_cast<int64_t>(bl.m0) * cp.ldc + bl.n0;
        const int64_t cleft = (static_cast<int64_t>(cp.M - bl.m0 - 1) * cp.ldc + (cp.N - bl.n0)) * ES;
        const uint32_t crec = cleft > 0x7ffffff0 ? 0x7ffffff0u : static_cast<uint32_t>(cleft);
        const uint64_t ca = reinterpret_cast<uint64_t>(ctile);
        const u32x4 crs = {static_cast<uint32_t>(ca), static_cast<uint32_t>(ca >> 32) & 0xffffu, crec, 0x00020000u};
        CT* dtile = g.d ? static_cast<CT*>(const_cast<void*>(g.d)) + static_cast<int64_t>(bl.m0) * cp.ldc + bl.n0 : ctile;
        const __amdgpu_buffer_rsrc_t crs_b = __builtin_amdgcn_make_buffer_rsrc(dtile, 0, static_cast<int>(crec), 0x00020000);
        const uint32_t cmask = bl.n0 + st_ch * ST::EPC < cp.N ? 0u : OUTSIDE;
        CT* cs = reinterpret_cast<CT*>(strip);
#pragma unroll
        for (int ph = 0; ph < ST::PHASES; ++ph) {
            const int i = CF32 ? ph / G::WGM : ph, ws = CF32 ? ph % G::WGM : 0;
            if (ks == 0 && (!CF32 || wm == ws)) {  // wavefront-uniform: the wavefronts that hold this strip's sums
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int qd = 0; qd < 4; ++qd) {
                        const int row = (CF32 ? 0 : wm * 32) + c32, col = (wn * FN + j) * 32 + qd * 8 + gh * 4;
                        if (CF32) {
                            const f32x4 v = {acc[i][j][qd * 4], acc[i][j][qd * 4 + 1], acc[i][j][qd * 4 + 2], acc[i][j][qd * 4 + 3]};
                            *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(cs) + row * ST::CP + col) = v;
                        } else {
                            const u32x2 v = {pack_bf16(acc[i][j][qd * 4], acc[i][j][qd * 4 + 1]),
                                             pack_bf16(acc[i][j][qd * 4 + 2], acc[i][j][qd * 4 + 3])};
                            *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(cs) + row * ST::CP + col) = v;
                        }
                    }
            }
            __syncthreads();
            // rows of C this strip holds start at tile row (ws FM + i) 32 (fp32) or i 32 (bf16, plus the lane's part)
            const uint32_t soff = static_cast<uint32_t>((CF32 ? ws * FM + i : i) * 32) * static_cast<uint32_t>(cp.ldc) * ES;
#pragma unroll
            for (int k = 0; k < ST::PER_PHASE; ++k) {
                const int srow = (static_cast<int>(threadIdx.x) + k * NTHR) / ST::CPR;
                u32x4 v = *reinterpret_cast<const u32x4*>(cs + srow * ST::CP + st_ch * ST::EPC);
                uint32_t off = coff[k];
                if (GROUPED) {  // the row pitch is the problem's
                    const int trow = CF32 ? srow : (srow >> 5) * FM * 32 + (srow & 31);
                    off = (static_cast<uint32_t>(trow) * static_cast<uint32_t>(cp.ldc) + st_ch * ST::EPC) * ES;
                }
                off |= cmask;
                if (g.beta) {
                    const u32x4 old = __builtin_amdgcn_raw_buffer_load_b128(crs_b, static_cast<int>(off), static_cast<int>(soff), 0);
                    if (CF32) {
                        f32x4 s = *reinterpret_cast<const f32x4*>(&old) + *reinterpret_cast<const f32x4*>(&v);
                        v = *reinterpret_cast<const u32x4*>(&s);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float lo = __uint_as_float(old[e] << 16) + __uint_as_float(v[e] << 16);
                            const float hi = __uint_as_float(old[e] & 0xffff0000u) + __uint_as_float(v[e] & 0xffff0000u);
                            v[e] = pack_bf16(lo, hi);
                        }
                    }
                }
                store16(v, off, crs, soff);
            }
            __syncthreads();
        }
    };

    // ---- the stream ----
    open();
    {
        int slot = 0;
        for (int s = 0; s < NS - 1; ++s) fetch(slot++);
    }
    Block cb;  // compute side: the block in hand
    int cv = next_block(static_cast<int>(blockIdx.x), cb);
    int c_slice = 0, c_nslices = (cb.k_end - cb.k_begin + BK - 1) / BK;
    int since_store = NS;  // waits since the last tile's stores were issued; below NS - 1 they are still counted
    zero_acc();
    for (;;) {
        bool done = false;
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            // Slice in hand landed: everything this wavefront issued after that slice's loads may still be in flight
            // -- the loads of NS - 2 later slices and, for the NS - 1 slices asked for before the last tile's
            // stores, those stores (memory operations complete in order).
            if (since_store < NS - 1)
                wait_loads<(NS - 2) * PERTOT + ST::NST>();
            else
                wait_loads<(NS - 2) * PERTOT>();
            since_store = min(since_store + 1, NS);
            barrier();                       // ... for every wavefront, and all have read the slice before
            fetch_begin((u + NS - 1) % NS);  // slice + NS - 1 of the stream goes into the slot the slice before leaves
            const uint8_t* As = lds + u * SLOT;
            const uint8_t* Bs = As + OA::BYTES;
            constexpr int SP = SPREAD ? KPW : 0;
            constexpr int PPK = SP == 0 ? 0 : (PERTOT + SP - 1) / SP;  // loads dropped behind each k-chunk's matrix instructions
            if constexpr (SP == 0) {
                fetch_pieces(std::integral_constant<int, 0>{}, std::integral_constant<int, 4>{});
                if constexpr (PERTOT > 4) fetch_pieces(std::integral_constant<int, 4>{}, std::integral_constant<int, PERTOT - 4>{});
            }
            auto chunk = [&](auto kqc) {
                constexpr int KQ = decltype(kqc)::value;
                const int kk = ks * KPW + KQ;
                bf16x8 fa[FM], fbb[FN];
#pragma unroll
                for (int i = 0; i < FM; ++i) fa[i] = read_a(As, i, KQ, kk);
#pragma unroll
                for (int j = 0; j < FN; ++j) fbb[j] = read_b(Bs, j, KQ, kk);
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j) acc[i][j] = mfma32(fbb[j], fa[i], acc[i][j]);
                constexpr int F = KQ * PPK, N = SP == 0 || F >= PERTOT ? 0 : (F + PPK <= PERTOT ? PPK : PERTOT - F);
                fetch_pieces(std::integral_constant<int, F>{}, std::integral_constant<int, (N > 4 ? 4 : N)>{});
                if constexpr (N > 4) fetch_pieces(std::integral_constant<int, F + 4>{}, std::integral_constant<int, N - 4>{});
            };
            chunk(std::integral_constant<int, 0>{});
            if constexpr (KPW > 1) chunk(std::integral_constant<int, 1>{});
            if constexpr (KPW > 2) chunk(std::integral_constant<int, 2>{});
            if constexpr (KPW > 3) chunk(std::integral_constant<int, 3>{});
            fetch_end();
            if (++c_slice == c_nslices) {  // wavefront-uniform
                if constexpr (EPI == 1) {
                    head_stats(cb);  // nothing goes through the slot, and no store joins the count of loads in flight
                } else {
                    if constexpr (EPI == 2) head_dlogits(cb);
                    barrier();  // every wavefront has read slot u: it takes the result on its way out
                    store_result(lds + u * SLOT, cb);
                    since_store = 0;
                }
                cv = next_block(cv + stride, cb);
                if (cv >= V) {
                    done = true;
                    break;
                }
                c_slice = 0;
                c_nslices = (cb.k_end - cb.k_begin + BK - 1) / BK;
                zero_acc();
            }
        }
        if (done) break;
    }
    wait_loads<0>();  // the zero-filling loads past the end write LDS: they must have landed before the workgroup ends
}

__global__ void sum_slices(const float* part, void* dst, int nparts, int64_t part_stride, int M, int N, int64_t ldc, int beta,
                           int c_f32) {
    const int64_t n4 = static_cast<int64_t>(M) * N / 4;
    for (int64_t i = blockIdx.x * 256LL + threadIdx.x; i < n4; i += static_cast<int64_t>(gridDim.x) * 256) {
        const int64_t e = i * 4, m = e / N, n = e % N;
        f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int p = 0; p < nparts; ++p) s += *reinterpret_cast<const f32x4*>(part + p * part_stride + e);
        if (c_f32) {
            f32x4* d = reinterpret_cast<f32x4*>(static_cast<float*>(dst) + m * ldc + n);
            *d = beta ? *d + s : s;
        } else {
            u32x2* d = reinterpret_cast<u32x2*>(static_cast<uint16_t*>(dst) + m * ldc + n);
            if (beta) {
                const u32x2 o = *d;
                s[0] += __uint_as_float(o[0] << 16);
                s[1] += __uint_as_float(o[0] & 0xffff0000u);
                s[2] += __uint_as_float(o[1] << 16);
                s[3] += __uint_as_float(o[1] & 0xffff0000u);
            }
            const u32x2 v = {pack_bf16(s[0], s[1]), pack_bf16(s[2], s[3])};
            *d = v;
        }
    }
}

// Joins a row's span statistics of the head's first pass, in span order: the row's maximum M, 1 / sum_j exp(z_j - M)
// and its loss -log(max(P_target, 1e-12)) (src/ops.cpp:360-368). 16 rows x 16 groups of spans per block.
__global__ __launch_bounds__(256) void head_rows(const float2* stats, const float* zt, int spans, int M, float* row_max,
                                                 float* row_inv, float* nll) {
    __shared__ float sh_m[16][16], sh_s[16][16];
    const int lr = threadIdx.x & 15, grp = threadIdx.x >> 4, r = blockIdx.x * 16 + lr;
    auto join = [](float& m, float& s, float m2, float s2) {
        const float nm = fmaxf(m, m2), ref = nm == -INFINITY ? 0.0f : nm;
        s = s * __builtin_amdgcn_exp2f((m - ref) * LOG2E) + s2 * __builtin_amdgcn_exp2f((m2 - ref) * LOG2E);
        m = nm;
    };
    float m = -INFINITY, s = 0.0f;
    if (r < M) {
        int p = grp;
        for (; p + 48 < spans; p += 64) {  // four loads in flight, joined in span order
            float2 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = stats[static_cast<int64_t>(p + 16 * u) * M + r];
#pragma unroll
            for (int u = 0; u < 4; ++u) join(m, s, v[u].x, v[u].y);
        }
        for (; p < spans; p += 16) {
            const float2 v = stats[static_cast<int64_t>(p) * M + r];
            join(m, s, v.x, v.y);
        }
    }
    sh_m[grp][lr] = m;
    sh_s[grp][lr] = s;
    __syncthreads();
    if (grp == 0 && r < M) {
        for (int q = 1; q < 16; ++q) join(m, s, sh_m[q][lr], sh_s[q][lr]);
        const float inv = 1.0f / s;
        row_max[r] = m;
        row_inv[r] = inv;
        nll[r] = -logf(fmaxf(__builtin_amdgcn_exp2f((zt[r] - m) * LOG2E) * inv, 1e-12f));
    }
}

template <typename G, bool CF32>
void launch_form(bool tA, bool tB, const GemmArgs& g, dim3 grid, hipStream_t st) {
    if (!tA && !tB) hipLaunchKernelGGL((gemm_bf16<G, false, false, CF32>), grid, dim3(G::NTHR), 0, st, g);
    if (!tA && tB) hipLaunchKernelGGL((gemm_bf16<G, false, true, CF32>), grid, dim3(G::NTHR), 0, st, g);
    if (tA && !tB) hipLaunchKernelGGL((gemm_bf16<G, true, false, CF32>), grid, dim3(G::NTHR), 0, st, g);
    if (tA && tB) hipLaunchKernelGGL((gemm_bf16<G, true, true, CF32>), grid, dim3(G::NTHR), 0, st, g);
}
template <typename G, bool CF32, int NS, bool SPREAD>
void launch_ring_form(bool tA, bool tB, const GemmArgs& g, dim3 grid, hipStream_t st) {
    if (!tA && !tB) hipLaunchKernelGGL((gemm_ring<G, false, false, CF32, NS, SPREAD>), grid, dim3(G::NTHR), 0, st, g, HeadArgs{}, GroupArgs{});
    if (!tA && tB) hipLaunchKernelGGL((gemm_ring<G, false, true, CF32, NS, SPREAD>), grid, dim3(G::NTHR), 0, st, g, HeadArgs{}, GroupArgs{});
    if (tA && !tB) hipLaunchKernelGGL((gemm_ring<G, true, false, CF32, NS, SPREAD>), grid, dim3(G::NTHR), 0, st, g, HeadArgs{}, GroupArgs{});
    if (tA && tB) hipLaunchKernelGGL((gemm_ring<G, true, true, CF32, NS, SPREAD>), grid, dim3(G::NTHR), 0, st, g, HeadArgs{}, GroupArgs{});
}
int cu_count() {
    static const int n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cus <= 0)
            return 256;
        return cus;
    }();
    return n;
}
template <typename G, int NS>
void launch_ring(bool tA, bool tB, GemmArgs g, int S, bool c_f32, hipStream_t st) {
    g.tiles_m = (g.M + G::BM - 1) / G::BM;
    g.tiles_n = (g.N + G::BN - 1) / G::BN;
    g.splits = S;
    // persistent: as many workgroups as the chip holds at once (a multiple of 8, one XCD's share each), or fewer
    constexpr int NW = G::NTHR / 64;
    constexpr int RING = NS * (RingOp<false, G::BM, NW>::BYTES + RingOp<false, G::BN, NW>::BYTES);  // same for every form
    const int64_t vblocks = (static_cast<int64_t>(g.tiles_m) * g.tiles_n * S + 7) / 8 * 8;
    const int64_t slots = static_cast<int64_t>(cu_count()) / 8 * 8 * (RING <= 80 * 1024 ? 2 : 1);
    const unsigned gx = static_cast<unsigned>(std::min(vblocks, slots));
    // When a slice's loads are issued. Spread behind the matrix instructions of the slice in hand they cost no issue
    // time of their own, but the last of them then leaves late: a ring of two slots has only the rest of that slice
    // to cover its latency, which pays where tiles change often (a short contraction, or the large tile whose slices
    // take long) and costs 10 % in the steady state of a long one; three and more slots always have the slack.
    const bool spread = NS > 2 || G::BM > 128 || std::min(g.K, g.k_per_split) <= 768;
    if constexpr (NS > 2 || (G::BM > 128)) {
        if (c_f32)
            launch_ring_form<G, true, NS, true>(tA, tB, g, dim3(gx), st);
        else
            launch_ring_form<G, false, NS, true>(tA, tB, g, dim3(gx), st);
    } else {
        if (c_f32 && spread) launch_ring_form<G, true, NS, true>(tA, tB, g, dim3(gx), st);
        if (c_f32 && !spread) launch_ring_form<G, true, NS, false>(tA, tB, g, dim3(gx), st);
        if (!c_f32 && spread) launch_ring_form<G, false, NS, true>(tA, tB, g, dim3(gx), st);
        if (!c_f32 && !spread) launch_ring_form<G, false, NS, false>(tA, tB, g, dim3(gx), st);
    }
    hip_check(hipGetLastError(), "gemm_ring launch");
}
template <typename G>
void launch_geo(bool tA, bool tB, GemmArgs g, int S, bool c_f32, hipStream_t st) {
    g.tiles_m = (g.M + G::BM - 1) / G::BM;
    g.tiles_n = (g.N + G::BN - 1) / G::BN;
    const unsigned gx = static_cast<unsigned>((g.tiles_m * g.tiles_n + 7) / 8 * 8);
    if (c_f32)
        launch_form<G, true>(tA, tB, g, dim3(gx, 1, static_cast<unsigned>(S)), st);
    else
        launch_form<G, false>(tA, tB, g, dim3(gx, 1, static_cast<unsigned>(S)), st);
    hip_check(hipGetLastError(), "gemm_bf16 launch");
}

bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

int g_force_geo = -1;  // -1: choose by shape; 0 / 1: small / large tiles always (measurement)

}  // namespace

void gemm_mfma_force_tiles(int which) { g_force_geo = which; }

namespace {
// How a product is run: tile geometry and kernel form, and into how many slices the contraction is cut.
struct Plan {
    bool large;  // 256 x 256 tiles
    int ring;    // 0: gemm_bf16 (register-staged tiles); otherwise a gemm_ring form (the numbers of pk_set_gemm_backend)
    int S;       // slices of the contraction, each multiplied into an fp32 partial product of its own
    int kps;     // contraction elements per slice (a multiple of BK)
};
Plan make_plan(bool tA, bool tB, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
    Plan p;
    // Which tiles (measured on the Linear shapes of a d = 512 block and of a 32000-word tied head). 256 x 256 where
    // the output gives nearly every CU a tile of its own and the contraction is long enough to pay for the larger
    // prologue, or where there are tiles for two rounds; 128 x 128 otherwise, two workgroups per CU -- except that an
    // output of at most one such tile per CU with a long contraction takes the two-set form with a deep ring, since
    // no second workgroup would come to share the CU.
    const int64_t tiles_large = ((M + 255) / 256) * ((N + 255) / 256);
    p.large = g_force_geo >= 0 ? (g_force_geo == 1 || g_force_geo == 8) : tiles_large >= 240 && (K >= 1024 || tiles_large >= 512);
    int64_t ntiles = p.large ? tiles_large : ((M + 127) / 128) * ((N + 127) / 128);
    // the ring kernels keep offsets and extents in 32 bits
    const int64_t ext_a = (tA ? K : M) * lda * 2, ext_b = (tB ? N : K) * ldb * 2;
    const int64_t ext_max = (int64_t{1} << 30) - 8192;
    const bool ring_ok = ext_a < ext_max && ext_b < ext_max && lda < (1 << 21) && ldb < (1 << 21) && ldc < (1 << 20);
    p.ring = 0;
    if (ring_ok && g_force_geo >= 5) p.ring = g_force_geo;
    if (ring_ok && g_force_geo < 0) p.ring = p.large ? 8 : (ntiles <= 256 && K >= 1024) ? 11 : 6;
    // Split the contraction when the tiles alone would leave most of the chip idle and the contraction is long: as
    // many slices as give every workgroup the chip holds at once one (tile, slice) -- a second round costs more than
    // longer slices -- but none shorter than 1024, since every slice is another partial product to write and add
    // (measured on [512, 1536], [512, 512], [512, 2752] and [1376, 512] outputs over 8192 tokens and on
    // [2048, 512] over 32000). Split products take 128 x 128 tiles: fewer than 64 of them in the two-set form, one
    // workgroup of eight wavefronts per CU, otherwise two workgroups of four per CU.
    p.S = 1;
    if (ntiles < 192 && K >= 2048) {
        if (ring_ok && g_force_geo < 0) p.ring = ntiles < 64 ? 11 : 6;
        // ... unless 256 x 256 tiles times slices of 1024 or more fill the chip by themselves (dh of a 4096-row head
        // chunk, [4096, 512] over 32000: 144 us against 162)
        const int64_t s_large = std::min<int64_t>({cu_count() / tiles_large, K / 1024, 16});
        if (ring_ok && g_force_geo < 0 && tiles_large * s_large >= 240) {
            p.large = true;
            p.ring = 8;
            ntiles = tiles_large;
        }
        const bool one_per_cu = p.ring == 5 || p.ring == 7 || p.ring == 8 || p.ring == 10 || p.ring == 11;
        const int64_t s = std::min<int64_t>({(one_per_cu ? cu_count() : 2 * cu_count()) / ntiles, K / 1024, 16});
        p.S = static_cast<int>(std::max<int64_t>(s, 1));
    }
    p.kps = static_cast<int>(((K + p.S - 1) / p.S + BK - 1) / BK * BK);
    p.S = static_cast<int>((K + p.kps - 1) / p.kps);
    return p;
}
void run_plan(const Plan& p, bool tA, bool tB, const GemmArgs& ga, int splits, bool f32, hipStream_t st) {
    switch (p.ring) {
        case 5: launch_ring<GeoSmall, 4>(tA, tB, ga, splits, f32, st); break;
        case 6: launch_ring<GeoSmall, 2>(tA, tB, ga, splits, f32, st); break;
        case 7: launch_ring<GeoSmall, 3>(tA, tB, ga, splits, f32, st); break;
        case 8: launch_ring<GeoLarge, 2>(tA, tB, ga, splits, f32, st); break;
        case 9: launch_ring<GeoSmallK2, 2>(tA, tB, ga, splits, f32, st); break;
        case 10: launch_ring<GeoSmallK2, 3>(tA, tB, ga, splits, f32, st); break;
        case 11: launch_ring<GeoSmallK2, 4>(tA, tB, ga, splits, f32, st); break;
        default:
            if (p.large)
                launch_geo<GeoLarge>(tA, tB, ga, splits, f32, st);
            else
                launch_geo<GeoSmall>(tA, tB, ga, splits, f32, st);
    }
}
bool takes(const void* a, bool tA, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return false;
    if (!aligned16(a) || !aligned16(b)) return false;
    if (lda % 8 || ldb % 8 || K % 8 || N % 8) return false;
    if (tA && M % 8) return false;  // A^T is read in 16-byte chunks along M
    return true;
}
GemmArgs gemm_args(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K) {
    GemmArgs g;
    g.a = static_cast<const uint16_t*>(a);
    g.b = static_cast<const uint16_t*>(b);
    g.c = nullptr;
    g.M = static_cast<int>(M), g.N = static_cast<int>(N), g.K = static_cast<int>(K);
    g.lda = lda, g.ldb = ldb, g.ldc = N;
    g.beta = 0;
    g.d = nullptr;
    g.k_per_split = g.K;
    g.part_stride = 0;
    g.tiles_m = g.tiles_n = 0;
    g.splits = 1;
    return g;
}
}  // namespace

// Returns false, having done nothing, for what the kernel does not take (fp32 operands, unaligned rows, sizes
// that are not multiples of 8): the caller then uses the library GEMM.
bool gemm_mfma_bf16(const void* a, bool tA, int64_t lda, const void* b, bool tB, int64_t ldb, void* c, int c_dtype,
                    int64_t M, int64_t N, int64_t K, int64_t ldc, float beta, hipStream_t st, const void* addend) {
    if (!takes(a, tA, lda, b, ldb, M, N, K) || !aligned16(c) || ldc % 8) return false;
    if (beta != 0.0f && beta != 1.0f) return false;
    GemmArgs g = gemm_args(a, lda, b, ldb, M, N, K);
    g.c = c;
    g.ldc = ldc;
    g.beta = beta != 0.0f;
    const Plan p = make_plan(tA, tB, M, N, K, lda, ldb, ldc);
    if (addend) {  // C = addend + product: in the epilogue of the ring kernels, whole contractions only
        if (beta != 1.0f || !aligned16(addend) || p.ring == 0 || p.S != 1) return false;
        g.d = addend;
    }
    if (p.S == 1) {
        run_plan(p, tA, tB, g, 1, c_dtype == PK_F32, st);
        return true;
    }
    Buffer part(sizeof(float) * static_cast<size_t>(p.S) * M * N);
    GemmArgs gp = g;
    gp.c = part.p;
    gp.ldc = N;
    gp.beta = 0;
    gp.k_per_split = p.kps;
    gp.part_stride = M * N;
    run_plan(p, tA, tB, gp, p.S, true, st);
    const int64_t n4 = M * N / 4;
    hipLaunchKernelGGL(sum_slices, dim3(static_cast<unsigned>(std::min<int64_t>((n4 + 255) / 256, 4096))), dim3(256), 0, st,
                       static_cast<const float*>(part.p), c, p.S, M * N, static_cast<int>(M), static_cast<int>(N), ldc,
                       g.beta, c_dtype == PK_F32 ? 1 : 0);
    hip_check(hipGetLastError(), "sum_slices launch");
    return true;
}

// The same product left as its fp32 partial products part[s][M][N], s < nparts (one where the contraction is not
// cut), for a caller that adds them itself on the way to where the result goes.
bool gemm_mfma_bf16_parts(const void* a, bool tA, int64_t lda, const void* b, bool tB, int64_t ldb, int64_t M, int64_t N,
                          int64_t K, hipStream_t st, std::unique_ptr<Buffer>& part, int& nparts) {
    if (!takes(a, tA, lda, b, ldb, M, N, K)) return false;
    const Plan p = make_plan(tA, tB, M, N, K, lda, ldb, N);
    part.reset(new Buffer(sizeof(float) * static_cast<size_t>(p.S) * M * N));
    GemmArgs g = gemm_args(a, lda, b, ldb, M, N, K);
    g.c = part->p;
    g.k_per_split = p.kps;
    g.part_stride = p.S > 1 ? M * N : 0;
    run_plan(p, tA, tB, g, p.S, true, st);
    nparts = p.S;
    return true;
}

// ---- the tied head's cross-entropy inside its logits product ----
namespace {
bool head_takes(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K) {
    if (!takes(a, false, lda, b, ldb, M, N, K)) return false;
    const int64_t ext_max = (int64_t{1} << 30) - 8192;
    return M * lda * 2 < ext_max && N * ldb * 2 < ext_max && lda < (1 << 21) && ldb < (1 << 21) && N < (1 << 20);
}
template <typename G, int EPI>
void launch_head(GemmArgs g, const HeadArgs& hd, hipStream_t st) {
    g.tiles_m = (g.M + G::BM - 1) / G::BM;
    g.tiles_n = (g.N + G::BN - 1) / G::BN;
    g.splits = 1;
    const int64_t vblocks = static_cast<int64_t>((g.tiles_m * g.tiles_n + 7) / 8 * 8);
    const int64_t slots = cu_count() / 8 * 8 * (G::BM > 128 ? 1 : 2);
    const unsigned gx = static_cast<unsigned>(std::min<int64_t>(vblocks, slots));
    hipLaunchKernelGGL((gemm_ring<G, false, true, false, 2, true, EPI>), dim3(gx), dim3(G::NTHR), 0, st, g, hd, GroupArgs{});
    hip_check(hipGetLastError(), "gemm_ring (head) launch");
}
}  // namespace

// 256 x 256 tiles, one workgroup of eight wavefronts per CU (128 x 128 tiles with two workgroups per CU, whose
// epilogues could overlap each other's matrix work, measured 15 % slower on [2048, 32000] x 512)
bool gemm_head_takes(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K) {
    return head_takes(a, lda, b, ldb, M, N, K);
}
int64_t gemm_head_spans(int64_t N) { return (N + GeoLarge::BN - 1) / GeoLarge::BN * GeoLarge::WGN; }

// Pass 1 over logits = A B^T (A [M, K] and B [N, K], bf16), which are formed tile by tile and never stored: per row
// its maximum, 1 / sum exp(z - maximum) and its loss against target[row]. `stats` is scratch of gemm_head_spans(N) * M
// pairs of floats, `zt` of M floats. False, with nothing done, for operands the kernel does not take.
bool gemm_head_rows(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K, const int* target,
                    void* stats, float* zt, float* row_max, float* row_inv, float* nll, hipStream_t st) {
    if (!head_takes(a, lda, b, ldb, M, N, K)) return false;
    GemmArgs g = gemm_args(a, lda, b, ldb, M, N, K);
    HeadArgs hd{};
    hd.target = target;
    hd.stats = static_cast<float2*>(stats);
    hd.zt = zt;
    launch_head<GeoLarge, 1>(g, hd, st);
    hipLaunchKernelGGL(head_rows, dim3(static_cast<unsigned>((M + 15) / 16)), dim3(256), 0, st, hd.stats, zt,
                       static_cast<int>(gemm_head_spans(N)), static_cast<int>(M), row_max, row_inv, nll);
    hip_check(hipGetLastError(), "head_rows launch");
    return true;
}

// Pass 2: the same tiles again, stored as dlogits[M, N] (bf16, row pitch ldc) =
// (exp(z - row_max) row_inv - [column == target]) gscale (src/ops.cpp:371-374).
bool gemm_head_dlogits(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                       const int* target, const float* row_max, const float* row_inv, float gscale, void* dl, int64_t ldc,
                       hipStream_t st) {
    if (!head_takes(a, lda, b, ldb, M, N, K) || !aligned16(dl) || ldc % 8 || ldc >= (1 << 20)) return false;
    GemmArgs g = gemm_args(a, lda, b, ldb, M, N, K);
    g.c = dl;
    g.ldc = ldc;
    HeadArgs hd{};
    hd.target = target;
    hd.row_max = row_max;
    hd.row_inv = row_inv;
    hd.gscale = gscale;
    launch_head<GeoLarge, 2>(g, hd, st);
    return true;
}

// ---- several small weight-gradient products as one launch ----
// C_p += A_p^T B_p, p < count <= GROUP_MAX: A_p [K, M_p] and B_p [K, N_p] bf16 with row pitches lda / ldb, C_p
// [M_p, N_p] fp32 with row pitch ldc, one contraction length K for all. The products of a layer's backward pass
// (X^T dY per weight, K = every token) are each a few dozen 128 x 128 tiles: alone each would cut its contraction into
// slices to fill the chip and add the partial products afterwards; together their tiles fill it with whole
// contractions. False, with nothing done, when an operand is not what the ring kernel takes or the tiles are too few
// to be worth it (the caller then multiplies them one by one).
bool gemm_mfma_grouped_tn(const GroupedProduct* ps, int count, int64_t K, hipStream_t st) {
    if (count < 2 || count > GROUP_MAX || K < 2048) return false;
    GroupArgs gr{};
    gr.count = count;
    int tiles = 0;
    const int64_t ext_max = (int64_t{1} << 30) - 8192;
    for (int p = 0; p < count; ++p) {
        const GroupedProduct& q = ps[p];
        if (!takes(q.a, true, q.lda, q.b, q.ldb, q.M, q.N, K) || !aligned16(q.c) || q.ldc % 4) return false;
        if (K * q.lda * 2 >= ext_max || K * q.ldb * 2 >= ext_max || q.lda >= (1 << 21) || q.ldb >= (1 << 21) || q.ldc >= (1 << 20))
            return false;
        gr.a[p] = static_cast<const uint16_t*>(q.a);
        gr.b[p] = static_cast<const uint16_t*>(q.b);
        gr.c[p] = q.c;
        gr.M[p] = static_cast<int>(q.M);
        gr.N[p] = static_cast<int>(q.N);
        gr.lda[p] = static_cast<int>(q.lda);
        gr.ldb[p] = static_cast<int>(q.ldb);
        gr.ldc[p] = static_cast<int>(q.ldc);
        gr.tiles_n[p] = static_cast<int>((q.N + 127) / 128);
        tiles += static_cast<int>((q.M + 127) / 128) * gr.tiles_n[p];
        gr.tile_end[p] = tiles;
    }
    for (int p = count; p < GROUP_MAX; ++p) gr.tile_end[p] = tiles;
    // worth it from about 3/8 of the CUs busy with whole contractions (measured: 196 tiles x 8192 in 69 us against 132
    // for the same four products one by one); with more tiles than CUs the 4-wavefront form, two workgroups per CU
    if (tiles < cu_count() * 3 / 8) return false;
    GemmArgs g = gemm_args(ps[0].a, ps[0].lda, ps[0].b, ps[0].ldb, ps[0].M, ps[0].N, K);
    g.beta = 1;
    g.splits = 1;
    g.tiles_m = g.tiles_n = 0;
    const int64_t vblocks = (static_cast<int64_t>(tiles) + 7) / 8 * 8;
    if (tiles <= cu_count()) {
        const unsigned gx = static_cast<unsigned>(std::min<int64_t>(vblocks, cu_count() / 8 * 8));
        hipLaunchKernelGGL((gemm_ring<GeoSmallK2, true, false, true, 4, true, 3>), dim3(gx), dim3(GeoSmallK2::NTHR), 0, st, g,
                           HeadArgs{}, gr);
    } else {
        const unsigned gx = static_cast<unsigned>(std::min<int64_t>(vblocks, cu_count() / 8 * 8 * 2));
        hipLaunchKernelGGL((gemm_ring<GeoSmall, true, false, true, 2, false, 3>), dim3(gx), dim3(GeoSmall::NTHR), 0, st, g,
                           HeadArgs{}, gr);
    }
    hip_check(hipGetLastError(), "gemm_ring (grouped) launch");
    return true;
}

}  // namespace pk
