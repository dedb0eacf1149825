// gfx950 (CDNA4) building blocks shared by the bf16 MFMA attention kernels.
//
// v_mfma_f32_32x32x16_bf16 operand layout (64-lane wavefront, g = lane / 32,
// c = lane % 32), verified on hardware:
//   A (32 x 16): lane holds row c,    k = 8g .. 8g+7   (8 bf16, 4 VGPRs)
//   B (16 x 32): lane holds column c, k = 8g .. 8g+7
//   C (32 x 32): lane holds column c, element r (0..15) is row (r/4)*8 + 4g + r%4
// The k index is a summation index, so A and B may use ANY common permutation
// of it. The kernels exploit that: a C tile whose rows are the contraction
// index of the next GEMM is fed back as a B operand directly from registers,
// elements 8h..8h+7 (h = 0, 1) forming one k-chunk, and the other operand is
// fetched with the matching row permutation {4g..4g+3} u {8+4g..8+4g+3}.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define PK_LDS __attribute__((address_space(3)))

__device__ inline f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Exchange a value with lane ^ 32 and combine (v_permlane32_swap: lanes 0..31
// of the second operand trade places with lanes 32..63 of the first).
__device__ inline float xhalf_max(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ inline float xhalf_sum(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Two fp32 -> packed bf16 (v_cvt_pk_bf16_f32, round to nearest even).
__device__ inline uint32_t pack_bf16(float lo, float hi) {
    f32x2 f = {lo, hi};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    return *reinterpret_cast<uint32_t*>(&h);
}

// Elements 8h .. 8h+7 of a C tile as one bf16 k-chunk (a B or A operand).
template <int H>
__device__ inline bf16x8 c_to_operand(const f32x16& c) {
    u32x4 u = {pack_bf16(c[8 * H + 0], c[8 * H + 1]), pack_bf16(c[8 * H + 2], c[8 * H + 3]),
               pack_bf16(c[8 * H + 4], c[8 * H + 5]), pack_bf16(c[8 * H + 6], c[8 * H + 7])};
    return *reinterpret_cast<bf16x8*>(&u);
}

// 16-byte LDS read of 8 consecutive bf16 (ds_read_b128).
__device__ inline bf16x8 lds_read8(const uint16_t* p) {
    return *reinterpret_cast<const bf16x8*>(p);
}

// Transposing LDS read (ds_read_b64_tr_b16). Within each group of 16 lanes,
// lane 4a+c receives element c of the four 8-byte rows addressed by lanes
// a, a+4, a+8, a+12 (verified on hardware). With lane j of a group pointing
// at  tile[row0 + j/4][col0 + 4*(j%4)]  lane i of the group ends up holding
// tile[row0 .. row0+3][col0 + i]: four consecutive ROWS of its own column.
__device__ inline s16x4 lds_read_tr4(const uint16_t* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((PK_LDS s16x4*)(p));
}

// Operand whose k-chunk is rows {row0+4g..+3} u {row0+8+4g..+3} of a row-major
// LDS tile, for the 32 columns col0 .. col0+31 (one per lane c). `stride` is
// the tile's row pitch in elements. Matches c_to_operand's row permutation.
__device__ inline bf16x8 lds_read_tr_operand(const uint16_t* tile, int stride, int row0, int col0,
                                             int lane) {
    const int g = lane >> 5, u = (lane >> 4) & 1, j = lane & 15;
    const uint16_t* p = tile + (row0 + 4 * g + (j >> 2)) * stride + col0 + 16 * u + 4 * (j & 3);
    s16x4 lo = lds_read_tr4(p);
    s16x4 hi = lds_read_tr4(p + 8 * stride);
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return *reinterpret_cast<bf16x8*>(&v);
}

// The same operand read from a tile whose row pitch is 4 banks past a multiple
// of 64 (the pitch that keeps 16-byte row reads conflict-free). With that
// pitch the natural column order would put two of the four rows of a
// transposing read on the same banks, so for head_dim 128 the 32 columns of
// MFMA block `db` are taken in a permuted order: lane 16u + 4a + c reads
// column 4*(8a + u + 2db) + c. Every 32-lane half then touches all 64 banks
// exactly once. The permutation only renames the rows of the product; tr_col0
// gives, for accumulator element group qd (= r/4) of block db on half g, the
// first of the 4 consecutive true columns that elements 4qd..4qd+3 hold.
template <int D>
struct TrMap;
template <>
struct TrMap<128> {
    __device__ static constexpr int src_col(int db, int u, int a) { return 4 * (8 * a + u + 2 * db); }
    __device__ static constexpr int col0(int db, int qd, int g) { return 32 * (2 * (qd & 1) + g) + 4 * (qd >> 1) + 8 * db; }
};
template <>
struct TrMap<64> {  // natural order
    __device__ static constexpr int src_col(int db, int u, int a) { return 32 * db + 16 * u + 4 * a; }
    __device__ static constexpr int col0(int db, int qd, int g) { return 32 * db + 8 * qd + 4 * g; }
};
// One 32 x 32 accumulator block (lane = row c32 of the output, elements 4qd .. 4qd+3 = four consecutive columns from
// TrMap<D>::col0(db, qd, g)) scaled and written as bf16 in 16-byte pieces instead of 8-byte ones: a lane's store is one
// request to the memory pipe whatever its size, and an epilogue of 8-byte pieces spends its time queueing requests.
// At head_dim 128 the pieces qd and qd + 2 of a lane are neighbours (4 columns apart); in the natural order of
// head_dim 64 a lane's neighbour piece sits in lane ^ 32, so pieces qd and qd + 1 trade halves first
// (v_permlane32_swap) and lane half g writes the eight columns from 32 db + 8 (2 qp + g). Both lanes of a pair must
// be active (they hold the same row, so a bound on the row keeps or drops them together).
// natural column order: elements 4qd .. 4qd+3 of half g are columns 32 db + 8 qd + 4 g ..
__device__ inline void store_acc_bf16_natural(uint16_t* row, int db, int g, const f32x16& acc, float sc) {
#pragma unroll
    for (int qp = 0; qp < 2; ++qp) {
        const int lo = qp * 8, hi = qp * 8 + 4;
        const uint32_t a0 = pack_bf16(acc[lo] * sc, acc[lo + 1] * sc), a1 = pack_bf16(acc[lo + 2] * sc, acc[lo + 3] * sc);
        const uint32_t b0 = pack_bf16(acc[hi] * sc, acc[hi + 1] * sc), b1 = pack_bf16(acc[hi + 2] * sc, acc[hi + 3] * sc);
        // (x, y) = swap(a, b): lanes 32..63 of a trade places with lanes 0..31 of b, so half 0 ends up with piece
        // 2qp of both halves and half 1 with piece 2qp + 1 of both
        const auto r0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
        const auto r1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
        u32x4 v = {r0[0], r1[0], r0[1], r1[1]};
        *reinterpret_cast<u32x4*>(row + 32 * db + 8 * (2 * qp + g)) = v;
    }
}
// column order of TrMap<D>
static_assert(TrMap<64>::col0(1, 2, 1) == 32 + 16 + 4 && TrMap<128>::col0(1, 2, 0) == TrMap<128>::col0(1, 0, 0) + 4,
              "head_dim 64 is in natural order; at 128 piece qd + 2 follows piece qd");
template <int D>
__device__ inline void store_acc_bf16(uint16_t* row, int db, int g, const f32x16& acc, float sc) {
    if (D != 128) return store_acc_bf16_natural(row, db, g, acc, sc);
#pragma unroll
    for (int qp = 0; qp < 2; ++qp) {
        const int lo = qp * 4, hi = (qp + 2) * 4;
        u32x4 v = {pack_bf16(acc[lo] * sc, acc[lo + 1] * sc), pack_bf16(acc[lo + 2] * sc, acc[lo + 3] * sc),
                   pack_bf16(acc[hi] * sc, acc[hi + 1] * sc), pack_bf16(acc[hi + 2] * sc, acc[hi + 3] * sc)};
        *reinterpret_cast<u32x4*>(row + TrMap<128>::col0(db, qp, g)) = v;
    }
}

// Where row r of a tile sits in LDS when the tile serves both 16-byte row reads and transposing reads at a pitch
// 4 banks past a multiple of 64. For head_dim 128 rows keep their order (the column permutation above does the
// work). For head_dim 64 a row is only 32 banks wide and no column order makes the four rows of a transposing
// read (r, r+1, r+2, r+3 of a 16-row group, 16 banks each) miss each other at that pitch; instead the rows of each
// 16-row group are stored in the order (4 (q % 4) + 9 (q / 4)) % 16, which puts rows 4i .. 4i+3 at bank offsets
// 16 apart and still gives the sixteen rows of a row read sixteen distinct 4-bank windows.
template <int D>
__device__ constexpr int lds_row(int r) {
    return D == 64 ? (r & ~15) | ((4 * (r & 3) + 9 * ((r >> 2) & 3)) & 15) : r;
}
// In that order the second four rows of a transposed operand (8 query rows on) always sit TR_HI_ROWS<D> LDS rows
// past the first four: (4t + 9g + 18) % 16 = (4t + 9g) % 16 + 2 for every t < 4, g < 2.
template <int D>
constexpr int TR_HI_ROWS = D == 64 ? 2 : 8;
static_assert(lds_row<64>(8 + 4 * 1 + 3) == lds_row<64>(4 * 1 + 3) + 2 && lds_row<64>(8 + 3) == lds_row<64>(3) + 2 &&
              lds_row<64>(8) == lds_row<64>(0) + 2 && lds_row<64>(12) == lds_row<64>(4) + 2, "second half two rows on");
template <int D>
__device__ inline bf16x8 lds_read_tr_operand_perm(const uint16_t* tile, int stride, int row0, int db,
                                                  int lane) {  // row0: a multiple of 16
    const int g = lane >> 5, u = (lane >> 4) & 1, j = lane & 15;
    const int col = TrMap<D>::src_col(db, u, j & 3);
    const uint16_t* p = tile + (row0 + lds_row<D>(4 * g + (j >> 2))) * stride + col;
    s16x4 lo = lds_read_tr4(p);
    s16x4 hi = lds_read_tr4(p + TR_HI_ROWS<D> * stride);
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return *reinterpret_cast<bf16x8*>(&v);
}

// Rows r0 .. of a [T, D] bf16 matrix (row stride `st` elements, first element at base + elem_off) as a
// buffer resource over what is left of the matrix from row r0 on. Tile loads then take a per-thread byte
// offset (row_in_tile * st + column) * 2 that never changes, the tile's position sits in the scalar
// resource, and rows past the end read as zero without a branch (offsets beyond num_records).
//
// This runs once per tile in loops where every scalar instruction is issue time, so it is written for few
// of them: the stride is below 2^22 and the row numbers below 2^24 (checked on the host before these kernels are
// chosen), hence 32 x 32 -> 64-bit products (two scalar instructions each) and a clamp without a 64-bit compare.
__device__ inline __amdgpu_buffer_rsrc_t tile_rsrc(const void* base, int64_t elem_off, int64_t st, int r0, int T, int D) {
    const uint32_t st32 = static_cast<uint32_t>(st);
    const uint32_t first = static_cast<uint32_t>(min(r0, T));
    const uint32_t rows = static_cast<uint32_t>(T) - first;  // rows left from r0 on
    const uint32_t some = rows != 0;
    const uint64_t left = (static_cast<uint64_t>(rows - some) * st32 + (some ? D : 0)) * 2;  // bytes up to the last row's end
    const uint32_t lo = static_cast<uint32_t>(left), hi = static_cast<uint32_t>(left >> 32);
    const uint32_t records = hi ? 0x7fffffffu : min(lo, 0x7fffffffu);
    const uint16_t* p = static_cast<const uint16_t*>(base) + elem_off + static_cast<uint64_t>(first) * st32;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p), 0, static_cast<int>(records), 0x00020000);
}
__device__ inline u32x4 tile_load16(__amdgpu_buffer_rsrc_t rsrc, int byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off, 0, 0);
}

// ---- tiles straight from memory into LDS (buffer_load_dwordx4 ... offen lds) ----
// One such instruction fills 1 KB of LDS lane after lane from M0 + immediate on; each lane names the 16 bytes of memory it
// fetches (lane offset + scalar offset + immediate, all counted by the range check of the descriptor; a lane outside
// the buffer writes zeros). The instructions are invisible to the compiler's count of memory operations in flight:
// the kernels that use them wait with wait_loads<N> on counts of their own.
// Offsets that are outside every buffer these kernels take (operands of less than 1 GiB): a lane offset, and a scalar
// offset whose sum with any lane offset and immediate still fits 32 bits.
constexpr uint32_t OUTSIDE = 0x80000000u, PAST_END = 0x40000000u;
// Descriptors start this far before the tile, so that a lane offset minus the instruction's immediate (below 4096)
// never goes negative.
constexpr int BIAS = 4096;
// PER consecutive 1 KB pieces of LDS from `lds_byte` on, lane offsets off[j] (already less j KB), scalar offset soff.
// m0 is set and used inside the one statement; the compiler never keeps a value of its own in m0 across other code.
template <int PER>
__device__ inline void dma_group(uint32_t lds_byte, const uint32_t (&off)[PER], u32x4 rsrc, uint32_t soff) {
    static_assert(PER == 1 || PER == 2 || PER == 4, "groups of one, two or four pieces");
    if constexpr (PER == 1)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds_byte), "v"(off[0]),
                     "s"(rsrc), "s"(soff)
                     : "memory");
    else if constexpr (PER == 2)
        asm volatile(
            "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
            "buffer_load_dwordx4 %1, %3, %4 offen lds\n\t"
            "buffer_load_dwordx4 %2, %3, %4 offen offset:1024 lds" ::"s"(lds_byte),
            "v"(off[0]), "v"(off[1]), "s"(rsrc), "s"(soff)
            : "memory");
    else
        asm volatile(
            "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
            "buffer_load_dwordx4 %1, %5, %6 offen lds\n\t"
            "buffer_load_dwordx4 %2, %5, %6 offen offset:1024 lds\n\t"
            "buffer_load_dwordx4 %3, %5, %6 offen offset:2048 lds\n\t"
            "buffer_load_dwordx4 %4, %5, %6 offen offset:3072 lds" ::"s"(lds_byte),
            "v"(off[0]), "v"(off[1]), "v"(off[2]), "v"(off[3]), "s"(rsrc), "s"(soff)
            : "memory");
}
// One piece of such a group on its own: the J-th 1 KB from `lds_byte` on (lane offset already less J KB), for kernels
// that drop their loads one by one between other instructions. No "memory" clobber: the compiler may move its own LDS
// reads across the statement (it keeps its place among the other volatile statements, the waits and barriers that
// guard the slot it fills), which a clobber would forbid -- every piece would then fence the fragment reads of the
// chunk after it from the matrix instructions of the chunk before.
template <int J>
__device__ inline void dma_piece(uint32_t lds_byte, uint32_t off, u32x4 rsrc, uint32_t soff) {
    static_assert(J >= 0 && J < 4, "immediate offsets below 4096");
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen offset:%4 lds" ::"s"(lds_byte), "v"(off),
                 "s"(rsrc), "s"(soff), "n"(J * 1024));
}
template <int N>
__device__ inline void wait_loads() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ inline void barrier() { asm volatile("s_barrier" ::: "memory"); }
// descriptor words for `bytes` bytes from p - BIAS on (raw buffer, no swizzle)
__device__ inline u32x4 dma_rsrc(const void* p, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(p) - BIAS;
    const u32x4 r = {static_cast<uint32_t>(a), static_cast<uint32_t>(a >> 32) & 0xffffu, bytes + BIAS, 0x00020000u};
    return r;
}

// XCD-aware workgroup -> tile mapping. The 256 CUs sit in 8 XCDs, each with
// its own 4 MB L2, and consecutive workgroup ids go round-robin over the XCDs.
// Every block of a (batch, KV head) unit re-reads that unit's K/V (or Q/dO),
// so all blocks of a unit -- and of the `rep` query heads sharing the KV head --
// are given ids that are congruent mod 8: one unit's tensors then live in ONE
// L2 instead of being fetched into all eight.
// Launch with grid.x = xcd_grid(nblk, rep, kv_units).
__host__ __device__ inline int xcd_grid(int nblk, int rep, int kv_units) {
    return nblk * rep * ((kv_units + 7) / 8) * 8;
}
// blk: block index inside the unit (0 = dispatched first); r: query head inside
// the GQA group; kvu: (batch, KV head) unit. Returns false for padding ids.
__device__ inline bool xcd_map(int nblk, int rep, int kv_units, int& blk, int& r, int& kvu) {
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    blk = j % nblk;
    r = (j / nblk) % rep;
    kvu = (j / (nblk * rep)) * 8 + xcd;
    return kvu < kv_units;
}
// The same ids in block-major order: block 0 of every unit and head of an XCD's share first, then every block 1, ...
// For causal blocks that are NOT paired, block 0 is the heaviest and the work falls linearly with the index, so this
// hands the CUs the longest workgroups first whatever the number of units (longest-processing-time order); with
// the unit-major order above the last units' heavy blocks start late and stretch the tail of the launch
// (512 unpaired workgroups of 256 queries at B x H = 32, T = 4096 took 232 us against 208 for the smaller kernel).
__device__ inline bool xcd_map_block_major(int nblk, int rep, int kv_units, int& blk, int& r, int& kvu) {
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int per = ((kv_units + 7) / 8) * rep;  // (unit, head) pairs of one XCD
    blk = j / per;
    r = (j % per) % rep;
    kvu = ((j % per) / rep) * 8 + xcd;
    return kvu < kv_units;
}

// The same mapping with block 0 of EVERY unit dispatched before any other block (rep = 1). With a
// band mask plus sink keys the workgroup that owns key block 0 walks all query tiles while the others
// walk a handful; started last it is the tail of the launch, started first it runs beside them.
__device__ inline bool xcd_map_block0_first(int nblk, int kv_units, int& blk, int& kvu) {
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int upx = (kv_units + 7) / 8;  // units per XCD
    if (j < upx) {
        blk = 0;
        kvu = j * 8 + xcd;
    } else {
        const int jj = j - upx;
        blk = 1 + jj % (nblk - 1);
        kvu = (jj / (nblk - 1)) * 8 + xcd;
    }
    return kvu < kv_units;
}

// Full-causal work per 128-row block grows linearly with its index, so the forward and dQ kernels
// give a workgroup blocks i and n-1-i back to back: equal work everywhere. That halves the number
// of workgroups; when the halved grid would not give every CU more than one workgroup (short
// sequences, few heads) the blocks are dispatched singly, heaviest first, and the hardware
// balances them (measured: 448 paired workgroups beat 896 single ones by 25 %, 128 paired lose
// to 256 single by 10 %).
__host__ __device__ inline bool pair_causal_blocks(int nblk, int units, int causal, int window) {
    return causal && window == 0 && static_cast<int64_t>((nblk + 1) / 2) * units > 256;
}

// Branch-free visibility tests (the reference's two ranges, paperkiln
// src/ops.cpp:879-880, 960-965). Written with non-short-circuit & and | so
// that each element costs a few compares and one select, never a branch.
//
// QueryVis: fixed query, varying key (lane = query kernels).
struct QueryVis {
    int hi;      // keys [0, hi) pass the causal / length test
    int win_lo;  // keys >= win_lo are inside the band
    int sinks;   // keys < sinks are always visible (0 without a band)
    __device__ QueryVis(int qi, int T, int causal, int window, int sinks_)
        : hi(qi < T ? (causal ? min(qi + 1, T) : T) : 0),
          win_lo(window > 0 ? qi + 1 - window : -0x40000000),
          sinks(window > 0 ? sinks_ : 0) {}
    __device__ bool operator()(int kj) const { return (kj < hi) & ((kj >= win_lo) | (kj < sinks)); }
};
// Which of QueryVis's three tests a block of keys [k0, k1] can fail at all for a wavefront whose queries are
// [qlo, qhi] -- wavefront-uniform, so the mask of a block becomes one scalar branch to a loop with ONE compare and
// one select per element instead of three compares, two mask combinations and a select: with a band of a few
// tiles every other live block of a wavefront lies on one of the band's edges and pays for its mask.
//   UPPER: only `kj < hi` can fail (the diagonal, or the end of the sequence);
//   LOWER: only `kj >= win_lo` can fail (the band's far edge; no sink key in the block);
//   SINKS: nothing of the block is inside any query's band: only `kj < sinks` decides;
//   ALL:   anything else.
enum class MaskKind { NONE, UPPER, LOWER, SINKS, ALL };
__device__ inline MaskKind mask_kind(int k0, int k1, int qlo, int qhi, int T, int causal, int window, int sinks) {
    const bool upper = k1 >= T || (causal && k1 > qlo);                 // some (query, key) pair fails kj < hi
    const bool lower = window > 0 && k0 + window <= qhi;                // some pair fails kj >= win_lo
    const bool has_sink = window > 0 && k0 < sinks;
    if (!upper && (!lower || (has_sink && k1 < sinks))) return MaskKind::NONE;
    if (upper && !lower) return MaskKind::UPPER;
    if (!upper && lower && !has_sink) return MaskKind::LOWER;
    if (!upper && lower && k1 + window <= qlo) return MaskKind::SINKS;  // wholly outside every band: sink keys only
    return MaskKind::ALL;
}
// x[r] of a C tile (lane = query, element r = key kbase + (r/4)*8 + r%4, kbase already carrying the lane's 4g) kept
// where the key is visible, else `fill`
__device__ inline void mask_block(f32x16& x, MaskKind kind, const QueryVis& vis, int kbase, float fill) {
    if (kind == MaskKind::UPPER) {
        const int lim = vis.hi - kbase;  // visible: offset < lim
#pragma unroll
        for (int r = 0; r < 16; ++r) x[r] = ((r >> 2) * 8 + (r & 3) < lim) ? x[r] : fill;
    } else if (kind == MaskKind::LOWER) {
        const int lim = vis.win_lo - kbase;  // visible: offset >= lim
#pragma unroll
        for (int r = 0; r < 16; ++r) x[r] = ((r >> 2) * 8 + (r & 3) >= lim) ? x[r] : fill;
    } else if (kind == MaskKind::SINKS) {
        const int lim = vis.sinks - kbase;
#pragma unroll
        for (int r = 0; r < 16; ++r) x[r] = ((r >> 2) * 8 + (r & 3) < lim) ? x[r] : fill;
    } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) x[r] = vis(kbase + (r >> 2) * 8 + (r & 3)) ? x[r] : fill;
    }
}

// KeyVis: fixed key, varying query (lane = key kernels).
struct KeyVis {
    int q_lo;    // queries >= q_lo pass the causal test
    int q_hi;    // queries < q_hi are inside the band (or the key is a sink)
    int T;
    __device__ KeyVis(int kj, int T_, int causal, int window, int sinks)
        : q_lo(kj < T_ ? (causal ? kj : 0) : 0x40000000),
          q_hi((window > 0 && kj >= sinks) ? kj + window : 0x40000000),
          T(T_) {}
    __device__ bool operator()(int qi) const { return (qi >= q_lo) & (qi < q_hi) & (qi < T); }
};

}  // namespace pk
