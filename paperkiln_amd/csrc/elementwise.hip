// Allocator, elementwise / rowwise kernels and the GEMM wrapper behind the
// host-side tape. They stand where the reference's device op set does
// (paperkiln src/cuda_ops.cu:76-381, write-through host->device->host per call)
// but are device-resident: operands and results stay in HBM between ops.
// Formulas are those of the CPU tape in src/ops.cpp, cited per kernel.
#include <hipcub/hipcub.hpp>
#include <rocblas/rocblas.h>

#include <atomic>
#include <type_traits>
#include <cstdlib>
#include <map>
#include <cmath>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "mfma_common.h"
#include "tensor.h"

namespace pk {

void hip_check(hipError_t e, const char* what) {
    if (e == hipSuccess) return;
    const std::string msg = std::string("HIP error: ") + hipGetErrorString(e) + " in " + what;
    throw Error(e == hipErrorOutOfMemory ? PK_ERR_OOM : PK_ERR_HIP, msg);
}
int status_of(const std::exception& e) {
    if (const Error* pe = dynamic_cast<const Error*>(&e)) return pe->code;
    if (dynamic_cast<const std::bad_alloc*>(&e)) return PK_ERR_OOM;
    return PK_ERR_ARGUMENT;
}
#define HIPCHK(x) ::pk::hip_check((x), #x)

// ---- allocator -------------------------------------------------------------
namespace {
struct Pool {
    std::mutex mu;
    // cached blocks by (stream that last used them, size): a block is handed out again without waiting for the
    // GPU, which is only safe for work queued behind its last use, i.e. on that same stream
    std::multimap<std::pair<hipStream_t, size_t>, void*> free_blocks;
    std::unordered_map<void*, size_t> sizes;          // every block handed out or cached
    std::unordered_map<void*, hipStream_t> handed_out;  // blocks a caller holds right now -> the stream that used them last
    size_t live = 0, peak = 0, reserved = 0;
    void release_cached() {  // give every cached block back to the driver (hipFree waits for the device)
        for (auto& kv : free_blocks) {
            (void)hipFree(kv.second);
            reserved -= kv.first.second;
            sizes.erase(kv.second);
        }
        free_blocks.clear();
    }
};
Pool& pool() {
    static Pool p;
    return p;
}
size_t round_up(size_t n) {
    if (n < 512) return 512;
    if (n < (1u << 20)) return (n + 511) & ~size_t(511);
    return (n + ((1u << 20) - 1)) & ~size_t((1u << 20) - 1);  // 1 MiB granules above 1 MiB
}
}  // namespace

void* dev_alloc(size_t bytes) {
    const size_t n = round_up(bytes);
    const hipStream_t st = tape_stream();
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    void* p = nullptr;
    auto it = P.free_blocks.lower_bound({st, n});
    auto fits = [&](decltype(it) i, hipStream_t s) {  // near-fitting only
        return i != P.free_blocks.end() && i->first.first == s && i->first.second <= n + n / 4 + 512;
    };
    if (!fits(it, st)) {
        // A block cached for ANOTHER stream may be taken over once that stream has nothing queued any more (its
        // last use of the block has then completed); otherwise blocks of a stream nobody uses again would sit in
        // the cache until an allocation fails. Streams are visited in key order, one query each.
        it = P.free_blocks.end();
        for (auto j = P.free_blocks.begin(); j != P.free_blocks.end(); j = P.free_blocks.upper_bound({j->first.first, SIZE_MAX})) {
            const hipStream_t other = j->first.first;
            if (other == st) continue;
            auto cand = P.free_blocks.lower_bound({other, n});
            if (!fits(cand, other)) continue;
            if (hipStreamQuery(other) == hipSuccess) {
                it = cand;
                break;
            }
            (void)hipGetLastError();  // still busy (or no longer a stream): leave its blocks alone
        }
    }
    if (it != P.free_blocks.end()) {
        p = it->second;
        P.live += it->first.second;
        P.free_blocks.erase(it);
    } else {
        hipError_t e = hipMalloc(&p, n);
        if (e != hipSuccess) {  // give cached blocks back and retry once
            (void)hipGetLastError();
            P.release_cached();
            e = hipMalloc(&p, n);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                throw Error(PK_ERR_OOM, "out of device memory: hipMalloc of " + std::to_string(n) + " bytes failed (" +
                                            hipGetErrorString(e) + ")");
            }
        }
        P.sizes[p] = n;
        P.reserved += n;
        P.live += n;
    }
    P.handed_out[p] = st;
    if (P.live > P.peak) P.peak = P.live;
    return p;
}

bool dev_free(void* p) {
    if (!p) return true;
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    auto held = P.handed_out.find(p);
    if (held == P.handed_out.end()) return false;
    // cached for the stream that used the block last (dev_touch), not for whichever context happens to free it: a
    // block used on stream S and freed outside any scope must not go to the next allocation of the null stream
    const hipStream_t last = held->second;
    P.handed_out.erase(held);
    const size_t n = P.sizes.at(p);
    P.live -= n;
    P.free_blocks.emplace(std::make_pair(last, n), p);
    return true;
}

void dev_touch(const void* p, void* stream) {
    if (!p) return;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    auto held = P.handed_out.find(const_cast<void*>(p));
    if (held != P.handed_out.end()) held->second = st;
}

bool dev_owns(const void* p) {
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    return P.handed_out.count(const_cast<void*>(p)) != 0;
}

size_t dev_live_bytes() {
    std::lock_guard<std::mutex> lk(pool().mu);
    return pool().live;
}
size_t dev_peak_bytes() {
    std::lock_guard<std::mutex> lk(pool().mu);
    return pool().peak;
}
void dev_reset_peak() {
    std::lock_guard<std::mutex> lk(pool().mu);
    pool().peak = pool().live;
}
void dev_trim() {
    Pool& P = pool();
    std::lock_guard<std::mutex> lk(P.mu);
    (void)hipDeviceSynchronize();
    P.release_cached();
}

// ---- element access --------------------------------------------------------
namespace {

__device__ inline float ldf(const float* p, int64_t i) { return p[i]; }
__device__ inline float ldf(const uint16_t* p, int64_t i) { return __uint_as_float(static_cast<uint32_t>(p[i]) << 16); }
__device__ inline void stf(float* p, int64_t i, float x) { p[i] = x; }
__device__ inline void stf(uint16_t* p, int64_t i, float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {  // NaN: keep it one (the rounding carry could turn it into an infinity)
        p[i] = static_cast<uint16_t>((u >> 16) | 0x0040u);
        return;
    }
    u += 0x7FFFu + ((u >> 16) & 1u);  // round to nearest even
    p[i] = static_cast<uint16_t>(u >> 16);
}

constexpr int NT = 256;
inline dim3 ew_grid(int64_t n) { return dim3(static_cast<unsigned>(std::min<int64_t>((n + NT - 1) / NT, 65535 * 16))); }

// dispatch one or two storage types
#define PK_DISPATCH1(T_, dt, ...)               \
    if ((dt) == PK_F32) {                       \
        using T_ = float;                       \
        __VA_ARGS__;                            \
    } else {                                    \
        using T_ = uint16_t;                    \
        __VA_ARGS__;                            \
    }

template <typename TA, typename TB, typename TY, int OP>
__global__ void ew_binary(const TA* a, const TB* b, TY* y, int64_t n) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        const float x = ldf(a, i), z = ldf(b, i);
        stf(y, i, OP == 0 ? x + z : x * z);
    }
}
template <typename TA, typename TY>
__global__ void ew_scale(const TA* a, float s, TY* y, int64_t n) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT)
        stf(y, i, ldf(a, i) * s);
}
template <typename TY, typename TX>
__global__ void ew_axpy(TY* y, float a, const TX* x, int64_t n) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT)
        stf(y, i, ldf(y, i) + a * ldf(x, i));
}
template <typename TY>
__global__ void ew_fill(TY* y, float v, int64_t n) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT)
        stf(y, i, v);
}
// ---- 8-wide bf16 forms -------------------------------------------------------
// The streaming kernels of the bf16 compute path move 16 bytes per lane and instruction when the
// element count (and any row pitch) is a multiple of 8 and the pointers are 16-byte aligned; the
// one-element kernels above and below remain for everything else. Same arithmetic, same rounding
// (nearest even; v_cvt_pk_bf16_f32 here, the integer form in stf).
struct F8 {
    float v[8];
};
__device__ inline F8 ld8(const uint16_t* p, int64_t e) {
    const u32x4 r = *reinterpret_cast<const u32x4*>(p + e);
    F8 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        o.v[2 * k] = __uint_as_float(r[k] << 16);
        o.v[2 * k + 1] = __uint_as_float(r[k] & 0xFFFF0000u);
    }
    return o;
}
__device__ inline F8 ld8(const float* p, int64_t e) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p + e), b = *reinterpret_cast<const f32x4*>(p + e + 4);
    return F8{{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]}};
}
__device__ inline void st8(uint16_t* p, int64_t e, const F8& x) {
    const u32x4 r = {pack_bf16(x.v[0], x.v[1]), pack_bf16(x.v[2], x.v[3]), pack_bf16(x.v[4], x.v[5]), pack_bf16(x.v[6], x.v[7])};
    *reinterpret_cast<u32x4*>(p + e) = r;
}
#define PK_EW8_LOOP(i, n8) \
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < (n8); i += static_cast<int64_t>(gridDim.x) * NT)
template <int OP>
__global__ void ew_binary8(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t n8) {
    PK_EW8_LOOP(i, n8) {
        const F8 x = ld8(a, i * 8), z = ld8(b, i * 8);
        F8 o;
#pragma unroll
        for (int k = 0; k < 8; ++k) o.v[k] = OP == 0 ? x.v[k] + z.v[k] : x.v[k] * z.v[k];
        st8(y, i * 8, o);
    }
}
__global__ void ew_scale8(const uint16_t* a, float s, uint16_t* y, int64_t n8) {
    PK_EW8_LOOP(i, n8) {
        F8 x = ld8(a, i * 8);
#pragma unroll
        for (int k = 0; k < 8; ++k) x.v[k] *= s;
        st8(y, i * 8, x);
    }
}
__global__ void ew_axpy8(uint16_t* y, float a, const uint16_t* x, int64_t n8) {
    PK_EW8_LOOP(i, n8) {
        F8 o = ld8(y, i * 8);
        const F8 z = ld8(x, i * 8);
#pragma unroll
        for (int k = 0; k < 8; ++k) o.v[k] = o.v[k] + a * z.v[k];
        st8(y, i * 8, o);
    }
}
// cols8, ld8: row length and row pitch of gate / up (and dgate / dup) in units of 8 elements
__global__ void ew_silu_mul_fwd8(const uint16_t* gate, const uint16_t* up, uint16_t* y, int64_t n8, int64_t cols8, int64_t ld8_) {
    PK_EW8_LOOP(i, n8) {
        const int64_t j = ((i / cols8) * ld8_ + i % cols8) * 8;
        const F8 g = ld8(gate, j), u = ld8(up, j);
        F8 o;
#pragma unroll
        for (int k = 0; k < 8; ++k) o.v[k] = (g.v[k] / (1.0f + expf(-g.v[k]))) * u.v[k];
        st8(y, i * 8, o);
    }
}
__global__ void ew_silu_mul_bwd8(const uint16_t* gate, const uint16_t* up, const uint16_t* dy, uint16_t* dgate, uint16_t* dup,
                                 int64_t n8, int64_t cols8, int64_t ld8_) {
    PK_EW8_LOOP(i, n8) {
        const int64_t j = ((i / cols8) * ld8_ + i % cols8) * 8;
        const F8 v = ld8(gate, j), u = ld8(up, j), g = ld8(dy, i * 8);
        F8 du, dg;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float sg = 1.0f / (1.0f + expf(-v.v[k]));
            du.v[k] = g.v[k] * (v.v[k] * sg);
            dg.v[k] = (g.v[k] * u.v[k]) * (sg * (1.0f + v.v[k] * (1.0f - sg)));
        }
        st8(dup, j, du);
        st8(dgate, j, dg);
    }
}
inline bool aligned16p(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

template <typename T>
__global__ void ew_silu_fwd(const T* x, T* y, int64_t n) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        const float v = ldf(x, i);
        stf(y, i, v / (1.0f + expf(-v)));  // ops.cpp:409
    }
}
template <typename T>
__global__ void ew_silu_bwd(const T* x, const T* dy, T* dx, int64_t n) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        const float v = ldf(x, i);
        const float s = 1.0f / (1.0f + expf(-v));
        stf(dx, i, ldf(dy, i) * s * (1.0f + v * (1.0f - s)));  // ops.cpp:419-420
    }
}

// silu(gate) .* up in one pass (the two tape nodes ops::silu, src/ops.cpp:404-424, and ops::mul, :76-83, of
// LlamaBlock's SwiGLU, src/llama.cpp:55-58) and the pair of closures in one pass back.
// gate, up (and dgate, dup) are [rows, cols] matrices with row pitch ld: ld == cols for separate
// contiguous matrices, ld == 2*cols for the two halves of one [rows, 2*cols] projection.
template <typename T>
__global__ void ew_silu_mul_fwd(const T* gate, const T* up, T* y, int64_t n, int64_t cols, int64_t ld) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        const int64_t j = (i / cols) * ld + i % cols;
        const float v = ldf(gate, j);
        stf(y, i, (v / (1.0f + expf(-v))) * ldf(up, j));
    }
}
template <typename T>
__global__ void ew_silu_mul_bwd(const T* gate, const T* up, const T* dy, T* dgate, T* dup, int64_t n, int64_t cols,
                                int64_t ld) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        const int64_t j = (i / cols) * ld + i % cols;
        const float v = ldf(gate, j), g = ldf(dy, i);
        const float s = 1.0f / (1.0f + expf(-v));
        stf(dup, j, g * (v * s));
        stf(dgate, j, (g * ldf(up, j)) * (s * (1.0f + v * (1.0f - s))));
    }
}

__device__ inline float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// One wavefront per row. y = x * rinv * w, rinv = 1/sqrt(mean(x^2) + eps).
template <typename T>
__global__ void rms_fwd(const T* x, const float* w, float eps, T* y, float* rinv, int64_t R, int C) {
    const int lane = threadIdx.x & 63;
    const int64_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= R) return;
    const T* xr = x + row * C;
    float ss = 0.0f;
    for (int j = lane; j < C; j += 64) {
        const float v = ldf(xr, j);
        ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss) / static_cast<float>(C);
    const float ri = 1.0f / sqrtf(ss + eps);
    if (lane == 0) rinv[row] = ri;
    for (int j = lane; j < C; j += 64) stf(y + row * C, j, ldf(xr, j) * ri * w[j]);
}
// dx = rinv * (dY*w - x * rinv^2 * sum_j(dY*w*x) / C)
template <typename T>
__global__ void rms_bwd_dx(const T* dy, const T* x, const float* rinv, const float* w, T* dx, int64_t R, int C) {
    const int lane = threadIdx.x & 63;
    const int64_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= R) return;
    const T* xr = x + row * C;
    const T* gr = dy + row * C;
    float term = 0.0f;
    for (int j = lane; j < C; j += 64) term = fmaf(ldf(gr, j) * w[j], ldf(xr, j), term);
    term = wave_sum(term);
    const float ri = rinv[row], k = ri * ri * term / static_cast<float>(C);
    for (int j = lane; j < C; j += 64) stf(dx + row * C, j, ri * (ldf(gr, j) * w[j] - ldf(xr, j) * k));
}
// 8-wide bf16 forms of the two row kernels above (C a multiple of 8): one 16-byte load per lane
// covers a 512-column row in a single step.
__global__ void rms_fwd8(const uint16_t* x, const float* w, float eps, uint16_t* y, float* rinv, int64_t R, int C) {
    const int lane = threadIdx.x & 63;
    const int64_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= R) return;
    const uint16_t* xr = x + row * C;
    float ss = 0.0f;
    for (int j = lane * 8; j < C; j += 512) {
        const F8 v = ld8(xr, j);
#pragma unroll
        for (int k = 0; k < 8; ++k) ss = fmaf(v.v[k], v.v[k], ss);
    }
    ss = wave_sum(ss) / static_cast<float>(C);
    const float ri = 1.0f / sqrtf(ss + eps);
    if (lane == 0) rinv[row] = ri;
    for (int j = lane * 8; j < C; j += 512) {
        F8 v = ld8(xr, j);
        const F8 g = ld8(w, j);
#pragma unroll
        for (int k = 0; k < 8; ++k) v.v[k] = v.v[k] * ri * g.v[k];
        st8(y + row * C, j, v);
    }
}
// The same with each row held in registers between the two passes (C <= 512 NP) and two rows of a wavefront in flight:
// 8 rows per block of four wavefronts.
template <int NP>
__global__ void rms_fwd8_reg(const uint16_t* x, const float* w, float eps, uint16_t* y, float* rinv, int64_t R, int C) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * 8 + wv;  // and row0 + 4
    if (row0 >= R) return;
    const bool two = row0 + 4 < R;
    const int64_t rows[2] = {row0, two ? row0 + 4 : row0};
    F8 v[2][NP], g[NP];
    float ss[2] = {0.0f, 0.0f};
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int j = lane * 8 + p * 512;
            if (j < C) v[q][p] = ld8(x + rows[q] * C, j);
        }
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int j = lane * 8 + p * 512;
        if (j < C) g[p] = ld8(w, j);
    }
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int j = lane * 8 + p * 512;
            if (j < C) {
#pragma unroll
                for (int k = 0; k < 8; ++k) ss[q] = fmaf(v[q][p].v[k], v[q][p].v[k], ss[q]);
            }
        }
    ss[0] = wave_sum(ss[0]) / static_cast<float>(C);
    ss[1] = wave_sum(ss[1]) / static_cast<float>(C);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        if (q == 1 && !two) break;
        const float ri = 1.0f / sqrtf(ss[q] + eps);
        if (lane == 0) rinv[rows[q]] = ri;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int j = lane * 8 + p * 512;
            if (j < C) {
                F8 o;
#pragma unroll
                for (int k = 0; k < 8; ++k) o.v[k] = v[q][p].v[k] * ri * g[p].v[k];
                st8(y + rows[q] * C, j, o);
            }
        }
    }
}
__global__ void rms_bwd_dx8(const uint16_t* dy, const uint16_t* x, const float* rinv, const float* w, uint16_t* dx, int64_t R,
                            int C) {
    const int lane = threadIdx.x & 63;
    const int64_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= R) return;
    const uint16_t* xr = x + row * C;
    const uint16_t* gr = dy + row * C;
    float term = 0.0f;
    for (int j = lane * 8; j < C; j += 512) {
        const F8 g = ld8(gr, j), v = ld8(xr, j), ww = ld8(w, j);
#pragma unroll
        for (int k = 0; k < 8; ++k) term = fmaf(g.v[k] * ww.v[k], v.v[k], term);
    }
    term = wave_sum(term);
    const float ri = rinv[row], kk = ri * ri * term / static_cast<float>(C);
    for (int j = lane * 8; j < C; j += 512) {
        const F8 g = ld8(gr, j), v = ld8(xr, j), ww = ld8(w, j);
        F8 o;
#pragma unroll
        for (int k = 0; k < 8; ++k) o.v[k] = ri * (g.v[k] * ww.v[k] - v.v[k] * kk);
        st8(dx + row * C, j, o);
    }
}
// dw_j = sum_i dY_ij x_ij rinv_i, in two deterministic stages: each block sums
// ROWS_PB rows into part[block][C], then one block per column chunk adds the parts.
constexpr int ROWS_PB = 32;  // 8192 rows -> 256 blocks, one per CU
template <typename T>
__global__ void rms_bwd_dw_part(const T* dy, const T* x, const float* rinv, float* part, int64_t R, int C) {
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * ROWS_PB;
    for (int j = threadIdx.x; j < C; j += NT) {
        float s = 0.0f;
        for (int64_t i = r0; i < min(r0 + ROWS_PB, R); ++i) s = fmaf(ldf(dy, i * C + j) * ldf(x, i * C + j), rinv[i], s);
        part[static_cast<int64_t>(blockIdx.x) * C + j] = s;
    }
}
// 8-wide bf16 form: C/8 threads cover a row, the block's NT / (C/8) row groups meet in LDS in a fixed order.
// Needs C % 8 == 0 and C/8 a divisor of NT.
__global__ void rms_bwd_dw_part8(const uint16_t* dy, const uint16_t* x, const float* rinv, float* part, int64_t R, int C) {
    extern __shared__ float sh_dw[];  // [NT / (C/8)][C]
    const int c8 = C / 8, col = (threadIdx.x % c8) * 8, rg = threadIdx.x / c8, nrg = NT / c8;
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * ROWS_PB, r1 = min(r0 + ROWS_PB, R);
    F8 acc{};
    for (int64_t i = r0 + rg; i < r1; i += nrg) {
        const F8 g = ld8(dy, i * C + col), v = ld8(x, i * C + col);
        const float ri = rinv[i];
#pragma unroll
        for (int k = 0; k < 8; ++k) acc.v[k] = fmaf(g.v[k] * v.v[k], ri, acc.v[k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) sh_dw[rg * C + col + k] = acc.v[k];
    __syncthreads();
    for (int j = threadIdx.x; j < C; j += NT) {
        float t = 0.0f;
        for (int q = 0; q < nrg; ++q) t += sh_dw[q * C + j];
        part[static_cast<int64_t>(blockIdx.x) * C + j] = t;
    }
}
// dx and the dW partial sums in one pass over dY and x (both are wanted in a training step, and each reads both
// tensors): a wavefront takes ROWS_PB / 8 rows of its block, two at a time, lane l the columns 8 l .. 8 l + 7 of
// every 512-column pass (NP passes, C <= 512 NP), keeps its rows' contribution to dW in registers, and the eight
// wavefronts meet in LDS in a fixed order.
// ADD: dx = addend + (the above), the gradient that reached x along another path (a residual connection), added
// before the one rounding to bf16.
template <int NP, bool ADD>
__global__ void rms_bwd_dx_dw8(const uint16_t* dy, const uint16_t* x, const float* rinv, const float* w,
                               const uint16_t* addend, uint16_t* dx, float* part, int64_t R, int C) {
    constexpr int NWV = 8;            // wavefronts per block
    extern __shared__ float sh_dw[];  // [NWV - 1][C]: wavefronts 1 .. NWV - 1
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * ROWS_PB, r1 = min(r0 + ROWS_PB, R);
    F8 acc[NP], ww[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int j = lane * 8 + p * 512;
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[p].v[k] = 0.0f;
        if (j < C) ww[p] = ld8(w, j);
    }
    // two rows of the wavefront at a time: their loads are in flight together, and so are the two row reductions
    for (int64_t row = r0 + wv; row < r1; row += 2 * NWV) {
        const bool two = row + NWV < r1;
        const int64_t rows[2] = {row, two ? row + NWV : row};
        F8 g[2][NP], v[2][NP], e[2][ADD ? NP : 1];
        float term[2] = {0.0f, 0.0f};
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const int j = lane * 8 + p * 512;
                if (j < C) {
                    g[q][p] = ld8(dy + rows[q] * C, j);
                    v[q][p] = ld8(x + rows[q] * C, j);
                    if (ADD) e[q][p] = ld8(addend + rows[q] * C, j);
                }
            }
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const int j = lane * 8 + p * 512;
                if (j < C) {
#pragma unroll
                    for (int k = 0; k < 8; ++k) term[q] = fmaf(g[q][p].v[k] * ww[p].v[k], v[q][p].v[k], term[q]);
                }
            }
        term[0] = wave_sum(term[0]);
        term[1] = wave_sum(term[1]);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if (q == 1 && !two) break;  // wavefront-uniform: an odd row count leaves the second row out
            const float ri = rinv[rows[q]], kk = ri * ri * term[q] / static_cast<float>(C);
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const int j = lane * 8 + p * 512;
                if (j < C) {
                    F8 o;
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        o.v[k] = ri * (g[q][p].v[k] * ww[p].v[k] - v[q][p].v[k] * kk);
                        if (ADD) o.v[k] += e[q][p].v[k];
                        acc[p].v[k] = fmaf(g[q][p].v[k] * v[q][p].v[k], ri, acc[p].v[k]);
                    }
                    st8(dx + rows[q] * C, j, o);
                }
            }
        }
    }
    if (wv > 0) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int j = lane * 8 + p * 512;
            if (j < C) {
#pragma unroll
                for (int k = 0; k < 8; ++k) sh_dw[(wv - 1) * C + j + k] = acc[p].v[k];
            }
        }
    }
    __syncthreads();
    if (wv == 0) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int j = lane * 8 + p * 512;
            if (j < C) {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    float t = acc[p].v[k];
#pragma unroll
                    for (int q = 0; q < NWV - 1; ++q) t += sh_dw[q * C + j + k];
                    part[static_cast<int64_t>(blockIdx.x) * C + j + k] = t;
                }
            }
        }
    }
}
__global__ void colsum_parts(const float* part, float* dw, int nparts, int C) {
    // 64 columns x 16 groups of parts per block (1024 threads: each walks a sixteenth of the
    // parts, the walk being a chain of dependent loads); the groups meet in a fixed order
    __shared__ float sh[16][64];
    const int col = blockIdx.x * 64 + (threadIdx.x & 63), grp = threadIdx.x >> 6;
    float s = 0.0f;
    if (col < C) {
        int p = grp;
        for (; p + 48 < nparts; p += 64) {  // four independent loads in flight, added in index order
            const float a0 = part[static_cast<int64_t>(p) * C + col], a1 = part[static_cast<int64_t>(p + 16) * C + col];
            const float a2 = part[static_cast<int64_t>(p + 32) * C + col], a3 = part[static_cast<int64_t>(p + 48) * C + col];
            s = (((s + a0) + a1) + a2) + a3;
        }
        for (; p < nparts; p += 16) s += part[static_cast<int64_t>(p) * C + col];
    }
    sh[grp][threadIdx.x & 63] = s;
    __syncthreads();
    if (grp == 0 && col < C) {
        float t = 0.0f;
        for (int q = 0; q < 16; ++q) t += sh[q][threadIdx.x];
        dw[col] += t;
    }
}
// dst[i] = beta * dst[i] + sum_s part[s][i], parts added in index order
template <typename T>
__global__ void add_parts(const float* part, T* dst, int nparts, int64_t n, float beta) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        float s = 0.0f;
        for (int p = 0; p < nparts; ++p) s += part[p * n + i];
        stf(dst, i, beta != 0.0f ? ldf(dst, i) + s : s);
    }
}

__global__ void add_parts4(const float* part, float* dst, int nparts, int64_t n4, float beta) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n4; i += static_cast<int64_t>(gridDim.x) * NT) {
        f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int p = 0; p < nparts; ++p) s += *reinterpret_cast<const f32x4*>(part + (p * n4 + i) * 4);
        f32x4* d = reinterpret_cast<f32x4*>(dst) + i;
        *d = beta != 0.0f ? *d + s : s;
    }
}

// The same sum, scattered: the [M, nsplit*N] result is cut into nsplit column blocks and block k
// goes to its own contiguous [M, N] destination (the gradients of weights that were multiplied as
// one concatenated matrix).
struct SplitDst {
    float* p[4];
};
__global__ void add_parts_split(const float* part, SplitDst dst, int nparts, int64_t M, int64_t N, int nsplit, float beta) {
    const int64_t W = N * nsplit, n = M * W;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        float s = 0.0f;
        for (int p = 0; p < nparts; ++p) s += part[p * n + i];
        const int64_t r = i / W, c = i % W;
        float* d = dst.p[c / N] + r * N + c % N;
        *d = beta != 0.0f ? *d + s : s;
    }
}
// four columns per thread (N a multiple of 4, so a group of four never straddles two destinations)
__global__ void add_parts_split4(const float* part, SplitDst dst, int nparts, int64_t M, int64_t N, int nsplit, float beta) {
    const int64_t W = N * nsplit, n4 = M * W / 4;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n4; i += static_cast<int64_t>(gridDim.x) * NT) {
        f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int p = 0; p < nparts; ++p) s += *reinterpret_cast<const f32x4*>(part + p * (n4 * 4) + i * 4);
        const int64_t r = (i * 4) / W, c = (i * 4) % W;
        f32x4* d = reinterpret_cast<f32x4*>(dst.p[c / N] + r * N + c % N);
        *d = beta != 0.0f ? *d + s : s;
    }
}
// dst[r][off + c] = src[r][c]: one column block of a concatenated matrix with row pitch ld
template <typename TA, typename TY>
__global__ void cast_cols_k(const TA* src, TY* dst, int64_t rows, int64_t cols, int64_t ld, int64_t off) {
    const int64_t n = rows * cols;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT)
        stf(dst, (i / cols) * ld + off + i % cols, ldf(src, i));
}

// Many casts of fp32 matrices into column blocks of bf16 matrices as one launch (the refresh of every compute-dtype
// weight copy after an optimizer step): job j covers blocks [block_begin[j], block_begin[j + 1]), eight elements a thread.
struct CastJobs {
    static constexpr int MAX = 64;
    int count;
    int block_begin[MAX + 1];
    const float* src[MAX];
    uint16_t* dst[MAX];
    int rows[MAX], cols[MAX], ld[MAX], off[MAX];
};
__global__ void cast_jobs_k(CastJobs jobs) {
    int j = 0;
    while (static_cast<int>(blockIdx.x) >= jobs.block_begin[j + 1]) ++j;
    const int cols = jobs.cols[j];
    const int64_t n8 = static_cast<int64_t>(jobs.rows[j]) * cols / 8;  // cols, ld and off are multiples of 8
    const int64_t i = (static_cast<int64_t>(blockIdx.x) - jobs.block_begin[j]) * NT + threadIdx.x;
    if (i >= n8) return;
    const int64_t e = i * 8, r = e / cols, c = e - r * cols;
    st8(jobs.dst[j], r * jobs.ld[j] + jobs.off[j] + c, ld8(jobs.src[j], e));
}

// apply_rope (ops.cpp:497-509 forward, :519-533 backward = rotation by -theta).
// The inverse frequencies come from the host, computed with the reference's own expression
// 1 / pow(theta, dim / head_dim): the angle pos * inv_freq is then the same fp32 number the
// reference feeds to cos / sin. An inv_freq one ulp off would be amplified by the position.
constexpr int ROPE_MAX_PAIRS = 128;  // head_dim <= 256
struct RopeFreq {
    float f[ROPE_MAX_PAIRS];
};
template <typename T>
__global__ void rope_k(const T* x, const int* pos, RopeFreq freq, int d, int head_dim, int rot_heads, float sign, T* y,
                       int64_t N) {
    const int d3 = 3 * d;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < N * (d3 / 2);
         i += static_cast<int64_t>(gridDim.x) * NT) {
        const int64_t row = i / (d3 / 2);
        const int c = static_cast<int>(i % (d3 / 2)) * 2;  // even column of the pair
        const int third = c / d, within = c % d;
        float x0 = ldf(x, row * d3 + c), x1 = ldf(x, row * d3 + c + 1);
        if (third < 2 && within < rot_heads * head_dim) {
            const int dim = within % head_dim;
            const float th = sign * static_cast<float>(pos[row]) * freq.f[dim >> 1];
            const float c_ = cosf(th), s_ = sinf(th);
            const float r0 = x0 * c_ - x1 * s_, r1 = x0 * s_ + x1 * c_;
            x0 = r0;
            x1 = r1;
        }
        stf(y, row * d3 + c, x0);
        stf(y, row * d3 + c + 1, x1);
    }
}

// The same rotation applied where the data lies: only the rotated columns (q and k thirds, the first
// rot_heads heads) are touched, everything else stays as it is.
template <typename T>
__global__ void rope_inplace_k(T* x, const int* pos, RopeFreq freq, int d, int head_dim, int rot_heads, float sign, int64_t N) {
    const int ppr = rot_heads * head_dim;  // rotated pairs per row: 2 thirds x rot_heads x head_dim / 2
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < N * ppr; i += static_cast<int64_t>(gridDim.x) * NT) {
        const int64_t row = i / ppr;
        const int p = static_cast<int>(i % ppr), third = p / (ppr / 2), within = (p % (ppr / 2)) * 2;
        const int64_t o = row * 3 * d + third * d + within;
        const float th = sign * static_cast<float>(pos[row]) * freq.f[(within % head_dim) >> 1];
        const float c_ = cosf(th), s_ = sinf(th);
        const float x0 = ldf(x, o), x1 = ldf(x, o + 1);
        stf(x, o, x0 * c_ - x1 * s_);
        stf(x, o + 1, x0 * s_ + x1 * c_);
    }
}

template <typename T>
__global__ void emb_fwd(const float* table, const int* ids, T* y, int64_t n, int d) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n * d; i += static_cast<int64_t>(gridDim.x) * NT)
        stf(y, i, table[static_cast<int64_t>(ids[i / d]) * d + i % d]);
}
// the same gather, eight columns a thread (d a multiple of 8, bf16 rows 16-byte aligned)
__global__ void emb_fwd8(const float* table, const int* ids, uint16_t* y, int64_t n, int d) {
    const int d8 = d / 8;
    const int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x;
    if (i >= n * d8) return;
    const int64_t r = i / d8;
    const int c = static_cast<int>(i - r * d8) * 8;
    st8(y, r * d + c, ld8(table, static_cast<int64_t>(ids[r]) * d + c));
}
// Scatter-add without atomics. The rows are visited in the order of a stable sort by id (sorted_id, row_of), so
// the rows that share an id are neighbours, in ascending row order. The block at the head of such a run adds the
// run's rows one after another and is the only writer of that table row; every other block leaves at once. The
// sum for an id is therefore formed in the reference's own order (rows ascending, src/ops.cpp:338-347) and is
// the same on every run.
__global__ void iota_i32(int* x, int n) {
    const int i = blockIdx.x * NT + threadIdx.x;
    if (i < n) x[i] = i;
}
// A run may be the whole input (every row the same id), so its columns are dealt to grid.y workgroups of one
// wavefront each and the rows are fetched EMB_ROWS at a time (independent loads in flight) and then added one by one.
constexpr int EMB_NT = 64, EMB_ROWS = 8;
template <typename T>
__global__ void __launch_bounds__(EMB_NT) emb_bwd_runs(const T* dy, const int* sorted_id, const int* row_of, float* dtable, int n, int d) {
    const int p = blockIdx.x;
    const int id = sorted_id[p];
    if (p > 0 && sorted_id[p - 1] == id) return;
    int end = p + 1;
    while (end < n && sorted_id[end] == id) ++end;
    const int c = blockIdx.y * EMB_NT + threadIdx.x;
    if (c >= d) return;
    float* dst = dtable + static_cast<int64_t>(id) * d + c;
    float acc = *dst;
    int r = p;
    for (; r + EMB_ROWS <= end; r += EMB_ROWS) {
        float v[EMB_ROWS];
#pragma unroll
        for (int u = 0; u < EMB_ROWS; ++u) v[u] = ldf(dy, static_cast<int64_t>(row_of[r + u]) * d + c);
#pragma unroll
        for (int u = 0; u < EMB_ROWS; ++u) acc += v[u];
    }
    for (; r < end; ++r) acc += ldf(dy, static_cast<int64_t>(row_of[r]) * d + c);
    *dst = acc;
}

__device__ inline float block_reduce(float x, bool is_max, float* sh) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float y = __shfl_xor(x, o, 64);
        x = is_max ? fmaxf(x, y) : x + y;
    }
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = x;
    __syncthreads();
    float r = sh[0];
    for (int i = 1; i < NT / 64; ++i) r = is_max ? fmaxf(r, sh[i]) : r + sh[i];
    __syncthreads();
    return r;
}
// One block per row: softmax, nll with the 1e-12 clamp, dlogits in place.
template <typename T>
__global__ void ce_rows(T* logits, const int* targets, float gscale, float* nll, int C) {
    __shared__ float sh[NT / 64];
    T* row = logits + static_cast<int64_t>(blockIdx.x) * C;
    const int t = targets[blockIdx.x];
    const float lt = ldf(row, t);  // read before any thread overwrites the row with dlogits
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < C; j += NT) mx = fmaxf(mx, ldf(row, j));
    mx = block_reduce(mx, true, sh);
    float z = 0.0f;
    for (int j = threadIdx.x; j < C; j += NT) z += expf(ldf(row, j) - mx);
    z = block_reduce(z, false, sh);
    const float inv = 1.0f / z;
    if (threadIdx.x == 0) nll[blockIdx.x] = -logf(fmaxf(expf(lt - mx) * inv, 1e-12f));
    for (int j = threadIdx.x; j < C; j += NT) {
        const float p = expf(ldf(row, j) - mx) * inv;
        stf(row, j, (p - (j == t ? 1.0f : 0.0f)) * gscale);
    }
}

// The same row operation for the chunked head (fp32 logits, vocabulary a multiple of 4 and at most
// 32768): 1024 threads hold the whole row in registers, so the logits are read ONCE; the forward pass
// writes nothing but the row's nll, the backward writes dlogits straight in the GEMM's operand type.
constexpr int CE_NT = 1024, CE_V4 = 8;  // 8 float4 per thread
template <typename TOut, bool WRITE>
__global__ __launch_bounds__(CE_NT) void ce_rows_reg(const float* logits, TOut* dl, const int* targets, float gscale,
                                                     float* nll, int C, int64_t dl_ld) {
    __shared__ float sh[CE_NT / 64];
    const float* row = logits + static_cast<int64_t>(blockIdx.x) * C;
    const int t = targets[blockIdx.x];
    f32x4 v[CE_V4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < CE_V4; ++i) {
        const int j = (threadIdx.x + i * CE_NT) * 4;
        if (j < C) {
            v[i] = *reinterpret_cast<const f32x4*>(row + j);
            mx = fmaxf(fmaxf(mx, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
        }
    }
    auto reduce = [&](float x, bool is_max) {
        for (int o = 32; o >= 1; o >>= 1) {
            const float y = __shfl_xor(x, o);
            x = is_max ? fmaxf(x, y) : x + y;
        }
        __syncthreads();  // sh is reused
        if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = x;
        __syncthreads();
        float r = sh[0];
        for (int w = 1; w < CE_NT / 64; ++w) r = is_max ? fmaxf(r, sh[w]) : r + sh[w];
        return r;
    };
    mx = reduce(mx, true);
    float z = 0.0f;
#pragma unroll
    for (int i = 0; i < CE_V4; ++i) {
        const int j = (threadIdx.x + i * CE_NT) * 4;
        if (j < C) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[i][e] = expf(v[i][e] - mx);
                z += v[i][e];
            }
        }
    }
    z = reduce(z, false);
    const float inv = 1.0f / z;
#pragma unroll
    for (int i = 0; i < CE_V4; ++i) {
        const int j = (threadIdx.x + i * CE_NT) * 4;
        if (j < C) {
            if (t >= j && t < j + 4) nll[blockIdx.x] = -logf(fmaxf(v[i][t - j] * inv, 1e-12f));
            if (WRITE) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (v[i][e] * inv - (j + e == t ? 1.0f : 0.0f)) * gscale;
                // dl may be the logits buffer itself (bf16 rows written over the fp32 row they came from):
                // every thread of the row has its logits in registers since before the first reduction
                TOut* dst = dl + static_cast<int64_t>(blockIdx.x) * dl_ld + j;
                if (sizeof(TOut) == 4) {
                    f32x4 w = {o[0], o[1], o[2], o[3]};
                    *reinterpret_cast<f32x4*>(dst) = w;
                } else {
                    u32x2 w = {pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
                    *reinterpret_cast<u32x2*>(dst) = w;
                }
            }
        }
    }
}

__global__ void sum_f32_k(const float* x, int64_t n, double* out) {
    __shared__ double sh[NT];
    double s = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += NT) s += static_cast<double>(x[i]);
    sh[threadIdx.x] = s;
    __syncthreads();
    for (int o = NT / 2; o >= 1; o >>= 1) {
        if (threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) *out = sh[0];
}
// mean of n floats, accumulated in double and rounded to float once: what the host does with
// k_sum_f32_to_host's result, without the round trip
__global__ __launch_bounds__(1024) void mean_f32_k(const float* x, int64_t n, float* out) {
    // thread t takes the elements sum_f32_k's thread t % NT takes, a quarter of them: the NT partial sums are formed
    // from four pieces each and then added in sum_f32_k's tree
    __shared__ double sh[1024];
    double s = 0.0;
    const int t = threadIdx.x % NT, q = threadIdx.x / NT;
    for (int64_t i = t + static_cast<int64_t>(q) * NT; i < n; i += 4 * NT) s += static_cast<double>(x[i]);
    sh[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x < NT) sh[threadIdx.x] = (sh[threadIdx.x] + sh[threadIdx.x + NT]) + (sh[threadIdx.x + 2 * NT] + sh[threadIdx.x + 3 * NT]);
    __syncthreads();
    for (int o = NT / 2; o >= 1; o >>= 1) {
        if (threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) *out = static_cast<float>(sh[0] / static_cast<double>(n));
}
__global__ void sumsq_part(const float* x, int64_t n, double* part) {
    __shared__ double sh[NT];
    double s = 0.0;
    if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {  // 16 bytes a lane, four chains of additions
        const int64_t n4 = n / 4;
        double q[4] = {0.0, 0.0, 0.0, 0.0};
        for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n4; i += static_cast<int64_t>(gridDim.x) * NT) {
            const f32x4 v = reinterpret_cast<const f32x4*>(x)[i];
#pragma unroll
            for (int e = 0; e < 4; ++e) q[e] += static_cast<double>(v[e]) * v[e];
        }
        s = (q[0] + q[1]) + (q[2] + q[3]);
        if (blockIdx.x == 0 && threadIdx.x < n - n4 * 4) {
            const float t = x[n4 * 4 + threadIdx.x];
            s += static_cast<double>(t) * t;
        }
    } else {
        for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT)
            s += static_cast<double>(x[i]) * x[i];
    }
    sh[threadIdx.x] = s;
    __syncthreads();
    for (int o = NT / 2; o >= 1; o >>= 1) {
        if (threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) part[blockIdx.x] = sh[0];
}
// CLIP: the gradient is scaled by gs first and the scaled value written back, as ops::clip_grad_norm leaves it
// (src/ops.cpp:1058-1062), in the same pass instead of one of its own.
template <bool CLIP>
__global__ void adamw_k(float* p, float* g, float* m, float* v, float lr, float b1, float b2, float eps, float wd, float c1,
                        float c2, float gs, int64_t n) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(NT) + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * NT) {
        float gi = g[i];
        if (CLIP) {
            gi *= gs;
            g[i] = gi;
        }
        const float mi = b1 * m[i] + (1.0f - b1) * gi;
        const float vi = b2 * v[i] + (1.0f - b2) * gi * gi;
        m[i] = mi;
        v[i] = vi;
        const float upd = (mi / c1) / (sqrtf(vi / c2) + eps);  // nn.cpp:317
        p[i] -= lr * (upd + wd * p[i]);
    }
}

void same_shape(const Tensor& a, const Tensor& b, const char* who) {
    if (a.rows != b.rows || a.cols != b.cols) throw std::runtime_error(std::string(who) + ": shape mismatch");
}
void post() { HIPCHK(hipGetLastError()); }

}  // namespace

void k_fill(const Tensor& y, float v) {
    PK_DISPATCH1(T, y.dtype, hipLaunchKernelGGL((ew_fill<T>), ew_grid(y.numel()), dim3(NT), 0, tape_stream(),
                                                static_cast<T*>(y.ptr()), v, y.numel()));
    post();
}
void k_cast(const Tensor& src, const Tensor& dst) {
    same_shape(src, dst, "cast");
    PK_DISPATCH1(TA, src.dtype, PK_DISPATCH1(TY, dst.dtype,
                 hipLaunchKernelGGL((ew_scale<TA, TY>), ew_grid(src.numel()), dim3(NT), 0, tape_stream(),
                                    static_cast<const TA*>(src.ptr()), 1.0f, static_cast<TY*>(dst.ptr()), src.numel())));
    post();
}
void k_cast_cols(const Tensor& src, const Tensor& dst, int64_t col_off) {
    if (src.rows != dst.rows || col_off < 0 || col_off + src.cols > dst.cols) throw std::runtime_error("cast_cols: shape mismatch");
    PK_DISPATCH1(TA, src.dtype, PK_DISPATCH1(TY, dst.dtype,
                 hipLaunchKernelGGL((cast_cols_k<TA, TY>), ew_grid(src.numel()), dim3(NT), 0, tape_stream(),
                                    static_cast<const TA*>(src.ptr()), static_cast<TY*>(dst.ptr()), src.rows, src.cols,
                                    dst.cols, col_off)));
    post();
}
// dst_k[:, off_k : off_k + cols_k] = bf16(src_k) for every job, one launch per 64 jobs. False, with nothing done,
// if a job is not an fp32 -> bf16 cast with column counts and offsets that are multiples of 8 (the caller casts one by one).
bool k_cast_many(const std::vector<CastJob>& list) {
    for (const CastJob& c : list)
        if (c.src.dtype != PK_F32 || c.dst.dtype != PK_BF16 || c.src.cols % 8 || c.dst.cols % 8 || c.col_off % 8 ||
            c.src.rows != c.dst.rows || c.col_off < 0 || c.col_off + c.src.cols > c.dst.cols ||
            c.src.numel() / 8 > (int64_t{1} << 30) || !aligned16p(c.src.ptr()) || !aligned16p(c.dst.ptr()))
            return false;
    size_t done = 0;
    while (done < list.size()) {
        CastJobs jobs{};
        int blocks = 0;
        while (done < list.size() && jobs.count < CastJobs::MAX) {
            const CastJob& c = list[done++];
            const int k = jobs.count++;
            jobs.block_begin[k] = blocks;
            jobs.src[k] = static_cast<const float*>(c.src.ptr());
            jobs.dst[k] = static_cast<uint16_t*>(c.dst.ptr());
            jobs.rows[k] = static_cast<int>(c.src.rows);
            jobs.cols[k] = static_cast<int>(c.src.cols);
            jobs.ld[k] = static_cast<int>(c.dst.cols);
            jobs.off[k] = static_cast<int>(c.col_off);
            blocks += static_cast<int>((c.src.numel() / 8 + NT - 1) / NT);
        }
        for (int k = jobs.count; k <= CastJobs::MAX; ++k) jobs.block_begin[k] = blocks;
        if (blocks > 0) {
            hipLaunchKernelGGL(cast_jobs_k, dim3(static_cast<unsigned>(blocks)), dim3(NT), 0, tape_stream(), jobs);
            post();
        }
    }
    return true;
}
template <int OP>
static void binary(const Tensor& a, const Tensor& b, const Tensor& y, const char* who) {
    same_shape(a, b, who);
    same_shape(a, y, who);
    if (a.dtype == PK_BF16 && b.dtype == PK_BF16 && y.dtype == PK_BF16 && a.numel() % 8 == 0 && aligned16p(a.ptr()) &&
        aligned16p(b.ptr()) && aligned16p(y.ptr())) {
        hipLaunchKernelGGL((ew_binary8<OP>), ew_grid(a.numel() / 8), dim3(NT), 0, tape_stream(),
                           static_cast<const uint16_t*>(a.ptr()), static_cast<const uint16_t*>(b.ptr()),
                           static_cast<uint16_t*>(y.ptr()), a.numel() / 8);
        post();
        return;
    }
    PK_DISPATCH1(TA, a.dtype, PK_DISPATCH1(TB, b.dtype, PK_DISPATCH1(TY, y.dtype,
                 hipLaunchKernelGGL((ew_binary<TA, TB, TY, OP>), ew_grid(a.numel()), dim3(NT), 0, tape_stream(),
                                    static_cast<const TA*>(a.ptr()), static_cast<const TB*>(b.ptr()),
                                    static_cast<TY*>(y.ptr()), a.numel()))));
    post();
}
void k_add(const Tensor& a, const Tensor& b, const Tensor& y) { binary<0>(a, b, y, "add"); }
void k_mul(const Tensor& a, const Tensor& b, const Tensor& y) { binary<1>(a, b, y, "mul"); }
void k_scale(const Tensor& a, float s, const Tensor& y) {
    same_shape(a, y, "scale");
    if (a.dtype == PK_BF16 && y.dtype == PK_BF16 && a.numel() % 8 == 0 && aligned16p(a.ptr()) && aligned16p(y.ptr())) {
        hipLaunchKernelGGL(ew_scale8, ew_grid(a.numel() / 8), dim3(NT), 0, tape_stream(), static_cast<const uint16_t*>(a.ptr()),
                           s, static_cast<uint16_t*>(y.ptr()), a.numel() / 8);
        post();
        return;
    }
    PK_DISPATCH1(TA, a.dtype, PK_DISPATCH1(TY, y.dtype,
                 hipLaunchKernelGGL((ew_scale<TA, TY>), ew_grid(a.numel()), dim3(NT), 0, tape_stream(),
                                    static_cast<const TA*>(a.ptr()), s, static_cast<TY*>(y.ptr()), a.numel())));
    post();
}
void k_axpy(const Tensor& y, float a, const Tensor& x) {
    if (x.rows != y.rows || x.cols != y.cols) throw std::runtime_error("accumulate: gradient shape mismatch");  // autograd.cpp:20-22
    if (x.dtype == PK_BF16 && y.dtype == PK_BF16 && y.numel() % 8 == 0 && aligned16p(x.ptr()) && aligned16p(y.ptr())) {
        hipLaunchKernelGGL(ew_axpy8, ew_grid(y.numel() / 8), dim3(NT), 0, tape_stream(), static_cast<uint16_t*>(y.ptr()), a,
                           static_cast<const uint16_t*>(x.ptr()), y.numel() / 8);
        post();
        return;
    }
    PK_DISPATCH1(TY, y.dtype, PK_DISPATCH1(TX, x.dtype,
                 hipLaunchKernelGGL((ew_axpy<TY, TX>), ew_grid(y.numel()), dim3(NT), 0, tape_stream(),
                                    static_cast<TY*>(y.ptr()), a, static_cast<const TX*>(x.ptr()), y.numel())));
    post();
}
void k_silu_fwd(const Tensor& x, const Tensor& y) {
    same_shape(x, y, "silu");
    PK_DISPATCH1(T, x.dtype, hipLaunchKernelGGL((ew_silu_fwd<T>), ew_grid(x.numel()), dim3(NT), 0, tape_stream(),
                                                static_cast<const T*>(x.ptr()), static_cast<T*>(y.ptr()), x.numel()));
    post();
}
void k_silu_bwd(const Tensor& x, const Tensor& dy, const Tensor& dx) {
    same_shape(x, dy, "silu");
    PK_DISPATCH1(T, x.dtype, hipLaunchKernelGGL((ew_silu_bwd<T>), ew_grid(x.numel()), dim3(NT), 0, tape_stream(),
                                                static_cast<const T*>(x.ptr()), static_cast<const T*>(dy.ptr()),
                                                static_cast<T*>(dx.ptr()), x.numel()));
    post();
}
namespace {
// gate, up: [rows, cols] with row pitch ld; y, dy contiguous; dgate, dup with pitch ld
void silu_mul_fwd_launch(const void* gate, const void* up, void* y, int dtype, int64_t rows, int64_t cols, int64_t ld) {
    const int64_t n = rows * cols;
    if (dtype == PK_BF16 && cols % 8 == 0 && ld % 8 == 0 && aligned16p(gate) && aligned16p(up) && aligned16p(y)) {
        hipLaunchKernelGGL(ew_silu_mul_fwd8, ew_grid(n / 8), dim3(NT), 0, tape_stream(), static_cast<const uint16_t*>(gate),
                           static_cast<const uint16_t*>(up), static_cast<uint16_t*>(y), n / 8, cols / 8, ld / 8);
    } else {
        PK_DISPATCH1(T, dtype, hipLaunchKernelGGL((ew_silu_mul_fwd<T>), ew_grid(n), dim3(NT), 0, tape_stream(),
                                                  static_cast<const T*>(gate), static_cast<const T*>(up),
                                                  static_cast<T*>(y), n, cols, ld));
    }
    post();
}
void silu_mul_bwd_launch(const void* gate, const void* up, const void* dy, void* dgate, void* dup, int dtype, int64_t rows,
                         int64_t cols, int64_t ld) {
    const int64_t n = rows * cols;
    if (dtype == PK_BF16 && cols % 8 == 0 && ld % 8 == 0 && aligned16p(gate) && aligned16p(up) && aligned16p(dy) &&
        aligned16p(dgate) && aligned16p(dup)) {
        hipLaunchKernelGGL(ew_silu_mul_bwd8, ew_grid(n / 8), dim3(NT), 0, tape_stream(), static_cast<const uint16_t*>(gate),
                           static_cast<const uint16_t*>(up), static_cast<const uint16_t*>(dy), static_cast<uint16_t*>(dgate),
                           static_cast<uint16_t*>(dup), n / 8, cols / 8, ld / 8);
    } else {
        PK_DISPATCH1(T, dtype, hipLaunchKernelGGL((ew_silu_mul_bwd<T>), ew_grid(n), dim3(NT), 0, tape_stream(),
                                                  static_cast<const T*>(gate), static_cast<const T*>(up),
                                                  static_cast<const T*>(dy), static_cast<T*>(dgate), static_cast<T*>(dup), n,
                                                  cols, ld));
    }
    post();
}
}  // namespace
void k_silu_mul_fwd(const Tensor& gate, const Tensor& up, const Tensor& y) {
    same_shape(gate, up, "mul");
    same_shape(gate, y, "mul");
    silu_mul_fwd_launch(gate.ptr(), up.ptr(), y.ptr(), gate.dtype, gate.rows, gate.cols, gate.cols);
}
void k_silu_mul_bwd(const Tensor& gate, const Tensor& up, const Tensor& dy, const Tensor& dgate, const Tensor& dup) {
    same_shape(gate, up, "mul");
    same_shape(gate, dy, "mul");
    same_shape(gate, dgate, "mul");
    same_shape(gate, dup, "mul");
    silu_mul_bwd_launch(gate.ptr(), up.ptr(), dy.ptr(), dgate.ptr(), dup.ptr(), gate.dtype, gate.rows, gate.cols, gate.cols);
}
void k_silu_mul_cat_fwd(const Tensor& gu, const Tensor& y) {
    if (gu.cols != 2 * y.cols || gu.rows != y.rows || gu.dtype != y.dtype) throw std::runtime_error("silu_mul: shape mismatch");
    const char* g = static_cast<const char*>(gu.ptr());
    silu_mul_fwd_launch(g, g + y.cols * gu.esize(), y.ptr(), gu.dtype, y.rows, y.cols, gu.cols);
}
void k_silu_mul_cat_bwd(const Tensor& gu, const Tensor& dy, const Tensor& dgu) {
    if (gu.cols != 2 * dy.cols || gu.rows != dy.rows || gu.dtype != dy.dtype) throw std::runtime_error("silu_mul: shape mismatch");
    same_shape(gu, dgu, "mul");
    const char* g = static_cast<const char*>(gu.ptr());
    char* d = static_cast<char*>(dgu.ptr());
    silu_mul_bwd_launch(g, g + dy.cols * gu.esize(), dy.ptr(), d, d + dy.cols * gu.esize(), gu.dtype, dy.rows, dy.cols, gu.cols);
}
void k_rmsnorm_fwd(const Tensor& x, const Tensor& w, float eps, const Tensor& y, float* rinv) {
    if (w.rows != 1 || w.cols != x.cols || w.dtype != PK_F32) throw std::runtime_error("rmsnorm: w must be [1, cols(x)]");
    if (x.dtype == PK_BF16 && x.cols % 8 == 0 && aligned16p(x.ptr()) && aligned16p(y.ptr()) && aligned16p(w.ptr())) {
        const int C = static_cast<int>(x.cols);
        auto launch = [&](auto np) {
            hipLaunchKernelGGL((rms_fwd8_reg<decltype(np)::value>), dim3((x.rows + 7) / 8), dim3(256), 0, tape_stream(),
                               static_cast<const uint16_t*>(x.ptr()), static_cast<const float*>(w.ptr()), eps,
                               static_cast<uint16_t*>(y.ptr()), rinv, x.rows, C);
        };
        if (C <= 512)
            launch(std::integral_constant<int, 1>{});
        else if (C <= 1024)
            launch(std::integral_constant<int, 2>{});
        else if (C <= 2048)
            launch(std::integral_constant<int, 4>{});
        else
            hipLaunchKernelGGL(rms_fwd8, dim3((x.rows + 3) / 4), dim3(NT), 0, tape_stream(), static_cast<const uint16_t*>(x.ptr()),
                               static_cast<const float*>(w.ptr()), eps, static_cast<uint16_t*>(y.ptr()), rinv, x.rows, C);
        post();
        return;
    }
    PK_DISPATCH1(T, x.dtype, hipLaunchKernelGGL((rms_fwd<T>), dim3((x.rows + 3) / 4), dim3(NT), 0, tape_stream(),
                                                static_cast<const T*>(x.ptr()), static_cast<const float*>(w.ptr()), eps,
                                                static_cast<T*>(y.ptr()), rinv, x.rows, static_cast<int>(x.cols)));
    post();
}
void k_rmsnorm_bwd(const Tensor& dy, const Tensor& x, const float* rinv, const Tensor& w, const Tensor* dw,
                   const Tensor* dx, const Tensor* addend) {
    const int C = static_cast<int>(x.cols);
    if (addend && (!dx || addend->rows != x.rows || addend->cols != x.cols || addend->dtype != dx->dtype))
        throw std::runtime_error("rmsnorm backward: the addend must have dx's shape and type");
    if (dx && dw && x.dtype == PK_BF16 && C % 8 == 0 && C <= 2048 && aligned16p(x.ptr()) && aligned16p(dy.ptr()) &&
        aligned16p(dx->ptr()) && aligned16p(w.ptr()) && (!addend || aligned16p(addend->ptr()))) {
        const int nparts = static_cast<int>((x.rows + ROWS_PB - 1) / ROWS_PB);
        Buffer part(sizeof(float) * static_cast<size_t>(nparts) * C);
        const size_t lds = sizeof(float) * 7 * C;
        auto launch = [&](auto np) {
            constexpr int NP = decltype(np)::value;
            if (addend)
                hipLaunchKernelGGL((rms_bwd_dx_dw8<NP, true>), dim3(nparts), dim3(512), lds, tape_stream(),
                                   static_cast<const uint16_t*>(dy.ptr()), static_cast<const uint16_t*>(x.ptr()), rinv,
                                   static_cast<const float*>(w.ptr()), static_cast<const uint16_t*>(addend->ptr()),
                                   static_cast<uint16_t*>(dx->ptr()), static_cast<float*>(part.p), x.rows, C);
            else
                hipLaunchKernelGGL((rms_bwd_dx_dw8<NP, false>), dim3(nparts), dim3(512), lds, tape_stream(),
                                   static_cast<const uint16_t*>(dy.ptr()), static_cast<const uint16_t*>(x.ptr()), rinv,
                                   static_cast<const float*>(w.ptr()), static_cast<const uint16_t*>(nullptr),
                                   static_cast<uint16_t*>(dx->ptr()), static_cast<float*>(part.p), x.rows, C);
        };
        if (C <= 512)
            launch(std::integral_constant<int, 1>{});
        else if (C <= 1024)
            launch(std::integral_constant<int, 2>{});
        else
            launch(std::integral_constant<int, 4>{});
        post();
        hipLaunchKernelGGL(colsum_parts, dim3((C + 63) / 64), dim3(1024), 0, tape_stream(),
                           static_cast<const float*>(part.p), static_cast<float*>(dw->ptr()), nparts, C);
        post();
        return;
    }
    if (dx) {
        if (x.dtype == PK_BF16 && C % 8 == 0 && aligned16p(x.ptr()) && aligned16p(dy.ptr()) && aligned16p(dx->ptr()) &&
            aligned16p(w.ptr())) {
            hipLaunchKernelGGL(rms_bwd_dx8, dim3((x.rows + 3) / 4), dim3(NT), 0, tape_stream(),
                               static_cast<const uint16_t*>(dy.ptr()), static_cast<const uint16_t*>(x.ptr()), rinv,
                               static_cast<const float*>(w.ptr()), static_cast<uint16_t*>(dx->ptr()), x.rows, C);
        } else {
            PK_DISPATCH1(T, x.dtype, hipLaunchKernelGGL((rms_bwd_dx<T>), dim3((x.rows + 3) / 4), dim3(NT), 0, tape_stream(),
                                                        static_cast<const T*>(dy.ptr()), static_cast<const T*>(x.ptr()), rinv,
                                                        static_cast<const float*>(w.ptr()), static_cast<T*>(dx->ptr()),
                                                        x.rows, C));
        }
        post();
        if (addend) k_add(*dx, *addend, *dx);  // elementwise, so in place is fine
    }
    if (dw) {
        const int nparts = static_cast<int>((x.rows + ROWS_PB - 1) / ROWS_PB);
        Buffer part(sizeof(float) * static_cast<size_t>(nparts) * C);
        if (x.dtype == PK_BF16 && C % 8 == 0 && NT % (C / 8) == 0 && aligned16p(x.ptr()) && aligned16p(dy.ptr())) {
            hipLaunchKernelGGL(rms_bwd_dw_part8, dim3(nparts), dim3(NT), sizeof(float) * (NT / (C / 8)) * C, tape_stream(),
                               static_cast<const uint16_t*>(dy.ptr()), static_cast<const uint16_t*>(x.ptr()), rinv,
                               static_cast<float*>(part.p), x.rows, C);
        } else {
            PK_DISPATCH1(T, x.dtype, hipLaunchKernelGGL((rms_bwd_dw_part<T>), dim3(nparts), dim3(NT), 0, tape_stream(),
                                                        static_cast<const T*>(dy.ptr()), static_cast<const T*>(x.ptr()), rinv,
                                                        static_cast<float*>(part.p), x.rows, C));
        }
        post();
        hipLaunchKernelGGL(colsum_parts, dim3((C + 63) / 64), dim3(1024), 0, tape_stream(),
                           static_cast<const float*>(part.p), static_cast<float*>(dw->ptr()), nparts, C);
        post();
    }
}
namespace {
RopeFreq rope_freq(const Tensor& x, float theta, int d, int head_dim) {
    if (x.cols != 3 * d) throw std::runtime_error("apply_rope: cols must be divisible by 3");
    if (head_dim % 2 != 0 || head_dim > d) throw std::runtime_error("apply_rope: head_dim must be even and <= d");
    if (head_dim > 2 * ROPE_MAX_PAIRS) throw std::runtime_error("apply_rope: head_dim above 256 is not supported");
    RopeFreq freq;
    for (int dim = 0; dim < head_dim; dim += 2)  // ops.cpp:499-500
        freq.f[dim >> 1] = 1.0f / std::pow(theta, static_cast<float>(dim) / static_cast<float>(head_dim));
    return freq;
}
}  // namespace
void k_rope(const Tensor& x, const int* pos, float theta, int d, int head_dim, int rot_heads, bool inverse,
            const Tensor& y) {
    const RopeFreq freq = rope_freq(x, theta, d, head_dim);
    PK_DISPATCH1(T, x.dtype, hipLaunchKernelGGL((rope_k<T>), ew_grid(x.numel() / 2), dim3(NT), 0, tape_stream(),
                                                static_cast<const T*>(x.ptr()), pos, freq, d, head_dim, rot_heads,
                                                inverse ? -1.0f : 1.0f, static_cast<T*>(y.ptr()), x.rows));
    post();
}
void k_rope_inplace(const Tensor& x, const int* pos, float theta, int d, int head_dim, int rot_heads, bool inverse) {
    const RopeFreq freq = rope_freq(x, theta, d, head_dim);
    if (rot_heads < 1 || rot_heads * head_dim > d) throw std::runtime_error("apply_rope: head_dim must be even and <= d");
    PK_DISPATCH1(T, x.dtype,
                 hipLaunchKernelGGL((rope_inplace_k<T>), ew_grid(x.rows * rot_heads * head_dim), dim3(NT), 0, tape_stream(),
                                    static_cast<T*>(x.ptr()), pos, freq, d, head_dim, rot_heads, inverse ? -1.0f : 1.0f, x.rows));
    post();
}
void k_embedding_fwd(const Tensor& table, const int* ids, const Tensor& y) {
    if (y.dtype == PK_BF16 && y.cols % 8 == 0 && aligned16p(y.ptr()) && aligned16p(table.ptr())) {
        const int64_t n8 = y.numel() / 8;
        hipLaunchKernelGGL(emb_fwd8, dim3(static_cast<unsigned>((n8 + NT - 1) / NT)), dim3(NT), 0, tape_stream(),
                           static_cast<const float*>(table.ptr()), ids, static_cast<uint16_t*>(y.ptr()), y.rows,
                           static_cast<int>(y.cols));
        post();
        return;
    }
    PK_DISPATCH1(T, y.dtype, hipLaunchKernelGGL((emb_fwd<T>), ew_grid(y.numel()), dim3(NT), 0, tape_stream(),
                                                static_cast<const float*>(table.ptr()), ids, static_cast<T*>(y.ptr()),
                                                y.rows, static_cast<int>(y.cols)));
    post();
}
void k_embedding_bwd(const Tensor& dy, const int* ids, const Tensor& dtable) {
    if (dy.rows > (1 << 30)) shape_fail("embedding: more than 2^30 rows");
    const int n = static_cast<int>(dy.rows), d = static_cast<int>(dy.cols);
    const hipStream_t st = tape_stream();
    Buffer rows_in(sizeof(int) * n), rows_out(sizeof(int) * n), ids_out(sizeof(int) * n);
    int* const r_in = static_cast<int*>(rows_in.p);
    int* const r_out = static_cast<int*>(rows_out.p);
    int* const i_out = static_cast<int*>(ids_out.p);
    hipLaunchKernelGGL(iota_i32, dim3((n + NT - 1) / NT), dim3(NT), 0, st, r_in, n);
    size_t tmp_bytes = 0;  // radix sort is stable: equal ids keep their rows in ascending order
    HIPCHK(hipcub::DeviceRadixSort::SortPairs(nullptr, tmp_bytes, ids, i_out, r_in, r_out, n, 0, 32, st));
    Buffer tmp(tmp_bytes ? tmp_bytes : 16);
    HIPCHK(hipcub::DeviceRadixSort::SortPairs(tmp.p, tmp_bytes, ids, i_out, r_in, r_out, n, 0, 32, st));
    PK_DISPATCH1(T, dy.dtype, hipLaunchKernelGGL((emb_bwd_runs<T>), dim3(n, (d + EMB_NT - 1) / EMB_NT), dim3(EMB_NT), 0, st,
                                                 static_cast<const T*>(dy.ptr()), i_out, r_out,
                                                 static_cast<float*>(dtable.ptr()), n, d));
    post();
}
void k_ce_rows(const Tensor& logits, const int* targets, float gscale, float* nll_rows) {
    PK_DISPATCH1(T, logits.dtype, hipLaunchKernelGGL((ce_rows<T>), dim3(logits.rows), dim3(NT), 0, tape_stream(),
                                                     static_cast<T*>(logits.ptr()), targets, gscale, nll_rows,
                                                     static_cast<int>(logits.cols)));
    post();
}
bool k_ce_rows_once(const Tensor& logits, const int* targets, float gscale, float* nll_rows, const Tensor* dl, int64_t dl_ld) {
    const int C = static_cast<int>(logits.cols);
    if (dl_ld == 0) dl_ld = C;
    if (logits.dtype != PK_F32 || C % 4 != 0 || C > CE_NT * CE_V4 * 4) return false;  // caller takes the generic kernel
    const float* src = static_cast<const float*>(logits.ptr());
    if (!dl) {
        hipLaunchKernelGGL((ce_rows_reg<float, false>), dim3(logits.rows), dim3(CE_NT), 0, tape_stream(), src,
                           static_cast<float*>(nullptr), targets, gscale, nll_rows, C, dl_ld);
    } else if (dl->dtype == PK_F32) {
        hipLaunchKernelGGL((ce_rows_reg<float, true>), dim3(logits.rows), dim3(CE_NT), 0, tape_stream(), src,
                           static_cast<float*>(dl->ptr()), targets, gscale, nll_rows, C, dl_ld);
    } else {
        hipLaunchKernelGGL((ce_rows_reg<uint16_t, true>), dim3(logits.rows), dim3(CE_NT), 0, tape_stream(), src,
                           static_cast<uint16_t*>(dl->ptr()), targets, gscale, nll_rows, C, dl_ld);
    }
    post();
    return true;
}
void k_mean_f32(const float* x, int64_t n, const Tensor& out) {
    if (out.dtype != PK_F32 || out.rows * out.cols != 1) throw std::runtime_error("mean: the result is one float");
    hipLaunchKernelGGL(mean_f32_k, dim3(1), dim3(1024), 0, tape_stream(), x, n, static_cast<float*>(out.ptr()));
    post();
}
double k_sum_f32_to_host(const float* x, int64_t n) {
    Buffer out(sizeof(double));
    hipLaunchKernelGGL(sum_f32_k, dim3(1), dim3(NT), 0, tape_stream(), x, n, static_cast<double*>(out.p));
    post();
    double h = 0.0;
    HIPCHK(hipMemcpyAsync(&h, out.p, sizeof(double), hipMemcpyDeviceToHost, tape_stream()));
    HIPCHK(hipStreamSynchronize(tape_stream()));
    return h;
}
int k_sumsq_parts(const Tensor& g, double* part_dev) {
    if (g.dtype != PK_F32) throw std::runtime_error("clip_grad_norm: gradients must be fp32");
    const int nb = static_cast<int>(std::min<int64_t>((g.numel() + NT - 1) / NT, SUMSQ_MAX_PARTS));
    hipLaunchKernelGGL(sumsq_part, dim3(nb), dim3(NT), 0, tape_stream(), static_cast<const float*>(g.ptr()), g.numel(),
                       part_dev);
    post();
    return nb;
}
double k_sum_f64_to_host(const double* part_dev, int64_t n) {
    std::vector<double> h(n);
    HIPCHK(hipMemcpyAsync(h.data(), part_dev, sizeof(double) * n, hipMemcpyDeviceToHost, tape_stream()));
    HIPCHK(hipStreamSynchronize(tape_stream()));
    double s = 0.0;
    for (double v : h) s += v;
    return s;
}
double k_sumsq_to_host(const Tensor& g) {
    Buffer part(sizeof(double) * SUMSQ_MAX_PARTS);
    const int nb = k_sumsq_parts(g, static_cast<double*>(part.p));
    return k_sum_f64_to_host(static_cast<const double*>(part.p), nb);
}
void k_adamw(const Tensor& p, const Tensor& g, const Tensor& m, const Tensor& v, float lr, float b1, float b2,
             float eps, float wd, float c1, float c2, float grad_scale) {
    if (grad_scale != 1.0f)
        hipLaunchKernelGGL(adamw_k<true>, ew_grid(p.numel()), dim3(NT), 0, tape_stream(), static_cast<float*>(p.ptr()),
                           static_cast<float*>(g.ptr()), static_cast<float*>(m.ptr()), static_cast<float*>(v.ptr()), lr, b1,
                           b2, eps, wd, c1, c2, grad_scale, p.numel());
    else
        hipLaunchKernelGGL(adamw_k<false>, ew_grid(p.numel()), dim3(NT), 0, tape_stream(), static_cast<float*>(p.ptr()),
                           static_cast<float*>(g.ptr()), static_cast<float*>(m.ptr()), static_cast<float*>(v.ptr()), lr, b1,
                           b2, eps, wd, c1, c2, 1.0f, p.numel());
    post();
}

// ---- GEMM -------------------------------------------------------------------
namespace {
rocblas_handle blas() {
    static thread_local rocblas_handle h = [] {  // a rocBLAS handle serves one host thread at a time
        rocblas_handle x;
        if (rocblas_create_handle(&x) != rocblas_status_success) throw std::runtime_error("rocblas_create_handle failed");
        // no atomics-based split-K: a recomputed (checkpointed) block must reproduce its first forward bit for bit
        rocblas_set_atomics_mode(x, rocblas_atomics_not_allowed);
        return x;
    }();
    return h;
}
}  // namespace

namespace {
// Process-wide and read by every model's thread, set by pk_set_gemm_backend from any thread: an atomic, relaxed
// (a product sees either the old or the new choice, both of which give the same numbers up to rounding order).
std::atomic<int> g_gemm_hand_written{[] {
    const char* v = std::getenv("PK_GEMM");
    return (v && std::string(v) == "library") ? 0 : 1;
}()};
}
void set_gemm_backend(int hand_written) { g_gemm_hand_written.store(hand_written, std::memory_order_relaxed); }
int gemm_backend() { return g_gemm_hand_written.load(std::memory_order_relaxed); }
namespace {
std::atomic<int> g_head_in_product{1};
}
void set_head_kernel(int in_product) { g_head_in_product.store(in_product != 0, std::memory_order_relaxed); }
int head_kernel() { return g_head_in_product.load(std::memory_order_relaxed); }

void gemm(const Tensor& A, bool tA, const Tensor& B, bool tB, void* C, int c_dtype, int64_t M, int64_t N, int64_t ldc,
          float beta, int64_t lda) {
    if (lda == 0) lda = A.cols;
    const int64_t Ka = tA ? A.rows : A.cols, Kb = tB ? B.cols : B.rows;
    const int64_t Ma = tA ? A.cols : A.rows, Nb = tB ? B.rows : B.cols;
    if (Ka != Kb) shape_fail("gemm: inner dimensions disagree");  // device.cpp:97
    if (Ma != M || Nb != N) shape_fail("gemm: output shape mismatch");
    if (A.dtype != B.dtype) throw std::runtime_error("gemm: operand dtypes differ");
    // Which kernel: measured per shape on the MI355X as GPU time from a kernel trace (timing launches from the host
    // measures the library's longer host path instead), on the Linear shapes of a d = 512 block and of the tied
    // head: the hand-written kernel is ahead of the library or level with it on all 15 products, so bf16 operands
    // go to it whenever it takes them (backends 1 and 2 alike); backend 0 sends everything to the library.
    const bool mine = gemm_backend() != 0;
    if (A.dtype == PK_BF16 && mine &&
        gemm_mfma_bf16(A.ptr(), tA, lda, B.ptr(), tB, B.cols, C, c_dtype, M, N, Ka, ldc, beta, tape_stream()))
        return;
    // Row-major C = op(A) op(B)  <=>  column-major C^T = op(B)^T op(A)^T.
    const rocblas_datatype ab = A.dtype == PK_F32 ? rocblas_datatype_f32_r : rocblas_datatype_bf16_r;
    const rocblas_datatype ct = c_dtype == PK_F32 ? rocblas_datatype_f32_r : rocblas_datatype_bf16_r;
    const float alpha = 1.0f;
    rocblas_set_stream(blas(), tape_stream());
    // Long contractions with a small output (weight gradients X^T dY over every token; dh = dlogits E over the
    // vocabulary): one GEMM would be a few hundred tiles at most and leave most of the chip idle. The contraction
    // axis is cut into slices that run as one strided-batched GEMM into separate fp32 partial products, which are
    // then added in slice order: no atomics, so the sum is the same on every run.
    if (!tB && ldc == N && Ka >= 2048 && M * N <= (int64_t{1} << 21) && (beta == 0.0f || beta == 1.0f)) {
        int S = 8;
        while (S > 1 && (Ka % S != 0 || Ka / S < 256)) S >>= 1;
        if (S > 1) {
            const int64_t Ks = Ka / S;
            Buffer part(sizeof(float) * static_cast<size_t>(S) * M * N);
            const float zero = 0.0f;
            const int64_t stride_a = tA ? Ks * lda : Ks, stride_b = Ks * B.cols;
            const rocblas_status st = rocblas_gemm_strided_batched_ex(
                blas(), rocblas_operation_none, tA ? rocblas_operation_transpose : rocblas_operation_none,
                static_cast<rocblas_int>(N), static_cast<rocblas_int>(M), static_cast<rocblas_int>(Ks), &alpha, B.ptr(), ab,
                static_cast<rocblas_int>(B.cols), stride_b, A.ptr(), ab, static_cast<rocblas_int>(lda), stride_a, &zero,
                part.p, rocblas_datatype_f32_r, static_cast<rocblas_int>(N), M * N, part.p, rocblas_datatype_f32_r,
                static_cast<rocblas_int>(N), M * N, S, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
            if (st != rocblas_status_success)
                throw std::runtime_error(std::string("rocblas_gemm_strided_batched_ex failed: ") + rocblas_status_to_string(st));
            if (c_dtype == PK_F32 && (M * N) % 4 == 0 && aligned16p(C))
                hipLaunchKernelGGL(add_parts4, ew_grid(M * N / 4), dim3(NT), 0, tape_stream(),
                                   static_cast<const float*>(part.p), static_cast<float*>(C), S, M * N / 4, beta);
            else if (c_dtype == PK_F32)
                hipLaunchKernelGGL((add_parts<float>), ew_grid(M * N), dim3(NT), 0, tape_stream(),
                                   static_cast<const float*>(part.p), static_cast<float*>(C), S, M * N, beta);
            else
                hipLaunchKernelGGL((add_parts<uint16_t>), ew_grid(M * N), dim3(NT), 0, tape_stream(),
                                   static_cast<const float*>(part.p), static_cast<uint16_t*>(C), S, M * N, beta);
            post();
            return;
        }
    }
    const rocblas_status st = rocblas_gemm_ex(
        blas(), tB ? rocblas_operation_transpose : rocblas_operation_none,
        tA ? rocblas_operation_transpose : rocblas_operation_none, static_cast<rocblas_int>(N),
        static_cast<rocblas_int>(M), static_cast<rocblas_int>(Ka), &alpha, B.ptr(), ab, static_cast<rocblas_int>(B.cols),
        A.ptr(), ab, static_cast<rocblas_int>(lda), &beta, C, ct, static_cast<rocblas_int>(ldc), C, ct,
        static_cast<rocblas_int>(ldc), rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    if (st != rocblas_status_success)
        throw std::runtime_error(std::string("rocblas_gemm_ex failed: ") + rocblas_status_to_string(st));
}

void gemm_tn_split(const Tensor& A, const Tensor& B, float* const* dst, int nsplit, float beta) {
    const int64_t K = A.rows, M = A.cols, W = B.cols;
    if (B.rows != K) throw std::runtime_error("gemm: inner dimensions disagree");
    if (nsplit < 1 || nsplit > 4 || W % nsplit != 0) throw std::runtime_error("gemm_tn_split: bad column split");
    if (A.dtype != B.dtype) throw std::runtime_error("gemm: operand dtypes differ");
    if (A.dtype == PK_BF16 && gemm_backend() != 0) {
        // the product [M, W] as fp32 partial products over slices of the tokens; the kernel that adds them deals the
        // column blocks to their tensors (measured ahead of the library's batched form on all four weight-gradient
        // shapes of a d = 512 block once the slices are one per resident workgroup)
        std::unique_ptr<Buffer> part;
        int nparts = 0;
        if (gemm_mfma_bf16_parts(A.ptr(), true, M, B.ptr(), false, W, M, W, K, tape_stream(), part, nparts)) {
            SplitDst d{};
            for (int k = 0; k < nsplit; ++k) d.p[k] = dst[k];
            bool vec = (W / nsplit) % 4 == 0;
            for (int k = 0; k < nsplit; ++k) vec = vec && aligned16p(dst[k]);
            if (vec)
                hipLaunchKernelGGL(add_parts_split4, ew_grid(M * W / 4), dim3(NT), 0, tape_stream(),
                                   static_cast<const float*>(part->p), d, nparts, M, W / nsplit, nsplit, beta);
            else
                hipLaunchKernelGGL(add_parts_split, ew_grid(M * W), dim3(NT), 0, tape_stream(),
                                   static_cast<const float*>(part->p), d, nparts, M, W / nsplit, nsplit, beta);
            post();
            return;
        }
    }
    const rocblas_datatype ab = A.dtype == PK_F32 ? rocblas_datatype_f32_r : rocblas_datatype_bf16_r;
    const float alpha = 1.0f, zero = 0.0f;
    rocblas_set_stream(blas(), tape_stream());
    // the contraction axis in slices, as in gemm(); short contractions run as one slice
    int S = 1;
    if (K >= 2048 && M * W <= (int64_t{1} << 21)) {
        S = 8;
        while (S > 1 && (K % S != 0 || K / S < 256)) S >>= 1;
    }
    const int64_t Ks = K / S;
    Buffer part(sizeof(float) * static_cast<size_t>(S) * M * W);
    const rocblas_status st = rocblas_gemm_strided_batched_ex(
        blas(), rocblas_operation_none, rocblas_operation_transpose, static_cast<rocblas_int>(W),
        static_cast<rocblas_int>(M), static_cast<rocblas_int>(Ks), &alpha, B.ptr(), ab, static_cast<rocblas_int>(W), Ks * W,
        A.ptr(), ab, static_cast<rocblas_int>(M), Ks * M, &zero, part.p, rocblas_datatype_f32_r,
        static_cast<rocblas_int>(W), M * W, part.p, rocblas_datatype_f32_r, static_cast<rocblas_int>(W), M * W, S,
        rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    if (st != rocblas_status_success)
        throw std::runtime_error(std::string("rocblas_gemm_strided_batched_ex failed: ") + rocblas_status_to_string(st));
    SplitDst d{};
    for (int k = 0; k < nsplit; ++k) d.p[k] = dst[k];
    bool vec = (W / nsplit) % 4 == 0;
    for (int k = 0; k < nsplit; ++k) vec = vec && aligned16p(dst[k]);
    if (vec)
        hipLaunchKernelGGL(add_parts_split4, ew_grid(M * W / 4), dim3(NT), 0, tape_stream(), static_cast<const float*>(part.p),
                           d, S, M, W / nsplit, nsplit, beta);
    else
        hipLaunchKernelGGL(add_parts_split, ew_grid(M * W), dim3(NT), 0, tape_stream(), static_cast<const float*>(part.p), d,
                           S, M, W / nsplit, nsplit, beta);
    post();
}

}  // namespace pk
