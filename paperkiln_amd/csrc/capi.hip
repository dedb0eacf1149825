// The C ABI of libpaperkiln_amd.so: argument checking, dispatch between the
// MFMA and the generic kernels, and the thread-local error string. There is
// no CPU path behind any entry: without a gfx950 device every call fails.
#include <cstdio>
#include <cstring>
#include <mutex>

#include "pk_internal.h"

namespace pk {

namespace {
thread_local std::string g_err;
}

// Scratch of pk_attn_bwd_static: the backward's workspace (row sums D_i and, for a band mask with sink keys, the
// partial sink rows) as a device array of the library itself, so that the call needs no allocation by anybody.
// `scratch` is a host-side stand-in for the symbol, never a device address: every GPU holds its own copy at its
// own address, looked up once per device with hipGetSymbolAddress and used through that pointer only.
constexpr size_t SCRATCH_BYTES = PK_ATTN_BWD_STATIC_MAX_WORKSPACE;
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[MAX_DEVICES] = {};

// The current device's copy of `scratch`; the lookup runs once per device, with that device current.
int scratch_of_current_device(void** out) {
    int dev = -1;
    PK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(PK_ERR_ARGUMENT, "device index beyond the scratch table");
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        PK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(PK_ERR_HIP, "hipGetSymbolAddress returned a null address for the scratch array");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return PK_OK;
}
}  // namespace

void set_error(const std::string& msg) { g_err = msg; }

int fail(int code, const std::string& msg) {
    g_err = msg;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    g_err = std::string("HIP error: ") + hipGetErrorString(e) + " in " + what;
    return PK_ERR_HIP;
}

namespace {

int check_shape(const pk_attn_shape* s, const char* who) {
    if (!s) return fail(PK_ERR_ARGUMENT, std::string(who) + ": null shape");
    if (s->B <= 0 || s->T <= 0 || s->Hq <= 0 || s->Hkv <= 0 || s->dk <= 0)
        return fail(PK_ERR_SHAPE, std::string(who) + ": shape mismatch (non-positive dimension)");
    if (s->Hq % s->Hkv != 0)
        return fail(PK_ERR_SHAPE, std::string(who) + ": shape mismatch (Hq not a multiple of Hkv)");
    if (s->T > (1 << 24))  // index + window sums stay far inside 32 bits
        return fail(PK_ERR_SHAPE, std::string(who) + ": more than 2^24 tokens per sequence not supported");
    if (s->dk > 256) return fail(PK_ERR_SHAPE, std::string(who) + ": head_dim > 256 not supported");
    if (s->window < 0 || s->sinks < 0)
        return fail(PK_ERR_ARGUMENT, std::string(who) + ": window and sinks must be >= 0");
    if (s->window > 0 && !s->causal)
        return fail(PK_ERR_ARGUMENT, std::string(who) + ": a window requires causal (swa_attention is causal)");
    if ((s->dtype != PK_F32 && s->dtype != PK_BF16) || (s->grad_dtype != PK_F32 && s->grad_dtype != PK_BF16))
        return fail(PK_ERR_ARGUMENT, std::string(who) + ": dtype must be PK_F32 or PK_BF16");
    return PK_OK;
}

bool bad(const pk_tensor4* t) { return !t || !t->ptr; }

// The mask the kernels run with. The reference takes size_t arguments and defines a window that covers the
// whole sequence as plain causal attention (tests/test_swa.cpp:47-57), so "window = INT32_MAX" is a legal way
// to ask for no band; the kernels add the window to key and query indices in 32-bit arithmetic, so the values
// are brought into [0, T] here, once, and every later use (tile skipping, sink tail, workspace size) sees these.
struct Mask {
    int window, sinks;
};
Mask effective_mask(const pk_attn_shape* s) {
    Mask m = {s->window, s->sinks};
    if (m.window >= s->T) m.window = 0, m.sinks = 0;  // every key at or before the query is inside the window
    if (m.window == 0) m.sinks = 0;                    // sinks only matter under a band
    if (m.sinks > s->T) m.sinks = s->T;
    return m;
}

// workspace = delta [B, Hq, T] fp32, then (band mask with 1..32 sink keys only) the sink-tail partial rows
size_t delta_bytes(const pk_attn_shape* s) { return sizeof(float) * static_cast<size_t>(s->B) * s->Hq * s->T; }
size_t tail_bytes(const pk_attn_shape* s) {
    const Mask m = effective_mask(s);
    const SinkTail t = sink_tail(s->T, m.window, m.sinks);
    if (t.nch == 0) return 0;
    const size_t pad = (256 - delta_bytes(s) % 256) % 256;
    return pad + sink_tail_bytes(s->B * s->Hkv, t.nch, s->dk);
}

// (GQA, band-free bf16 only) the per-split partial dK / dV of the dK/dV launch, after delta and the sink tail
int head_split_of(const pk_attn_shape* s) {
    const Mask m = effective_mask(s);
    return gqa_head_split(s->B, s->T, s->Hq, s->Hkv, s->dk, s->causal != 0, m.window, s->dtype == PK_BF16);
}
size_t part_bytes(const pk_attn_shape* s) {
    const int hs = head_split_of(s);
    if (hs <= 1) return 0;
    const size_t before = delta_bytes(s) + tail_bytes(s);
    return (256 - before % 256) % 256 + gqa_part_bytes(s->B * s->Hkv, hs, s->T, s->dk);
}

int bwd_stages(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k, const pk_tensor4* v,
               const pk_tensor4* o, const float* lse, const pk_tensor4* d_o, const pk_tensor4* dq, const pk_tensor4* dk,
               const pk_tensor4* dv, void* workspace, size_t workspace_bytes, int stages, bool split_heads, void* stream);

void fill_common(AttnArgs& a, const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k,
                 const pk_tensor4* v, const pk_tensor4* o) {
    std::memset(&a, 0, sizeof a);
    a.q = q->ptr; a.q_sb = q->stride_b; a.q_st = q->stride_t; a.q_sh = q->stride_h;
    a.k = k->ptr; a.k_sb = k->stride_b; a.k_st = k->stride_t; a.k_sh = k->stride_h;
    a.v = v->ptr; a.v_sb = v->stride_b; a.v_st = v->stride_t; a.v_sh = v->stride_h;
    a.o = o->ptr; a.o_sb = o->stride_b; a.o_st = o->stride_t; a.o_sh = o->stride_h;
    a.B = s->B; a.T = s->T; a.Hq = s->Hq; a.Hkv = s->Hkv; a.dk_dim = s->dk;
    const Mask m = effective_mask(s);
    a.causal = s->causal != 0; a.window = m.window; a.sinks = m.sinks;
    a.scale = s->scale;
    a.grad_f32 = s->grad_dtype == PK_F32;
    a.head_split = 1;
}

}  // namespace
}  // namespace pk

using namespace pk;

extern "C" {

const char* pk_last_error(void) { return g_err.c_str(); }

int pk_init(int device, char* arch, size_t arch_len) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0)
        return fail(PK_ERR_HIP, "pk_init: no HIP device visible (this library has no CPU path)");
    if (device < 0 || device >= n) return fail(PK_ERR_ARGUMENT, "pk_init: device index out of range");
    PK_HIP(hipSetDevice(device));
    hipDeviceProp_t p;
    PK_HIP(hipGetDeviceProperties(&p, device));
    if (arch && arch_len) {
        std::snprintf(arch, arch_len, "%s", p.gcnArchName);
    }
    if (std::strncmp(p.gcnArchName, "gfx950", 6) != 0)
        return fail(PK_ERR_HIP, std::string("pk_init: kernels are built for gfx950 only, found ") + p.gcnArchName);
    void* scratch_ptr = nullptr;  // this device's copy of the static scratch, so the first static call finds it
    return scratch_of_current_device(&scratch_ptr);
}

int pk_attn_fwd(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k, const pk_tensor4* v,
                const pk_tensor4* o, float* lse, void* stream) {
    if (int rc = check_shape(s, "pk_attn_fwd")) return rc;
    if (bad(q) || bad(k) || bad(v) || bad(o) || !lse)
        return fail(PK_ERR_ARGUMENT, "pk_attn_fwd: null tensor");
    AttnArgs a;
    fill_common(a, s, q, k, v, o);
    a.lse = lse;
    const void* used[] = {q->ptr, k->ptr, v->ptr, o->ptr, lse};
    for (const void* p : used) dev_touch(p, stream);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->dtype == PK_BF16 && mfma_supported(a)) return launch_mfma_fwd(a, st);
    if (s->dtype == PK_F32 && f32_mfma_supported(a)) return launch_f32_mfma_fwd(a, st);
    return launch_generic_fwd(a, s->dtype == PK_BF16, st);
}

size_t pk_attn_bwd_workspace_bytes(const pk_attn_shape* s) {
    if (check_shape(s, "pk_attn_bwd_workspace_bytes")) return 0;
    return delta_bytes(s) + tail_bytes(s) + part_bytes(s);
}

int pk_attn_bwd(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k, const pk_tensor4* v,
                const pk_tensor4* o, const float* lse, const pk_tensor4* d_o, const pk_tensor4* dq,
                const pk_tensor4* dk, const pk_tensor4* dv, void* workspace, size_t workspace_bytes,
                void* stream) {
    return pk_attn_bwd_stages(s, q, k, v, o, lse, d_o, dq, dk, dv, workspace, workspace_bytes,
                              PK_BWD_ALL, stream);
}

int pk_attn_bwd_static(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k, const pk_tensor4* v,
                       const pk_tensor4* o, const float* lse, const pk_tensor4* d_o, const pk_tensor4* dq,
                       const pk_tensor4* dk, const pk_tensor4* dv, void* stream) {
    if (int rc = check_shape(s, "pk_attn_bwd_static")) return rc;
    // The GQA head split of the dK/dV launch needs room for its partial sums; where that does not fit the array the
    // heads of a group are walked by one workgroup as before (same results up to the order of summation).
    size_t need = delta_bytes(s) + tail_bytes(s);
    const bool split_heads = need + part_bytes(s) <= SCRATCH_BYTES;
    if (split_heads) need += part_bytes(s);
    if (need > SCRATCH_BYTES)
        return fail(PK_ERR_WORKSPACE, "pk_attn_bwd_static: this shape needs " + std::to_string(need) +
                                          " bytes of scratch, the static array holds " + std::to_string(SCRATCH_BYTES) +
                                          " (PK_ATTN_BWD_STATIC_MAX_WORKSPACE); use pk_attn_bwd with a workspace");
    void* ws = nullptr;
    if (int rc = scratch_of_current_device(&ws)) return rc;
    // Every word of the workspace the kernels read they have written earlier in the same call (D_i by the dQ
    // kernel, each piece's partial sink rows and each split's partial dK / dV by its own workgroup), so nothing has
    // to be cleared between calls.
    return bwd_stages(s, q, k, v, o, lse, d_o, dq, dk, dv, ws, SCRATCH_BYTES, PK_BWD_ALL, split_heads, stream);
}

int pk_attn_bwd_stages(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k,
                       const pk_tensor4* v, const pk_tensor4* o, const float* lse,
                       const pk_tensor4* d_o, const pk_tensor4* dq, const pk_tensor4* dk,
                       const pk_tensor4* dv, void* workspace, size_t workspace_bytes, int stages,
                       void* stream) {
    return bwd_stages(s, q, k, v, o, lse, d_o, dq, dk, dv, workspace, workspace_bytes, stages, true, stream);
}

}  // extern "C"

namespace pk {
namespace {

int bwd_stages(const pk_attn_shape* s, const pk_tensor4* q, const pk_tensor4* k, const pk_tensor4* v,
               const pk_tensor4* o, const float* lse, const pk_tensor4* d_o, const pk_tensor4* dq, const pk_tensor4* dk,
               const pk_tensor4* dv, void* workspace, size_t workspace_bytes, int stages, bool split_heads, void* stream) {
    if (int rc = check_shape(s, "pk_attn_bwd")) return rc;
    if (stages <= 0 || (stages & ~PK_BWD_ALL))
        return fail(PK_ERR_ARGUMENT, "pk_attn_bwd_stages: stages must be a non-empty subset of PK_BWD_ALL");
    if (bad(q) || bad(k) || bad(v) || bad(o) || !lse || bad(d_o) || bad(dq) || bad(dk) || bad(dv))
        return fail(PK_ERR_ARGUMENT, "pk_attn_bwd: null tensor");
    const size_t before_part = delta_bytes(s) + tail_bytes(s);
    if (!workspace || workspace_bytes < before_part + (split_heads ? part_bytes(s) : 0))
        return fail(PK_ERR_WORKSPACE, "pk_attn_bwd: workspace smaller than pk_attn_bwd_workspace_bytes()");
    if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return fail(PK_ERR_ARGUMENT, "pk_attn_bwd: workspace must be 16-byte aligned");
    AttnArgs a;
    fill_common(a, s, q, k, v, o);
    a.lse = const_cast<float*>(lse);
    a.d_o = d_o->ptr; a.do_sb = d_o->stride_b; a.do_st = d_o->stride_t; a.do_sh = d_o->stride_h;
    a.dq = dq->ptr; a.dq_sb = dq->stride_b; a.dq_st = dq->stride_t; a.dq_sh = dq->stride_h;
    a.dk = dk->ptr; a.dk_sb = dk->stride_b; a.dk_st = dk->stride_t; a.dk_sh = dk->stride_h;
    a.dv = dv->ptr; a.dv_sb = dv->stride_b; a.dv_st = dv->stride_t; a.dv_sh = dv->stride_h;
    const void* used[] = {q->ptr, k->ptr, v->ptr, o->ptr, lse, d_o->ptr, dq->ptr, dk->ptr, dv->ptr, workspace};
    for (const void* p : used) dev_touch(p, stream);
    a.delta = static_cast<float*>(workspace);
    if (tail_bytes(s)) {
        const size_t db = delta_bytes(s);
        a.tail = reinterpret_cast<float*>(static_cast<char*>(workspace) + db + (256 - db % 256) % 256);
    }
    if (split_heads && part_bytes(s)) {
        a.head_split = head_split_of(s);
        a.part = reinterpret_cast<float*>(static_cast<char*>(workspace) + before_part + (256 - before_part % 256) % 256);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->dtype == PK_BF16 && mfma_supported(a)) return launch_mfma_bwd(a, stages, st);
    if (s->dtype == PK_F32 && f32_mfma_supported(a)) return launch_f32_mfma_bwd(a, stages, st);
    return launch_generic_bwd(a, s->dtype == PK_BF16, stages, st);
}

}  // namespace
}  // namespace pk
