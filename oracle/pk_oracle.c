/* TEST INFRASTRUCTURE ONLY -- see pk_oracle.h. Plain C, one thread, fp32,
 * the [rows,rows] weight matrix materialised exactly as the reference does. */
#include "pk_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* C[M,N] = A[M,K] . B[K,N], k ascending, plain fp32 adds. The reference goes
 * through device::gemm -> matmul_optimized (src/device.cpp:91-125), whose AVX2
 * lanes sum in a different order; the two agree to fp32 rounding, not bitwise. */
static void gemm_nn(const float* A, const float* B, float* C, size_t M, size_t K, size_t N) {
    memset(C, 0, M * N * sizeof(float));
    for (size_t i = 0; i < M; ++i) {
        float* c = C + i * N;
        for (size_t k = 0; k < K; ++k) {
            const float a = A[i * K + k];
            const float* b = B + k * N;
            for (size_t j = 0; j < N; ++j) c[j] += a * b[j];
        }
    }
}

/* Materialised transpose, as device::gemm does for Trans::T operands on the
 * CPU path (src/device.cpp:121-124). */
static float* transposed(const float* X, size_t R, size_t C) {
    float* t = (float*)malloc(R * C * sizeof(float));
    if (!t) return NULL;
    for (size_t i = 0; i < R; ++i)
        for (size_t j = 0; j < C; ++j) t[j * R + i] = X[i * C + j];
    return t;
}

/* Visible set of query row i as two half-open ranges [a0,a1) u [b0r,b1r).
 * window == 0: fused_attention, src/ops.cpp:879-880.
 * window >= 1: swa_attention's `ranges` lambda, src/ops.cpp:960-965. */
static void visible(size_t i, size_t sl, int causal, size_t window, size_t sinks, size_t* a0,
                    size_t* a1, size_t* b0r, size_t* b1r) {
    const size_t b0 = (i / sl) * sl;
    if (window == 0) {
        *a0 = *a1 = b0;
        *b0r = b0;
        *b1r = causal ? i + 1 : b0 + sl;
        return;
    }
    const size_t ii = i - b0;
    const size_t win_lo = b0 + (ii + 1 > window ? ii + 1 - window : 0);
    const size_t smin = sinks < ii + 1 ? sinks : ii + 1;
    size_t sink_hi = b0 + smin;
    if (sink_hi > win_lo) sink_hi = win_lo;
    *a0 = b0;
    *a1 = sink_hi;
    *b0r = win_lo;
    *b1r = i + 1;
}

static int check_args(size_t rows, size_t seq_len, int causal, size_t window, size_t* sl) {
    if (rows == 0) return 1;
    *sl = seq_len == 0 ? rows : seq_len;
    if (rows % *sl != 0) return 2;
    if (window != 0 && !causal) return 3;
    return 0;
}

int pko_attn_head_fwd(const float* q, const float* k, const float* v, size_t rows, size_t dk,
                      size_t dv, float scale, size_t seq_len, int causal, size_t window,
                      size_t sinks, float* y, float* lse, float* A) {
    size_t sl;
    int rc = check_args(rows, seq_len, causal, window, &sl);
    if (rc) return rc;
    const size_t T = rows;
    float* kt = transposed(k, T, dk);
    if (!kt) return 4;
    gemm_nn(q, kt, A, T, dk, T); /* A = Q K^T, src/ops.cpp:876-877 */
    free(kt);
    for (size_t i = 0; i < T; ++i) {
        size_t a0, a1, b0, b1;
        visible(i, sl, causal, window, sinks, &a0, &a1, &b0, &b1);
        float* row = A + i * T;
        float mx = -1e30f; /* src/ops.cpp:881 */
        for (size_t j = a0; j < a1; ++j) {
            row[j] *= scale;
            mx = row[j] > mx ? row[j] : mx;
        }
        for (size_t j = b0; j < b1; ++j) {
            row[j] *= scale;
            mx = row[j] > mx ? row[j] : mx;
        }
        float z = 0.0f;
        for (size_t j = a0; j < a1; ++j) {
            row[j] = expf(row[j] - mx);
            z += row[j];
        }
        for (size_t j = b0; j < b1; ++j) {
            row[j] = expf(row[j] - mx);
            z += row[j];
        }
        for (size_t j = 0; j < T; ++j) {
            const int vis = (j >= a0 && j < a1) || (j >= b0 && j < b1);
            row[j] = vis ? row[j] / z : 0.0f; /* hard zero, src/ops.cpp:890-896 */
        }
        if (lse) lse[i] = mx + logf(z);
    }
    gemm_nn(A, v, y, T, T, dv); /* Y = A V, src/ops.cpp:899-900 */
    return 0;
}

int pko_attn_head_bwd(const float* q, const float* k, const float* v, const float* A,
                      const float* dy, size_t rows, size_t dk, size_t dv, float scale,
                      size_t seq_len, int causal, size_t window, size_t sinks, float* dq,
                      float* dk_out, float* dv_out) {
    size_t sl;
    int rc = check_args(rows, seq_len, causal, window, &sl);
    if (rc) return rc;
    const size_t T = rows;
    float* At = transposed(A, T, T);
    float* vt = transposed(v, T, dv);
    float* ds = (float*)malloc(T * T * sizeof(float));
    if (!At || !vt || !ds) {
        free(At);
        free(vt);
        free(ds);
        return 4;
    }
    gemm_nn(At, dy, dv_out, T, T, dv); /* dV = A^T dY, src/ops.cpp:907-910 */
    gemm_nn(dy, vt, ds, T, dv, T);     /* dP = dY V^T, src/ops.cpp:915-916 */
    free(At);
    free(vt);
    for (size_t i = 0; i < T; ++i) {
        size_t a0, a1, b0, b1;
        visible(i, sl, causal, window, sinks, &a0, &a1, &b0, &b1);
        const float* arow = A + i * T;
        float* drow = ds + i * T;
        /* src/ops.cpp:920-921 sums over [b0,hi), :1015-1016 over [b0,i]; the
         * masked entries in between carry A == 0 and add exactly 0. */
        float dot = 0.0f;
        for (size_t j = a0; j < b1; ++j) dot += drow[j] * arow[j];
        for (size_t j = 0; j < T; ++j) {
            const int vis = (j >= a0 && j < a1) || (j >= b0 && j < b1);
            drow[j] = vis ? scale * arow[j] * (drow[j] - dot) : 0.0f;
        }
    }
    float* dst = transposed(ds, T, T);
    if (!dst) {
        free(ds);
        return 4;
    }
    gemm_nn(ds, k, dq, T, T, dk);      /* dQ = dS K,   src/ops.cpp:927-929 */
    gemm_nn(dst, q, dk_out, T, T, dk); /* dK = dS^T Q, src/ops.cpp:930-932 */
    free(ds);
    free(dst);
    return 0;
}

/* Copy head h of batch b out of / into a [B,T,H,dk] tensor: the slice_cols /
 * concat_cols pair of src/llama.cpp:48-53. */
static void gather_head(const float* x, size_t b, size_t h, size_t T, size_t H, size_t dk,
                        float* out) {
    for (size_t t = 0; t < T; ++t)
        memcpy(out + t * dk, x + ((b * T + t) * H + h) * dk, dk * sizeof(float));
}
static void scatter_head(float* x, size_t b, size_t h, size_t T, size_t H, size_t dk,
                         const float* in, int accumulate) {
    for (size_t t = 0; t < T; ++t) {
        float* dst = x + ((b * T + t) * H + h) * dk;
        if (accumulate) {
            for (size_t j = 0; j < dk; ++j) dst[j] += in[t * dk + j];
        } else {
            memcpy(dst, in + t * dk, dk * sizeof(float));
        }
    }
}

int pko_attn_fwd(const float* q, const float* k, const float* v, size_t B, size_t T, size_t Hq,
                 size_t Hkv, size_t dk, float scale, int causal, size_t window, size_t sinks,
                 float* o, float* lse) {
    if (Hkv == 0 || Hq % Hkv != 0) return 1;
    const size_t rep = Hq / Hkv;
    float* buf = (float*)malloc((4 * T * dk + T * T) * sizeof(float));
    if (!buf) return 4;
    float *qh = buf, *kh = buf + T * dk, *vh = buf + 2 * T * dk, *yh = buf + 3 * T * dk;
    float* A = buf + 4 * T * dk;
    int rc = 0;
    for (size_t b = 0; b < B && !rc; ++b)
        for (size_t h = 0; h < Hq && !rc; ++h) {
            gather_head(q, b, h, T, Hq, dk, qh);
            gather_head(k, b, h / rep, T, Hkv, dk, kh);
            gather_head(v, b, h / rep, T, Hkv, dk, vh);
            rc = pko_attn_head_fwd(qh, kh, vh, T, dk, dk, scale, 0, causal, window, sinks, yh,
                                   lse ? lse + (b * Hq + h) * T : NULL, A);
            scatter_head(o, b, h, T, Hq, dk, yh, 0);
        }
    free(buf);
    return rc;
}

int pko_attn_bwd(const float* q, const float* k, const float* v, const float* d_o, size_t B,
                 size_t T, size_t Hq, size_t Hkv, size_t dk, float scale, int causal,
                 size_t window, size_t sinks, float* dq, float* dk_out, float* dv_out) {
    if (Hkv == 0 || Hq % Hkv != 0) return 1;
    const size_t rep = Hq / Hkv;
    float* buf = (float*)malloc((8 * T * dk + T * T) * sizeof(float));
    if (!buf) return 4;
    float *qh = buf, *kh = qh + T * dk, *vh = kh + T * dk, *yh = vh + T * dk, *dyh = yh + T * dk,
          *dqh = dyh + T * dk, *dkh = dqh + T * dk, *dvh = dkh + T * dk;
    float* A = buf + 8 * T * dk;
    memset(dk_out, 0, B * T * Hkv * dk * sizeof(float));
    memset(dv_out, 0, B * T * Hkv * dk * sizeof(float));
    int rc = 0;
    for (size_t b = 0; b < B && !rc; ++b)
        for (size_t h = 0; h < Hq && !rc; ++h) {
            gather_head(q, b, h, T, Hq, dk, qh);
            gather_head(k, b, h / rep, T, Hkv, dk, kh);
            gather_head(v, b, h / rep, T, Hkv, dk, vh);
            gather_head(d_o, b, h, T, Hq, dk, dyh);
            rc = pko_attn_head_fwd(qh, kh, vh, T, dk, dk, scale, 0, causal, window, sinks, yh,
                                   NULL, A);
            if (rc) break;
            rc = pko_attn_head_bwd(qh, kh, vh, A, dyh, T, dk, dk, scale, 0, causal, window,
                                   sinks, dqh, dkh, dvh);
            scatter_head(dq, b, h, T, Hq, dk, dqh, 0);
            /* one K/V Variable parented by `rep` head nodes: grads add up
             * (diamond rule, tests/test_gradcheck.cpp:111-123). */
            scatter_head(dk_out, b, h / rep, T, Hkv, dk, dkh, 1);
            scatter_head(dv_out, b, h / rep, T, Hkv, dk, dvh, 1);
        }
    free(buf);
    return rc;
}

int pko_attention_mask(size_t rows, size_t seq_len, int causal, float* out) {
    if (seq_len == 0) seq_len = rows;
    if (rows == 0 || rows % seq_len != 0) return 2;
    for (size_t i = 0; i < rows; ++i) {
        const size_t blk = i / seq_len;
        for (size_t j = 0; j < rows; ++j) {
            const int vis = (j / seq_len == blk) && (!causal || j <= i);
            out[i * rows + j] = vis ? 0.0f : -1e9f;
        }
    }
    return 0;
}

unsigned long long pko_visible_pairs(size_t T, int causal, size_t window, size_t sinks) {
    unsigned long long n = 0;
    for (size_t i = 0; i < T; ++i) {
        size_t a0, a1, b0, b1;
        visible(i, T, causal, window, sinks, &a0, &a1, &b0, &b1);
        n += (a1 - a0) + (b1 - b0);
    }
    return n;
}

/* ---- Llama block ops ------------------------------------------------------ */

void pko_rmsnorm_fwd(const float* x, const float* w, size_t R, size_t C, float eps, float* y, float* rms_inv) {
    for (size_t i = 0; i < R; ++i) { /* src/ops.cpp:438-444 */
        float rms_sq = 0.0f;
        for (size_t j = 0; j < C; ++j) rms_sq += x[i * C + j] * x[i * C + j];
        rms_sq /= (float)C;
        rms_inv[i] = 1.0f / sqrtf(rms_sq + eps);
        for (size_t j = 0; j < C; ++j) y[i * C + j] = x[i * C + j] * rms_inv[i] * w[j];
    }
}

void pko_rmsnorm_bwd(const float* dy, const float* x, const float* rms_inv, const float* w, size_t R, size_t C,
                     float* dw, float* dx) {
    for (size_t j = 0; j < C; ++j) dw[j] = 0.0f;
    for (size_t i = 0; i < R; ++i) /* src/ops.cpp:457-459 */
        for (size_t j = 0; j < C; ++j) dw[j] += dy[i * C + j] * x[i * C + j] * rms_inv[i];
    for (size_t i = 0; i < R; ++i) { /* src/ops.cpp:466-474 */
        float term = 0.0f;
        for (size_t j = 0; j < C; ++j) term += dy[i * C + j] * w[j] * x[i * C + j];
        const float ri2 = rms_inv[i] * rms_inv[i];
        const float n_inv = 1.0f / (float)C;
        for (size_t j = 0; j < C; ++j)
            dx[i * C + j] = rms_inv[i] * (dy[i * C + j] * w[j] - x[i * C + j] * ri2 * term * n_inv);
    }
}

void pko_silu_fwd(const float* x, size_t n, float* y) {
    for (size_t i = 0; i < n; ++i) y[i] = x[i] / (1.0f + expf(-x[i])); /* src/ops.cpp:408-409 */
}

void pko_silu_bwd(const float* x, const float* dy, size_t n, float* dx) {
    for (size_t i = 0; i < n; ++i) { /* src/ops.cpp:418-420 */
        const float s = 1.0f / (1.0f + expf(-x[i]));
        dx[i] = dy[i] * (s * (1.0f + x[i] * (1.0f - s)));
    }
}

int pko_rope(const float* x, const int* pos, size_t T, size_t d3, float theta_base, size_t head_dim, int inverse,
             float* y) {
    if (d3 % 3 != 0) return -1;                  /* src/ops.cpp:483-485 */
    const size_t d = d3 / 3;
    if (head_dim % 2 != 0 || head_dim > d) return -1; /* src/ops.cpp:487-489 */
    memcpy(y, x, T * d3 * sizeof(float));
    for (size_t i = 0; i < T; ++i) {
        const float m = (float)pos[i];
        for (size_t start = 0; start < 2 * d; start += d)     /* q third, k third; v untouched */
            for (size_t dim = 0; dim < head_dim; dim += 2) {  /* only the first head's columns, as written */
                const float inv_freq = 1.0f / powf(theta_base, (float)dim / (float)head_dim);
                const float th = inverse ? -m * inv_freq : m * inv_freq;
                const float c = cosf(th), s = sinf(th);
                const float x0 = y[i * d3 + start + dim], x1 = y[i * d3 + start + dim + 1];
                y[i * d3 + start + dim] = x0 * c - x1 * s;
                y[i * d3 + start + dim + 1] = x0 * s + x1 * c;
            }
    }
    return 0;
}

int pko_embedding_fwd(const float* table, size_t V, size_t d, const int* ids, size_t n, float* y) {
    for (size_t i = 0; i < n; ++i) {
        if (ids[i] < 0 || (size_t)ids[i] >= V) return -1; /* src/ops.cpp:333-335 */
        memcpy(y + i * d, table + (size_t)ids[i] * d, d * sizeof(float));
    }
    return 0;
}

int pko_embedding_bwd(const float* dy, const int* ids, size_t n, size_t V, size_t d, float* dtable) {
    memset(dtable, 0, V * d * sizeof(float));
    for (size_t i = 0; i < n; ++i) { /* src/ops.cpp:345-346, in id order */
        if (ids[i] < 0 || (size_t)ids[i] >= V) return -1;
        for (size_t j = 0; j < d; ++j) dtable[(size_t)ids[i] * d + j] += dy[i * d + j];
    }
    return 0;
}

int pko_cross_entropy(const float* logits, const int* targets, size_t R, size_t C, float* loss, float* dlogits) {
    float* P = (float*)malloc(R * C * sizeof(float));
    if (!P) return -2;
    double nll = 0.0;
    for (size_t i = 0; i < R; ++i) { /* components.cpp:232-250 */
        float mx = -INFINITY;
        for (size_t j = 0; j < C; ++j) mx = fmaxf(mx, logits[i * C + j]);
        float sum = 0.0f;
        for (size_t j = 0; j < C; ++j) {
            const float e = expf(logits[i * C + j] - mx);
            P[i * C + j] = e;
            sum += e;
        }
        for (size_t j = 0; j < C; ++j) P[i * C + j] /= sum;
        if (targets[i] < 0 || (size_t)targets[i] >= C) { /* src/ops.cpp:363-365 */
            free(P);
            return -1;
        }
        nll -= log((double)fmaxf(P[i * C + targets[i]], 1e-12f)); /* std::log(float) summed into a double */
    }
    *loss = (float)(nll / (double)R);
    if (dlogits) { /* src/ops.cpp:371-374 with upstream grad 1 */
        const float g = 1.0f / (float)R;
        for (size_t i = 0; i < R; ++i)
            for (size_t j = 0; j < C; ++j)
                dlogits[i * C + j] = (P[i * C + j] - ((size_t)targets[i] == j ? 1.0f : 0.0f)) * g;
    }
    free(P);
    return 0;
}

void pko_adamw(float* p, const float* g, float* m, float* v, size_t n, float lr, float b1, float b2, float eps,
               float wd, int t) {
    const float c1 = 1.0f - powf(b1, (float)t); /* src/nn.cpp:305-306 */
    const float c2 = 1.0f - powf(b2, (float)t);
    for (size_t i = 0; i < n; ++i) { /* src/nn.cpp:312-318 */
        m[i] = b1 * m[i] + (1.0f - b1) * g[i];
        v[i] = b2 * v[i] + (1.0f - b2) * g[i] * g[i];
        const float update = (m[i] / c1) / (sqrtf(v[i] / c2) + eps);
        p[i] -= lr * (update + wd * p[i]);
    }
}

float pko_clip_grad_norm(float* const* grads, const size_t* sizes, size_t nparams, float max_norm) {
    double sq = 0.0; /* src/ops.cpp:1047-1053 */
    for (size_t k = 0; k < nparams; ++k)
        for (size_t i = 0; i < sizes[k]; ++i) sq += (double)grads[k][i] * grads[k][i];
    const float total = (float)sqrt(sq);
    if (total > max_norm && total > 0.0f) { /* src/ops.cpp:1055-1062 */
        const float scale = max_norm / total;
        for (size_t k = 0; k < nparams; ++k)
            for (size_t i = 0; i < sizes[k]; ++i) grads[k][i] *= scale;
    }
    return total;
}
