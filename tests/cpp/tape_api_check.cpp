// The C++ tape interface of libpaperkiln_amd.so (include/paperkiln_amd.hpp) used the way the reference's own
// tests use its tape (paperkiln tests/test_gradcheck.cpp:196-238, tests/test_checkpointing.cpp:46-90,
// tests/test_swa.cpp:47-57): build Variables, call ops::fused_attention / ops::swa_attention / checkpoint,
// run backward, read gradients. Compiled with plain g++ against the public header only -- no HIP header, no
// internal header -- and linked against the shared library. Expected values come from a float64 evaluation
// of the textbook formulas written out below (tiny sizes), not from the library.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "paperkiln_amd.hpp"

namespace {

int g_failures = 0;
void check(bool ok, const char* label, double measured) {
    std::printf("  [%s] %-62s %.3e\n", ok ? "ok" : "FAIL", label, measured);
    if (!ok) ++g_failures;
}

// splitmix64 -> uniform in (-1, 1)
struct Rng {
    uint64_t s;
    double next() {
        s += 0x9E3779B97F4A7C15ull;
        uint64_t z = s;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        return (static_cast<double>(z >> 11) + 0.5) / 9007199254740992.0 * 2.0 - 1.0;
    }
};
std::vector<float> draw(size_t n, uint64_t seed, double amp) {
    Rng r{seed};
    std::vector<float> v(n);
    for (auto& x : v) x = static_cast<float>(r.next() * amp);
    return v;
}
double max_abs_diff(const std::vector<float>& a, const std::vector<double>& b) {
    double w = 0.0;
    for (size_t i = 0; i < a.size(); ++i) w = std::fmax(w, std::fabs(static_cast<double>(a[i]) - b[i]));
    return w;
}
std::vector<float> host(const pk::Tensor& t) {
    std::vector<float> h(static_cast<size_t>(t.rows * t.cols));
    pk::download(t, h.data());
    return h;
}

// Softmax attention of one head, rows = B stacked sequences of seq_len, and the mean cross-entropy of its
// output rows against `target` columns, with every gradient, in float64.
struct Exact {
    std::vector<double> y, dq, dk, dv;
    double loss;
};
bool visible(int i, int j, int sl, bool causal, int window, int sinks) {
    const int b0 = i / sl * sl;
    if (j < b0 || j >= b0 + sl) return false;
    if (causal && j > i) return false;
    if (window > 0 && j + window <= i && j - b0 >= sinks) return false;
    return true;
}
Exact exact(const std::vector<float>& q, const std::vector<float>& k, const std::vector<float>& v,
            const std::vector<int>& target, int T, int dk, double scale, int sl, bool causal, int window, int sinks) {
    Exact e;
    if (sl == 0) sl = T;  // seq_len 0 = one sequence (src/ops.cpp:869)
    std::vector<double> P(static_cast<size_t>(T) * T, 0.0);
    e.y.assign(static_cast<size_t>(T) * dk, 0.0);
    for (int i = 0; i < T; ++i) {
        double mx = -1e300, z = 0.0;
        std::vector<double> s(T, 0.0);
        for (int j = 0; j < T; ++j) {
            if (!visible(i, j, sl, causal, window, sinks)) continue;
            for (int d = 0; d < dk; ++d) s[j] += static_cast<double>(q[i * dk + d]) * k[j * dk + d];
            s[j] *= scale;
            mx = std::fmax(mx, s[j]);
        }
        for (int j = 0; j < T; ++j)
            if (visible(i, j, sl, causal, window, sinks)) z += (P[i * T + j] = std::exp(s[j] - mx));
        for (int j = 0; j < T; ++j) {
            P[i * T + j] /= z;
            for (int d = 0; d < dk; ++d) e.y[i * dk + d] += P[i * T + j] * v[j * dk + d];
        }
    }
    // loss = mean_i -log softmax(y_i)[target_i];  dy = (softmax(y) - onehot) / T
    std::vector<double> dy(static_cast<size_t>(T) * dk);
    e.loss = 0.0;
    for (int i = 0; i < T; ++i) {
        double mx = -1e300, z = 0.0;
        for (int d = 0; d < dk; ++d) mx = std::fmax(mx, e.y[i * dk + d]);
        for (int d = 0; d < dk; ++d) z += std::exp(e.y[i * dk + d] - mx);
        for (int d = 0; d < dk; ++d) dy[i * dk + d] = std::exp(e.y[i * dk + d] - mx) / z / T;
        e.loss -= std::log(dy[i * dk + target[i]] * T) / T;
        dy[i * dk + target[i]] -= 1.0 / T;
    }
    e.dq.assign(static_cast<size_t>(T) * dk, 0.0);
    e.dk.assign(static_cast<size_t>(T) * dk, 0.0);
    e.dv.assign(static_cast<size_t>(T) * dk, 0.0);
    for (int i = 0; i < T; ++i) {
        std::vector<double> dp(T, 0.0);
        double dot = 0.0;
        for (int j = 0; j < T; ++j) {
            for (int d = 0; d < dk; ++d) dp[j] += dy[i * dk + d] * v[j * dk + d];
            dot += dp[j] * P[i * T + j];
        }
        for (int j = 0; j < T; ++j) {
            const double ds = scale * P[i * T + j] * (dp[j] - dot);
            for (int d = 0; d < dk; ++d) {
                e.dq[i * dk + d] += ds * k[j * dk + d];
                e.dk[j * dk + d] += ds * q[i * dk + d];
                e.dv[j * dk + d] += P[i * T + j] * dy[i * dk + d];
            }
        }
    }
    return e;
}

std::shared_ptr<pk::Buffer> device_ints(const std::vector<int>& h) {
    // integer targets travel as the bit patterns of a float32 row (upload converts nothing in fp32)
    static_assert(sizeof(int) == sizeof(float), "int and float are both 4 bytes");
    pk::Tensor t = pk::upload(reinterpret_cast<const float*>(h.data()), 1, static_cast<int64_t>(h.size()), PK_F32);
    return t.buf;
}

void attention_case(const char* name, int T, int dk, int sl, bool causal, int window, int sinks) {
    const double scale = 1.0 / std::sqrt(static_cast<double>(dk));
    const auto hq = draw(static_cast<size_t>(T) * dk, 11, 1.5), hk = draw(static_cast<size_t>(T) * dk, 12, 1.5),
               hv = draw(static_cast<size_t>(T) * dk, 13, 1.5);
    std::vector<int> target(T);
    for (int i = 0; i < T; ++i) target[i] = (7 * i + 3) % dk;
    const Exact want = exact(hq, hk, hv, target, T, dk, scale, sl, causal, window, sinks);

    pk::Var q = pk::make_var(pk::upload(hq.data(), T, dk), true);
    pk::Var k = pk::make_var(pk::upload(hk.data(), T, dk), true);
    pk::Var v = pk::make_var(pk::upload(hv.data(), T, dk), true);
    pk::Var y = window > 0 ? pk::ops::swa_attention(q, k, v, static_cast<float>(scale), window, sinks, sl)
                           : pk::ops::fused_attention(q, k, v, static_cast<float>(scale), sl, causal);
    pk::Var loss = pk::ops::cross_entropy(y, device_ints(target));
    pk::backward(loss);
    std::printf("%s (T=%d dk=%d seq_len=%d causal=%d window=%d sinks=%d)\n", name, T, dk, sl, causal, window, sinks);
    check(max_abs_diff(host(y->data), want.y) < 1e-5, "forward y vs float64", max_abs_diff(host(y->data), want.y));
    check(std::fabs(host(loss->data)[0] - want.loss) < 1e-5, "loss vs float64", std::fabs(host(loss->data)[0] - want.loss));
    check(max_abs_diff(host(q->grad), want.dq) < 1e-5, "dQ vs float64", max_abs_diff(host(q->grad), want.dq));
    check(max_abs_diff(host(k->grad), want.dk) < 1e-5, "dK vs float64", max_abs_diff(host(k->grad), want.dk));
    check(max_abs_diff(host(v->grad), want.dv) < 1e-5, "dV vs float64", max_abs_diff(host(v->grad), want.dv));
}

void checkpoint_case() {
    std::printf("checkpoint(fn, x) against the plain tape\n");
    const int T = 24, d = 16;
    const auto hx = draw(static_cast<size_t>(T) * d, 21, 1.0), hw = draw(static_cast<size_t>(d) * d, 22, 0.3),
               hg = draw(d, 23, 1.0);
    std::vector<int> target(T);
    for (int i = 0; i < T; ++i) target[i] = (5 * i + 1) % d;
    auto tg = device_ints(target);
    struct Run {
        float loss;
        std::vector<float> gx, gw, gg;
        size_t live;
    };
    auto run = [&](bool ckpt) {
        const size_t live0 = pk::live_variables();
        pk::Var x = pk::make_var(pk::upload(hx.data(), T, d), true);
        pk::Var w = pk::make_var(pk::upload(hw.data(), d, d), true);
        pk::Var gain = pk::make_var(pk::upload(hg.data(), 1, d), true);
        w->is_param = gain->is_param = true;
        auto block = [w, gain](const pk::Var& in) {
            pk::Var h = pk::ops::rmsnorm(in, gain);
            pk::Var p = pk::ops::linear(h, w);
            pk::Var a = pk::ops::fused_attention(p, p, h, 0.25f, 12, true);
            return pk::ops::add(in, pk::ops::silu(a));
        };
        pk::Var h = x;
        for (int i = 0; i < 3; ++i) h = ckpt ? pk::checkpoint(block, h) : block(h);
        pk::Var loss = pk::ops::cross_entropy(h, tg);
        h.reset();
        Run r;
        r.live = pk::live_variables() - live0;
        pk::backward(loss);
        r.loss = host(loss->data)[0];
        r.gx = host(x->grad);
        r.gw = host(w->grad);
        r.gg = host(gain->grad);
        return r;
    };
    const Run plain = run(false), ck = run(true);
    auto diff = [](const std::vector<float>& a, const std::vector<float>& b) {
        double w = 0.0;
        for (size_t i = 0; i < a.size(); ++i) w = std::fmax(w, std::fabs(static_cast<double>(a[i]) - b[i]));
        return w;
    };
    check(plain.loss == ck.loss, "loss equal", std::fabs(plain.loss - ck.loss));
    check(diff(plain.gx, ck.gx) < 1e-6, "input gradient", diff(plain.gx, ck.gx));
    check(diff(plain.gw, ck.gw) < 1e-6, "weight gradient (parameter inside the segment)", diff(plain.gw, ck.gw));
    check(diff(plain.gg, ck.gg) < 1e-6, "gain gradient", diff(plain.gg, ck.gg));
    check(ck.live * 2 < plain.live, "live variables after forward more than halved", static_cast<double>(ck.live));
    std::printf("  live variables after forward: plain %zu, checkpointed %zu\n", plain.live, ck.live);
}

// Gradients that reach a Variable along two paths. Both parents of an add take the node's gradient tensor itself
// (shared, read-only), so writing one parent's gradient afterwards -- a later accumulation, zero_grad -- must not
// show in the other's; and rmsnorm's backward adds the gradient its input already has inside the kernel.
void shared_gradient_case(int dtype, const char* name, double tol) {
    std::printf("gradients along two paths, %s\n", name);
    const int T = 48, d = 64;
    const auto hx = draw(static_cast<size_t>(T) * d, 41, 1.0), hu = draw(static_cast<size_t>(T) * d, 42, 1.0),
               hg = draw(d, 43, 1.0);
    std::vector<int> target(T);
    for (int i = 0; i < T; ++i) target[i] = (7 * i + 3) % d;
    auto tg = device_ints(target);
    auto diff = [](const std::vector<float>& a, const std::vector<float>& b, double fb) {
        double w = 0.0;
        for (size_t i = 0; i < a.size(); ++i) w = std::fmax(w, std::fabs(static_cast<double>(a[i]) - fb * b[i]));
        return w;
    };
    {
        pk::Var x = pk::make_var(pk::upload(hx.data(), T, d, dtype), true);
        pk::Var u = pk::make_var(pk::upload(hu.data(), T, d, dtype), true);
        auto pass = [&] { pk::backward(pk::ops::cross_entropy(pk::ops::add(x, u), tg)); };
        pass();
        const auto g1 = host(x->grad);
        double size = 0.0;
        for (float v : g1) size = std::fmax(size, std::fabs(v));
        check(size > 1e-4, "add: the gradient is not zero", size);
        check(host(u->grad) == g1, "add: both parents hold the node's gradient", 0.0);
        pass();  // accumulates onto gradients that share storage
        check(diff(host(x->grad), g1, 2.0) <= tol * size, "second backward doubles the first parent's", diff(host(x->grad), g1, 2.0));
        check(diff(host(u->grad), g1, 2.0) <= tol * size, "... and the second parent's, once each", diff(host(u->grad), g1, 2.0));
        pk::Var x2 = pk::make_var(pk::upload(hx.data(), T, d, dtype), true);
        pk::Var u2 = pk::make_var(pk::upload(hu.data(), T, d, dtype), true);
        pk::backward(pk::ops::cross_entropy(pk::ops::add(x2, u2), tg));
        pk::zero_grad({x2});
        check(diff(host(x2->grad), g1, 0.0) == 0.0, "zero_grad of one parent zeroes it", 0.0);
        check(host(u2->grad) == g1, "... and leaves the other parent's gradient alone", 0.0);
    }
    {
        // z = x + rmsnorm(x): one Variable on both paths against two leaves with the same values, one per path
        pk::Var gain = pk::make_var(pk::upload(hg.data(), 1, d), true);
        gain->is_param = true;
        pk::Var x = pk::make_var(pk::upload(hx.data(), T, d, dtype), true);
        pk::backward(pk::ops::cross_entropy(pk::ops::add(x, pk::ops::rmsnorm(x, gain)), tg));
        const auto both = host(x->grad), gg = host(gain->grad);
        pk::zero_grad({gain});
        pk::Var xa = pk::make_var(pk::upload(hx.data(), T, d, dtype), true);
        pk::Var xb = pk::make_var(pk::upload(hx.data(), T, d, dtype), true);
        pk::backward(pk::ops::cross_entropy(pk::ops::add(xa, pk::ops::rmsnorm(xb, gain)), tg));
        const auto ga = host(xa->grad), gb = host(xb->grad);
        double w = 0.0, size = 0.0;
        for (size_t i = 0; i < both.size(); ++i) {
            w = std::fmax(w, std::fabs(static_cast<double>(both[i]) - (static_cast<double>(ga[i]) + gb[i])));
            size = std::fmax(size, std::fabs(static_cast<double>(ga[i]) + gb[i]));
        }
        check(w <= tol * size, "x + rmsnorm(x): gradient = residual path + norm path", w);
        check(diff(host(gain->grad), gg, 1.0) <= 1e-6, "gain gradient the same either way", diff(host(gain->grad), gg, 1.0));
    }
}

// r + x W with the add inside the product's epilogue (bf16) against the two ops it stands for; edge tiles in both
// directions, and a contraction long enough for the two-wavefront-set form of the kernel.
void linear_add_case(int dtype, const char* name, int T, int din, int dout, double tol) {
    std::printf("linear_add, %s, [%d, %d] x [%d, %d]\n", name, T, din, din, dout);
    const auto hx = draw(static_cast<size_t>(T) * din, 51, 1.0), hw = draw(static_cast<size_t>(din) * dout, 52, 0.2),
               hr = draw(static_cast<size_t>(T) * dout, 53, 2.0);
    std::vector<int> target(T);
    for (int i = 0; i < T; ++i) target[i] = (3 * i + 1) % dout;
    auto tg = device_ints(target);
    pk::set_compute_dtype(dtype);  // the weight's compute-dtype copy follows it
    struct Run {
        std::vector<float> y, gx, gw, gr;
    };
    auto run = [&](bool fused) {
        pk::Var x = pk::make_var(pk::upload(hx.data(), T, din, dtype), true);
        pk::Var r = pk::make_var(pk::upload(hr.data(), T, dout, dtype), true);
        pk::Var w = pk::make_var(pk::upload(hw.data(), din, dout), true);
        w->is_param = true;
        pk::Var y = fused ? pk::ops::linear_add(x, w, r) : pk::ops::add(r, pk::ops::linear(x, w));
        Run out;
        out.y = host(y->data);
        pk::backward(pk::ops::cross_entropy(y, tg));
        out.gx = host(x->grad);
        out.gw = host(w->grad);
        out.gr = host(r->grad);
        pk::invalidate_shadows();
        return out;
    };
    const Run two = run(false), one = run(true);
    auto rel = [](const std::vector<float>& a, const std::vector<float>& b) {
        double w = 0.0, size = 0.0;
        for (size_t i = 0; i < a.size(); ++i) {
            w = std::fmax(w, std::fabs(static_cast<double>(a[i]) - b[i]));
            size = std::fmax(size, std::fabs(static_cast<double>(b[i])));
        }
        return w / std::fmax(size, 1e-30);
    };
    check(rel(one.y, two.y) <= tol, "r + x W vs add(r, linear(x, W))", rel(one.y, two.y));
    check(rel(one.gx, two.gx) <= 4 * tol, "dX", rel(one.gx, two.gx));
    check(rel(one.gw, two.gw) <= 4 * tol, "dW", rel(one.gw, two.gw));
    check(rel(one.gr, two.gr) <= 4 * tol, "dr", rel(one.gr, two.gr));
    pk::set_compute_dtype(PK_F32);
}

// The chunked tied head with the cross-entropy inside the logits product against the same head through fp32 logits
// and the row kernel, on logits of a few tens in size (far from the ~0.01 of a freshly initialised model): the
// in-product path carries the row maximum and the scaling in the exponent of exp2, which is where a large logit
// would show.
void head_case() {
    std::printf("linear_cross_entropy, logits of size ~50: inside the product vs fp32 logits + row kernel\n");
    const int T = 300, d = 64, V = 1000;
    const auto hh = draw(static_cast<size_t>(T) * d, 61, 3.0), he = draw(static_cast<size_t>(V) * d, 62, 3.0);
    std::vector<int> target(T);
    for (int i = 0; i < T; ++i) target[i] = (37 * i + 11) % V;
    auto tg = device_ints(target);
    pk::set_compute_dtype(PK_BF16);
    struct Run {
        float loss;
        std::vector<float> gh, ge;
    };
    auto run = [&](int in_product) {
        const int before = pk_set_head_kernel(in_product);
        pk::Var h = pk::make_var(pk::upload(hh.data(), T, d, PK_BF16), true);
        pk::Var E = pk::make_var(pk::upload(he.data(), V, d), true);
        E->is_param = true;
        pk::Var loss = pk::ops::linear_cross_entropy(h, E, tg, 128);  // 3 chunks, the last of 44 rows
        pk::backward(loss);
        Run r{host(loss->data)[0], host(h->grad), host(E->grad)};
        pk::invalidate_shadows();
        pk_set_head_kernel(before);
        return r;
    };
    const Run rows = run(0), prod = run(1);
    auto rel = [](const std::vector<float>& a, const std::vector<float>& b) {
        double w = 0.0, size = 0.0;
        for (size_t i = 0; i < a.size(); ++i) {
            w = std::fmax(w, std::fabs(static_cast<double>(a[i]) - b[i]));
            size = std::fmax(size, std::fabs(static_cast<double>(b[i])));
        }
        return w / std::fmax(size, 1e-30);
    };
    check(std::isfinite(prod.loss) && prod.loss > 10.0f, "loss is finite and large (the logits are)", prod.loss);
    check(std::fabs(prod.loss - rows.loss) <= 2e-5 * rows.loss, "loss", std::fabs(prod.loss - rows.loss));
    check(rel(prod.gh, rows.gh) <= 1.0 / 64, "dh", rel(prod.gh, rows.gh));
    check(rel(prod.ge, rows.ge) <= 1.0 / 64, "dE", rel(prod.ge, rows.ge));
    pk::set_compute_dtype(PK_F32);
}

// Weight gradients of several Linears over 2056 tokens: in the default setting the backward pass holds the X^T dY
// products back and multiplies them as one grouped launch; pk_set_gemm_backend(2) multiplies them one by one. Output
// widths that are not multiples of the 128-wide tile, two different inputs (row pitches 512 and 136, the second
// with a ragged last row tile), one pair sharing a concatenated product, one weight used by two Linears (whose two
// products must not run in one launch: they add into the same gradient).
void grouped_weight_gradient_case() {
    std::printf("weight gradients held back and multiplied as one grouped launch vs one by one\n");
    const int T = 2056, d = 512;  // not a multiple of the kernel's 64-deep slices: the last slice is 8 tokens
    const int widths[6] = {1376, 520, 520, 136, 512, 512};  // Wa, {Wb | Wc}, W0 (feeds Wf), We, Wf [136, 512]
    const auto hx = draw(static_cast<size_t>(T) * d, 71, 1.0);
    std::vector<std::vector<float>> hw;
    for (int k = 0; k < 5; ++k) hw.push_back(draw(static_cast<size_t>(d) * widths[k], 72 + k, 0.05));
    hw.push_back(draw(static_cast<size_t>(136) * 512, 78, 0.05));
    std::vector<int> target(T);
    for (int i = 0; i < T; ++i) target[i] = (5 * i + 2) % 136;
    auto tg = device_ints(target);
    pk::set_compute_dtype(PK_BF16);
    auto run = [&](int backend) {
        const int before = pk_set_gemm_backend(backend);
        pk::Var x = pk::make_var(pk::upload(hx.data(), T, d, PK_BF16), true);
        std::vector<pk::Var> W;
        for (int k = 0; k < 5; ++k) W.push_back(pk::make_var(pk::upload(hw[k].data(), d, widths[k]), true));
        W.push_back(pk::make_var(pk::upload(hw[5].data(), 136, 512), true));
        for (auto& w : W) w->is_param = true;
        pk::Var ya = pk::ops::linear(x, W[0]);
        pk::Var ybc = pk::ops::linear_cat(x, {W[1], W[2]});
        pk::Var y0 = pk::ops::linear(x, W[3]);
        pk::Var ye = pk::ops::linear(pk::ops::linear(x, W[4]), W[4]);  // one weight used twice
        pk::Var yf = pk::ops::linear_add(y0, W[5], ye);
        pk::Var loss = pk::ops::add(pk::ops::add(pk::ops::cross_entropy(ya, tg), pk::ops::cross_entropy(ybc, tg)),
                                    pk::ops::cross_entropy(yf, tg));
        pk::backward(loss);
        std::vector<std::vector<float>> g;
        for (auto& w : W) g.push_back(host(w->grad));
        pk::invalidate_shadows();
        pk_set_gemm_backend(before);
        return g;
    };
    const auto one = run(2), grouped = run(1);
    const char* names[6] = {"dW [512, 1376]", "dW [512, 520] (first of a pair)", "dW [512, 520] (second of a pair)", "dW [512, 136]",
                            "dW [512, 512]", "dW [136, 512]"};
    for (int k = 0; k < 6; ++k) {
        double w = 0.0, size = 0.0;
        for (size_t i = 0; i < one[k].size(); ++i) {
            w = std::fmax(w, std::fabs(static_cast<double>(one[k][i]) - grouped[k][i]));
            size = std::fmax(size, std::fabs(static_cast<double>(one[k][i])));
        }
        check(size > 0.0 && w <= 1e-4 * size, names[k], w / std::fmax(size, 1e-30));
    }
    pk::set_compute_dtype(PK_F32);
}

void behaviour_case() {
    std::printf("tape behaviour and errors\n");
    const auto h = draw(8 * 4, 31, 1.0);
    pk::Var q = pk::make_var(pk::upload(h.data(), 8, 4), true);
    const size_t live0 = pk::live_variables();
    {
        pk::NoGrad off;
        pk::Var y = pk::ops::fused_attention(q, q, q, 0.5f, 0, true);
        check(!y->requires_grad && y->is_leaf(), "NoGrad: nothing recorded", 0.0);
    }
    check(pk::live_variables() == live0, "live_variables back to the baseline", static_cast<double>(pk::live_variables() - live0));
    auto throws = [](const char* label, int want_code, const std::function<void()>& f) {
        int code = -1;
        std::string what;
        try {
            f();
        } catch (const pk::Error& e) {
            code = e.code;
            what = e.what();
        } catch (const std::exception& e) {
            code = -2;
            what = e.what();
        }
        check(code == want_code, label, static_cast<double>(code));
        if (code != want_code) std::printf("      got: %s\n", what.c_str());
    };
    pk::Var short_k = pk::make_var(pk::upload(h.data(), 4, 4), true);
    throws("fused_attention: shape mismatch -> PK_ERR_SHAPE", PK_ERR_SHAPE,
           [&] { pk::ops::fused_attention(q, short_k, q, 0.5f, 0, true); });
    throws("fused_attention: rows not a multiple of seq_len -> PK_ERR_SHAPE", PK_ERR_SHAPE,
           [&] { pk::ops::fused_attention(q, q, q, 0.5f, 3, true); });
    throws("swa_attention: window 0 throws", -2, [&] { pk::ops::swa_attention(q, q, q, 0.5f, 0, 0, 0); });
    throws("backward: root must be a scalar", -2, [&] { pk::backward(pk::ops::fused_attention(q, q, q, 0.5f, 0, true)); });
    // window >= seq_len, no sinks == causal, bit for bit (tests/test_swa.cpp:47-57)
    pk::Var a = pk::ops::fused_attention(q, q, q, 0.5f, 0, true), b = pk::ops::swa_attention(q, q, q, 0.5f, 8, 0, 0);
    check(host(a->data) == host(b->data), "swa(window >= T, sinks = 0) == causal, bitwise", 0.0);
}

}  // namespace

int main() {
    std::setvbuf(stdout, nullptr, _IOLBF, 0);
    char arch[64] = {0};
    if (pk_init(0, arch, sizeof arch) != PK_OK) {
        std::printf("tape_api_check: %s\n", pk_last_error());
        return 2;
    }
    std::printf("device: %s\n", arch);
    attention_case("fused_attention, one sequence", 13, 8, 0, true, 0, 0);
    attention_case("fused_attention, two stacked sequences, bidirectional", 16, 8, 8, false, 0, 0);
    attention_case("fused_attention, head_dim 32 (fp32 matrix-core kernels)", 40, 32, 20, true, 0, 0);
    attention_case("swa_attention, window 3 + 2 sinks", 18, 8, 9, true, 3, 2);
    checkpoint_case();
    shared_gradient_case(PK_F32, "float32", 1e-6);
    shared_gradient_case(PK_BF16, "bfloat16 (the fused row kernel)", 1.0 / 128);
    linear_add_case(PK_F32, "float32 (product, then add)", 40, 24, 16, 1e-6);
    linear_add_case(PK_BF16, "bfloat16, edge tiles", 200, 72, 136, 1.0 / 128);
    linear_add_case(PK_BF16, "bfloat16, long contraction", 300, 1376, 64, 1.0 / 128);
    head_case();
    grouped_weight_gradient_case();
    behaviour_case();
    if (g_failures == 0) {
        std::printf("tape_api_check PASSED\n");
        return 0;
    }
    std::printf("tape_api_check: %d FAILURE(S)\n", g_failures);
    return 1;
}
