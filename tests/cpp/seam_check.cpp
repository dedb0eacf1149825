// paperkiln's own tape (compiled from the reference's sources, untouched) running over the HIP device seam of
// paperkiln_amd/adapter/microtorch_hip_seam.cpp instead of src/device.cpp + src/device_cache.cpp. Each leg runs
// the same computation twice on identical inputs -- device CPU (the reference's host loops and AVX2 GEMM), then
// device GPU through libpaperkiln_amd.so -- and compares, as tests/test_cuda_ops.cpp:263-300 and
// tests/test_step_residency.cpp:142-172 of the reference do for its CUDA seam:
//   1. the op-set entries (add, sub, mul, scale, axpy, fill, rmsnorm, silu) against the host formulas;
//   2. device::gemm with all four transpose combinations, and the explicit residency table
//      (make_resident / invalidate / evict_all / resident_count) with the reference's mutate -> invalidate ->
//      resident-again leg;
//   3. ops::fused_attention / ops::swa_attention (host loops, [T,T] weights kept) against the O + logsumexp
//      nodes fused_attention_hip / swa_attention_hip: output and dQ, dK, dV within 1e-5;
//   4. a whole nn::Llama forward + cross-entropy + backward, plain and with checkpointed blocks, with the
//      GEMMs and RMSNorm on the GPU (and operands cached inside a step window) against the all-host run.
// Built by oracle/Makefile (target seam) into oracle/_ref/, only where the reference tree is present.
#include <cmath>
#include <cstdio>
#include <random>
#include <vector>

#include "microtorch/device.hpp"
#include "microtorch/device_cache.hpp"
#include "microtorch/llama.hpp"
#include "microtorch/ops.hpp"
#include "microtorch_hip_seam.hpp"

namespace mt = microtorch;
namespace device = microtorch::device;
namespace devops = microtorch::device::devops;
using mt::Var;

namespace {

int g_failures = 0;
void check(bool ok, const char* label, double measured) {
    std::printf("  [%s] %-58s %.3e\n", ok ? "ok" : "FAIL", label, measured);
    if (!ok) ++g_failures;
}
Matrix filled(size_t r, size_t c, unsigned seed, float amp = 1.5f) {
    Matrix m(r, c);
    std::mt19937 rng(seed);
    std::uniform_real_distribution<float> u(-amp, amp);
    for (size_t i = 0; i < r * c; ++i) m.get_data()[i] = u(rng);
    return m;
}
double max_abs_diff(const Matrix& x, const Matrix& y) {
    double worst = x.rows() == y.rows() && x.cols() == y.cols() ? 0.0 : 1e30;
    for (size_t i = 0; i < x.rows() * x.cols() && worst < 1e30; ++i)
        worst = std::fmax(worst, std::fabs(static_cast<double>(x.get_data()[i]) - y.get_data()[i]));
    return worst;
}
struct OnGpu {  // GPU device + op set for one scope
    OnGpu() {
        device::set(device::Device::CUDA);
        device::set_device_ops(true);
    }
    ~OnGpu() {
        device::set_device_ops(false);
        device::set(device::Device::CPU);
    }
};

void leg_op_set() {
    std::printf("-- op set against the host formulas --\n");
    const size_t R = 67, C = 133;
    const Matrix a = filled(R, C, 1), b = filled(R, C, 2), w = filled(1, C, 3);
    OnGpu gpu;
    Matrix dev(R, C), host(R, C);
    auto each = [&](auto f) {
        for (size_t i = 0; i < R * C; ++i) host.get_data()[i] = f(a.get_data()[i], b.get_data()[i]);
    };
    check(devops::add(a, b, dev), "add handled", 0.0);
    each([](float x, float y) { return x + y; });
    check(max_abs_diff(dev, host) <= 1e-6, "add", max_abs_diff(dev, host));
    check(devops::sub(a, b, dev), "sub handled", 0.0);
    each([](float x, float y) { return x - y; });
    check(max_abs_diff(dev, host) <= 1e-6, "sub", max_abs_diff(dev, host));
    check(devops::mul(a, b, dev), "mul handled", 0.0);
    each([](float x, float y) { return x * y; });
    check(max_abs_diff(dev, host) <= 1e-6, "mul", max_abs_diff(dev, host));
    check(devops::scale(a, 0.37f, dev), "scale handled", 0.0);
    each([](float x, float) { return x * 0.37f; });
    check(max_abs_diff(dev, host) <= 1e-6, "scale", max_abs_diff(dev, host));
    Matrix yd = filled(R, C, 4), yh = yd;
    check(devops::axpy(yd, 0.61f, a), "axpy handled", 0.0);
    for (size_t i = 0; i < R * C; ++i) yh.get_data()[i] += 0.61f * a.get_data()[i];
    check(max_abs_diff(yd, yh) <= 1e-6, "axpy", max_abs_diff(yd, yh));
    check(devops::fill(dev, -2.5f), "fill handled", 0.0);
    each([](float, float) { return -2.5f; });
    check(max_abs_diff(dev, host) <= 0.0, "fill", max_abs_diff(dev, host));
    check(!devops::gelu_fwd(a, dev) && !devops::softmax_fwd(a, dev), "gelu / softmax: not handled (host loop runs)", 0.0);

    // silu and its derivative (src/ops.cpp:404-424)
    check(devops::silu_fwd(a, dev), "silu_fwd handled", 0.0);
    each([](float x, float) { return x / (1.0f + std::exp(-x)); });
    check(max_abs_diff(dev, host) <= 1e-6, "silu_fwd", max_abs_diff(dev, host));
    check(devops::silu_bwd(a, b, dev), "silu_bwd handled", 0.0);
    each([](float x, float g) {
        const float s = 1.0f / (1.0f + std::exp(-x));
        return g * s * (1.0f + x * (1.0f - s));
    });
    check(max_abs_diff(dev, host) <= 1e-5, "silu_bwd", max_abs_diff(dev, host));

    // rmsnorm (src/ops.cpp:426-479)
    const float eps = 1e-5f;
    Matrix yc(R, C);
    std::vector<float> rid, ric(R);
    check(devops::rmsnorm_fwd(a, w, eps, dev, rid), "rmsnorm_fwd handled", 0.0);
    for (size_t i = 0; i < R; ++i) {
        float ss = 0.0f;
        for (size_t j = 0; j < C; ++j) ss += a(i, j) * a(i, j);
        ric[i] = 1.0f / std::sqrt(ss / static_cast<float>(C) + eps);
        for (size_t j = 0; j < C; ++j) yc(i, j) = a(i, j) * ric[i] * w(0, j);
    }
    check(max_abs_diff(dev, yc) <= 1e-5, "rmsnorm_fwd", max_abs_diff(dev, yc));
    Matrix dwd(1, C), dxd(R, C), dwc(1, C), dxc(R, C);
    check(devops::rmsnorm_bwd(b, a, ric, w, true, &dwd, true, &dxd), "rmsnorm_bwd handled", 0.0);
    for (size_t i = 0; i < R; ++i) {
        float term = 0.0f;
        for (size_t j = 0; j < C; ++j) {
            dwc(0, j) += b(i, j) * a(i, j) * ric[i];
            term += b(i, j) * w(0, j) * a(i, j);
        }
        for (size_t j = 0; j < C; ++j)
            dxc(i, j) = ric[i] * (b(i, j) * w(0, j) - a(i, j) * ric[i] * ric[i] * term / static_cast<float>(C));
    }
    check(max_abs_diff(dwd, dwc) <= 1e-4, "rmsnorm_bwd dw", max_abs_diff(dwd, dwc));
    check(max_abs_diff(dxd, dxc) <= 1e-5, "rmsnorm_bwd dx", max_abs_diff(dxd, dxc));
}

void leg_gemm() {
    std::printf("-- device::gemm, four transpose combinations, GPU against host --\n");
    const size_t M = 70, K = 131, N = 45;
    const char* names[4] = {"N N", "T N", "N T", "T T"};
    for (int combo = 0; combo < 4; ++combo) {
        const bool ta = combo & 1, tb = combo & 2;
        const Matrix A = ta ? filled(K, M, 11) : filled(M, K, 11), B = tb ? filled(N, K, 12) : filled(K, N, 12);
        const auto tA = ta ? device::Trans::T : device::Trans::N, tB = tb ? device::Trans::T : device::Trans::N;
        const Matrix host = device::gemm(A, nullptr, tA, B, nullptr, tB);
        Matrix gpu(1, 1);
        {
            OnGpu on;
            gpu = device::gemm(A, nullptr, tA, B, nullptr, tB);
        }
        check(max_abs_diff(gpu, host) <= 2e-4, names[combo], max_abs_diff(gpu, host));
    }
}

// Explicit residency, the legs of tests/test_resident_parity.cpp:65-104 of the reference: both operands resident,
// one resident and one uploaded per call, and the contract leg -- mutate host data, invalidate, make resident again,
// and the product must be that of the mutated operand. One leg more than the reference has: a resident copy that
// was NOT refreshed after a host mutation must still give the OLD product, which shows that the table is really
// what the product reads (stubs that upload on every call would pass every other leg).
void leg_residency() {
    std::printf("-- explicit residency: make_resident / invalidate / evict_all / resident_count --\n");
    const size_t M = 37, K = 53, N = 41;
    Matrix A = filled(M, K, 31), B = filled(K, N, 32);
    const Matrix c_ref = device::matmul(A, B);  // host
    device::set(device::Device::CUDA);
    device::set_residency(true);
    check(device::residency_enabled(), "residency_enabled after set_residency(true)", 0.0);
    device::make_resident(A);
    device::make_resident(B);
    check(device::resident_count() == 2, "resident_count after 2 uploads", static_cast<double>(device::resident_count()));
    const Matrix c_b1 = device::matmul(A, B);
    check(max_abs_diff(c_ref, c_b1) <= 1e-4, "both operands resident vs host", max_abs_diff(c_ref, c_b1));
    device::make_resident(A);  // same pointer, same shape: refreshed in place, no second entry
    check(device::resident_count() == 2, "make_resident twice keeps one entry", static_cast<double>(device::resident_count()));
    device::invalidate(B);
    check(device::resident_count() == 1, "resident_count after invalidate", static_cast<double>(device::resident_count()));
    const Matrix c_mixed = device::matmul(A, B);
    check(max_abs_diff(c_ref, c_mixed) <= 1e-4, "A resident, B uploaded per call vs host", max_abs_diff(c_ref, c_mixed));
    // host mutation without a refresh: the device copy is the old one, by contract
    A.get_data()[0] += 0.5f;
    A.get_data()[M * K - 1] -= 0.25f;
    const Matrix c_stale = device::matmul(A, B);
    check(max_abs_diff(c_ref, c_stale) <= 1e-4, "stale resident copy gives the old product", max_abs_diff(c_ref, c_stale));
    // the contract leg
    device::invalidate(A);
    device::make_resident(A);
    device::make_resident(B);
    device::set(device::Device::CPU);
    const Matrix c_ref2 = device::matmul(A, B);
    device::set(device::Device::CUDA);
    const Matrix c_after = device::matmul(A, B);
    check(max_abs_diff(c_ref2, c_after) <= 1e-4, "mutate -> invalidate -> resident again matches the new host product",
          max_abs_diff(c_ref2, c_after));
    check(max_abs_diff(c_ref, c_ref2) > 1e-2, "(the mutation does change the product)", max_abs_diff(c_ref, c_ref2));
    device::evict_all();
    check(device::resident_count() == 0, "evict_all empties the table", static_cast<double>(device::resident_count()));
    device::set_residency(false);
    device::set(device::Device::CPU);
}

struct HeadRun {
    Matrix y, dq, dk, dv;
};
HeadRun run_head(bool hip_node, size_t T, size_t dk, size_t sl, bool causal, size_t window, size_t sinks) {
    Var q = mt::make_var(filled(T, dk, 21, 1.0f), true), k = mt::make_var(filled(T, dk, 22, 1.0f), true),
        v = mt::make_var(filled(T, dk, 23, 1.0f), true), g = mt::make_var(filled(T, dk, 24, 1.0f), false);
    const float scale = 1.0f / std::sqrt(static_cast<float>(dk));
    Var y;
    if (hip_node)
        y = window ? mt::ops::swa_attention_hip(q, k, v, scale, window, sinks, sl)
                   : mt::ops::fused_attention_hip(q, k, v, scale, sl, causal);
    else
        y = window ? mt::ops::swa_attention(q, k, v, scale, window, sinks, sl)
                   : mt::ops::fused_attention(q, k, v, scale, sl, causal);
    mt::backward(mt::ops::mean(mt::ops::mul(y, g)));
    return HeadRun{y->data, q->grad, k->grad, v->grad};
}
void leg_attention() {
    std::printf("-- attention tape nodes: host loops ([T,T] kept) against the O + logsumexp node on the GPU --\n");
    struct Case {
        const char* name;
        size_t T, dk, sl, window, sinks;
        bool causal;
    } cases[] = {
        {"fused_attention causal, T=128 d=32 (BASELINE config 1 head)", 128, 32, 0, 0, 0, true},
        {"fused_attention two stacked sequences, bidirectional", 96, 16, 48, 0, 0, false},
        {"fused_attention causal, T=200 d=64", 200, 64, 0, 0, 0, true},
        {"swa_attention window 7 + 2 sinks, stacked", 120, 32, 60, 7, 2, true},
        {"swa_attention window past the sequence (== causal)", 64, 32, 0, 1000, 0, true},
    };
    for (const Case& c : cases) {
        const HeadRun host = run_head(false, c.T, c.dk, c.sl, c.causal, c.window, c.sinks);
        HeadRun gpu;
        {
            OnGpu on;
            gpu = run_head(true, c.T, c.dk, c.sl, c.causal, c.window, c.sinks);
        }
        std::printf(" %s\n", c.name);
        check(max_abs_diff(gpu.y, host.y) <= 1e-5, "y", max_abs_diff(gpu.y, host.y));
        check(max_abs_diff(gpu.dq, host.dq) <= 1e-5, "dQ", max_abs_diff(gpu.dq, host.dq));
        check(max_abs_diff(gpu.dk, host.dk) <= 1e-5, "dK", max_abs_diff(gpu.dk, host.dk));
        check(max_abs_diff(gpu.dv, host.dv) <= 1e-5, "dV", max_abs_diff(gpu.dv, host.dv));
    }
    // with the device off the new node IS the old one
    const HeadRun a = run_head(false, 40, 8, 0, true, 0, 0), b = run_head(true, 40, 8, 0, true, 0, 0);
    check(max_abs_diff(a.y, b.y) == 0.0 && max_abs_diff(a.dq, b.dq) == 0.0, "device off: falls through to the host loops, bitwise", 0.0);
}

struct ModelRun {
    float loss;
    std::vector<Matrix> grads;
};
ModelRun run_llama(bool ckpt, bool window) {
    mt::nn::LlamaConfig cfg;
    cfg.vocab = 97;
    cfg.d = 32;
    cfg.n_layers = 2;
    cfg.n_heads = 4;
    cfg.d_ff = 64;
    cfg.n_ctx = 16;
    mt::nn::Llama model(cfg, 42);
    model.train();
    model.checkpoint_blocks = ckpt;
    std::vector<int> ids(32), tg(32);
    for (int i = 0; i < 32; ++i) {
        ids[i] = (7 * i + 3) % 97;
        tg[i] = (11 * i + 5) % 97;
    }
    if (window) device::step_begin();
    Var loss = mt::ops::cross_entropy(model.forward(ids, 16), tg);
    mt::backward(loss);
    if (window) device::step_end();
    ModelRun r;
    r.loss = loss->data(0, 0);
    for (const auto& p : model.parameters()) r.grads.push_back(p->grad);
    return r;
}
void leg_llama() {
    std::printf("-- nn::Llama forward + cross-entropy + backward: GEMMs and RMSNorm on the GPU against all-host --\n");
    for (int ckpt = 0; ckpt < 2; ++ckpt) {
        const ModelRun host = run_llama(ckpt != 0, false);
        ModelRun gpu;
        {
            OnGpu on;
            device::set_step_residency(true);
            gpu = run_llama(ckpt != 0, true);
            device::set_step_residency(false);
        }
        double worst = 0.0;
        for (size_t i = 0; i < host.grads.size(); ++i) worst = std::fmax(worst, max_abs_diff(gpu.grads[i], host.grads[i]));
        std::printf(" checkpoint_blocks = %d: loss host %.7f gpu %.7f\n", ckpt, host.loss, gpu.loss);
        check(std::fabs(host.loss - gpu.loss) <= 1e-5, "loss", std::fabs(host.loss - gpu.loss));
        check(worst <= 1e-5, "every parameter gradient", worst);
    }
}

}  // namespace

int main() {
    std::setvbuf(stdout, nullptr, _IOLBF, 0);
    try {
        device::set(device::Device::CUDA);  // throws without a gfx950 device
        device::set(device::Device::CPU);
        leg_op_set();
        leg_gemm();
        leg_residency();
        leg_attention();
        leg_llama();
    } catch (const std::exception& e) {
        std::printf("seam_check: exception: %s\n", e.what());
        return 2;
    }
    if (g_failures == 0) {
        std::printf("seam_check PASSED\n");
        return 0;
    }
    std::printf("seam_check: %d FAILURE(S)\n", g_failures);
    return 1;
}
