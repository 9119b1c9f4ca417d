// Benchmark-configuration harness written against the Juzhen API
// (Matrix<D>, operators, ml/layer.hpp layers).  The same source is compiled
// twice: with plain g++ against the reference tree (D = float: the reference's
// own CPU path, the parity oracle and CPU baseline) and with hipcc -DROCM_HIP
// against the MI355X backend (D = ROCMfloat).  All inputs and initial weights
// are generated on the host from explicit mt19937 seeds, so both builds see
// identical numbers.  Results are printed as `RESULT <name> <values...>` lines
// and dumped as raw float32 files for element-wise comparison.
//
// Selected through the environment (the library owns main(), cpp/launcher.cu):
//   JZ_CONFIG = c1 | c2 | c3      JZ_STEPS = training steps      JZ_OUT = dump dir
//   JZ_SCALE  = full | small      (small shrinks batch/width for quick runs)
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <iomanip>
#include <list>
#include <random>
#include <string>
#include <vector>

#include "../ml/layer.hpp"

using namespace Juzhen;

#ifdef ROCM_HIP
typedef ROCMfloat D;
static const char* kBackend = "rocm";
static Matrix<float> host(const Matrix<D>& m) { return m.to_host(); }
#else
typedef float D;
static const char* kBackend = "cpu";
static Matrix<float> host(const Matrix<D>& m) { return m; }
#endif

namespace {

std::string env(const char* k, const char* dflt) {
    const char* v = std::getenv(k);
    return v ? v : dflt;
}

Matrix<float> host_normal(int r, int c, std::mt19937& g, float scale) {
    std::normal_distribution<float> n(0.f, 1.f);
    Matrix<float> m("h", r, c);
    float* p = const_cast<float*>(m.data());
    for (size_t i = 0; i < (size_t)r * c; ++i) p[i] = n(g) * scale;
    return m;
}
Matrix<float> host_uniform(int r, int c, std::mt19937& g) {
    std::uniform_real_distribution<float> u(0.f, 1.f);
    Matrix<float> m("h", r, c);
    float* p = const_cast<float*>(m.data());
    for (size_t i = 0; i < (size_t)r * c; ++i) p[i] = u(g);
    return m;
}

void dump(const std::string& dir, const std::string& name, const Matrix<float>& m) {
    // logical content, column-major float32
    const std::string path = dir + "/" + name + "." + kBackend + ".f32";
    FILE* f = std::fopen(path.c_str(), "wb");
    if (!f) { std::printf("cannot write %s\n", path.c_str()); return; }
    for (size_t j = 0; j < m.num_col(); ++j)
        for (size_t i = 0; i < m.num_row(); ++i) {
            const float v = m.elem(i, j);
            std::fwrite(&v, sizeof v, 1, f);
        }
    std::fclose(f);
}

double now_ms() {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// ── C1: expression chain (README.md:29-31), row softmax, row / column sums ──
int run_c1(const std::string& out, bool small) {
    const int n = small ? 192 : 1024;
    std::mt19937 ga(1), gb(2);
    const Matrix<float> Ah = host_normal(n, n, ga, 1.0f / std::sqrt((float)n));
    const Matrix<float> Bh = host_normal(n, n, gb, 1.0f / std::sqrt((float)n));
    const Matrix<D> A(Ah), B(Bh);
    // each op separately, as the configuration asks
    Matrix<D> P = A * B;
    dump(out, "c1_gemm", host(P));
    Matrix<D> E = exp(P);
    dump(out, "c1_exp", host(E));
    Matrix<D> E1 = E + 1.0;
    Matrix<D> L = log(E1);
    dump(out, "c1_log", host(L));
    Matrix<D> C = L / 5.0;
    dump(out, "c1_chain", host(C));
    // the one-expression form must agree with the stepwise one
    Matrix<D> C2 = log(exp(A * B) + 1.0f) / 5.0f;
    dump(out, "c1_chain_expr", host(C2));
    Matrix<D> S = row_softmax(C);
    dump(out, "c1_softmax", host(S));
    dump(out, "c1_rowsum", host(sum(S, 1)));
    dump(out, "c1_colsum", host(sum(S, 0)));
    dump(out, "c1_chain_rowsum", host(sum(C, 1)));
    dump(out, "c1_chain_colsum", host(sum(C, 0)));
    // timing of the whole chain (3 warm-ups, 10 iterations; tests/benchmarkCoreOps.cu:35-54)
    for (int i = 0; i < 3; ++i) { Matrix<D> t = log(exp(A * B) + 1.0f) / 5.0f; (void)host(sum(t, 1)); }
    const double t0 = now_ms();
    for (int i = 0; i < 10; ++i) { Matrix<D> t = log(exp(A * B) + 1.0f) / 5.0f; (void)host(sum(t, 1)); }
    std::printf("RESULT c1_chain_ms %.4f\n", (now_ms() - t0) / 10);
    return 0;
}

// ── C2: MLP regression, MSE, Adam (examples/helloworld_nn.cu:72-99) ─────────
int run_c2(const std::string& out, bool small, int steps) {
    const int nb = small ? 256 : 4096, din = 16, hid = small ? 64 : 256;
    std::mt19937 g(7);
    const Matrix<float> Xh = host_normal(din, nb, g, 1.0f);
    Matrix<float> Yh("y", 1, nb);
    {
        std::normal_distribution<float> noise(0.f, 0.1f);
        for (int c = 0; c < nb; ++c) {
            float s = 0.f;
            for (int r = 0; r < din; ++r) s += std::sin(Xh.elem(r, c));
            Yh.elem(0, c) = s + noise(g);
        }
    }
    ReluLayer<D> L0(hid, din, nb), L1(hid, hid, nb);
    LinearLayer<D> L2(1, hid, nb);
    std::list<Layer<D>*> net({&L2, &L1, &L0});
    for (Layer<D>* l : net) {
        // He-normal weights, zero biases, Adam alpha 1e-3
        const int fan_in = (int)l->W().num_col();
        l->W() = Matrix<D>(host_normal((int)l->W().num_row(), fan_in, g, std::sqrt(2.0f / fan_in)));
        l->b() = Matrix<D>(Matrix<float>::zeros(l->b().num_row(), 1));
        l->adamWstate().alpha = 1e-3f;
        l->adambstate().alpha = 1e-3f;
    }
    const Matrix<D> X(Xh), Y(Yh);
    Matrix<float> losses("losses", 1, steps);
    double t0 = 0;
    for (int it = 0; it < steps; ++it) {
        if (it == 3) t0 = now_ms();
        forward(net, X);
        LossLayer<D> loss(nb, Y);
        loss.eval(L2.value());
        losses.elem(0, it) = item(loss.value());
        net.push_front(&loss);
        backprop(net, X);
        net.pop_front();
    }
    if (steps > 3) std::printf("RESULT c2_ms_per_step %.4f\n", (now_ms() - t0) / (steps - 3));
    std::printf("RESULT c2_loss_first %.8g\nRESULT c2_loss_last %.8g\n", losses.elem(0, 0), losses.elem(0, steps - 1));
    dump(out, "c2_losses", losses);
    dump(out, "c2_W0", host(L0.W()));
    dump(out, "c2_W2", host(L2.W()));
    return 0;
}

// ── C3: MNIST-shaped CNN, softmax cross-entropy, Adam (examples/demo_cnn_mnist.cu:251-288) ──
int run_c3(const std::string& out, bool small, int steps) {
    const int nb = small ? 16 : 128, C1 = small ? 8 : 32, C2 = small ? 16 : 64, H = 28, k = 10;
    std::mt19937 g(11);
    const Matrix<float> Xh = host_uniform(H * H, nb, g);
    Matrix<float> Yh("y", k, nb);
    Yh.zeros();
    {
        std::uniform_int_distribution<int> lab(0, k - 1);
        for (int c = 0; c < nb; ++c) Yh.elem(lab(g), c) = 1.0f;
    }
    ConvLayer conv1(nb, 1, H, H, C1, 3, 3, 1, 1, true);
    ConvLayer conv2(nb, C1, H, H, C2, 3, 3, 1, 2, true);
    const int H2 = (H + 2 - 3) / 2 + 1;
    LinearLayer<D> fc(k, C2 * H2 * H2, nb);
    std::list<Layer<D>*> net({&fc, &conv2, &conv1});
    for (Layer<D>* l : net) {
        l->W() = Matrix<D>(host_normal((int)l->W().num_row(), (int)l->W().num_col(), g, 0.01f));
        l->b() = Matrix<D>(host_normal((int)l->b().num_row(), 1, g, 0.01f));
        l->adamWstate().alpha = 1e-3f;
        l->adambstate().alpha = 1e-3f;
    }
    const Matrix<D> X(Xh), Y(Yh);
    Matrix<float> losses("losses", 1, steps);
    double t0 = 0;
    for (int it = 0; it < steps; ++it) {
        if (it == 2) t0 = now_ms();
        forward(net, X);
        LogisticLayer<D> loss(nb, Y);
        loss.eval(fc.value());
        losses.elem(0, it) = item(loss.value());
        net.push_front(&loss);
        backprop(net, X);
        net.pop_front();
    }
    if (steps > 2) std::printf("RESULT c3_ms_per_step %.4f\n", (now_ms() - t0) / (steps - 2));
    std::printf("RESULT c3_loss_first %.8g\nRESULT c3_loss_last %.8g\n", losses.elem(0, 0), losses.elem(0, steps - 1));
    dump(out, "c3_losses", losses);
    dump(out, "c3_conv1_W", host(conv1.W()));
    dump(out, "c3_fc_b", host(fc.b()));
    return 0;
}

}  // namespace

int compute() {
    const std::string cfg = env("JZ_CONFIG", "c1");
    const std::string out = env("JZ_OUT", "/tmp");
    const bool small = env("JZ_SCALE", "full") == "small";
    const int steps = std::atoi(env("JZ_STEPS", "100").c_str());
    std::printf("RESULT backend %s\n", kBackend);
    if (cfg == "c1") return run_c1(out, small);
    if (cfg == "c2") return run_c2(out, small, steps);
    if (cfg == "c3") return run_c3(out, small, steps);
    std::printf("unknown JZ_CONFIG %s\n", cfg.c_str());
    return 1;
}
