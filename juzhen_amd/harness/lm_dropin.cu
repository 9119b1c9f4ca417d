// The character-LM train step written only with the reference's own classes
// on Matrix<ROCMfloat>: LinearLayer embed on stacked one-hot [token; position]
// columns, `layers` TransformerLayer blocks, LinearLayer projection,
// LogisticLayer loss, Adam — the wiring of examples/demo_transformer.cu:285-383,
// timed the way tests/benchmarkTrainingStep.cu:47-88 times one block (warm-up,
// per-step wall clock closed by a device synchronisation, mean / p50 / p95).
// It measures what a user of the drop-in API gets for the benchmark's model
// size, beside the hand-scheduled harness (juzhen_amd/harness/lm.cpp) that
// reaches the same mathematics through the C ABI.
//
// Environment: JZ_SCALE = full | small, JZ_STEPS (default 10), JZ_WARMUP (3).
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <list>
#include <memory>
#include <numeric>
#include <random>
#include <string>
#include <vector>

#include "../ml/layer.hpp"

using namespace Juzhen;

#ifdef ROCM_HIP
typedef ROCMfloat D;
static const char* kBackend = "rocm";
static Matrix<float> host(const Matrix<D>& m) { return m.to_host(); }
extern "C" int jzhip_synchronize(void);
static void device_sync() { jzhip_synchronize(); }
#else
typedef float D;
static const char* kBackend = "cpu";
static Matrix<float> host(const Matrix<D>& m) { return m; }
static void device_sync() {}
#endif

namespace {
int env_int(const char* k, int dflt) {
    const char* v = std::getenv(k);
    return v ? std::atoi(v) : dflt;
}
double now_ms() {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
Matrix<float> host_normal(int r, int c, std::mt19937& g, float scale) {
    std::normal_distribution<float> n(0.f, 1.f);
    Matrix<float> m("h", r, c);
    float* p = const_cast<float*>(m.data());
    for (size_t i = 0; i < (size_t)r * c; ++i) p[i] = n(g) * scale;
    return m;
}
}  // namespace

int compute() {
    const char* sc = std::getenv("JZ_SCALE");
    const bool small = sc && std::string(sc) == "small";
    const int V = small ? 32 : 256, d = small ? 64 : 512, heads = small ? 4 : 8, ff = small ? 128 : 2048;
    const int L = small ? 2 : 6, S = small ? 32 : 256, B = small ? 4 : 64;
    const int N = S * B, in_dim = V + S;
    const int steps = env_int("JZ_STEPS", 10), warmup = env_int("JZ_WARMUP", 3);

    // token ids Zipf(s = 1.1), one-hot inputs and targets built on the host
    std::mt19937 g(1234);
    std::vector<double> cdf(V);
    double acc = 0;
    for (int i = 0; i < V; ++i) cdf[i] = (acc += 1.0 / std::pow(i + 1.0, 1.1));
    std::uniform_real_distribution<double> u(0.0, acc);
    auto draw = [&] { return (int)(std::lower_bound(cdf.begin(), cdf.end(), u(g)) - cdf.begin()); };
    Matrix<float> Xh = Matrix<float>::zeros(in_dim, N), Yh = Matrix<float>::zeros(V, N);
    for (int b = 0; b < B; ++b) {
        int tok = draw();
        for (int s = 0; s < S; ++s) {
            const int n = b * S + s, next = draw();
            Xh.elem(tok, n) = 1.f;
            Xh.elem(V + s, n) = 1.f;
            Yh.elem(next, n) = 1.f;
            tok = next;
        }
    }

    LinearLayer<D> embed(d, in_dim, N);
    LinearLayer<D> proj(V, d, N);
    std::vector<std::unique_ptr<TransformerLayer<D>>> blocks;
    for (int i = 0; i < L; ++i) blocks.push_back(std::make_unique<TransformerLayer<D>>(d, d, ff, S, B, heads));
    // weights from the host so that the run does not depend on the device generator
    embed.W() = Matrix<D>(host_normal(d, in_dim, g, 0.02f));
    proj.W() = Matrix<D>(host_normal(V, d, g, 1.0f / std::sqrt((float)d)));
    const float lr = 3e-4f;
    embed.adamWstate().alpha = lr; embed.adambstate().alpha = lr;
    proj.adamWstate().alpha = lr;  proj.adambstate().alpha = lr;
    for (auto& b : blocks) b->set_lr(lr);

    std::list<Layer<D>*> net;
    net.push_back(&proj);
    for (int i = L - 1; i >= 0; --i) net.push_back(blocks[i].get());
    net.push_back(&embed);

    const Matrix<D> X(Xh), Y(Yh);
    float last_loss = 0.f, first_loss = 0.f;
    auto step = [&](bool read_loss) {
        // examples/demo_transformer.cu:368-376
        forward(net, X);
        LogisticLayer<D> loss(N, Matrix<D>(Y));
        net.push_front(&loss);
        backprop(net, X);
        net.pop_front();
        if (read_loss) {
            net.push_front(&loss);
            last_loss = host(forward(net, X)).elem(0, 0);
            net.pop_front();
        }
    };
    step(true);
    first_loss = last_loss;
    for (int i = 1; i < warmup; ++i) step(false);
    device_sync();
    std::vector<double> samples;
    const double t_all = now_ms();
    for (int i = 0; i < steps; ++i) {
        const double t0 = now_ms();
        step(false);
        device_sync();
        samples.push_back(now_ms() - t0);
    }
    const double wall = now_ms() - t_all;
    step(true);
    std::sort(samples.begin(), samples.end());
    const double mean = std::accumulate(samples.begin(), samples.end(), 0.0) / samples.size();
    const double p50 = samples[(size_t)(0.50 * (samples.size() - 1))], p95 = samples[(size_t)(0.95 * (samples.size() - 1))];
    std::printf("RESULT dropin backend=%s config=V%d,d%d,h%d,ff%d,L%d,S%d,B%d warmup=%d steps=%d mean_ms=%.3f p50_ms=%.3f "
                "p95_ms=%.3f tokens_per_second=%.1f loss_first=%.4f loss_last=%.4f wall_ms=%.1f\n",
                kBackend, V, d, heads, ff, L, S, B, warmup, steps, mean, p50, p95, N * 1000.0 / mean, first_loss,
                last_loss, wall);
    return (last_loss == last_loss) ? 0 : 1;   // NaN check
}
