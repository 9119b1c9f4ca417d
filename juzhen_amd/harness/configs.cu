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
//   JZ_CONFIG = c1 | c2 | c3 | c5  JZ_STEPS = training steps     JZ_OUT = dump dir
//   JZ_SCALE  = full | small      (small shrinks batch/width for quick runs)
//   JZ_GRAPH  = 1                 (ROCm build, c2 and c3: record the step once, replay it as a HIP graph)
//   JZ_STREAM = 1                 (ROCm build: run on a created stream instead of the null stream)
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

// Wait for everything issued so far (reading any device value does): timing marks only.
template <class M>
void sync_device(const std::vector<M>& kept) {
    if (!kept.empty()) (void)item(kept.back());
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
    // Losses stay on the device while the loop runs and are read after it: reading one
    // per step (item(), ml/util.cuh:112-124) would drain the device once per step.
    std::vector<Matrix<D>> loss_dev;
    loss_dev.reserve(steps);
    double t0 = 0;
#ifdef ROCM_HIP
    if (env("JZ_GRAPH", "0") == "1") {
        // three ordinary steps (they also fill the pool with every buffer size), then the step
        // is recorded once and replayed: one graph launch per step instead of ~60 kernel launches
        RocmStepGraph graph;
        LossLayer<D> loss(nb, Y);
        Matrix<D> loss_now("loss_now", 1, 1);   // backprop overwrites the loss layer's value
        const bool every = env("JZ_GRAPH_LOSSES", "1") == "1";
        auto one_step = [&] {
            forward(net, X);
            loss.eval(L2.value());
            copy(loss_now, loss.value());
            net.push_front(&loss);
            backprop(net, X);
            net.pop_front();
        };
        for (int it = 0; it < steps; ++it) {
            if (it == 3) {
                sync_device(loss_dev);
                graph.begin();
                one_step();
                graph.end();
                t0 = now_ms();
            }
            if (it < 3) one_step(); else graph.replay();
            // a copy on the device, ordered after the replay (JZ_GRAPH_LOSSES=0: only the last one)
            if (every || it == steps - 1) loss_dev.push_back(loss_now);
            else loss_dev.push_back(Matrix<D>("skipped", 1, 1));
        }
    } else
#endif
    for (int it = 0; it < steps; ++it) {
        if (it == 3) { sync_device(loss_dev); t0 = now_ms(); }
        forward(net, X);
        LossLayer<D> loss(nb, Y);
        loss.eval(L2.value());
        loss_dev.push_back(loss.value());
        net.push_front(&loss);
        backprop(net, X);
        net.pop_front();
    }
    sync_device(loss_dev);
    if (steps > 3) std::printf("RESULT c2_ms_per_step %.4f\n", (now_ms() - t0) / (steps - 3));
    for (int it = 0; it < steps; ++it) losses.elem(0, it) = item(loss_dev[it]);
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
    std::vector<Matrix<D>> loss_dev;
    loss_dev.reserve(steps);
    double t0 = 0;
#ifdef ROCM_HIP
    if (env("JZ_GRAPH", "0") == "1") {
        RocmStepGraph graph;
        LogisticLayer<D> loss(nb, Y);
        auto one_step = [&] {
            forward(net, X);
            loss.eval(fc.value());
            net.push_front(&loss);
            backprop(net, X);
            net.pop_front();
        };
        for (int it = 0; it < steps; ++it) {
            if (it == 2) {
                sync_device(loss_dev);
                graph.begin();
                one_step();
                graph.end();
                t0 = now_ms();
            }
            if (it < 2) one_step(); else graph.replay();
            loss_dev.push_back(loss.value());
        }
    } else
#endif
    for (int it = 0; it < steps; ++it) {
        if (it == 2) { sync_device(loss_dev); t0 = now_ms(); }
        forward(net, X);
        LogisticLayer<D> loss(nb, Y);
        loss.eval(fc.value());
        loss_dev.push_back(loss.value());
        net.push_front(&loss);
        backprop(net, X);
        net.pop_front();
    }
    sync_device(loss_dev);
    if (steps > 2) std::printf("RESULT c3_ms_per_step %.4f\n", (now_ms() - t0) / (steps - 2));
    for (int it = 0; it < steps; ++it) losses.elem(0, it) = item(loss_dev[it]);
    std::printf("RESULT c3_loss_first %.8g\nRESULT c3_loss_last %.8g\n", losses.elem(0, 0), losses.elem(0, steps - 1));
    dump(out, "c3_losses", losses);
    dump(out, "c3_conv1_W", host(conv1.W()));
    dump(out, "c3_fc_b", host(fc.b()));
    return 0;
}

// ── C5: rectified-flow conv UNet, CIFAR-10 shape (wiring of
//    examples/demo_cnn_rectified.cu:210-315 and its step :476-535, with two
//    conv+ReLU blocks per level and an additive sinusoidal time embedding) ──
struct UNet {
    int nb, H, c1, c2, c3;
    ConvLayer e1a, e1b, e2a, e2b, e3a, e3b, d2a, d2b, d1a, d1b, head;
    ConvTransLayer up2, up1;
    Matrix<D> T1, T2, T3, Td2, Td1;                       // time embeddings, one per level
    Matrix<D> a1, s1, a2, s2, a3, m, cat2, ad2, dd2, cat1, ad1, dd1;

    UNet(int nb_, int H_, int c1_, int c2_, int c3_)
        : nb(nb_), H(H_), c1(c1_), c2(c2_), c3(c3_),
          e1a(nb, 3, H, H, c1, 3, 3, 1, 1, true), e1b(nb, c1, H, H, c1, 3, 3, 1, 1, true),
          e2a(nb, c1, H, H, c2, 3, 3, 1, 2, true), e2b(nb, c2, H / 2, H / 2, c2, 3, 3, 1, 1, true),
          e3a(nb, c2, H / 2, H / 2, c3, 3, 3, 1, 2, true), e3b(nb, c3, H / 4, H / 4, c3, 3, 3, 1, 1, true),
          d2a(nb, 2 * c2, H / 2, H / 2, c2, 3, 3, 1, 1, true), d2b(nb, c2, H / 2, H / 2, c2, 3, 3, 1, 1, true),
          d1a(nb, 2 * c1, H, H, c1, 3, 3, 1, 1, true), d1b(nb, c1, H, H, c1, 3, 3, 1, 1, true),
          head(nb, c1, H, H, 3, 3, 3, 1, 1, false),
          up2(nb, c3, H / 4, H / 4, c2, 4, 4, 1, 2, true), up1(nb, c2, H / 2, H / 2, c1, 4, 4, 1, 2, true) {}

    std::vector<Layer<D>*> layers() {
        return {&e1a, &e1b, &e2a, &e2b, &e3a, &e3b, &up2, &d2a, &d2b, &up1, &d1a, &d1b, &head};
    }

    // emb(c*P + p, n) = sin(2^(c/2) * pi * t_n) for even c, cos(...) for odd c
    static Matrix<float> time_embedding(int C, int P, const std::vector<float>& t) {
        Matrix<float> e("temb", C * P, (int)t.size());
        for (size_t n = 0; n < t.size(); ++n)
            for (int c = 0; c < C; ++c) {
                const float f = std::ldexp(3.14159265358979323846f, (c / 2) % 6);
                const float v = 0.1f * ((c & 1) ? std::cos(f * t[n]) : std::sin(f * t[n]));
                for (int p = 0; p < P; ++p) e.elem((size_t)c * P + p, n) = v;
            }
        return e;
    }
    void set_time(const std::vector<float>& t) {
        const int P = H * H;
        T1 = Matrix<D>(time_embedding(c1, P, t));
        T2 = Matrix<D>(time_embedding(c2, P / 4, t));
        T3 = Matrix<D>(time_embedding(c3, P / 16, t));
        Td2 = Matrix<D>(time_embedding(c2, P / 4, t));
        Td1 = Matrix<D>(time_embedding(c1, P, t));
    }

    const Matrix<D>& fwd(const Matrix<D>& x) {
        e1a.eval(x);    a1 = e1a.value() + T1;
        e1b.eval(a1);   s1 = e1b.value();
        e2a.eval(s1);   a2 = e2a.value() + T2;
        e2b.eval(a2);   s2 = e2b.value();
        e3a.eval(s2);   a3 = e3a.value() + T3;
        e3b.eval(a3);   m = e3b.value();
        up2.eval(m);    cat2 = vstack(std::vector<MatrixView<D>>{MatrixView<D>(up2.value()), MatrixView<D>(s2)});
        d2a.eval(cat2); ad2 = d2a.value() + Td2;
        d2b.eval(ad2);  dd2 = d2b.value();
        up1.eval(dd2);  cat1 = vstack(std::vector<MatrixView<D>>{MatrixView<D>(up1.value()), MatrixView<D>(s1)});
        d1a.eval(cat1); ad1 = d1a.value() + Td1;
        d1b.eval(ad1);  dd1 = d1b.value();
        head.eval(dd1);
        return head.value();
    }
    void bwd(const Matrix<D>& x, Matrix<D>&& g) {
        auto g0 = head.backward(dd1, std::move(g));
        auto g1 = d1b.backward(ad1, std::move(g0));
        auto gc1 = d1a.backward(cat1, std::move(g1));
        const size_t k1 = (size_t)c1 * H * H;
        auto gu1 = gc1.rows(0, k1);
        auto gs1 = gc1.rows(k1, gc1.num_row());
        auto g2 = up1.backward(dd2, std::move(gu1));
        auto g3 = d2b.backward(ad2, std::move(g2));
        auto gc2 = d2a.backward(cat2, std::move(g3));
        const size_t k2 = (size_t)c2 * (H / 2) * (H / 2);
        auto gu2 = gc2.rows(0, k2);
        auto gs2 = gc2.rows(k2, gc2.num_row());
        auto g4 = up2.backward(m, std::move(gu2));
        auto g5 = e3b.backward(a3, std::move(g4));
        auto g6 = e3a.backward(s2, std::move(g5));
        g6 = g6 + gs2;
        auto g7 = e2b.backward(a2, std::move(g6));
        auto g8 = e2a.backward(s1, std::move(g7));
        g8 = g8 + gs1;
        auto g9 = e1b.backward(a1, std::move(g8));
        e1a.backward(x, std::move(g9));
    }
};

int run_c5(const std::string& out, bool small, int steps) {
    const int nb = small ? 4 : 128, H = small ? 16 : 32;
    const int c1 = small ? 8 : 64, c2 = small ? 16 : 128, c3 = small ? 32 : 256;
    const int d = 3 * H * H;
    std::mt19937 g(23);
    UNet net(nb, H, c1, c2, c3);
    for (Layer<D>* l : net.layers()) {
        // He-normal over the patch fan-in, zero biases, Adam alpha 2e-4
        const size_t nw = l->W().num_row() * l->W().num_col();
        const size_t cout = l->b().num_row();
        const float sd = std::sqrt(2.0f / (float)(nw / cout));
        l->W() = Matrix<D>(host_normal((int)l->W().num_row(), (int)l->W().num_col(), g, sd));
        l->b() = Matrix<D>(Matrix<float>::zeros(cout, 1));
        l->adamWstate().alpha = 2e-4f;
        l->adambstate().alpha = 2e-4f;
    }
    // one fixed batch: x1 = clip(N(0,1), -1, 1), x0 = N(0,1), t = U[0,1]
    Matrix<float> x1h = host_normal(d, nb, g, 1.0f);
    for (size_t i = 0; i < (size_t)d * nb; ++i) {
        float& v = const_cast<float*>(x1h.data())[i];
        v = v < -1.f ? -1.f : (v > 1.f ? 1.f : v);
    }
    const Matrix<float> x0h = host_normal(d, nb, g, 1.0f);
    std::vector<float> t(nb);
    {
        std::uniform_real_distribution<float> u(0.f, 1.f);
        for (float& v : t) v = u(g);
    }
    // x_t = (1-t) x0 + t x1 and the target velocity x1 - x0, formed on the host
    Matrix<float> xth("xt", d, nb), vth("vt", d, nb);
    for (int n = 0; n < nb; ++n)
        for (int p = 0; p < d; ++p) {
            xth.elem(p, n) = (1.f - t[n]) * x0h.elem(p, n) + t[n] * x1h.elem(p, n);
            vth.elem(p, n) = x1h.elem(p, n) - x0h.elem(p, n);
        }
    const Matrix<D> xt(xth), vt(vth);
    net.set_time(t);
    Matrix<float> losses("losses", 1, steps);
    std::vector<Matrix<D>> loss_dev;
    loss_dev.reserve(steps);
    double t0 = 0;
    for (int it = 0; it < steps; ++it) {
        if (it == 1) { sync_device(loss_dev); t0 = now_ms(); }
        const Matrix<D>& pred = net.fwd(xt);
        if (it == 0) dump(out, "c5_pred0", host(pred));
        Matrix<D> diff = pred - vt;
        loss_dev.push_back(sum(sum(square(Matrix<D>(diff)), 0), 1));   // demo_cnn_rectified.cu:531-534
        Matrix<D> grad = 2.0f * diff / (float)nb;
        net.bwd(xt, std::move(grad));
    }
    sync_device(loss_dev);
    if (steps > 1) std::printf("RESULT c5_ms_per_step %.4f\n", (now_ms() - t0) / (steps - 1));
    for (int it = 0; it < steps; ++it) losses.elem(0, it) = item(loss_dev[it]) / (float)nb;
    std::printf("RESULT c5_loss_first %.8g\nRESULT c5_loss_last %.8g\n", losses.elem(0, 0), losses.elem(0, steps - 1));
    dump(out, "c5_losses", losses);
    dump(out, "c5_head_W", host(net.head.W()));
    dump(out, "c5_e1a_W", host(net.e1a.W()));
    dump(out, "c5_up2_W", host(net.up2.W()));
    return 0;
}

}  // namespace

int compute() {
    const std::string cfg = env("JZ_CONFIG", "c1");
    const std::string out = env("JZ_OUT", "/tmp");
    const bool small = env("JZ_SCALE", "full") == "small";
    const int steps = std::atoi(env("JZ_STEPS", "100").c_str());
    std::printf("RESULT backend %s\n", kBackend);
#ifdef ROCM_HIP
    if (env("JZ_STREAM", "0") == "1") {   // everything on a stream of its own instead of the null stream
        void* s = nullptr;
        if (jzhip_stream_create(&s) != 0 || jzhip_set_stream(s) != 0) return 1;
    }
#endif
    if (cfg == "c1") return run_c1(out, small);
    if (cfg == "c2") return run_c2(out, small, steps);
    if (cfg == "c3") return run_c3(out, small, steps);
    if (cfg == "c5") return run_c5(out, small, steps);
    std::printf("unknown JZ_CONFIG %s\n", cfg.c_str());
    return 1;
}
