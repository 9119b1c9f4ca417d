// Forward-mode tangents (jvp) on Matrix<ROCMfloat> against the CPU Matrix<float>:
// the reference's own tests/testJVP.cu skips on ROCm (:26-30), so this program
// runs its three checks for the layers that have a ROCm tangent path --
//   (a) the tangent against the CPU tangent of a layer with identical weights,
//   (b) adjoint consistency <W, J u> == <J^T W, u> against backprop on the device,
//   (c) central finite differences of the device forward pass along u --
// for a TransformerLayer (batched attention tangent, fused LayerNorm tangent)
// with and without the causal mask, and for a tanh -> relu -> linear stack of
// the dense layers (generic Layer::jvp on device matrices).
// Exit status 0 when every check passes.
#include <cmath>
#include <cstdio>
#include <list>
#include <random>
#include <string>

#include "../ml/layer.hpp"

using namespace Juzhen;

namespace {

Matrix<float> host_normal(int r, int c, std::mt19937& g, float scale) {
    std::normal_distribution<float> n(0.f, 1.f);
    Matrix<float> m("h", r, c);
    float* p = const_cast<float*>(m.data());
    for (size_t i = 0; i < (size_t)r * c; ++i) p[i] = n(g) * scale;
    return m;
}
Matrix<float> down(const Matrix<float>& m) { return m; }
#ifdef ROCM_HIP
typedef ROCMfloat Dev;
Matrix<float> down(const Matrix<ROCMfloat>& m) { return m.to_host(); }
Matrix<ROCMfloat> up(const Matrix<float>& h) { return Matrix<ROCMfloat>(h); }
#else
typedef float Dev;
Matrix<float> up(const Matrix<float>& h) { return h; }
#endif

double dotd(const Matrix<float>& a, const Matrix<float>& b) {
    double s = 0;
    for (size_t j = 0; j < a.num_col(); ++j)
        for (size_t i = 0; i < a.num_row(); ++i) s += (double)a.elem(i, j) * b.elem(i, j);
    return s;
}
// Relative error over all columns but the worst one, and the number of columns
// outside `tol`.  A ReLU pre-activation within rounding of zero may fall on either
// side on the two backends; that changes the tangent of that one token column
// and nothing else (the feed-forward part acts per column), so one such column
// is tolerated and reported.
double rel_but_one(const Matrix<float>& got, const Matrix<float>& want, double tol, int& outliers) {
    double num = 0, den = 0, worst_num = 0;
    outliers = 0;
    for (size_t j = 0; j < want.num_col(); ++j) {
        double n = 0, d = 0;
        for (size_t i = 0; i < want.num_row(); ++i) {
            const double e = (double)got.elem(i, j) - want.elem(i, j);
            n += e * e;
            d += (double)want.elem(i, j) * want.elem(i, j);
        }
        if (std::sqrt(n / (d + 1e-30)) > tol) ++outliers;
        worst_num = std::max(worst_num, n);
        num += n;
        den += d;
    }
    return std::sqrt((num - worst_num) / (den + 1e-30));
}
double rel(const Matrix<float>& got, const Matrix<float>& want) {
    double num = 0, den = 0;
    for (size_t j = 0; j < want.num_col(); ++j)
        for (size_t i = 0; i < want.num_row(); ++i) {
            const double d = (double)got.elem(i, j) - want.elem(i, j);
            num += d * d;
            den += (double)want.elem(i, j) * want.elem(i, j);
        }
    return std::sqrt(num / (den + 1e-30));
}

template <class D>
void copy_block_weights(const TransformerLayer<float>& src, TransformerLayer<D>& dst) {
    dst.set_Wq(Matrix<D>(src.get_Wq())); dst.set_Wk(Matrix<D>(src.get_Wk())); dst.set_Wv(Matrix<D>(src.get_Wv()));
    dst.set_Wo(Matrix<D>(src.get_Wo())); dst.set_bo(Matrix<D>(src.get_bo()));
    dst.set_W1(Matrix<D>(src.get_W1())); dst.set_b1(Matrix<D>(src.get_b1()));
    dst.set_W2(Matrix<D>(src.get_W2())); dst.set_b2(Matrix<D>(src.get_b2()));
    dst.set_ln1_gamma(Matrix<D>(src.get_ln1_gamma())); dst.set_ln1_beta(Matrix<D>(src.get_ln1_beta()));
    dst.set_ln2_gamma(Matrix<D>(src.get_ln2_gamma())); dst.set_ln2_beta(Matrix<D>(src.get_ln2_beta()));
}

// checks (a)-(c) for one network given as CPU and device layer lists with identical weights
int check(const std::string& name, std::list<Layer<float>*> cpu, std::list<Layer<Dev>*> dev, int d_in, int nb,
          std::mt19937& g, double tol_parity) {
    const Matrix<float> xh = host_normal(d_in, nb, g, 0.7f), uh = host_normal(d_in, nb, g, 1.0f);
    const Matrix<Dev> x = up(xh), u = up(uh);
    const Matrix<float> Ju_cpu = jvp(cpu, xh, uh);
    const Matrix<Dev> Ju_dev = jvp(dev, x, u);
    const Matrix<float> Ju = down(Ju_dev);
    int kinked = 0;
    const double parity = rel_but_one(Ju, Ju_cpu, 30 * tol_parity, kinked);
    // adjoint consistency on the device
    const Matrix<float> Wh = host_normal((int)Ju.num_row(), (int)Ju.num_col(), g, 1.0f);
    const Matrix<Dev> W = up(Wh);
    const Matrix<float> JTW = down(grad(dev, x, W));
    const double lhs = dotd(Wh, Ju), rhs = dotd(JTW, uh);
    // relative to the inner product as tests/testJVP.cu:60-66 does, with a floor at fp32
    // rounding of the terms it sums (the product can cancel to a small value by chance)
    const double terms = std::sqrt(dotd(Wh, Wh) * dotd(Ju, Ju));
    const double adj = std::fabs(lhs - rhs) / (std::fabs(lhs) + 1e-2 * terms + 1e-12);
    // central differences of the device forward pass, best of three steps (ReLU kinks)
    double fd = 1e30;
    for (float e : {1e-2f, 2.5e-3f, 6.25e-4f}) {
        const Matrix<float> fp = down(forward(dev, x + e * u)), fm = down(forward(dev, x - e * u));
        const Matrix<float> d = (fp - fm) * (0.5f / e);
        fd = std::min(fd, rel(d, Ju));
    }
    const bool ok = parity <= tol_parity && kinked <= 1 && adj <= 1e-4 && fd <= 5e-2;
    std::printf("%s %-34s tangent vs CPU %.2e%s  adjoint %.2e  finite differences %.2e\n", ok ? "ok  " : "FAIL",
                name.c_str(), parity, kinked ? " (one column at a ReLU kink set aside)" : "", adj, fd);
    return ok ? 0 : 1;
}

int transformer_case(int d, int ff, int S, int B, int heads, bool causal, std::mt19937& g) {
    TransformerLayer<float> cpu(d, d, ff, S, B, heads, causal);
    TransformerLayer<Dev> dev(d, d, ff, S, B, heads, causal);
    // biases and gains away from their trivial initial values so every path is live
    cpu.set_bo(host_normal(d, 1, g, 0.1f)); cpu.set_b1(host_normal(ff, 1, g, 0.1f)); cpu.set_b2(host_normal(d, 1, g, 0.1f));
    cpu.set_ln1_gamma(host_normal(d, 1, g, 0.2f) + 1.0); cpu.set_ln1_beta(host_normal(d, 1, g, 0.1f));
    cpu.set_ln2_gamma(host_normal(d, 1, g, 0.2f) + 1.0); cpu.set_ln2_beta(host_normal(d, 1, g, 0.1f));
    copy_block_weights(cpu, dev);
    char name[96];
    std::snprintf(name, sizeof name, "transformer d%d ff%d S%d B%d h%d%s", d, ff, S, B, heads, causal ? " causal" : "");
    return check(name, {&cpu}, {&dev}, d, S * B, g, 1e-3);
}

int mlp_case(std::mt19937& g) {
    const int nb = 33, d0 = 7, d1 = 19, d2 = 12, d3 = 5;
    Layer<float> c1(d1, d0, nb);   ReluLayer<float> c2(d2, d1, nb); LinearLayer<float> c3(d3, d2, nb);
    Layer<Dev> g1(d1, d0, nb);     ReluLayer<Dev> g2(d2, d1, nb);   LinearLayer<Dev> g3(d3, d2, nb);
    Layer<float>* cl[] = {&c1, &c2, &c3};
    Layer<Dev>* gl[] = {&g1, &g2, &g3};
    const int dims[] = {d0, d1, d2, d3};
    for (int l = 0; l < 3; ++l) {
        cl[l]->W() = host_normal(dims[l + 1], dims[l], g, 1.0f / std::sqrt((float)dims[l]));
        cl[l]->b() = host_normal(dims[l + 1], 1, g, 0.1f);
        gl[l]->W() = Matrix<Dev>(cl[l]->W());
        gl[l]->b() = Matrix<Dev>(cl[l]->b());
    }
    // forward()/jvp() walk the list from the back
    return check("dense tanh -> relu -> linear", {&c3, &c2, &c1}, {&g3, &g2, &g1}, d0, nb, g, 1e-4);
}

int layernorm_case(int dim, int N, std::mt19937& g) {
    LayerNorm<float> c(dim, N);
    LayerNorm<Dev> d(dim, N);
    const Matrix<float> gm = host_normal(dim, 1, g, 0.3f) + 1.0, bt = host_normal(dim, 1, g, 0.2f);
    c.set_gamma(gm); c.set_beta(bt);
    d.set_gamma(Matrix<Dev>(gm)); d.set_beta(Matrix<Dev>(bt));
    const Matrix<float> xh = host_normal(dim, N, g, 1.5f), uh = host_normal(dim, N, g, 1.0f);
    c.forward(xh);
    d.forward(up(xh));
    const double e1 = rel(down(d.jvp(up(uh))), c.jvp(uh));
    // transposed tangent operand
    const Matrix<float> uth = host_normal(N, dim, g, 1.0f);
    const double e2 = rel(down(d.jvp(up(uth).T())), c.jvp(uth.T()));
    const bool ok = e1 <= 1e-4 && e2 <= 1e-4;
    std::printf("%s layernorm jvp dim %d N %d            vs CPU %.2e, transposed tangent %.2e\n", ok ? "ok  " : "FAIL", dim,
                N, e1, e2);
    return ok ? 0 : 1;
}

}  // namespace

int compute() {
    std::mt19937 g(2024);
    int bad = 0;
    bad += layernorm_case(16, 9, g);
    bad += layernorm_case(512, 70, g);
    bad += layernorm_case(1030, 5, g);
    bad += mlp_case(g);
    bad += transformer_case(16, 32, 7, 2, 4, true, g);      // unfused attention path (S not a multiple of 32)
    bad += transformer_case(16, 32, 7, 2, 4, false, g);
    bad += transformer_case(128, 256, 64, 3, 2, true, g);   // fused attention core, d_h 64
    bad += transformer_case(64, 96, 32, 2, 2, true, g);     // d_h 32
    bad += transformer_case(128, 256, 96, 2, 2, false, g);  // S a multiple of 32 but not of 64
    bad += transformer_case(128, 256, 128, 2, 4, true, g);
    std::printf("%s: %d failures\n", bad ? "FAILED" : "PASSED", bad);
    return bad ? 1 : 0;
}
