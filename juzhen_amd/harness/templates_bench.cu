// Timing of the two user-functor templates of Matrix<ROCMfloat>, elemwise<F>
// and reduce<F> (cpp/hipmatrix.cuh:164-250 in the reference), which launch from
// the including translation unit and therefore cannot be measured through the
// C ABI.  HIP events on the library's stream, 3 warm-ups and the median of 20
// samples (tests/benchmarkCoreOps.cu:35-54).  Prints one Markdown table row per
// case in the format of the per-entry-point report.
#include <algorithm>
#include <cstdio>
#include <vector>

#include "../ml/layer.hpp"

using namespace Juzhen;
typedef Matrix<ROCMfloat> MD;

namespace {
template <class F>
double median_us(F&& fn) {
    hipStream_t s = static_cast<hipStream_t>(jzhip_get_stream());
    hipEvent_t a, b;
    hipEventCreate(&a);
    hipEventCreate(&b);
    for (int i = 0; i < 3; ++i) fn();
    std::vector<double> t;
    for (int i = 0; i < 20; ++i) {
        hipEventRecord(a, s);
        fn();
        hipEventRecord(b, s);
        hipEventSynchronize(b);
        float ms = 0;
        hipEventElapsedTime(&ms, a, b);
        t.push_back(ms * 1e3);
    }
    std::sort(t.begin(), t.end());
    hipEventDestroy(a);
    hipEventDestroy(b);
    return t[t.size() / 2];
}
void row(const char* what, const char* shape, double us, double bytes) {
    const double gbs = bytes / us * 1e-3;
    std::printf("| template | %s | %s | %.1f | | %.2f MB | %.0f GB/s | hbm | %.2f |\n", what, shape, us, bytes / 1e6, gbs,
                gbs / 8000.0);
}
}  // namespace

int compute() {
    auto relu_f = [] __GPU_CPU__(float x) { return x > 0.0 ? x : 0.0; };   // ml/util.cuh:76 (double result)
    for (size_t lg : {24, 26, 28}) {
        const size_t n = size_t(1) << lg;
        MD A = MD::ones(n / 4096, 4096);
        char shape[64];
        std::snprintf(shape, sizeof shape, "2^%zu", lg);
        row("elemwise<F> (const&, relu functor)", shape, median_us([&] { MD t = elemwise(relu_f, A); }), 8.0 * n);
        row("elemwise<F> (&&, in place)", shape, median_us([&] { A = elemwise(relu_f, std::move(A)); }), 8.0 * n);
    }
    auto max_f = [] __GPU_CPU__(float* v, float* out, int len, int) {   // ml/layer.hpp:2346-2351
        float m = -1e30f;
        for (int i = 0; i < len; ++i) m = m > v[i] ? m : v[i];
        out[0] = m;
    };
    auto sel_f = [] __GPU_CPU__(float* v, float* out, int len, int k) {  // overwrites its vector (examples/knn.cu:61-78)
        for (int j = 0; j < k; ++j) {
            int at = 0;
            for (int i = 1; i < len; ++i)
                if (v[i] < v[at]) at = i;
            out[j] = (float)at;
            v[at] = 1e30f;
        }
    };
    const int shapes[][2] = {{10, 1 << 20}, {256, 1 << 18}, {1024, 1 << 16}, {4096, 1 << 14}};
    for (const auto& s : shapes) {
        MD A = MD::randn(s[0], s[1]);
        char shape[64];
        std::snprintf(shape, sizeof shape, "%dx%d, dim 0", s[0], s[1]);
        const double n = (double)s[0] * s[1];
        row("reduce<F> (column max)", shape, median_us([&] { MD t = reduce(max_f, A, 0, 1); }), 4.0 * (n + s[1]));
        row("reduce<F> (selection of 2, overwrites its input)", shape, median_us([&] { MD t = reduce(sel_f, A, 0, 2); }),
            4.0 * (2 * n + 2 * s[1]));
    }
    return 0;
}
