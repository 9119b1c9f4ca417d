// Transpose-flag and ownership semantics of Matrix<ROCMfloat> against the CPU
// Matrix<float>, in one program written against the Juzhen API.  A ROCm build of
// the reference's own tests/testbasic.cu and tests/testStackOps.cu exercises
// Matrix<float> only (their GPU sections are CUDA-only), and
// tests/testRocmCpuParity.cu never hands a transposed operand to add, hadmd,
// reduce, slice or the stacks, so this program runs every such case once per
// backend from the same template and compares the two runs.
//
// Inputs are multiples of 1/4 of small magnitude: sums, products, quotients
// by powers of two and dot products are then exact in fp32 in any order, so
// everything except the transcendental chains must agree bit for bit; those
// are held to the elementwise tolerance 1e-5.  Result shape, transpose flag
// and (for rvalue overloads) reuse of the operand's buffer are compared too.
//
// Exit status 0 when every check passes (the library owns main(),
// cpp/launcher.cu).  Needs <PROJECT_DIR>/tests/basic.testdata for the golden
// chain of tests/testbasic.cu:11-16.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <string>
#include <vector>

#include "../ml/layer.hpp"

using namespace Juzhen;

namespace {

struct Rec {
    std::string name;
    size_t rows = 0, cols = 0;
    int flag = 0;
    int reused = -1;            // -1: not applicable; else whether the result aliases the rvalue operand
    double tol = 0.0;           // 0: bit-exact
    std::vector<float> v;       // logical content, column-major
};

Matrix<float> down(const Matrix<float>& m) { return m; }
Matrix<float> up(const Matrix<float>& h, float*) { return h; }
Matrix<float> hs(std::vector<MatrixView<float>> v) { return hstack<float>(v); }
Matrix<float> vs(std::vector<MatrixView<float>> v) { return vstack<float>(v); }
// copy(dest, src) exists for the device type only (cpp/hipmatrix.cuh:157); on the CPU it is assignment
void copy_into(Matrix<float>& dst, const Matrix<float>& src) { dst = src; }
#ifdef ROCM_HIP
typedef ROCMfloat Dev;
Matrix<float> down(const Matrix<ROCMfloat>& m) { return m.to_host(); }
Matrix<ROCMfloat> up(const Matrix<float>& h, ROCMfloat*) { return Matrix<ROCMfloat>(h); }
void copy_into(Matrix<ROCMfloat>& dst, const Matrix<ROCMfloat>& src) { copy(dst, src); }
Matrix<ROCMfloat> hs(std::vector<MatrixView<ROCMfloat>> v) { return hstack(v); }
Matrix<ROCMfloat> vs(std::vector<MatrixView<ROCMfloat>> v) { return vstack(v); }
#else
typedef float Dev;   // a CPU-only build compares the CPU path with itself (a check of this program)
#endif

// A deep copy that keeps the flag.  `Matrix<D> X(A.T())` would not be one: T()
// returns a prvalue, so X would be that view itself and alias A's buffer.
template <class D>
Matrix<D> deep(const Matrix<D>& m) {
    return Matrix<D>(m);
}

template <class D>
Rec rec(const std::string& name, const Matrix<D>& m, double tol = 0.0, int reused = -1) {
    Rec r;
    r.name = name;
    r.rows = m.num_row();
    r.cols = m.num_col();
    r.flag = (int)m.get_transpose();
    r.reused = reused;
    r.tol = tol;
    const Matrix<float> h = down(m);
    r.v.resize(r.rows * r.cols);
    for (size_t j = 0; j < r.cols; ++j)
        for (size_t i = 0; i < r.rows; ++i) r.v[j * r.rows + i] = h.elem(i, j);
    return r;
}

Matrix<float> quarters(int r, int c, unsigned seed, bool nonzero = false) {
    std::mt19937 g(seed);
    std::uniform_int_distribution<int> d(-12, 12);
    Matrix<float> m("h", r, c);
    float* p = const_cast<float*>(m.data());
    for (size_t i = 0; i < (size_t)r * c; ++i) {
        int q = d(g);
        if (nonzero) {   // divisors: powers of two, so quotients stay exact
            static const float pw[] = {0.25f, 0.5f, 1.f, 2.f, 4.f, -0.5f, -1.f, -2.f};
            p[i] = pw[(q + 12) % 8];
        } else {
            p[i] = 0.25f * q;
        }
    }
    return m;
}

// One battery of cases for an (r x c) matrix A and a (c x r) matrix B, so that
// B.T() has A's logical shape.
template <class D>
void battery(std::vector<Rec>& out, int r, int c, const std::string& tag) {
    D* const sel = nullptr;
    const Matrix<float> Ah = quarters(r, c, 11 + r), Bh = quarters(c, r, 23 + c), Ph = quarters(c, r, 5, true);
    const Matrix<D> A = up(Ah, sel), B = up(Bh, sel), P = up(Ph, sel);
    auto N = [&](const char* n) { return tag + "." + n; };

    // const add / subtract with mismatched flags: logical index, result flag 0 (cpp/core.hpp:414-431)
    out.push_back(rec(N("A+Bt"), A + B.T()));
    out.push_back(rec(N("A-Bt"), A - B.T()));
    out.push_back(rec(N("Bt+A"), B.T() + A));
    out.push_back(rec(N("At+B"), A.T() + B));
    out.push_back(rec(N("At-B"), A.T() - B));
    out.push_back(rec(N("At+At"), A.T() + A.T()));
    out.push_back(rec(N("add(Bt,2,-.5)"), A.add(B.T(), 2.0f, -0.5f)));
    // rvalue operands of the operators (cpp/operators.hpp:116-171 steals one side)
    out.push_back(rec(N("mv(A)+Bt"), Matrix<D>(A) + B.T()));
    out.push_back(rec(N("Bt-mv(A)"), B.T() - Matrix<D>(A)));
    out.push_back(rec(N("mv(At)+B"), deep(A.T()) + B));
    // in place with mismatched flags keeps the target's own layout (cpp/core.hpp:435-449)
    {
        Matrix<D> X(A);
        X += B.T();
        out.push_back(rec(N("A+=Bt"), X));
        X -= B.T();
        out.push_back(rec(N("A+=Bt-=Bt"), X));
        Matrix<D> Y = deep(A.T());   // carries the flag
        Y += B;
        out.push_back(rec(N("At+=B"), Y));
        Y.add(B, 0.5f, -2.0f);
        out.push_back(rec(N("At.add(B,.5,-2)"), Y));
    }
    // scalar forms keep the source flag (cpp/core.hpp:454,478)
    out.push_back(rec(N("At+1.5"), A.T() + 1.5));
    out.push_back(rec(N("At*0.5"), A.T() * 0.5));
    out.push_back(rec(N("At/4"), A.T() / 4.0));
    out.push_back(rec(N("-At"), -A.T()));
    out.push_back(rec(N("2/Pt"), 2.0 / P.T()));
    out.push_back(rec(N("Pt.eleminv(1)"), P.T().eleminv(1.0)));
    // division = hadmd(A, B.eleminv(1)) (cpp/operators.hpp:270-280)
    out.push_back(rec(N("A/Pt"), A / P.T()));
    out.push_back(rec(N("At/P"), A.T() / P));
    // hadmd, all four overloads, mismatched flags (cpp/matrix.hpp:428-474)
    out.push_back(rec(N("hadmd(A,Bt)"), hadmd(A, B.T())));
    out.push_back(rec(N("hadmd(At,B)"), hadmd(A.T(), B)));
    {
        Matrix<D> X = deep(B.T());
        const void* p = X.data();
        Matrix<D> R = hadmd(A, std::move(X));
        out.push_back(rec(N("hadmd(A,mv(Bt))"), R, 0.0, p == (const void*)R.data()));
    }
    {
        Matrix<D> X(A);
        const void* p = X.data();
        Matrix<D> R = hadmd(std::move(X), B.T());
        out.push_back(rec(N("hadmd(mv(A),Bt)"), R, 0.0, p == (const void*)R.data()));
    }
    {
        Matrix<D> X = deep(A.T()), Y(B);
        const void* py = Y.data();
        Matrix<D> R = hadmd(std::move(X), std::move(Y));
        out.push_back(rec(N("hadmd(mv(At),mv(B))"), R, 0.0, py == (const void*)R.data()));
    }
    // unary maps keep layout and flag; rvalue forms reuse the buffer
    out.push_back(rec(N("square(At)"), square(A.T())));
    out.push_back(rec(N("exp(At)"), exp(A.T()), 1e-5));
    out.push_back(rec(N("tanh(At)"), tanh(A.T()), 1e-5));
    out.push_back(rec(N("d_tanh(At)"), d_tanh(A.T()), 1e-5));
    out.push_back(rec(N("log(square(At)+1)"), log(square(A.T()) + 1.0), 1e-5));
    {
        Matrix<D> X = deep(A.T());
        const void* p = X.data();
        Matrix<D> R = exp(std::move(X));
        out.push_back(rec(N("exp(mv(At))"), R, 1e-5, p == (const void*)R.data()));
    }
    // products with every flag combination (cpp/core.hpp:395-411)
    out.push_back(rec(N("A*B"), A * B));
    out.push_back(rec(N("Bt*At"), B.T() * A.T()));
    out.push_back(rec(N("A*At"), A * A.T()));
    out.push_back(rec(N("At*A"), A.T() * A));
    out.push_back(rec(N("Bt*B"), B.T() * B));
    // sums of a transposed matrix (cpp/matrix.hpp:74-91)
    out.push_back(rec(N("sum(A,0)"), sum(A, 0)));
    out.push_back(rec(N("sum(A,1)"), sum(A, 1)));
    out.push_back(rec(N("sum(At,0)"), sum(A.T(), 0)));
    out.push_back(rec(N("sum(At,1)"), sum(A.T(), 1)));
    out.push_back(rec(N("sum(sum(At,0),1)"), sum(sum(A.T(), 0), 1)));
    // reduce<F> orientation table (cpp/matrix.hpp:202-250), k = 1 and k = 2
    {
        auto sum_f = [] __GPU_CPU__(float* src, float* dst, int n, int) {
            float s = 0.0f;
            for (int i = 0; i < n; ++i) s += src[i];
            dst[0] = s;
        };
        auto stats_f = [] __GPU_CPU__(float* src, float* dst, int n, int) {
            float s = 0.0f, m = src[0];
            for (int i = 0; i < n; ++i) {
                s += src[i];
                m = m > src[i] ? m : src[i];
            }
            dst[0] = s;
            dst[1] = m;
        };
        out.push_back(rec(N("reduce(sum,A,0)"), reduce(sum_f, A, 0, 1)));
        out.push_back(rec(N("reduce(sum,A,1)"), reduce(sum_f, A, 1, 1)));
        out.push_back(rec(N("reduce(sum,At,0)"), reduce(sum_f, A.T(), 0, 1)));
        out.push_back(rec(N("reduce(sum,At,1)"), reduce(sum_f, A.T(), 1, 1)));
        out.push_back(rec(N("reduce(stats,A,0,2)"), reduce(stats_f, A, 0, 2)));
        out.push_back(rec(N("reduce(stats,A,1,2)"), reduce(stats_f, A, 1, 2)));
        out.push_back(rec(N("reduce(stats,At,0,2)"), reduce(stats_f, A.T(), 0, 2)));
        out.push_back(rec(N("reduce(stats,At,1,2)"), reduce(stats_f, A.T(), 1, 2)));
        // the input of a reduce is left as it was
        out.push_back(rec(N("A after reduce"), A));
        // a functor that overwrites its vector (the selection of examples/knn.cu:61-78): when the
        // vectors are the matrix's own columns the caller sees them overwritten, on both backends;
        // along the other dimension the functor works on a private transposed copy
        auto min2_f = [] __GPU_CPU__(float* src, float* dst, int n, int k) {
            for (int j = 0; j < k; ++j) {
                int at = 0;
                for (int i = 1; i < n; ++i)
                    if (src[i] < src[at]) at = i;
                dst[j] = (float)at;
                src[at] = 1e30f;
            }
        };
        Matrix<D> X(A), Y(A);
        out.push_back(rec(N("reduce(min2,X,0,2)"), reduce(min2_f, X, 0, 2)));
        out.push_back(rec(N("X after overwriting reduce"), X));
        out.push_back(rec(N("reduce(min2,Y,1,2)"), reduce(min2_f, Y, 1, 2)));
        out.push_back(rec(N("Y after overwriting reduce"), Y));
    }
    // elemwise<F> keeps layout and flag; rvalue reuses the buffer
    {
        auto ew = [] __GPU_CPU__(float x) { return x * x + 2.0f * x - 0.5f; };
        out.push_back(rec(N("elemwise(At)"), elemwise(ew, A.T())));
        Matrix<D> X = deep(A.T());
        const void* p = X.data();
        Matrix<D> R = elemwise(ew, std::move(X));
        out.push_back(rec(N("elemwise(mv(At))"), R, 0.0, p == (const void*)R.data()));
        out.push_back(rec(N("relu(At)"), relu(deep(A.T()))));
        out.push_back(rec(N("d_relu(At)"), d_relu(deep(A.T()))));
    }
    // slices of a transposed matrix; slice-assign with both flags (cpp/core.hpp:353-373)
    {
        const size_t lr = A.T().num_row(), lc = A.T().num_col();   // c x r
        auto lo = [](size_t n) { return n / 4; };
        auto hi = [](size_t n) { return n - n / 4; };                // hi(n) > lo(n) for n >= 1
        out.push_back(rec(N("At.slice"), A.T().slice(lo(lr), hi(lr), lo(lc), hi(lc))));
        out.push_back(rec(N("At.rows"), A.T().rows(lr / 3, lr)));
        out.push_back(rec(N("At.columns"), A.T().columns(0, (lc + 1) / 2)));
        out.push_back(rec(N("A.slice"), A.slice(lo(r), hi(r), lo(c), hi(c))));
        Matrix<D> X = deep(A.T());                                        // target carries the flag
        X.slice(lo(lr), hi(lr), lo(lc), hi(lc), B.slice(lo(lr), hi(lr), lo(lc), hi(lc)));   // plain source
        out.push_back(rec(N("At.slice=B.slice"), X));
        X.rows(0, 2, A.columns(0, 2).T());                          // transposed source
        out.push_back(rec(N("At.rows=(A.columns).T"), X));
        Matrix<D> Y(A);
        Y.columns(1, 3, B.rows(1, 3).T());
        out.push_back(rec(N("A.columns=(B.rows).T"), Y));
    }
    // stacks with transposed inputs (cpp/matrix.hpp:93-150): result flag 0
    out.push_back(rec(N("vstack{A,Bt}"), vs({A, B.T()})));
    out.push_back(rec(N("vstack{At,B}"), vs({A.T(), B})));
    out.push_back(rec(N("vstack{At,Bt.T}"), vs({A.T(), B.T().T()})));
    out.push_back(rec(N("hstack{A,Bt}"), hs({A, B.T()})));
    out.push_back(rec(N("hstack{At,B,At}"), hs({A.T(), B, A.T()})));
    // softmax of a transposed matrix (ml/layer.hpp:2344-2367)
    out.push_back(rec(N("col_softmax(At)"), col_softmax(A.T()), 1e-4));
    out.push_back(rec(N("row_softmax(At)"), row_softmax(A.T()), 1e-4));
    out.push_back(rec(N("row_softmax(A)"), row_softmax(A), 1e-4));
    // predict_one_hot (ml/util.cuh:258-279): plain result, every entry tied with its column's
    // maximum gets a 1 (the quarter-integer inputs tie often)
    out.push_back(rec(N("predict_one_hot(A)"), predict_one_hot(A)));
    out.push_back(rec(N("predict_one_hot(At)"), predict_one_hot(A.T())));
    // copies keep the flag, T() aliases, to_host carries flag and physical dims
    {
        Matrix<D> X = deep(A.T());
        out.push_back(rec(N("copy-ctor(At)"), X));
        Matrix<D> Y("y", 3, 3);
        Y = A.T();
        out.push_back(rec(N("assign(At)"), Y));
        Matrix<D> Z("z", 3, 3);
        copy_into(Z, A.T());
        out.push_back(rec(N("copy(At)"), Z));
        const Matrix<D> V = A.T();
        out.push_back(rec(N("T() aliases"), V, 0.0, (const void*)V.data() == (const void*)A.data()));
        out.push_back(rec(N("At.T"), A.T().T()));
    }
}

// tests/testbasic.cu:11-16 on Matrix<D>, compared with tests/basic.testdata
template <class D>
int golden_chain(const char* what) {
    D* const sel = nullptr;
    const Matrix<float> Ah("A", {{1, 2, 3}, {3, 4, 5}}), Bh("B", {{6, 7, 8}, {9, 10, 11}});
    const Matrix<D> A = up(Ah, sel), B = up(Bh, sel);
    auto C = log(exp(-A / B) + exp(hadmd(B, A))) - (A.T() * B).rows(0, 2);
    const Matrix<float> bench = read<float>(std::string(PROJECT_DIR) + "/tests/basic.testdata");
    const float err = (down(C) - bench).norm();
    std::printf("%s golden chain: |C - basic.testdata| = %.3g\n", what, err);
    return err < 1e-5f ? 0 : 1;
}

// the ten shape-mismatch exceptions of tests/testbasic.cu:114-249 and the stack /
// slice error paths of tests/testStackOps.cu:146-198 on Matrix<D>
template <class D>
int exceptions(const char* what) {
    const Matrix<D> A = Matrix<D>::ones(3, 4), B = Matrix<D>::ones(3, 3);
    int caught = 0, wanted = 0;
    auto expect = [&](const char* name, std::function<void()> f, bool range = false) {
        ++wanted;
        try {
            f();
            std::printf("%s %s: no exception\n", what, name);
        } catch (const std::invalid_argument&) {
            caught += range ? 0 : 1;
        } catch (const std::out_of_range&) {
            caught += range ? 1 : 0;
        }
    };
    expect("A+B", [&] { auto t = A + B; });
    expect("A-B", [&] { auto t = A - B; });
    expect("A*B", [&] { auto t = A * B; });
    expect("A/B", [&] { auto t = A / B; });
    expect("hadmd(A,B)", [&] { auto t = hadmd(A, B); });
    expect("A+Bt", [&] { auto t = A + B.T(); });
    expect("A-Bt", [&] { auto t = A - B.T(); });
    expect("A*Bt", [&] { auto t = A * B.T(); });
    expect("A/Bt", [&] { auto t = A / B.T(); });
    expect("hadmd(A,Bt)", [&] { auto t = hadmd(A, B.T()); });
    expect("A+=At", [&] { Matrix<D> X(A); X += A.T(); });
    expect("hstack rows", [&] { auto t = hs({Matrix<D>::ones(2, 2), Matrix<D>::ones(3, 1)}); });
    expect("vstack cols", [&] { auto t = vs({Matrix<D>::ones(2, 2), Matrix<D>::ones(1, 3)}); });
    expect("hstack empty", [&] { auto t = hs(std::vector<MatrixView<D>>{}); });
    expect("vstack empty", [&] { auto t = vs(std::vector<MatrixView<D>>{}); });
    if (!std::is_same<D, float>::value) {  // the CPU slice checks neither (cpp/hipmatrix.cpp:269-271,296-304 add both)
        expect("slice assign shape", [&] { Matrix<D> X(A); X.slice(0, 2, 0, 2, B); });
        expect("slice range", [&] { auto t = A.slice(0, 5, 0, 2); }, true);
    }
    std::printf("%s exceptions: %d of %d\n", what, caught, wanted);
    return caught == wanted ? 0 : 1;
}

// write/read of the .matrix layout (three ints numrow, numcol, transpose, then the
// physical payload; cpp/core.hpp:484-525) through Matrix<D>: the file a device
// matrix writes must be byte-identical to the CPU writer's, for both transpose
// flags, and read back into a device matrix must give the same matrix.
template <class D>
int io_roundtrip(const char* what) {
    D* const sel = nullptr;
    int bad = 0;
    const std::string dir = std::string(PROJECT_DIR) + "/res/";
    for (int flag = 0; flag < 2; ++flag) {
        const Matrix<float> base = quarters(7, 5, 77 + flag);
        const Matrix<float> Mh = flag ? deep(base.T()) : base;
        const Matrix<D> Md = up(Mh, sel);
        const std::string f_cpu = dir + "io_cpu.matrix", f_dev = dir + "io_dev.matrix";
        FILE* fp = std::fopen(f_cpu.c_str(), "wb");
        if (!fp) { std::printf("%s io: cannot write %s\n", what, f_cpu.c_str()); return 1; }
        write(fp, Mh);
        std::fclose(fp);
        fp = std::fopen(f_dev.c_str(), "wb");
        write(fp, Md);
        std::fclose(fp);
        auto slurp = [](const std::string& p) {
            std::vector<unsigned char> b;
            if (FILE* f = std::fopen(p.c_str(), "rb")) {
                unsigned char buf[4096];
                size_t n;
                while ((n = std::fread(buf, 1, sizeof buf, f)) > 0) b.insert(b.end(), buf, buf + n);
                std::fclose(f);
            }
            return b;
        };
        const auto a = slurp(f_cpu), b = slurp(f_dev);
        int hdr[3] = {0, 0, 0};
        if (a.size() >= 12) std::memcpy(hdr, a.data(), 12);
        const bool header_ok = a.size() == 12 + 35 * sizeof(float) && hdr[0] == 7 && hdr[1] == 5 &&
                               hdr[2] == flag;   // physical dims travel, the flag beside them
        if (!header_ok || a != b) {
            std::printf("FAIL %s io flag %d: files differ or header wrong (%zu vs %zu bytes, header %d %d %d)\n", what,
                        flag, a.size(), b.size(), hdr[0], hdr[1], hdr[2]);
            ++bad;
        }
        Matrix<D> R("r", 2, 2);
        fp = std::fopen(f_dev.c_str(), "rb");
        read(fp, R);
        std::fclose(fp);
        const Rec want = rec("io", Mh), got = rec("io", R);
        if (want.rows != got.rows || want.cols != got.cols || want.flag != got.flag || want.v != got.v) {
            std::printf("FAIL %s io flag %d: read back %zux%zu flag %d\n", what, flag, got.rows, got.cols, got.flag);
            ++bad;
        }
    }
    std::printf("%s .matrix round trip: %d failures\n", what, bad);
    return bad;
}

// Uploads must not disturb work in flight and must deliver the host values as
// they were at the call: the converting constructor copies through page-locked
// staging buffers and returns before the device has run the copy.
template <class D>
int uploads_in_flight(const char* what) {
    D* const sel = nullptr;
    int bad = 0;
    const Matrix<float> Wh = quarters(256, 256, 3);
    const Matrix<D> W = up(Wh, sel);
    Matrix<D> acc = W * W;                               // work in flight while batches are uploaded
    std::vector<Matrix<D>> kept;
    std::vector<Matrix<float>> want;
    Matrix<float> batch = quarters(300, 41, 9);
    for (int i = 0; i < 12; ++i) {
        float* p = const_cast<float*>(batch.data());
        for (int j = 0; j < 300 * 41; ++j) p[j] += 0.25f;   // the host buffer is reused right after each upload
        kept.push_back(up(batch, sel));
        want.push_back(batch);
        acc = acc * W * (1.0 / 4096.0);
    }
    for (size_t i = 0; i < kept.size(); ++i)
        if (rec("u", kept[i]).v != rec("u", want[i]).v) {
            std::printf("FAIL %s upload %zu differs from the host values at the call\n", what, i);
            ++bad;
        }
    // one larger than a staging buffer is expected to hold
    const Matrix<float> big = quarters(4096, 5000, 5);
    if (rec("u", up(big, sel)).v != rec("u", big).v) {
        std::printf("FAIL %s large upload\n", what);
        ++bad;
    }
    std::printf("%s uploads beside work in flight: %d failures\n", what, bad);
    return bad;
}

int compare(const std::vector<Rec>& cpu, const std::vector<Rec>& gpu) {
    int bad = 0;
    if (cpu.size() != gpu.size()) {
        std::printf("FAIL record counts differ: %zu vs %zu\n", cpu.size(), gpu.size());
        return 1;
    }
    for (size_t i = 0; i < cpu.size(); ++i) {
        const Rec &a = cpu[i], &b = gpu[i];
        std::string why;
        if (a.rows != b.rows || a.cols != b.cols) why = "shape";
        else if (a.flag != b.flag) why = "transpose flag";
        else if (a.reused != b.reused) why = "buffer reuse";
        else if (a.reused == 0) why = "rvalue operand not reused";
        else {
            double worst = 0.0, scale = 0.0;
            for (size_t k = 0; k < a.v.size(); ++k) scale = std::max(scale, (double)std::fabs(a.v[k]));
            for (size_t k = 0; k < a.v.size(); ++k) {
                if (a.tol == 0.0) {
                    if (std::memcmp(&a.v[k], &b.v[k], sizeof(float)) != 0 && !(a.v[k] == 0.0f && b.v[k] == 0.0f))
                        worst = std::max(worst, std::fabs((double)a.v[k] - b.v[k]) + 1e-30);
                } else {
                    worst = std::max(worst, std::fabs((double)a.v[k] - b.v[k]) / std::max(std::fabs((double)a.v[k]), 1e-3 * scale + 1e-30));
                }
            }
            if (worst > a.tol) why = "values (worst " + std::to_string(worst) + ")";
        }
        if (!why.empty()) {
            std::printf("FAIL %-32s %s: cpu %zux%zu flag %d reused %d | rocm %zux%zu flag %d reused %d\n", a.name.c_str(),
                        why.c_str(), a.rows, a.cols, a.flag, a.reused, b.rows, b.cols, b.flag, b.reused);
            ++bad;
        }
    }
    return bad;
}

}  // namespace

int compute() {
    int bad = 0;
    const int shapes[][2] = {{5, 7}, {37, 70}, {128, 64}, {130, 257}, {1, 9}, {300, 4}};
    size_t checks = 0;
    for (const auto& s : shapes) {
        std::vector<Rec> cpu, gpu;
        const std::string tag = std::to_string(s[0]) + "x" + std::to_string(s[1]);
        battery<float>(cpu, s[0], s[1], tag);
        battery<Dev>(gpu, s[0], s[1], tag);
        const int b = compare(cpu, gpu);
        std::printf("shape %s: %zu cases, %d mismatches\n", tag.c_str(), cpu.size(), b);
        checks += cpu.size();
        bad += b;
    }
    bad += golden_chain<float>("cpu");
    bad += golden_chain<Dev>("rocm");
    bad += io_roundtrip<Dev>("rocm");
    bad += uploads_in_flight<Dev>("rocm");
    bad += exceptions<float>("cpu");
    bad += exceptions<Dev>("rocm");
    std::printf("%s: %zu cases, %d failures\n", bad ? "FAILED" : "PASSED", checks, bad);
    return bad ? 1 : 0;
}
