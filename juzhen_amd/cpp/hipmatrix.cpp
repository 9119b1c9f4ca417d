// Matrix<ROCMfloat> on MI355X: every member is a thin call into the C ABI of
// libjzhip.so (include/jzhip.h).  Replaces the reference's cpp/hipmatrix.cpp.
//
// Semantics follow the CPU Matrix<float> (cpp/core.hpp, cpp/matrix.hpp), which
// is the parity oracle — in particular binary ops index *logically*, so
// operands with different transpose flags combine correctly, const forms of
// add/hadmd return a non-transposed result while unary forms keep the source's
// flag, and dot() checks the inner dimension.
#include "hipmatrix.cuh"

#include <algorithm>
#include <cstring>

#include "jzhip.h"

#ifdef ROCM_HIP

namespace {

[[noreturn]] void die(const char* what, int rc) {
    // the reference's convention for device failures: log and exit(1)
    // (cpp/hipmatrix.cpp:147-150, ERROR_OUT cpp/helper.hpp:135)
    std::cerr << "juzhen rocm: " << what << " failed with code " << rc << " (" << jzhip_error_string(rc)
              << ")" << std::endl;
    LOG_ERROR("{} failed with code {}", what, rc);
    ERROR_OUT;
}

inline void ok(int rc, const char* what) {
    if (rc != 0) die(what, rc);
}

inline int as_int(size_t v) { return static_cast<int>(v); }

void pool_release(ROCMfloat* p) { Memory<ROCMfloat>::free(p); }

// Host -> device uploads.  The reference's converting constructor is a blocking
// copy from pageable memory (cpp/hipmatrix.cpp:60-63): it waits for everything
// in flight, so a training loop that uploads a batch per step
// (ml/dataloader.hpp:88-113, examples/demo_transformer.cu:378-380) drains the
// device once per step.  Here the host data is copied into one of two
// page-locked staging buffers and an asynchronous copy is enqueued behind the
// work in flight; the call returns once the staging buffer holds the data, so
// the caller may reuse or free its buffer at once, as with the blocking copy.
// A staging buffer is reused only after the event behind its last copy has
// passed.  Uploads beyond the staging cap take the blocking copy.
struct Staging {
    void* buf = nullptr;
    size_t cap = 0;
    void* event = nullptr;
    bool busy = false;
};
constexpr size_t kStagingCap = size_t(64) << 20;
Staging g_staging[2];
int g_staging_next = 0;

void upload(float* dst, const float* src, size_t count) {
    const size_t bytes = count * sizeof(float);
    if (bytes == 0) return;
    if (bytes > kStagingCap) {
        ok(jzhip_memcpy_h2d(dst, src, count), "upload");
        return;
    }
    Staging& st = g_staging[g_staging_next];
    g_staging_next ^= 1;
    if (st.busy) {
        ok(jzhip_event_synchronize(st.event), "upload (staging wait)");
        st.busy = false;
    }
    if (st.cap < bytes) {
        if (st.buf) ok(jzhip_host_free(st.buf), "upload (staging free)");
        st.buf = nullptr;
        st.cap = (bytes + (size_t(1) << 20) - 1) >> 20 << 20;
        ok(jzhip_host_alloc(&st.buf, st.cap), "upload (staging alloc)");
    }
    if (!st.event) ok(jzhip_event_create(&st.event), "upload (event)");
    std::memcpy(st.buf, src, bytes);
    ok(jzhip_memcpy_h2d_async(dst, st.buf, bytes), "upload");
    ok(jzhip_event_record(st.event), "upload (event record)");
    st.busy = true;
}

}  // namespace

using MR = Matrix<ROCMfloat>;

// ── construction ─────────────────────────────────────────────────────────────

MR::Matrix(const char* name, size_t numrow, size_t numcol, int trans,
           std::shared_ptr<ROCMfloat[]> elements)
    : numcol(numcol), numrow(numrow), transpose(trans != 0), name(name), elements(std::move(elements)) {}

// Buffers created while a step is being recorded (jzhip_graph_begin) are written by every
// replay of the graph, so they must not go back to the pool while the graph lives: each gets
// one more owner here, which RocmStepGraph takes over when the recording ends.
static std::vector<std::shared_ptr<ROCMfloat[]>>& recording_pins() {
    static std::vector<std::shared_ptr<ROCMfloat[]>> pins;
    return pins;
}
std::vector<std::shared_ptr<ROCMfloat[]>> JzRocmFused::take_recording_pins() {
    std::vector<std::shared_ptr<ROCMfloat[]>> out;
    out.swap(recording_pins());
    return out;
}

MR::Matrix(const char* name, size_t numrow, size_t numcol, int trans)
    : numcol(numcol), numrow(numrow), transpose(trans != 0), name(name) {
    elements.reset(Memory<ROCMfloat>::allocate(numrow * numcol), pool_release);
    if (jzhip_graph_recording()) recording_pins().push_back(elements);
}

MR::Matrix(const Matrix<float>& M)
    : MR(M.get_name().c_str(), M.numrow, M.numcol, M.transpose) {
    // physical dims and the flag travel unchanged (cpp/hipmatrix.cpp:60-63)
    upload(dev(), M.data(), count());
}

MR::Matrix(const MR& M) : MR(M.name.c_str(), M.numrow, M.numcol, M.transpose) {
    ok(jzhip_copy(dev(), M.dev(), count()), "copy");
}

MR::Matrix(MR&& M) noexcept
    : numcol(M.numcol), numrow(M.numrow), transpose(M.transpose), name(M.name), elements(std::move(M.elements)) {
    M.elements = nullptr;
}

MR& MR::operator=(const MR& M) {
    if (this == &M) return *this;
    if (!elements || count() != M.count() || elements.use_count() != 1) {
        elements.reset(Memory<ROCMfloat>::allocate(M.count()), pool_release);
    }
    name = M.name;
    numrow = M.numrow;
    numcol = M.numcol;
    transpose = M.transpose;
    ok(jzhip_copy(dev(), M.dev(), count()), "copy");
    return *this;
}

MR& MR::operator=(MR&& M) noexcept {
    if (this == &M) return *this;
    name = M.name;
    numrow = M.numrow;
    numcol = M.numcol;
    transpose = M.transpose;
    elements = std::move(M.elements);
    M.elements = nullptr;
    return *this;
}

// ── fill / factories ─────────────────────────────────────────────────────────

void MR::ones() { ok(jzhip_fill(dev(), count(), 1.0f), "fill"); }
void MR::zeros() { ok(jzhip_fill(dev(), count(), 0.0f), "fill"); }

MR MR::ones(size_t m, size_t n) {
    MR r("ones", m, n);
    r.ones();
    return r;
}
MR MR::zeros(size_t m, size_t n) {
    MR r("zeros", m, n);
    r.zeros();
    return r;
}
MR MR::randn(size_t m, size_t n) {
    MR r("randn", m, n);
    ok(jzhip_rand_normal(r.dev(), m * n, 0.0f, 1.0f, 0), "rand_normal");
    return r;
}
MR MR::rand(size_t m, size_t n) {
    MR r("rand", m, n);
    ok(jzhip_rand_uniform(r.dev(), m * n, 0), "rand_uniform");
    return r;
}

// ── products and sums ────────────────────────────────────────────────────────

MR MR::dot(const MR& B) const {
    if (num_col() != B.num_row()) {
        throw std::invalid_argument("Matrix dimensions are not compatible");  // cpp/core.hpp:397-399
    }
    const size_t m = num_row(), n = B.num_col(), k = num_col();
    MR C("dot", m, n);
    if (m == 0 || n == 0) return C;
    if (k == 0) {
        C.zeros();
        return C;
    }
    ok(jzhip_gemm(dev(), B.dev(), C.dev(), as_int(m), as_int(n), as_int(k), transpose, B.transpose,
                  as_int(numrow), as_int(B.numrow), as_int(m), 1.0f, 0.0f),
       "gemm");
    return C;
}

MR MR::add(const MR& B, float s1, float s2) const {
    if (num_col() != B.num_col() || num_row() != B.num_row()) {
        throw std::invalid_argument("Matrix dimensions are not compatible");
    }
    // result is a fresh non-transposed rows x cols matrix (cpp/core.hpp:420)
    MR C("add", num_row(), num_col(), 0);
    ok(jzhip_axpby2d(C.dev(), as_int(C.numrow), 0, dev(), as_int(numrow), transpose, B.dev(),
                     as_int(B.numrow), B.transpose, as_int(num_row()), as_int(num_col()), s1, s2),
       "axpby2d");
    return C;
}

void MR::add(const MR& B, float s1, float s2) {
    if (num_col() != B.num_col() || num_row() != B.num_row()) {
        throw std::invalid_argument("Matrix dimensions are not compatible");
    }
    // in place: this keeps its own layout (cpp/core.hpp:435-449)
    ok(jzhip_axpby2d(dev(), as_int(numrow), transpose, dev(), as_int(numrow), transpose, B.dev(),
                     as_int(B.numrow), B.transpose, as_int(num_row()), as_int(num_col()), s1, s2),
       "axpby2d");
}

MR MR::add(float a, float s1) const {
    MR C("add", numrow, numcol, transpose);  // keeps the source flag (cpp/core.hpp:454)
    ok(jzhip_affine(C.dev(), dev(), count(), s1, a), "affine");
    return C;
}

void MR::add(float a, float s1) { ok(jzhip_affine_inplace(dev(), count(), s1, a), "affine"); }

void MR::scale(float s1) { add(0.0f, s1); }

void MR::eleminv(double l) { ok(jzhip_eleminv(dev(), dev(), count(), l), "eleminv"); }

MR MR::eleminv(double l) const {
    MR C((name + "reci").c_str(), numrow, numcol, transpose);
    ok(jzhip_eleminv(C.dev(), dev(), count(), l), "eleminv");
    return C;
}

float MR::norm() const {
    MR acc("norm", 1, 1);
    ok(jzhip_nrm2(acc.dev(), dev(), count()), "nrm2");
    float v = 0.0f;
    ok(jzhip_memcpy_d2h(&v, acc.dev(), 1), "download");
    return v;
}

const MR MR::T() const { return MR((name + "_T").c_str(), numrow, numcol, !transpose, elements); }

Matrix<float> MR::to_host() const {
    Matrix<float> H(name.c_str(), numrow, numcol);
    H.transpose = transpose;
    ok(jzhip_memcpy_d2h(H.elements.get(), dev(), count()), "download");
    return H;
}

MR sum(const MR& M, int dim) {
    // dim 0 sums over logical rows (result 1 x cols, stored as a transposed
    // cols x 1 column); dim 1 over logical columns (cpp/matrix.hpp:74-91)
    const bool over_phys_rows = (dim == 0) != M.transpose;  // reduce along the contiguous dimension
    const size_t len = over_phys_rows ? M.numcol : M.numrow;
    MR out("sumM", len, 1, 0);
    if (M.numrow == 0 || M.numcol == 0) {
        out.zeros();
    } else if (over_phys_rows) {
        ok(jzhip_sum_cols(out.dev(), M.dev(), as_int(M.numrow), as_int(M.numcol), as_int(M.numrow)), "sum_cols");
    } else {
        ok(jzhip_sum_rows(out.dev(), M.dev(), as_int(M.numrow), as_int(M.numcol), as_int(M.numrow)), "sum_rows");
    }
    if (dim == 0) out.transpose = 1;
    return out;
}

// ── slices and stacks ────────────────────────────────────────────────────────

MR MR::slice(size_t rstart, size_t rend, size_t cstart, size_t cend) const {
    if (rstart > rend || cstart > cend || rend > num_row() || cend > num_col()) {
        throw std::out_of_range("slice indices out of range");
    }
    const size_t r = rend - rstart, c = cend - cstart;
    MR out("submatrix", r, c, 0);
    ok(jzhip_slice_extract(out.dev(), r, dev(), numrow, transpose, rstart, cstart, r, c), "slice_extract");
    return out;
}

void MR::slice(size_t rstart, size_t rend, size_t cstart, size_t cend, const MR& M) {
    if (rstart > rend || cstart > cend || rend > num_row() || cend > num_col()) {
        throw std::out_of_range("slice indices out of range");
    }
    const size_t r = rend - rstart, c = cend - cstart;
    if (M.num_row() != r || M.num_col() != c) {
        throw std::invalid_argument("slice assignment matrix dimensions do not match target range");
    }
    ok(jzhip_slice_assign(dev(), numrow, transpose, rstart, cstart, M.dev(), M.numrow, M.transpose, r, c),
       "slice_assign");
}

MR MR::rows(size_t rstart, size_t rend) const { return slice(rstart, rend, 0, num_col()); }
void MR::rows(size_t rstart, size_t rend, const MR& M) { slice(rstart, rend, 0, num_col(), M); }
MR MR::columns(size_t cstart, size_t cend) const { return slice(0, num_row(), cstart, cend); }
void MR::columns(size_t cstart, size_t cend, const MR& M) { slice(0, num_row(), cstart, cend, M); }

namespace {
// physical row/column counts behind a view (a view only reports logical ones)
inline size_t view_numrow(const MatrixView<ROCMfloat>& v) { return v.get_transpose() ? v.num_col() : v.num_row(); }
inline size_t view_numcol(const MatrixView<ROCMfloat>& v) { return v.get_transpose() ? v.num_row() : v.num_col(); }

void drop_empty(std::vector<MatrixView<ROCMfloat>>& v) {
    v.erase(std::remove_if(v.begin(), v.end(),
                           [](const MatrixView<ROCMfloat>& m) { return m.num_row() == 0 || m.num_col() == 0; }),
            v.end());
}
}  // namespace

MR hstack(std::vector<MatrixView<ROCMfloat>> matrices) {
    drop_empty(matrices);
    if (matrices.empty()) throw std::invalid_argument("hstack: input list is empty or contains only empty matrices");
    const size_t nrow = matrices[0].num_row();
    size_t ncol = 0;
    for (const auto& m : matrices) {
        if (m.num_row() != nrow) throw std::invalid_argument("hstack: all matrices must have the same row count");
        ncol += m.num_col();
    }
    MR result("hstack", nrow, ncol, 0);
    size_t at = 0;
    for (const auto& m : matrices) {
        ok(jzhip_stack_copy_cols(result.dev(), nrow, at, reinterpret_cast<const float*>(m.data()), view_numrow(m),
                                 view_numcol(m), m.get_transpose() != 0),
           "stack_copy_cols");
        at += m.num_col();
    }
    return result;
}

MR vstack(std::vector<MatrixView<ROCMfloat>> matrices) {
    drop_empty(matrices);
    if (matrices.empty()) throw std::invalid_argument("vstack: input list is empty or contains only empty matrices");
    const size_t ncol = matrices[0].num_col();
    size_t nrow = 0;
    for (const auto& m : matrices) {
        if (m.num_col() != ncol) throw std::invalid_argument("vstack: all matrices must have the same column count");
        nrow += m.num_row();
    }
    MR result("vstack", nrow, ncol, 0);
    size_t at = 0;
    for (const auto& m : matrices) {
        ok(jzhip_stack_copy_rows(result.dev(), nrow, at, reinterpret_cast<const float*>(m.data()), view_numrow(m),
                                 view_numcol(m), m.get_transpose() != 0),
           "stack_copy_rows");
        at += m.num_row();
    }
    return result;
}

// ── unary maps: keep layout and flag; rvalue forms work in place ─────────────

#define JZ_UNARY(NAME, CALL)                                              \
    MR NAME(const MR& M) {                                                \
        MR out(#NAME, M.numrow, M.numcol, M.transpose);                   \
        ok(CALL(out.dev(), M.dev(), M.count()), #NAME);                   \
        return out;                                                       \
    }
#define JZ_UNARY_RVALUE(NAME, CALL)                                       \
    MR NAME(MR&& M) {                                                     \
        ok(CALL(M.dev(), M.dev(), M.count()), #NAME);                     \
        return std::move(M);                                              \
    }

JZ_UNARY(exp, jzhip_exp)
JZ_UNARY_RVALUE(exp, jzhip_exp)
JZ_UNARY(log, jzhip_log)
JZ_UNARY(tanh, jzhip_tanh)
JZ_UNARY_RVALUE(tanh, jzhip_tanh)
JZ_UNARY(d_tanh, jzhip_dtanh)
JZ_UNARY_RVALUE(d_tanh, jzhip_dtanh)
JZ_UNARY(square, jzhip_square)
JZ_UNARY_RVALUE(square, jzhip_square)

MR relu(MR&& M) {
    ok(jzhip_relu(JzRocmFused::ptr(M), JzRocmFused::ptr(M), M.num_row() * M.num_col()), "relu");
    return std::move(M);
}
MR d_relu(MR&& M) {
    ok(jzhip_drelu(JzRocmFused::ptr(M), JzRocmFused::ptr(M), M.num_row() * M.num_col()), "drelu");
    return std::move(M);
}

MR& fill(MR& M, double a) {
    ok(jzhip_fill(M.dev(), M.count(), static_cast<float>(a)), "fill");
    return M;
}

void copy(MR& dest, const MR& src) {
    if (!dest.elements || dest.count() != src.count() || dest.elements.use_count() != 1) {
        dest.elements.reset(Memory<ROCMfloat>::allocate(src.count()), pool_release);
    }
    dest.numrow = src.numrow;
    dest.numcol = src.numcol;
    dest.transpose = src.transpose;
    ok(jzhip_copy(dest.dev(), src.dev(), src.count()), "copy");
}

// ── Hadamard products (cpp/matrix.hpp:428-474) ───────────────────────────────

namespace {
void check_same_shape(const MR& a, const MR& b) {
    if (a.num_row() != b.num_row() || a.num_col() != b.num_col()) {
        throw std::invalid_argument("Matrix dimensions are not compatible");
    }
}
}  // namespace

MR hadmd(const MR& M1, const MR& M2) {
    check_same_shape(M1, M2);
    MR out("hadmd", M1.num_row(), M1.num_col(), 0);
    ok(jzhip_hadamard2d(out.dev(), as_int(out.numrow), 0, M1.dev(), as_int(M1.numrow), M1.transpose, M2.dev(),
                        as_int(M2.numrow), M2.transpose, as_int(M1.num_row()), as_int(M1.num_col())),
       "hadamard2d");
    return out;
}

MR hadmd(const MR& M1, MR&& M2) {
    check_same_shape(M1, M2);
    ok(jzhip_hadamard2d(M2.dev(), as_int(M2.numrow), M2.transpose, M2.dev(), as_int(M2.numrow), M2.transpose,
                        M1.dev(), as_int(M1.numrow), M1.transpose, as_int(M1.num_row()), as_int(M1.num_col())),
       "hadamard2d");
    return std::move(M2);
}

MR hadmd(MR&& M1, const MR& M2) {
    check_same_shape(M1, M2);
    ok(jzhip_hadamard2d(M1.dev(), as_int(M1.numrow), M1.transpose, M1.dev(), as_int(M1.numrow), M1.transpose,
                        M2.dev(), as_int(M2.numrow), M2.transpose, as_int(M1.num_row()), as_int(M1.num_col())),
       "hadamard2d");
    return std::move(M1);
}

MR hadmd(MR&& M1, MR&& M2) { return hadmd(M1, std::move(M2)); }

// ── fused softmax / argmax helpers used by the layer templates ──────────────

MR JzRocmFused::materialise(const MR& M) {
    MR out("materialised", M.num_row(), M.num_col(), 0);
    ok(jzhip_copy2d(out.dev(), as_int(out.numrow), 0, 0, 0, M.dev(), as_int(M.numrow), M.transpose, 0, 0,
                    M.num_row(), M.num_col()),
       "copy2d");
    return out;
}

namespace Juzhen {

// softmax along logical columns; result is a plain rows x cols matrix
MR col_softmax(const MR& M) {
    MR out = JzRocmFused::make("softmax", M.num_row(), M.num_col(), 0);
    if (M.num_row() == 0 || M.num_col() == 0) return out;
    const int pr = as_int(JzRocmFused::phys_rows(M)), pc = as_int(JzRocmFused::phys_cols(M));
    if (!M.get_transpose()) {
        ok(jzhip_softmax_cols(JzRocmFused::ptr(out), JzRocmFused::ptr(M), pr, pc, pr), "softmax_cols");
        return out;
    }
    // logical columns are physical rows: row-softmax the buffer, then return the
    // logical (transposed) content as a plain matrix
    MR tmp = JzRocmFused::like("softmax_t", M);
    ok(jzhip_softmax_rows(JzRocmFused::ptr(tmp), JzRocmFused::ptr(M), pr, pc, pr), "softmax_rows");
    return JzRocmFused::materialise(tmp);
}

}  // namespace Juzhen

// 1 where an entry is within 1e-5 of its logical column's maximum, else 0; a plain
// rows x cols matrix, as the generic chain of ml/util.cuh:258-279 returns
MR predict_one_hot(const MR& input) {
    MR out = JzRocmFused::make("one_hot_pred", input.num_row(), input.num_col(), 0);
    if (input.num_row() == 0 || input.num_col() == 0) return out;
    if (!input.get_transpose()) {
        const int pr = as_int(JzRocmFused::phys_rows(input)), pc = as_int(JzRocmFused::phys_cols(input));
        ok(jzhip_predict_one_hot(JzRocmFused::ptr(out), JzRocmFused::ptr(input), pr, pc, pr), "predict_one_hot");
        return out;
    }
    // logical columns are strided in a transposed view: lay them out contiguously first
    MR plain = JzRocmFused::materialise(input);
    ok(jzhip_predict_one_hot(JzRocmFused::ptr(out), JzRocmFused::ptr(plain), as_int(input.num_row()),
                             as_int(input.num_col()), as_int(input.num_row())),
       "predict_one_hot");
    return out;
}

namespace Juzhen {

// row_softmax(M) = col_softmax(M.T()).T()  (ml/layer.hpp:2364-2367): the result
// is always a transposed view of a plain (cols x rows) buffer, like the CPU's.
MR row_softmax(const MR& M) {
    if (M.num_row() == 0 || M.num_col() == 0) return MR(JzRocmFused::make("softmax", M.num_col(), M.num_row(), 0).T());
    if (M.get_transpose()) {
        // logical rows are contiguous physical columns already
        const int pr = as_int(JzRocmFused::phys_rows(M)), pc = as_int(JzRocmFused::phys_cols(M));
        MR out = JzRocmFused::like("softmax", M);
        ok(jzhip_softmax_cols(JzRocmFused::ptr(out), JzRocmFused::ptr(M), pr, pc, pr), "softmax_cols");
        return out;
    }
    // plain input: lay the rows out contiguously, then the column kernel in place
    MR t = JzRocmFused::materialise(M.T());
    const int pr = as_int(JzRocmFused::phys_rows(t)), pc = as_int(JzRocmFused::phys_cols(t));
    ok(jzhip_softmax_cols(JzRocmFused::ptr(t), JzRocmFused::ptr(t), pr, pc, pr), "softmax_cols");
    return MR(t.T());
}

}  // namespace Juzhen

// ── device API of cpp/hipbackend.hpp that lived in this file upstream ────────
// (RocmGemm / RocmGemmNN / RocmGemv, cpp/hipmatrix.cpp:605-707)

int Juzhen::RocmGemm(const float* A_device, const float* B_device, float* C_device, int m, int n, int k,
                     bool transA, bool transB, int lda, int ldb, int ldc, float alpha, float beta) {
    return jzhip_gemm(A_device, B_device, C_device, m, n, k, transA, transB, lda, ldb, ldc, alpha, beta);
}

int Juzhen::RocmGemmNN(const float* A_device, const float* B_device, float* C_device, int m, int n, int k,
                       float alpha, float beta) {
    return jzhip_gemm_nn(A_device, B_device, C_device, m, n, k, alpha, beta);
}

int Juzhen::RocmGemv(const float* A_device, const float* x_device, float* y_device, int m, int n, bool transA,
                     int lda, int incx, int incy, float alpha, float beta) {
    return jzhip_gemv(A_device, x_device, y_device, m, n, transA, lda, incx, incy, alpha, beta);
}

// ── host staging: printing and the .matrix file format ──────────────────────

std::ostream& operator<<(std::ostream& os, const MR& M) {
    os << M.to_host();
    return os;
}

template <>
void write(FILE* fp, const MR& M) {
    write(fp, M.to_host());
}

template <>
void read(FILE* fp, MR& M) {
    Matrix<float> tmp;
    read(fp, tmp);
    if (!M.elements || M.count() != tmp.numrow * tmp.numcol || M.elements.use_count() != 1) {
        M.elements.reset(Memory<ROCMfloat>::allocate(tmp.numrow * tmp.numcol), pool_release);
    }
    M.numrow = tmp.numrow;
    M.numcol = tmp.numcol;
    M.transpose = tmp.transpose;
    upload(M.dev(), tmp.elements.get(), M.count());
}

#endif  // ROCM_HIP
