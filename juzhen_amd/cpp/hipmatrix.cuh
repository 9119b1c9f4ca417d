// Matrix<ROCMfloat> for MI355X (gfx950): drop-in for the reference's
// cpp/hipmatrix.cuh.  The public surface (constructors, members, friends and the
// free functions) is the one the reference declares (cpp/hipmatrix.cuh:40-162),
// so cpp/operators.hpp, ml/layer.hpp and user programs compile unchanged.
// Behind it every operation is one call into the C ABI of libjzhip.so
// (include/jzhip.h); semantics are those of the CPU Matrix<float>
// (cpp/core.hpp, cpp/matrix.hpp), including transpose flags on both operands.
//
// Additions over the reference header, all ROCm-only and found by ordinary
// overload resolution (a non-template overload beats the generic template, the
// mechanism the reference uses for its Metal backend, ml/layer.hpp:2333-2339):
// fused col_softmax/row_softmax, relu/d_relu and predict_one_hot here, adam_update and the
// layer classes in hipfused_util.hpp / hipfused.hpp.
#ifndef HIPMATRIX_CUH
#define HIPMATRIX_CUH

#ifdef __HIPCC__
#include <hip/hip_runtime.h>
#endif

#include <stdexcept>
#include <vector>

#include "core.hpp"
#include "hipbackend.hpp"
#include "matrix.hpp"
#include "operators.hpp"

// ── pool allocator hooks (cpp/memory.hpp:36-37) ─────────────────────────────
template <>
inline ROCMfloat* Memory<ROCMfloat>::_alloc(size_t size) {
    float* p = nullptr;
    if (Juzhen::RocmMalloc(&p, size ? size : 1) != 0 || p == nullptr) throw std::bad_alloc();
    return reinterpret_cast<ROCMfloat*>(p);
}

template <>
inline void Memory<ROCMfloat>::_free(ROCMfloat* ptr) {
    Juzhen::RocmFree(reinterpret_cast<float*>(ptr));
}

template <class T>
struct adam_state;

// The stream every library call is enqueued on (include/jzhip.h); the
// templates below launch on the same one so program order stays device order.
extern "C" void* jzhip_get_stream(void);

template <>
class Matrix<ROCMfloat> {
    // Field names are part of the contract: MatrixView<ROCMfloat> and the
    // reduce/elemwise templates read them directly.
    size_t numcol;
    size_t numrow;
    bool transpose;
    std::string name;
    std::shared_ptr<ROCMfloat[]> elements;

    // view constructor: shares `elements`
    Matrix<ROCMfloat>(const char* name, size_t numrow, size_t numcol, int trans,
                      std::shared_ptr<ROCMfloat[]> elements);
    // owning constructor: takes an uninitialised block from the pool
    Matrix<ROCMfloat>(const char* name, size_t numrow, size_t numcol, int trans);

    float* dev() const { return reinterpret_cast<float*>(elements.get()); }
    size_t count() const { return numrow * numcol; }

   public:
    // ── construction / assignment ──
    Matrix<ROCMfloat>() : Matrix<ROCMfloat>("un_init", 2, 2, 0) {}
    Matrix<ROCMfloat>(const char* name, size_t numrow, size_t numcol)
        : Matrix<ROCMfloat>(name, numrow, numcol, 0) {}
    explicit Matrix<ROCMfloat>(const Matrix<float>& M);  // upload, keeps dims and flag
    Matrix<ROCMfloat>(const Matrix<ROCMfloat>& M);       // deep copy
    Matrix<ROCMfloat>(Matrix<ROCMfloat>&& M) noexcept;   // steals the buffer
    Matrix<ROCMfloat>& operator=(const Matrix<ROCMfloat>& M);
    Matrix<ROCMfloat>& operator=(Matrix<ROCMfloat>&& M) noexcept;

    // ── shape / storage ──
    inline size_t idx(size_t i, size_t j) const { return transpose ? i * numrow + j : j * numrow + i; }
    inline size_t num_col() const { return transpose ? numrow : numcol; }
    inline size_t num_row() const { return transpose ? numcol : numrow; }
    inline size_t get_transpose() const { return transpose; }
    std::string get_name() const { return name; }
    const ROCMfloat* data() const { return elements.get(); }
    // Device memory is not host-addressable; kept only so generic code that
    // names elem() still compiles.  Use to_host() to read values.
    inline ROCMfloat elem(size_t i, size_t j) const { return elements[idx(i, j)]; }
    inline ROCMfloat& elem(size_t i, size_t j) { return elements[idx(i, j)]; }

    // ── fill / factories ──
    void ones();
    void zeros();
    static Matrix<ROCMfloat> randn(size_t m, size_t n);
    static Matrix<ROCMfloat> rand(size_t m, size_t n);
    static Matrix<ROCMfloat> ones(size_t m, size_t n);
    static Matrix<ROCMfloat> zeros(size_t m, size_t n);

    // ── the four operator concepts (cpp/operators.hpp:47-96) ──
    Matrix<ROCMfloat> dot(const Matrix<ROCMfloat>& B) const;
    Matrix<ROCMfloat> add(const Matrix<ROCMfloat>& B, float s1, float s2) const;
    void add(const Matrix<ROCMfloat>& B, float s1, float s2);
    Matrix<ROCMfloat> add(float a, float s1) const;
    void add(float a, float s1);
    Matrix<ROCMfloat> scale(float s1) const { return add(0, s1); }
    void scale(float s1);
    void eleminv(double l);
    Matrix<ROCMfloat> eleminv(double l) const;

    float norm() const;
    const Matrix<ROCMfloat> T() const;
    Matrix<float> to_host() const;

    // ── rectangular views ──
    Matrix<ROCMfloat> slice(size_t rstart, size_t rend, size_t cstart, size_t cend) const;
    void slice(size_t rstart, size_t rend, size_t cstart, size_t cend, const Matrix<ROCMfloat>& M);
    Matrix<ROCMfloat> rows(size_t rstart, size_t rend) const;
    void rows(size_t rstart, size_t rend, const Matrix<ROCMfloat>& M);
    Matrix<ROCMfloat> columns(size_t cstart, size_t cend) const;
    void columns(size_t cstart, size_t cend, const Matrix<ROCMfloat>& M);

    // ── friends (same set as the reference declares) ──
    friend class MatrixView<ROCMfloat>;
    friend Matrix<ROCMfloat> sum(const Matrix<ROCMfloat>& M, int dim);
    friend Matrix<ROCMfloat> hadmd(const Matrix<ROCMfloat>& M1, const Matrix<ROCMfloat>& M2);
    friend Matrix<ROCMfloat> hadmd(const Matrix<ROCMfloat>& M1, Matrix<ROCMfloat>&& M2);
    friend Matrix<ROCMfloat> hadmd(Matrix<ROCMfloat>&& M1, const Matrix<ROCMfloat>& M2);
    friend Matrix<ROCMfloat> hadmd(Matrix<ROCMfloat>&& M1, Matrix<ROCMfloat>&& M2);
    friend Matrix<ROCMfloat> exp(const Matrix<ROCMfloat>& M);
    friend Matrix<ROCMfloat> exp(Matrix<ROCMfloat>&& M);
    friend Matrix<ROCMfloat> log(const Matrix<ROCMfloat>& M);
    friend Matrix<ROCMfloat> tanh(const Matrix<ROCMfloat>& M);
    friend Matrix<ROCMfloat> tanh(Matrix<ROCMfloat>&& M);
    friend Matrix<ROCMfloat> d_tanh(const Matrix<ROCMfloat>& M);
    friend Matrix<ROCMfloat> d_tanh(Matrix<ROCMfloat>&& M);
    friend Matrix<ROCMfloat> square(const Matrix<ROCMfloat>& M);
    friend Matrix<ROCMfloat> square(Matrix<ROCMfloat>&& M);
    friend void copy(Matrix<ROCMfloat>& dest, const Matrix<ROCMfloat>& src);
    friend Matrix<ROCMfloat>& fill(Matrix<ROCMfloat>& M, double a);
    friend Matrix<ROCMfloat> hstack(std::vector<MatrixView<ROCMfloat>> matrices);
    friend Matrix<ROCMfloat> vstack(std::vector<MatrixView<ROCMfloat>> matrices);
    template <class Function>
    friend Matrix<ROCMfloat> reduce(Function func, const Matrix<ROCMfloat>& M, int dim, int k);
    template <class Function>
    friend Matrix<ROCMfloat> elemwise(Function func, const Matrix<ROCMfloat>& M);
    template <class Function>
    friend Matrix<ROCMfloat> elemwise(Function func, Matrix<ROCMfloat>&& M);
    friend std::ostream& operator<<(std::ostream& os, const Matrix<ROCMfloat>& M);
    friend void write<ROCMfloat>(FILE* fp, const Matrix<ROCMfloat>& M);
    friend void read<ROCMfloat>(FILE* fp, Matrix<ROCMfloat>& M);

    // fused ROCm paths (defined in hipmatrix.cpp)
    friend struct JzRocmFused;
};

Matrix<ROCMfloat> sum(const Matrix<ROCMfloat>& M, int dim);
std::ostream& operator<<(std::ostream& os, const Matrix<ROCMfloat>& M);
Matrix<ROCMfloat> exp(const Matrix<ROCMfloat>& M);
Matrix<ROCMfloat> exp(Matrix<ROCMfloat>&& M);
Matrix<ROCMfloat> log(const Matrix<ROCMfloat>& M);
Matrix<ROCMfloat> tanh(const Matrix<ROCMfloat>& M);
Matrix<ROCMfloat> tanh(Matrix<ROCMfloat>&& M);
Matrix<ROCMfloat> d_tanh(const Matrix<ROCMfloat>& M);
Matrix<ROCMfloat> d_tanh(Matrix<ROCMfloat>&& M);
Matrix<ROCMfloat> square(const Matrix<ROCMfloat>& M);
Matrix<ROCMfloat> square(Matrix<ROCMfloat>&& M);
void copy(Matrix<ROCMfloat>& dest, const Matrix<ROCMfloat>& src);
Matrix<ROCMfloat>& fill(Matrix<ROCMfloat>& M, double a);
Matrix<ROCMfloat> hstack(std::vector<MatrixView<ROCMfloat>> matrices);
Matrix<ROCMfloat> vstack(std::vector<MatrixView<ROCMfloat>> matrices);

// ── fused overloads picked up by the unmodified layer templates ─────────────
// relu / d_relu (ml/util.cuh:74-82): the generic templates go through a
// device lambda; these call the fixed-function kernels and, unlike the
// generic ones, really do reuse the rvalue's buffer.
Matrix<ROCMfloat> relu(Matrix<ROCMfloat>&& M);
Matrix<ROCMfloat> d_relu(Matrix<ROCMfloat>&& M);
namespace Juzhen {
// col_softmax / row_softmax (ml/layer.hpp:2344-2367): single-pass kernels.
Matrix<ROCMfloat> col_softmax(const Matrix<ROCMfloat>& M);
Matrix<ROCMfloat> row_softmax(const Matrix<ROCMfloat>& M);
}  // namespace Juzhen
// predict_one_hot (ml/util.cuh:258-279): column maximum and threshold in one launch
// instead of reduce<F>, a rank-1 product, a subtraction and elemwise<F>.
Matrix<ROCMfloat> predict_one_hot(const Matrix<ROCMfloat>& input);

// Internal access point for the fused paths.
struct JzRocmFused {
    static float* ptr(const Matrix<ROCMfloat>& M) { return M.dev(); }
    static Matrix<ROCMfloat> like(const char* name, const Matrix<ROCMfloat>& M) {
        return Matrix<ROCMfloat>(name, M.numrow, M.numcol, M.transpose);
    }
    static Matrix<ROCMfloat> make(const char* name, size_t r, size_t c, int trans) {
        return Matrix<ROCMfloat>(name, r, c, trans);
    }
    // A dense r x c matrix that starts `offset` floats into M's buffer and keeps that buffer alive
    // (several matrices laid out back to back for one strided-batched launch).
    static Matrix<ROCMfloat> block(const char* name, const Matrix<ROCMfloat>& M, size_t offset, size_t r, size_t c) {
        std::shared_ptr<ROCMfloat[]> alias(M.elements, M.elements.get() + offset);
        return Matrix<ROCMfloat>(name, r, c, 0, alias);
    }
    static size_t phys_rows(const Matrix<ROCMfloat>& M) { return M.numrow; }
    static size_t phys_cols(const Matrix<ROCMfloat>& M) { return M.numcol; }
    // Materialise the logical transpose of M as a plain (flag 0) matrix.
    static Matrix<ROCMfloat> materialise(const Matrix<ROCMfloat>& M);
    // The buffers created since jzhip_graph_begin (each with one extra owner): whoever takes
    // them keeps them out of the pool for as long as the recorded graph may be replayed.
    static std::vector<std::shared_ptr<ROCMfloat[]>> take_recording_pins();
};

// adam_update (ml/util.cuh:166-256) as one fused kernel with the arithmetic of
// the CPU loop (ml/util.cuh:223-245).  adam_state is only forward-declared
// here, so the body is a template that is instantiated at the end of the
// including translation unit, where ml/util.cuh has completed the type.
extern "C" int jzhip_graph_recording(void);
extern "C" int jzhip_adam_update(float* g, float* m, float* v, size_t count, float alpha, float beta1,
                                 float beta2, float eps, int iteration);

template <class State>
Matrix<ROCMfloat> jz_rocm_adam_update(Matrix<ROCMfloat>&& g, State& st) {
    if (jzhip_graph_recording()) {
        // the step count is a by-value argument of this launch: a replay would repeat step `iteration`
        LOG_ERROR("adam_update cannot be recorded into a graph: update parameters through a layer's backward()");
        ERROR_OUT;
    }
    if (!g.get_transpose() && !st.m.get_transpose() && !st.v.get_transpose()) {
        const int rc = jzhip_adam_update(JzRocmFused::ptr(g), JzRocmFused::ptr(st.m), JzRocmFused::ptr(st.v),
                                         g.num_row() * g.num_col(), st.alpha, st.beta1, st.beta2, st.eps,
                                         st.iteration);
        if (rc != 0) {
            LOG_ERROR("jzhip_adam_update failed with code {}", rc);
            ERROR_OUT;
        }
        st.iteration++;
        return std::move(g);
    }
    // transposed operands: the generic formulation (ml/util.cuh:247-255)
    st.m = st.beta1 * st.m + (1 - st.beta1) * g;
    st.v = st.beta2 * st.v + (1 - st.beta2) * square(g);
    auto m_hat = st.m / (1 - pow(st.beta1, st.iteration));
    auto v_hat = st.v / (1 - pow(st.beta2, st.iteration));
    g = st.alpha * m_hat / (sqrt(v_hat) + st.eps);
    st.iteration++;
    return std::move(g);
}

// Declared here so that it is visible before the layer templates are parsed;
// defined in hipfused_util.hpp, which is included at the end of ml/util.cuh
// (where adam_state is complete), the way ml/util.cuh:147-192 hooks CUDA.
inline Matrix<ROCMfloat> adam_update(Matrix<ROCMfloat>&& g, adam_state<ROCMfloat>& state);

#ifdef __HIPCC__

// ── user-functor templates ──────────────────────────────────────────────────
// elemwise<F> and reduce<F> take arbitrary device functors, so they have to be
// header templates that launch from the user's translation unit.  elemwise
// applies the functor per lane over float4 loads, one float4 per thread with
// the grid covering the data once (workgroups are dispatched in id order, so
// the resident ones stream one compact window of memory).  reduce keeps the
// reference contract "one functor call per reduced vector, on a contiguous
// vector the functor may overwrite" (cpp/matrix.hpp:202-250) but moves the
// data with the whole workgroup: a group of vectors is read into LDS in
// coalesced rows, each vector's functor call then runs on its LDS copy, and
// whatever the functor changed is written back the same way, so the caller
// sees the same overwritten input as on the CPU (examples/knn.cu:61-78 relies
// on overwriting its input while it selects minima).

namespace jzrocm {
constexpr size_t kStreamingBytes = size_t(384) << 20;   // launches from this size on stream past the caches
constexpr int kThreads = 256;
inline hipStream_t stream() { return static_cast<hipStream_t>(jzhip_get_stream()); }
inline unsigned grid_cover(size_t items) {
    size_t need = (items + kThreads - 1) / kThreads;
    if (need < 1) need = 1;
    if (need > 0x7fffffffull) need = 0x7fffffffull;   // the kernels keep a stride loop for the excess
    return static_cast<unsigned>(need);
}

// NT: loads and stores with the non-temporal hint, for launches that move more than the
// last-level cache can hold (a map over 2^28 floats: 6.1 -> 6.5 TB/s).
template <bool NT, class Function>
__global__ __launch_bounds__(kThreads) void elemwise_kernel(Function func, float* dst,
                                                            const float* src, size_t n, int vec) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
    const size_t tid = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (vec) {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride) {
            f4 x, y;
            if constexpr (NT) x = __builtin_nontemporal_load(reinterpret_cast<const f4*>(src) + i);
            else x = reinterpret_cast<const f4*>(src)[i];
            y.x = func(x.x);
            y.y = func(x.y);
            y.z = func(x.z);
            y.w = func(x.w);
            if constexpr (NT) __builtin_nontemporal_store(y, reinterpret_cast<f4*>(dst) + i);
            else reinterpret_cast<f4*>(dst)[i] = y;
        }
        for (size_t j = n4 * 4 + tid; j < n; j += stride) dst[j] = func(src[j]);
    } else {
        for (size_t j = tid; j < n; j += stride) dst[j] = func(src[j]);
    }
}

// One thread per vector, straight from global memory: vectors too long for
// the staged form below.
template <class Function>
__global__ __launch_bounds__(kThreads) void reduce_kernel(Function func, float* vecdes, float* vec,
                                                          size_t lenvec, size_t lenvecdes,
                                                          size_t numvecs) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; i < numvecs; i += stride)
        func(&vec[i * lenvec], &vecdes[i * lenvecdes], lenvec, lenvecdes);
}

// Staged form: a workgroup takes `group` consecutive vectors (group * lenvec
// floats, contiguous in memory), keeps two copies in LDS with an odd pitch
// (lanes that walk their own vectors in step hit distinct banks), runs one
// functor call per vector on the first copy, then compares the copies and
// writes the group back only when a call changed its vector.
constexpr int kReduceLdsFloats = 8128;   // per copy: two copies fill the 64 KiB a workgroup may declare
template <class Function>
__global__ __launch_bounds__(kThreads) void reduce_staged_kernel(Function func, float* vecdes, float* vec,
                                                                 int lenvec, int lenvecdes,
                                                                 size_t numvecs, int group, int pitch) {
    __shared__ float work[kReduceLdsFloats];
    __shared__ float keep[kReduceLdsFloats];
    __shared__ int changed;
    // element e = threadIdx.x + i*kThreads of the group is (vector v, row r): stepped without divisions
    const int v0 = threadIdx.x / lenvec, r0 = threadIdx.x % lenvec;
    const int dv = kThreads / lenvec, dr = kThreads % lenvec;
    for (size_t first = static_cast<size_t>(blockIdx.x) * group; first < numvecs;
         first += static_cast<size_t>(gridDim.x) * group) {
        const int nv = numvecs - first < static_cast<size_t>(group) ? static_cast<int>(numvecs - first) : group;
        const int total = nv * lenvec;
        float* base = vec + first * lenvec;
        if (threadIdx.x == 0) changed = 0;
        for (int e = threadIdx.x, v = v0, r = r0; e < total; e += kThreads) {
            const float x = base[e];
            work[v * pitch + r] = x;
            keep[v * pitch + r] = x;
            v += dv; r += dr;
            if (r >= lenvec) { r -= lenvec; ++v; }
        }
        __syncthreads();
        if (threadIdx.x < nv)
            func(&work[threadIdx.x * pitch], &vecdes[(first + threadIdx.x) * lenvecdes], lenvec, lenvecdes);
        __syncthreads();
        int diff = 0;
        for (int e = threadIdx.x, v = v0, r = r0; e < total; e += kThreads) {
            // bit comparison: a functor that writes the same value, or a NaN, counts as it should
            diff |= __float_as_uint(work[v * pitch + r]) != __float_as_uint(keep[v * pitch + r]);
            v += dv; r += dr;
            if (r >= lenvec) { r -= lenvec; ++v; }
        }
        if (diff) changed = 1;
        __syncthreads();
        if (changed) {
            for (int e = threadIdx.x, v = v0, r = r0; e < total; e += kThreads) {
                base[e] = work[v * pitch + r];
                v += dv; r += dr;
                if (r >= lenvec) { r -= lenvec; ++v; }
            }
        }
        __syncthreads();
    }
}

template <class Function>
inline void launch_reduce(Function func, float* dst, float* src, size_t lenvec, size_t k, size_t numvecs) {
    if (numvecs == 0) return;
    // Staging pays for vectors of a few dozen to a few hundred elements (measured on
    // MI355X, column max over 2^28 bytes: 252 us staged against 374 us direct at length
    // 256, 677 against 3557 us for a functor that overwrites its vector).  Shorter
    // vectors are read well enough directly (a wavefront's 64 vectors form one
    // contiguous block); longer ones leave too few functor calls per workgroup to keep
    // its lanes busy (length 1024: 428 us staged against 148 us direct).
    if (lenvec > 16 && lenvec <= 512) {
        const int pitch = static_cast<int>(lenvec | 1);                       // odd: conflict-free column walks
        int group = kReduceLdsFloats / pitch;
        if (group > kThreads) group = kThreads;
        const size_t blocks = (numvecs + group - 1) / group;
        reduce_staged_kernel<<<static_cast<unsigned>(blocks < 0x7fffffffull ? blocks : 0x7fffffffull), kThreads, 0,
                               stream()>>>(func, dst, src, static_cast<int>(lenvec), static_cast<int>(k), numvecs,
                                           group, pitch);
        return;
    }
    reduce_kernel<<<grid_cover(numvecs), kThreads, 0, stream()>>>(func, dst, src, lenvec, k, numvecs);
}
}  // namespace jzrocm

template <class Function>
Matrix<ROCMfloat> elemwise(Function func, const Matrix<ROCMfloat>& M) {
    Matrix<ROCMfloat> result("resM", M.numrow, M.numcol, M.transpose);
    const size_t n = M.count();
    const int vec = ((reinterpret_cast<uintptr_t>(M.dev()) | reinterpret_cast<uintptr_t>(result.dev())) & 15) == 0;
    if (n * 2 * sizeof(float) >= jzrocm::kStreamingBytes)
        jzrocm::elemwise_kernel<true><<<jzrocm::grid_cover(vec ? n / 4 + 1 : n), jzrocm::kThreads, 0, jzrocm::stream()>>>(
            func, result.dev(), M.dev(), n, vec);
    else
        jzrocm::elemwise_kernel<false><<<jzrocm::grid_cover(vec ? n / 4 + 1 : n), jzrocm::kThreads, 0, jzrocm::stream()>>>(
            func, result.dev(), M.dev(), n, vec);
    return result;
}

template <class Function>
Matrix<ROCMfloat> elemwise(Function func, Matrix<ROCMfloat>&& M) {
    const size_t n = M.count();
    const int vec = (reinterpret_cast<uintptr_t>(M.dev()) & 15) == 0;
    if (n * sizeof(float) >= jzrocm::kStreamingBytes)   // in place: one buffer
        jzrocm::elemwise_kernel<true><<<jzrocm::grid_cover(vec ? n / 4 + 1 : n), jzrocm::kThreads, 0, jzrocm::stream()>>>(
            func, M.dev(), M.dev(), n, vec);
    else
        jzrocm::elemwise_kernel<false><<<jzrocm::grid_cover(vec ? n / 4 + 1 : n), jzrocm::kThreads, 0, jzrocm::stream()>>>(
            func, M.dev(), M.dev(), n, vec);
    return std::move(M);
}

// Orientation table of the CPU oracle (cpp/matrix.hpp:202-250): the functor is
// handed the physical columns directly when they are the vectors to reduce,
// otherwise a private transposed copy.
template <class Function>
Matrix<ROCMfloat> reduce(Function func, const Matrix<ROCMfloat>& M, int dim, int k) {
    const bool direct = (dim == 0) == !M.transpose;
    if (direct) {
        Matrix<ROCMfloat> result("resM", k, M.numcol);
        jzrocm::launch_reduce(func, result.dev(), M.dev(), M.numrow, k, M.numcol);
        return M.transpose ? Matrix<ROCMfloat>(result.T()) : result;
    }
    // physical transpose of the buffer: its columns are the vectors to reduce
    Matrix<ROCMfloat> t = JzRocmFused::materialise(M.transpose ? M : M.T());
    Matrix<ROCMfloat> result("resM", k, t.numcol);
    jzrocm::launch_reduce(func, result.dev(), t.dev(), t.numrow, k, t.numcol);
    return M.transpose ? result : Matrix<ROCMfloat>(result.T());
}

#endif  // __HIPCC__

#endif
