/*
 * jzhip.h — C ABI of the MI355X (gfx950) device library behind Juzhen's
 * Matrix<ROCMfloat>.
 *
 * Conventions (all entry points):
 *   - plain C: device pointers are `float*`, element counts `size_t`, matrix
 *     dimensions `int`, flags `int` (0/1).  No C++ or torch types cross it.
 *   - return value: 0 = success, -1 = invalid argument (null pointer,
 *     non-positive dimension, unsupported flag), -2 = the workspace could not
 *     be created, -3 = a size beyond the fixed scratch of a no-allocation
 *     entry point, otherwise a positive hipError_t value.  `jzhip_error_string` turns it into text.
 *   - matrices are fp32, column-major: element (i,j) of a matrix with
 *     physical row count `ld` lives at `p[j*ld + i]`.  A "trans" flag means
 *     the logical matrix is the transpose of the physical one
 *     (reference: cpp/hipmatrix.cuh:64-66).
 *   - ordering: every call enqueues on the library's current stream (the
 *     null stream unless `jzhip_set_stream` was called) and returns without
 *     synchronising; issue order is execution order, exactly as the
 *     reference's null-stream launches (cpp/hipkernels.cpp:610-622).  Only
 *     the memcpy calls and `jzhip_synchronize` block the host.
 *   - threads: the current stream is one setting for the whole process, as the
 *     reference's null stream is (cpp/hipkernels.cpp:458-461).  Drive the library
 *     from one host thread, or serialise `jzhip_set_stream` plus the calls that
 *     depend on it under a lock of your own: two threads that select different
 *     streams at the same time would enqueue on each other's stream and share
 *     its workspace.  The internal tables themselves (workspaces, one-time
 *     kernel attributes) tolerate concurrent callers.
 *   - no entry point allocates device memory behind the caller's back except
 *     `jzhip_malloc` and the lazily created reduction workspace, one per
 *     stream that needs it (see `jzhip_workspace_bytes`).
 *
 * Citations `file:line` refer to the reference tree (anewgithubname/Juzhen).
 */
#ifndef JZHIP_H
#define JZHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ── runtime ─────────────────────────────────────────────────────────── */

/* Replaces Juzhen::RocmRuntimeAvailable (cpp/hipbackend.hpp:10). 1 when a
 * gfx950 device is usable, else 0. */
int jzhip_runtime_available(void);
/* Library ABI version (major*100+minor). */
int jzhip_version(void);
/* Text for a return code of this library. Never NULL. */
const char* jzhip_error_string(int rc);
/* Number of compute units of the current device (0 on failure). */
int jzhip_num_compute_units(void);

/* Replaces Juzhen::RocmMalloc / RocmFree (cpp/hipbackend.hpp:12-13,
 * cpp/hipkernels.cpp:513-533). `count` is in floats; count==0 allocates one. */
int jzhip_malloc(float** ptr, size_t count);
int jzhip_free(float* ptr);
/* Replaces Juzhen::RocmMemcpyH2D/D2H/D2D (cpp/hipbackend.hpp:14-16,
 * cpp/hipkernels.cpp:535-569). Synchronous with respect to the host, ordered
 * after all work previously issued on the current stream. */
int jzhip_memcpy_h2d(float* dst_device, const float* src_host, size_t count);
int jzhip_memcpy_d2h(float* dst_host, const float* src_device, size_t count);
int jzhip_memcpy_d2d(float* dst_device, const float* src_device, size_t count);

/* No reference counterpart (the reference uses the null stream only,
 * cpp/hipkernels.cpp:458-461): select the hipStream_t every later call of
 * this process enqueues on (one setting for all host threads, see "threads"
 * above); NULL restores the null stream. */
int jzhip_set_stream(void* hip_stream);
void* jzhip_get_stream(void);
/* Block until the current stream is idle. */
int jzhip_synchronize(void);
/* Bytes of the lazily created reduction workspaces (0 before first use): one
 * per stream that has run a call needing partial results, so that calls
 * issued on different streams never share scratch storage. */
size_t jzhip_workspace_bytes(void);
/* No reference counterpart (cpp/hipkernels.cpp:458-461 runs everything on the
 * null stream): a second stream and the events that order work between
 * streams, for callers that overlap independent products (weight gradients
 * against the gradient chain).  `jzhip_stream_create` makes a non-blocking
 * stream of default priority; `jzhip_event_record` marks the current stream's
 * position and `jzhip_stream_wait_event` makes everything issued afterwards
 * on the current stream wait for that mark.  Neither blocks the host.
 * `jzhip_stream_destroy` waits for the stream, frees the workspace the stream
 * may have acquired and restores the null stream if it was the current one. */
int jzhip_stream_create(void** out_stream);
int jzhip_stream_destroy(void* hip_stream);
int jzhip_event_create(void** out_event);
int jzhip_event_destroy(void* event);
int jzhip_event_record(void* event);
int jzhip_stream_wait_event(void* event);
/* Block the host until the work marked by `jzhip_event_record` has run. */
int jzhip_event_synchronize(void* event);
/* No reference counterpart: record the calls of a launch-bound loop body once and
 * replay them as one HIP graph launch.  Between `jzhip_graph_begin` and
 * `jzhip_graph_end` every call of this library is recorded on an internal stream
 * instead of run (the current stream is switched for that span and restored by
 * `jzhip_graph_end`; `jzhip_set_stream` is refused meanwhile); pointers, sizes and
 * scalar arguments are fixed at recording time, so the replay works on the same
 * buffers.  What must not happen while recording: host reads of device data
 * (`jzhip_memcpy_d2h`, `jzhip_synchronize`), uploads from pageable memory, and
 * calls whose scalar arguments change from step to step (an optimiser step
 * count: use `jzhip_adamw_step_multi_counted`).  Device memory may be allocated
 * while recording (it is allocated at once, not replayed).  `jzhip_graph_launch`
 * enqueues one replay on the current stream (the null stream included) and
 * returns without waiting.  `jzhip_graph_recording` is 1 between begin and end.
 * `jzhip_graph_destroy` waits for every stream the graph was replayed on, then
 * destroys it (-1 while another recording is in progress): after it returns the
 * caller may free the buffers the recording used.  Every recording bakes the
 * record stream's one workspace (split-K partials, reduction partials, flipped
 * convolution weights) into its nodes: replays of recorded graphs must therefore
 * be serialised with each other and with eager calls made while recording, i.e.
 * launched on one stream or ordered with events; two graphs replayed on two
 * streams at once race on that workspace.  The record stream is a blocking
 * stream, so work that other code puts on the legacy null stream while a
 * recording is open invalidates the recording (`jzhip_graph_end` then fails).
 * What it buys on MI355X: the MLP step of ~60 kernels 0.196 -> 0.186 ms, the CNN
 * step 0.341 -> 0.334 ms; such steps are bound by the device's dispatch of short
 * dependent kernels, which a graph does not remove, not by host launch cost. */
int jzhip_graph_begin(void);
int jzhip_graph_end(void** out_graph);
int jzhip_graph_recording(void);
int jzhip_graph_launch(void* graph);
int jzhip_graph_destroy(void* graph);
/* No reference counterpart: the reference reads a batch into pageable host
 * memory and uploads it with a blocking copy in Matrix<ROCMfloat>'s converting
 * constructor (ml/dataloader.hpp:88-113, cpp/hipmatrix.cpp:60-63), which drains
 * the stream before every batch.  `jzhip_host_alloc` returns page-locked host
 * memory; `jzhip_memcpy_h2d_async` / `_d2h_async` enqueue a copy of `bytes`
 * bytes on the current stream and return at once when the host side is such
 * memory (from pageable memory the copy is still ordered but may block; an
 * upload of up to 1 MiB from page-locked memory is done by a kernel that reads
 * the host buffer directly, so it never leaves the compute queue).  The
 * host buffer must stay untouched until the stream has passed the copy: record
 * an event after it and `jzhip_event_synchronize` before reusing the buffer. */
int jzhip_host_alloc(void** ptr, size_t bytes);
int jzhip_host_free(void* ptr);
int jzhip_memcpy_h2d_async(void* dst_device, const void* src_host, size_t bytes);
int jzhip_memcpy_d2h_async(void* dst_host, const void* src_device, size_t bytes);

/* ── random numbers ──────────────────────────────────────────────────── */

/* Replace Juzhen::RocmRandUniform / RocmRandNormal (cpp/hipbackend.hpp:18-20,
 * cpp/hipkernels.cpp:571-608; rocRAND there, Philox4x32-10 + Box-Muller here).
 * seed==0 continues the library's running stream; seed!=0 restarts it. */
int jzhip_rand_uniform(float* dst, size_t count, uint64_t seed);
int jzhip_rand_normal(float* dst, size_t count, float mean, float stddev,
                      uint64_t seed);

/* ── flat elementwise ops (operate on `count` contiguous floats) ─────── */

/* Juzhen::RocmFill (cpp/hipbackend.hpp:22). */
int jzhip_fill(float* dst, size_t count, float value);
/* Juzhen::RocmExpInplace / RocmLogInplace (cpp/hipbackend.hpp:23-24);
 * oracle exp/log loops cpp/matrix.hpp:253-279. */
int jzhip_exp_inplace(float* x, size_t count);
int jzhip_log_inplace(float* x, size_t count);
/* Out-of-place forms (one pass instead of the reference's D2D copy + in-place
 * kernel, cpp/hipmatrix.cpp:338-353). out may equal in. */
int jzhip_exp(float* out, const float* in, size_t count);
int jzhip_log(float* out, const float* in, size_t count);
/* Juzhen::RocmAxpby (cpp/hipbackend.hpp:25-26): out = s1*a + s2*b, same
 * physical layout for all three; out may alias a or b.
 * Oracle cpp/core.hpp:414-449. */
int jzhip_axpby(float* out, const float* a, const float* b, size_t count,
                float s1, float s2);
/* Juzhen::RocmAffineInplace (cpp/hipbackend.hpp:27): x = s1*x + a.
 * Oracle cpp/core.hpp:453-469. */
int jzhip_affine_inplace(float* x, size_t count, float s1, float a);
/* One-pass out-of-place form of the above (cpp/hipmatrix.cpp:190-201). */
int jzhip_affine(float* out, const float* in, size_t count, float s1, float a);
/* Juzhen::RocmHadamard / RocmHadamardInplace (cpp/hipbackend.hpp:28-31).
 * Oracle cpp/matrix.hpp:428-474. */
int jzhip_hadamard(float* out, const float* a, const float* b, size_t count);
int jzhip_hadamard_inplace(float* x, const float* other, size_t count);
/* Juzhen::RocmElemInvInplace (cpp/hipbackend.hpp:32): x = l / x. */
int jzhip_eleminv_inplace(float* x, size_t count, float l);
/* out = (float)(l / (double)in), the oracle's arithmetic
 * (cpp/core.hpp:472-482 divides in double, then rounds). out may equal in. */
int jzhip_eleminv(float* out, const float* in, size_t count, double l);
/* Juzhen::RocmCopy (cpp/hipbackend.hpp:33). */
int jzhip_copy(float* dst, const float* src, size_t count);
/* Juzhen::RocmSquare(Inplace), RocmTanh(Inplace), RocmDTanh(Inplace)
 * (cpp/hipbackend.hpp:34-39); oracle cpp/matrix.hpp:280-326,407-425. */
int jzhip_square(float* out, const float* in, size_t count);
int jzhip_square_inplace(float* x, size_t count);
int jzhip_tanh(float* out, const float* in, size_t count);
int jzhip_tanh_inplace(float* x, size_t count);
int jzhip_dtanh(float* out, const float* in, size_t count);
int jzhip_dtanh_inplace(float* x, size_t count);
/* Fixed-function forms of the functors the layers pass to elemwise<F>:
 * relu / d_relu (ml/util.cuh:74-82), sqrt (cpp/juzhen.hpp:71-79),
 * clamp (ml/util.cuh:84-89). out may equal in. */
int jzhip_relu(float* out, const float* in, size_t count);
int jzhip_drelu(float* out, const float* in, size_t count);
int jzhip_sqrt(float* out, const float* in, size_t count);
int jzhip_clamp(float* out, const float* in, size_t count, float lo, float hi);
/* out = d_relu(pre) * up in one pass: the product every backward() forms as
 * hadmd(d_relu(Matrix(val)), upstream) (ml/layer.hpp:100,1672-1674,3189). */
int jzhip_drelu_mul(float* out, const float* pre, const float* up, size_t count);
/* The squared-error head (LossLayer, ml/layer.hpp:204-227) in one launch each:
 * out_device[0] = scale * sum((target - pred)^2) over `count` elements, which eval()
 * forms as sum(sum(square(output - input), 0), 1) / nb, and
 * out = ((pred - target) * 2) * inv_nb, which grad() forms as 2.0 * (input - output) / nb
 * (every step rounded as the separate operations round; out may equal pred). Flat
 * buffers: both operands stored the same way. */
int jzhip_mse_loss(float* out_device, const float* target, const float* pred, size_t count, float scale);
int jzhip_mse_grad(float* out, const float* pred, const float* target, size_t count, float inv_nb);
/* GELU (exact erf form) and its derivative times an upstream gradient. No
 * reference counterpart (the reference FFN is ReLU, ml/layer.hpp:3018); used
 * by the character-LM configuration. */
int jzhip_gelu(float* out, const float* in, size_t count);
int jzhip_dgelu_mul(float* out, const float* pre, const float* up, size_t count);

/* ── 2-D elementwise ops honouring transpose flags ───────────────────── */

/* out(i,j) = s1*a(i,j) + s2*b(i,j) over logical rows x cols, each operand
 * with its own physical leading dimension and transpose flag. This is the
 * logical-index semantics of the CPU oracle (cpp/core.hpp:414-449) that the
 * reference's flat RocmAxpby call ignores (cpp/hipmatrix.cpp:154-188).
 * out may alias a (same ld and flag) for the in-place form. */
int jzhip_axpby2d(float* out, int ldo, int trans_o,
                  const float* a, int lda, int trans_a,
                  const float* b, int ldb, int trans_b,
                  int rows, int cols, float s1, float s2);
/* Same for the Hadamard product (oracle cpp/matrix.hpp:428-474). */
int jzhip_hadamard2d(float* out, int ldo, int trans_o,
                     const float* a, int lda, int trans_a,
                     const float* b, int ldb, int trans_b,
                     int rows, int cols);
/* dst(dr0+i, dc0+j) = src(sr0+i, sc0+j) for a logical rows x cols block. */
int jzhip_copy2d(float* dst, int ldd, int trans_d, size_t dr0, size_t dc0,
                 const float* src, int lds, int trans_s, size_t sr0, size_t sc0,
                 size_t rows, size_t cols);

/* Juzhen::RocmStackCopyCols / RocmStackCopyRows (cpp/hipbackend.hpp:40-53,
 * kernels cpp/hipkernels.cpp:116-158; oracle hstack/vstack
 * cpp/matrix.hpp:93-150). */
int jzhip_stack_copy_cols(float* dst, size_t dst_numrow, size_t dst_col_offset,
                          const float* src, size_t src_numrow, size_t src_numcol,
                          int src_transpose);
int jzhip_stack_copy_rows(float* dst, size_t dst_numrow, size_t dst_row_offset,
                          const float* src, size_t src_numrow, size_t src_numcol,
                          int src_transpose);
/* Juzhen::RocmSliceExtract / RocmSliceAssign (cpp/hipbackend.hpp:54-72,
 * kernels cpp/hipkernels.cpp:160-206; oracle slice cpp/core.hpp:353-373). */
int jzhip_slice_extract(float* dst, size_t dst_numrow,
                        const float* src, size_t src_numrow, int src_transpose,
                        size_t rstart, size_t cstart, size_t rows, size_t cols);
int jzhip_slice_assign(float* dst, size_t dst_numrow, int dst_transpose,
                       size_t rstart, size_t cstart,
                       const float* src, size_t src_numrow, int src_transpose,
                       size_t rows, size_t cols);

/* No reference counterpart as a kernel: the reference's language-model demo
 * feeds one-hot matrices through dense layers (examples/demo_transformer.cu,
 * LinearLayer ml/layer.hpp:83-105), i.e. x0 = E*onehot(tokens) +
 * P*onehot(positions) + b*ones.  A product with a one-hot matrix copies one
 * column per token, so this lookup gives the same bits:
 * out(:, n) = E(:, tokens[n]) + P(:, n % S) (+ bias), all column-major with
 * leading dimension d; an id outside [0, vocab) selects no column.  (The
 * gradient of the position table is jzhip_sum_rows over the (d*S) x (N/S)
 * view of the gradient; the token table keeps the one-hot product.) */
int jzhip_embedding_fwd(float* out, const float* E, const float* P, const float* bias,
                        const int32_t* tokens, int d, int vocab, int S, int N);

/* The device form of one_hot (ml/util.cuh:295-303), which fills a k x n
 * column-major matrix on the host (zeros, then elem(Y(0,j), j) = 1) and leaves
 * the caller to upload k*n floats: here the labels are n int32 values already
 * on the device.  A label outside [0, k) leaves its column zero. */
int jzhip_one_hot(float* out, const int32_t* labels, int k, size_t n);

/* ── reductions ──────────────────────────────────────────────────────── */

/* Sums over a physical column-major numrow x numcol buffer; replace the
 * ones-vector GEMV of sum(M,dim) (cpp/hipmatrix.cpp:529-555; oracle
 * cpp/matrix.hpp:74-91).
 *   jzhip_sum_cols: out[j] = sum_i a[j*ld+i]   (numcol outputs)
 *   jzhip_sum_rows: out[i] = sum_j a[j*ld+i]   (numrow outputs) */
int jzhip_sum_cols(float* out, const float* a, int numrow, int numcol, int ld);
int jzhip_sum_rows(float* out, const float* a, int numrow, int numcol, int ld);
/* No counterpart in the reference.  For callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  Same result as jzhip_sum_rows (the column-chunk partial
 * sums are combined in the same fixed order), but the partials live in a fixed
 * 4 MiB array inside the library's code object instead of the lazily created
 * workspace, so the call performs no hipMalloc/hipFree at all.  Limit:
 * numrow <= 65536, otherwise rc -3 (any numcol).  Every call on one GPU shares
 * that GPU's array: calls that may overlap on one GPU (different streams, or
 * different host threads) race and must be ordered by the caller. */
int jzhip_sum_rows_noalloc(float* out, const float* a, int numrow, int numcol, int ld);
/* out[0] = sqrt(sum x^2): replaces hipblasSnrm2 in norm()
 * (cpp/hipmatrix.cpp:232-254; oracle cpp/core.hpp:337-344). */
int jzhip_nrm2(float* out_device, const float* x, size_t count);
/* out[j] = max_i a[j*ld+i], the functor col_softmax / predict_one_hot pass to
 * reduce<F> (ml/layer.hpp:2346-2351, ml/util.cuh:260-272). */
int jzhip_max_cols(float* out, const float* a, int numrow, int numcol, int ld);
/* out[j] = index (stored as int32) of the first maximum of column j: the
 * first-maximum rule of std::max_element (ml/util.cuh:104-110,
 * examples/demo_transformer.cu:350-357). Bit-exact. */
int jzhip_argmax_cols(int32_t* out, const float* a, int numrow, int numcol, int ld);
/* predict_one_hot (ml/util.cuh:258-279: reduce<F> column maximum, rank-1 product,
 * subtraction, elemwise<F> threshold) as one launch: out (numrow x numcol, dense) holds
 * 1 where (double)(a - max of its column) > -1e-5, else 0; bit-identical to the chain,
 * ties and NaNs included.  out must not alias a. */
int jzhip_predict_one_hot(float* out, const float* a, int numrow, int numcol, int ld);

/* ── GEMM family ─────────────────────────────────────────────────────── */

/* Juzhen::RocmGemm (cpp/hipbackend.hpp:77-81, hipBLAS there
 * cpp/hipmatrix.cpp:605-652): C(m x n) = alpha*op(A)(m x k)*op(B)(k x n)
 * + beta*C, column-major, fp32 MFMA with fp32 accumulation. Returns -1 for
 * m,n,k <= 0 or null pointers, as the reference does (:611-612).
 * Oracle: Matrix::dot -> gemm (cpp/core.hpp:395-411, cpp/cpulinalg.hpp:46-91). */
int jzhip_gemm(const float* A, const float* B, float* C, int m, int n, int k,
               int trans_a, int trans_b, int lda, int ldb, int ldc,
               float alpha, float beta);
/* GEMM with the layer's elementwise tail fused into the store of C, for the
 * chains dense layers issue after a product (ml/layer.hpp:83-105 `W*x + b*ones`,
 * :335-345 activation, :3005-3024 residual adds of TransformerLayer): with
 * v = alpha*op(A)op(B) + beta*C element by element, in this order
 *   bias != NULL      : v += bias[row]                    (RocmGemm k=1 broadcast + RocmAxpby)
 *   act 1 relu, 2 gelu: aux(row,col) = v when aux != NULL (the pre-activation
 *                       the backward pass needs), then v = act(v)
 *   act 3, 4          : v *= relu'(aux(row,col)) / gelu'(aux(row,col))   (hadmd(d_act(pre), up))
 *   residual != NULL  : v += residual(row,col)
 * Each step rounds like the separate kernel it replaces, so the result is
 * bit-identical to jzhip_gemm followed by jzhip_add_bias / jzhip_gelu /
 * jzhip_dgelu_mul / jzhip_axpby(1,1).  aux has leading dimension ld_aux,
 * residual ldr; residual may alias C. */
int jzhip_gemm_fused(const float* A, const float* B, float* C, int m, int n,
                     int k, int trans_a, int trans_b, int lda, int ldb, int ldc,
                     float alpha, float beta, const float* bias, int act,
                     float* aux, int ld_aux, const float* residual, int ldr);
/* jzhip_gemm_fused plus rowsum[i] = sum_j C(i, j) over the values it stores: an
 * upstream gradient formed as (W^T t) .* act'(pre) and the bias gradient
 * `sum(., 1)` of the layer below it (ml/layer.hpp:98-100; dF1 and db1 of
 * TransformerLayer::backward) without a second pass over the (m x n) result.
 * Each workgroup of the tiled kernel adds up what it stores per row and leaves
 * one partial sum per tile column; they are summed in a fixed order (equal to
 * jzhip_sum_rows over C to rounding).  C as jzhip_gemm_fused bit for bit.
 * Products that take a form without a fused store (see jzhip_gemm_fused) run
 * jzhip_sum_rows over C afterwards.  rowsum must not alias the other operands. */
int jzhip_gemm_fused_rowsum(const float* A, const float* B, float* C, float* rowsum,
                            int m, int n, int k, int trans_a, int trans_b, int lda,
                            int ldb, int ldc, float alpha, float beta, const float* bias,
                            int act, float* aux, int ld_aux, const float* residual, int ldr);
/* A layer's two parameter gradients from one pass over the upstream gradient
 * (`gW = t * input.T(); gb = sum(t, 1);`, ml/layer.hpp:99-100; the same pair in
 * TransformerLayer::backward for Wo / W1 / W2 and their biases): jzhip_gemm as
 * above plus rowsum[i] = sum_p op(A)(i, p), i < m.  With A plain, B transposed
 * and every extent a whole number of tiles (16-byte aligned operands, leading
 * dimensions in multiples of 4) the workgroups of the first tile column add up
 * their A panel on its way into LDS, so the sums cost no second pass over A;
 * they are then the sum over K chunks of per-thread partial sums in a fixed
 * order, equal to jzhip_sum_rows to rounding (<= 1e-5 relative at k = 16384),
 * not bit for bit.  Every other shape runs jzhip_gemm followed by
 * jzhip_sum_rows / jzhip_sum_cols.  rowsum must not alias A, B or C. */
int jzhip_gemm_rowsum(const float* A, const float* B, float* C, float* rowsum, int m,
                      int n, int k, int trans_a, int trans_b, int lda, int ldb, int ldc,
                      float alpha, float beta);
/* Juzhen::RocmGemmNN (cpp/hipbackend.hpp:94-95). */
int jzhip_gemm_nn(const float* A, const float* B, float* C, int m, int n, int k,
                  float alpha, float beta);
/* Juzhen::RocmGemv (cpp/hipbackend.hpp:84-91; oracle cpp/cpulinalg.hpp:96-131):
 * y = alpha*op(A)*x + beta*y, A physically m x n. */
int jzhip_gemv(const float* A, const float* x, float* y, int m, int n,
               int trans_a, int lda, int incx, int incy, float alpha, float beta);
/* Strided-batched GEMM, the shape contract of the reference's CUDA attention
 * path (cublasSgemmStridedBatched, ml/layer.hpp:2896-2927): batch b uses
 * A + b*stride_a, B + b*stride_b, C + b*stride_c. */
int jzhip_gemm_strided_batched(const float* A, const float* B, float* C,
                               int m, int n, int k, int trans_a, int trans_b,
                               int lda, int ldb, int ldc,
                               long long stride_a, long long stride_b,
                               long long stride_c, int batch,
                               float alpha, float beta);
/* Measurement aid, no reference counterpart: while enabled, every launch of
 * the tiled MFMA kernel is bracketed by HIP events on its stream.
 * jzhip_profile_gemm_report synchronises and writes a JSON array with, per
 * kernel instantiation, the launch count, the summed duration in ms and the
 * summed algorithmic flops (2*m*n*k), then forgets the records. */
int jzhip_profile_gemm(int enable);
int jzhip_profile_gemm_report(char* json_out, size_t capacity);
/* y(rows x cols, column-major, ld=rows) += b[i] broadcast over columns: the
 * rank-1 product `b * ones(1,N)` the layers use for every bias
 * (ml/layer.hpp:79,120,2797; CUDA add_bias_kernel ml/layer.hpp:2538-2542). */
int jzhip_add_bias(float* y, const float* b, int rows, int cols);

/* ── softmax family ──────────────────────────────────────────────────── */

/* Column softmax of a physical numrow x numcol buffer (each contiguous
 * column is one distribution): out = exp(x-max) * 1/(sum+1e-12), the
 * arithmetic of col_softmax (ml/layer.hpp:2344-2358). out may equal in. */
int jzhip_softmax_cols(float* out, const float* in, int numrow, int numcol, int ld);
/* Row softmax of the same buffer (each physical row, stride ld, is one
 * distribution): row_softmax = col_softmax(M.T()).T() (ml/layer.hpp:2364-2367). */
int jzhip_softmax_rows(float* out, const float* in, int numrow, int numcol, int ld);
/* Attention softmax over `nblk` column-major S x S score blocks stored back
 * to back, with the score scale and the causal mask fused: x = in*scale,
 * masked entries (key index > query index) are set to -1e9 before the
 * softmax exactly as the reference does (host loop ml/layer.hpp:2979-2994,
 * CUDA causal_mask_kernel :2401-2412, softmax_rows_batched_kernel
 * :2373-2399), then p = exp(x-max) * 1/(sum+1e-12).
 *   keys_along_rows == 0: element (query a, key b) of a block at a + b*S —
 *       the reference's cached_A layout; the softmax runs along a block row.
 *   keys_along_rows == 1: element (key b, query a) at b + a*S — the
 *       transposed block; the softmax runs along a contiguous column.
 * out may equal in. */
int jzhip_attn_softmax(float* out, const float* in, int S, int nblk,
                       float scale, int causal, int keys_along_rows);
/* Softmax backward for the same two layouts: dS = A*(dA - sum_keys A*dA)*scale
 * (CUDA softmax_backward_rows_kernel ml/layer.hpp:2418-2445; generic form
 * :3343-3350). dS may equal dA. */
int jzhip_attn_softmax_bwd(float* dS, const float* A, const float* dA, int S,
                           int nblk, float scale, int keys_along_rows);
/* Softmax cross-entropy of logits (K x N, one sample per column) against
 * integer labels: loss_out[0] = -(1/N) sum_n log softmax(x_n)[label_n] and,
 * when dlogits != NULL, dlogits = (softmax - onehot)/N: LogisticLayer's
 * value and gradient (ml/layer.hpp:232-284) without materialising the
 * one-hot matrix. */
int jzhip_softmax_xent(float* loss_out, float* dlogits, const float* logits,
                       const int32_t* labels, int K, int N, int ld);
/* The same against a K x N matrix of targets (leading dimension ld, as the logits), which is
 * how LogisticLayer holds them: loss_out[0] = -inv_nb * sum_n (sum_k x*y - lse_n)
 * (ml/layer.hpp:272-283) and dlogits = -(y - softmax) * inv_nb (ml/layer.hpp:252-262).
 * Either output may be NULL. */
int jzhip_softmax_xent_dense(float* loss_out, float* dlogits, const float* logits, const float* target,
                             int K, int N, int ld, float inv_nb);

/* Multi-head self-attention core over the layouts TransformerLayer keeps
 * (ml/layer.hpp:2843-2848): Q, K, V, H are (d_k, S*B) column-major with head hh
 * in rows [hh*d_h, (hh+1)*d_h) and sequence b in columns [b*S, (b+1)*S); A is
 * (S, S*B*heads) with block hh*B + b holding A[query, key].  Forward computes
 * A = softmax_keys(Q_i^T K_i / sqrt(d_h), causal mask) and H_i = V_i A_i^T for
 * every (head, sequence): the generic loop of ml/layer.hpp:2967-3006 (CUDA
 * path :2880-2927) as batched launches with the mask applied on the device. */
int jzhip_attention_fwd(float* H, float* A, const float* Q, const float* K,
                        const float* V, int d_k, int heads, int S, int B,
                        int causal);
/* Backward of the above (ml/layer.hpp:3329-3363; CUDA path :3214-3283): from dH
 * and the cached Q, K, V, A writes dQ, dK, dV; dA_scratch is caller-provided
 * storage of the size of A. */
int jzhip_attention_bwd(float* dQ, float* dK, float* dV, float* dA_scratch,
                        const float* dH, const float* Q, const float* K,
                        const float* V, const float* A, int d_k, int heads,
                        int S, int B);
/* The same two calls for operands that live inside wider matrices (Q, K, V as
 * row blocks of one stacked (3*d_k, S*B) projection and likewise dQ, dK, dV):
 * ld_qkv / ld_dqkv / ld_h / ld_dh are the leading dimensions of those buffers.
 * causal != 0 in the backward call states that A came from a causal forward
 * call (exact zeros above the diagonal), which lets it skip those key tiles.
 * causal == 2 additionally states that the entries above the diagonal of the
 * output score buffer (A forward, dA_scratch backward) already hold the zeros
 * an earlier call with causal == 1 wrote into the same buffer, so the fused
 * kernel does not write them again (a training loop reuses both buffers every
 * step; nearly half of each is such zeros).
 * For head widths 32 and 64 with S a multiple of 32 up to 256 both calls run
 * as one fused kernel per pass (scores, softmax and the second product in
 * registers); other shapes take batched GEMMs and the softmax kernels. */
int jzhip_attention_fwd_ld(float* H, int ld_h, float* A, const float* Q,
                           const float* K, const float* V, int ld_qkv, int d_k,
                           int heads, int S, int B, int causal);
int jzhip_attention_bwd_ld(float* dQ, float* dK, float* dV, int ld_dqkv,
                           float* dA_scratch, const float* dH, int ld_dh,
                           const float* Q, const float* K, const float* V,
                           int ld_qkv, const float* A, int d_k, int heads, int S,
                           int B, int causal);
/* No reference counterpart (the reference caches four S x S x batch x heads buffers per
 * block, ml/layer.hpp:2843-2848): the same attention core without any S x S matrix in
 * memory.  `jzhip_attention_flash_fwd` computes H as jzhip_attention_fwd_ld does and keeps,
 * instead of the probabilities A, two floats per query: stats, 2*S*heads*B floats, holds
 * for block hh*B + b the S row maxima of the scaled, masked scores followed by the S
 * values 1/(sum + 1e-12).  `jzhip_attention_flash_bwd` recomputes the probabilities tile
 * by tile from Q, K and stats, forms the score gradients in registers and writes dQ, dK
 * and dV from one kernel; it also needs H, the forward output (the row term of the
 * softmax derivative is sum_d dH .* H).  Every element is summed in a fixed order, so
 * results are reproducible bit for bit; against the materialising pair above they agree
 * to rounding (1e-6 relative).  Shapes: head width 32 or 64, S a multiple of 32 up to 256,
 * leading dimensions multiples of 4 and 16-byte aligned pointers; causal is 0 or 1.
 * `jzhip_attention_flash_supported` says whether a shape qualifies (1) or not (0); the two
 * calls return -1 for shapes that do not, and callers then use the pair above.  The first
 * backward call for a given (S, causal) uploads a 268-byte visiting order with a blocking
 * copy, so make that call outside a graph recording.  At S 256, 8 heads of 64, batch 64
 * the six blocks of the character model keep 1.6 MB of stats instead of 1.6 GB of
 * probabilities, and the shared 268 MB score-gradient scratch is not needed. */
int jzhip_attention_flash_supported(int d_k, int heads, int S, int B);
/* Host only, no GPU needed: the order in which jzhip_attention_flash_bwd visits the
 * (query tile, key tile) cells of one S x S block (tiles of 16).  The kernel runs S/32
 * waves; in step j wave o works on cells[2*(j*S/32 + o)] (query tile) and
 * cells[2*(j*S/32 + o) + 1] (key tile).  Returns the number of steps (S/16 + 1 with the
 * causal mask, 2*S/16 without) or -1 (bad arguments, capacity below 2*steps*S/32 ints).
 * What makes the result reproducible bit for bit: the waves of one step are on distinct
 * query tiles, every cell is visited exactly once, and a wave finishes one key tile
 * before it starts its other one. */
int jzhip_attention_flash_order(int S, int causal, int* cells, int capacity);
int jzhip_attention_flash_fwd(float* H, int ld_h, float* stats, const float* Q, const float* K,
                              const float* V, int ld_qkv, int d_k, int heads, int S, int B,
                              int causal);
int jzhip_attention_flash_bwd(float* dQ, float* dK, float* dV, int ld_dqkv, const float* dH,
                              int ld_dh, const float* Q, const float* K, const float* V,
                              int ld_qkv, const float* H, int ld_h, const float* stats, int d_k,
                              int heads, int S, int B, int causal);

/* ── LayerNorm ───────────────────────────────────────────────────────── */

/* Per column of x (dim x N): mean, biased variance, inv = 1/sqrt(var+1e-5),
 * xhat = (x-mean)*inv, y = gamma*xhat + beta; writes y, xhat (dim x N) and
 * inv_std (N). LayerNorm<D>::forward (ml/layer.hpp:2632-2639; CUDA kernel
 * :2483-2508). */
int jzhip_layernorm_fwd(float* y, float* xhat, float* inv_std, const float* x,
                        const float* gamma, const float* beta, int dim, int N);
/* dx = inv*(dxh - mean(dxh) - xhat*mean(dxh*xhat)), dxh = gamma*dy
 * (ml/layer.hpp:2674-2681; CUDA kernel :2512-2534). */
int jzhip_layernorm_bwd(float* dx, const float* dy, const float* gamma,
                        const float* xhat, const float* inv_std, int dim, int N);
/* dx = layernorm_bwd(dy) + res in one pass (res may be NULL or alias dx): the
 * residual branch of a pre-LN block adds the skip gradient right after the
 * LayerNorm backward (ml/layer.hpp:3287-3299, 3372-3376); rounds like the
 * separate add. */
int jzhip_layernorm_bwd_residual(float* dx, const float* dy, const float* gamma,
                                 const float* xhat, const float* inv_std,
                                 const float* res, int dim, int N);
/* Everything a pre-LN block's backward pass sums over the tokens around one
 * LayerNorm, in the sweep that forms dx: jzhip_layernorm_bwd_residual and
 * jzhip_layernorm_param_grads (ml/layer.hpp:2674-2686) plus, where asked for
 * (non-NULL), sum_dx[i] = sum_c dx(i, c) and sum_res[i] = sum_c res(i, c) --
 * the `sum(t, 1)` bias gradients (ml/layer.hpp:100) of the dense layers that
 * receive dx and res as their upstream gradients.  dy, xhat and res are read
 * once instead of two to three times.  dx as jzhip_layernorm_bwd_residual bit
 * for bit; the sums are added per wave over a run of columns, then over
 * workgroups in a fixed order: equal to the separate entry points to rounding
 * (<= 1e-5 relative), not bit for bit.  Takes dim <= 512 in multiples of 4
 * with 16-byte aligned operands and N >= 1024 in one sweep; other shapes run
 * the separate entry points.  sum_res needs res; res may alias dx. */
int jzhip_layernorm_bwd_residual_sums(float* dx, const float* dy, const float* gamma,
                                      const float* xhat, const float* inv_std,
                                      const float* res, float* dgamma, float* dbeta,
                                      float* sum_dx, float* sum_res, int dim, int N);
/* Tangent through the normalisation at the point cached by the forward call:
 * out = gamma .* inv*(dx - mean(dx) - xhat*mean(dx*xhat)), LayerNorm<D>::jvp
 * (ml/layer.hpp:2690-2702: two sums, three rank-1 products and four Hadamard
 * products there). */
int jzhip_layernorm_jvp(float* out, const float* dx, const float* gamma,
                        const float* xhat, const float* inv_std, int dim, int N);
/* dgamma[i] = sum_c dy*xhat, dbeta[i] = sum_c dy in one pass over dy/xhat:
 * the two sum(...,1) calls of ml/layer.hpp:2683-2686. */
int jzhip_layernorm_param_grads(float* dgamma, float* dbeta, const float* dy,
                                const float* xhat, int dim, int N);

/* ── optimisers ──────────────────────────────────────────────────────── */

/* adam_update (ml/util.cuh:166-256): m,v updated in place, g overwritten by
 * the step alpha*m_hat/(sqrt(v_hat)+eps) with the exact float expression of
 * the CPU loop (:223-245); `iteration` is the 1-based step counter the
 * caller keeps in adam_state. */
int jzhip_adam_update(float* g, float* m, float* v, size_t count, float alpha,
                      float beta1, float beta2, float eps, int iteration);
/* Adam step with the weight update fused: w -= step (the `W -= adam_update`
 * of ml/layer.hpp:108-111), and decoupled weight decay w -= alpha*wd*w when
 * wd != 0 (AdamW; no reference counterpart). g is left untouched. */
int jzhip_adamw_step(float* w, const float* g, float* m, float* v, size_t count,
                     float alpha, float beta1, float beta2, float eps,
                     float weight_decay, int iteration);

/* The same step for several tensors in one launch: a layer's weights and bias
 * (the two adam_update calls plus two in-place subtractions of Layer::update,
 * ml/layer.hpp:108-111), or all parameter tensors of a small model, where one
 * launch per tensor costs more than the arithmetic.  Each tensor carries its
 * own hyper-parameters and step counter; element for element the result is
 * that of jzhip_adamw_step. */
typedef struct jzhip_adam_tensor {
    float* w;
    const float* g;
    float* m;
    float* v;
    size_t count;
    float alpha, beta1, beta2, eps, weight_decay;
    int iteration;
} jzhip_adam_tensor;
int jzhip_adamw_step_multi(const jzhip_adam_tensor* tensors, int n_tensors);
/* The same launch in a form that can be recorded once and replayed for successive
 * steps (jzhip_graph_begin below): the step number of tensor i is
 * tensors[i].iteration + *replays_device, read when the kernel runs, and the bias
 * corrections 1/(1 - beta^step) of ml/util.cuh:226-227 are formed on the device
 * (in double, as on the host).  No reference counterpart: adam_update passes its
 * step count by value (ml/util.cuh:166-172).  jzhip_counter_add adds `delta` to an
 * int in device memory on the current stream (record it after the step's last
 * optimiser launch so that every replay advances the step). */
int jzhip_adamw_step_multi_counted(const jzhip_adam_tensor* tensors, int n_tensors,
                                   const int* replays_device);
int jzhip_counter_add(int* counter_device, int delta);

/* ── convolution data movement ───────────────────────────────────────── */

/* Juzhen::RocmIm2col / RocmCol2im (cpp/hipbackend.hpp:99-111; oracle
 * make_im2col / col2im ml/layer.hpp:1897-1925,1975-1999). Bit-exact. */
int jzhip_im2col(const float* input, float* col, int C_in, int H_in, int W_in,
                 int kH, int kW, int pad_h, int pad_w, int stride_h,
                 int stride_w, int H_out, int W_out, int N);
int jzhip_col2im(const float* col, float* dx, int C_in, int H_in, int W_in,
                 int kH, int kW, int pad_h, int pad_w, int stride_h,
                 int stride_w, int H_out, int W_out, int N);
/* Juzhen::RocmConvForwardReshapeBias / RocmConvBackwardReshape
 * (cpp/hipbackend.hpp:113-117; oracle ml/layer.hpp:1942-1973). */
int jzhip_conv_forward_reshape_bias(const float* y2d, float* out,
                                    const float* bias, int C_out, int P, int N);
int jzhip_conv_backward_reshape(const float* t, float* t2d, int C_out, int P,
                                int N);
/* Juzhen::RocmConvTransScatter / Gather / Reshape (cpp/hipbackend.hpp:119-136;
 * oracle ml/layer.hpp:2112-2221). */
int jzhip_convtrans_scatter(const float* patches, float* out, const float* bias,
                            int C_out, int H_out, int W_out, int H_in, int W_in,
                            int kH, int kW, int pad_h, int pad_w, int stride_h,
                            int stride_w, int N);
int jzhip_convtrans_gather(const float* t, float* tp, int C_out, int H_out,
                           int W_out, int H_in, int W_in, int kH, int kW,
                           int pad_h, int pad_w, int stride_h, int stride_w,
                           int N);
int jzhip_convtrans_reshape(const float* src, float* dst, int C, int spatial,
                            int N, int direction);

/* ── convolution without the patch matrix ─────────────────────────────── */

/* The three products of ConvLayer (ml/layer.hpp:1611-1719) with the patch
 * matrix formed on the fly inside the product (implicit GEMM) instead of being
 * written by RocmIm2col and read back.  Layouts are the layer's own: input
 * (C_in*H_in*W_in, N), weights the stored (K, C_out) column-major matrix with
 * K = C_in*kH*kW (ml/layer.hpp:1566-1569), out and t (C_out*H_out*W_out, N).
 *   jzhip_conv2d_forward          replaces RocmIm2col + RocmGemm(W^T col) +
 *                                 RocmConvForwardReshapeBias (+ relu when relu != 0;
 *                                 bias may be NULL)                          (:1611-1637)
 *   jzhip_conv2d_backward_weights replaces RocmConvBackwardReshape + RocmIm2col +
 *                                 RocmGemm(col t2d^T): dW in the stored (K, C_out)
 *                                 layout, t the upstream gradient after the
 *                                 activation derivative                       (:1679-1696)
 * 3x3, stride-1, pad-1 layers whose shape qualifies (jzhip_conv2d_check with which = 4, 5,
 * 6) run from image strips staged in LDS instead: every pixel is fetched once per stage, the
 * taps are the same strip at another offset.  The same geometry with one to four input
 * channels, rows in multiples of four pixels and eight or more output channels (forward and
 * backward_weights) runs as plain vector kernels bound by the output or the upstream
 * gradient passing through memory once.
 *   jzhip_conv2d_backward_data    replaces RocmGemm(W t2d) + RocmCol2im for stride 1
 *                                 (returns -1 for other strides: those keep the
 *                                 patch-matrix route); the taps of one input
 *                                 pixel are summed inside the product, so the
 *                                 result agrees with the col2im order to
 *                                 rounding, not bit for bit                   (:1698-1709) */
int jzhip_conv2d_forward(const float* input, const float* weights, const float* bias,
                         float* out, int C_in, int H_in, int W_in, int C_out, int kH,
                         int kW, int pad_h, int pad_w, int stride_h, int stride_w,
                         int H_out, int W_out, int N, int relu);
int jzhip_conv2d_backward_weights(const float* input, const float* t, float* dW, int C_in,
                                  int H_in, int W_in, int C_out, int kH, int kW, int pad_h,
                                  int pad_w, int stride_h, int stride_w, int H_out,
                                  int W_out, int N);
int jzhip_conv2d_backward_data(const float* t, const float* weights, float* dx, int C_in,
                               int H_in, int W_in, int C_out, int kH, int kW, int pad_h,
                               int pad_w, int stride_h, int stride_w, int H_out, int W_out,
                               int N);
/* Transposed convolution without the patch matrix:
 *   out(co, oy, ox; n) = bias(co) + sum over (ci, ky, kx) with (oy + pad_h - ky) % stride_h == 0 and
 *                        (ox + pad_w - kx) % stride_w == 0 of
 *                        x(ci, (oy + pad_h - ky)/stride_h, (ox + pad_w - kx)/stride_w; n) * W((co, ky, kx), ci),
 * taps outside the input counting as zero, [relu].  x is (C_in*H_in*W_in, N), out
 * (C_out*H_out*W_out, N), W the (C_out*kH*kW, C_in) column-major matrix convtransLayer stores
 * (ml/layer.hpp:1728-1766); bias may be NULL.  Replaces RocmConvTransReshape + RocmGemm +
 * RocmConvTransScatter (+ relu) of convtransLayer::eval (ml/layer.hpp:1770-1790; oracle
 * :2112-2160).  The stored (K, C_out) weights of a ConvLayer are the same bytes as the
 * (C_in*kH*kW, C_out) matrix of the transposed layer that maps its output grid back onto its
 * input grid, so with x = the upstream gradient t, C_in = the layer's C_out, C_out = the
 * layer's C_in and (H_out, W_out) = the layer's input grid this call is the input gradient of
 * a strided convolution, RocmGemm(W t2d) + RocmCol2im (ml/layer.hpp:1698-1709).  The output
 * rows with equal (oy + pad_h) % stride_h share their taps: each of the stride_h*stride_w
 * residue classes is a stride-1 convolution with the sub-kernel of those taps, run through the
 * forward kernel in one launch and stored to every stride-th pixel; the weights are regrouped
 * per class in the workspace first.  Results agree with the scatter / col2im order to
 * rounding, not bit for bit.  Limits: stride_h*stride_w <= 4, kH >= stride_h, kW >= stride_w,
 * C_in*kH*kW*C_out <= 16 Mi, H_out at most stride_h - 1 beyond (H_in-1)*stride_h - 2*pad_h + kH
 * (likewise W_out); -1 otherwise (`jzhip_conv2d_check` with which = 3 asks without launching). */
int jzhip_conv2d_transposed(const float* x, const float* weights, const float* bias, float* out,
                            int C_in, int H_in, int W_in, int C_out, int kH, int kW, int pad_h,
                            int pad_w, int stride_h, int stride_w, int H_out, int W_out, int N,
                            int relu);
/* No reference counterpart.  0 when the entry point above named by `which` (0 forward,
 * 1 backward_weights, 2 backward_data, 3 transposed) accepts this geometry, -1 when it would refuse it:
 * a dimension that is not positive, an index product beyond the kernels' 32-bit
 * arithmetic (C*H*W of an image >= 2^30, K = C_in*kH*kW >= 2^24), a patch grid larger
 * than (H_in + 2*pad - kH)/stride + 1, and for backward_data a stride other than 1,
 * pad > k - 1, H_in != H_out + kH - 1 - 2*pad or more than 16 Mi weights (they are
 * flipped into the workspace).  which = 4 asks whether backward_weights takes its kernel for
 * 3x3, stride-1, pad-1 layers that stages image strips in LDS (rows of 8, 16, 32 or 64
 * pixels, a whole number of 64-pixel stages per image and four or more in all, channel
 * counts in multiples of 32 on both sides, operands 16-byte aligned and under 2 GiB each);
 * other accepted shapes run the general kernel.  which = 5 and 6 ask the same of forward
 * and backward_data, whose strip kernel takes 3x3, stride-1, pad-1 layers with rows of 8, 16
 * or 32 pixels in whole tiles of 8, 8 or 4 rows, the product's input channels in multiples
 * of 8 and its output channels in multiples of 64 (for backward_data the product's input is
 * t and its output dx), operands 16-byte aligned and under 2 GiB each; the weights are
 * regrouped into the workspace by one small launch first.  Nothing is launched.  Callers that have a
 * patch-matrix route to fall back to (ConvLayer, convtransLayer) pick their route with it. */
int jzhip_conv2d_check(int which, int C_in, int H_in, int W_in, int C_out, int kH, int kW,
                       int pad_h, int pad_w, int stride_h, int stride_w, int H_out,
                       int W_out, int N);

#ifdef __cplusplus
}
#endif
#endif /* JZHIP_H */
