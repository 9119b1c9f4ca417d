// ROCm hook for ml/layer.hpp: include at the very end of that file,
//
//     #ifdef ROCM_HIP
//     #include "../cpp/hipfused.hpp"
//     #endif
//
// the counterpart of the `#ifdef CUDA` / `#ifdef APPLE_SILICON` blocks the
// reference keeps inside LayerNorm and TransformerLayer (ml/layer.hpp:2595-2631,
// 2646-2673, 2772-2798, 2880-2965, 3214-3283).  The members below are explicit
// specialisations for ROCMfloat, so user code and the rest of ml/layer.hpp stay
// untouched; without this include the generic formulation still compiles, but
// TransformerLayer's causal mask is then written from the host into device
// memory while the kernels that produce the scores are still in flight
// (ml/layer.hpp:2979-2994), which races.
//
// What changes against the generic path:
//   LayerNorm::forward / backward   one kernel each (+ one for dgamma/dbeta)
//   TransformerLayer::add_bias      one broadcast kernel instead of a rank-1 GEMM
//   TransformerLayer::eval/backward attention for all heads and sequences as
//                                   batched GEMMs with the mask and softmax
//                                   (and its backward) on the device; causal
//                                   blocks of a supported shape keep no S x S
//                                   matrix at all (two floats per query)
#ifndef JZ_HIPFUSED_HPP
#define JZ_HIPFUSED_HPP

#include <cstdlib>
#include <initializer_list>
#include <vector>
#include <typeinfo>

#include "jzhip.h"

namespace Juzhen {

namespace rocm_detail {
inline float* p(const Matrix<ROCMfloat>& m) { return JzRocmFused::ptr(m); }
inline void must(int rc, const char* what) {
    if (rc != 0) {
        std::cerr << "juzhen rocm: " << what << " failed with code " << rc << " (" << jzhip_error_string(rc)
                  << ")" << std::endl;
        ERROR_OUT;
    }
}
// plain column-major copy of a possibly transposed operand
inline Matrix<ROCMfloat> plain(const Matrix<ROCMfloat>& m) {
    return m.get_transpose() ? JzRocmFused::materialise(m) : Matrix<ROCMfloat>(m);
}

// `W -= adam_update(g, state)` for several parameter tensors in one launch
// (ml/layer.hpp:108-111, 2683-2686, 3377-3387 issue an Adam kernel and an
// in-place subtraction per tensor).  Element for element the arithmetic is the
// same; tensors held as transposed views take the per-tensor path.
struct AdamItem {
    Matrix<ROCMfloat>* w;
    Matrix<ROCMfloat>* g;
    adam_state<ROCMfloat>* st;
};
// What a recording in progress (RocmStepGraph below) needs from the optimiser launches it
// records: the device counter of replays their step numbers are offset by, and the list
// of optimiser states whose host-side step count a replay has to advance.
struct GraphRecording {
    int* replays_device = nullptr;
    std::vector<adam_state<ROCMfloat>*> states;
};
inline GraphRecording*& current_recording() {
    static GraphRecording* r = nullptr;
    return r;
}
inline void fused_update(std::initializer_list<AdamItem> items) {
    bool all_plain = items.size() <= 16;
    for (const AdamItem& it : items) {
        const size_t n = it.w->num_row() * it.w->num_col();
        all_plain = all_plain && !it.w->get_transpose() && !it.g->get_transpose() && !it.st->m.get_transpose() &&
                    !it.st->v.get_transpose() && it.g->num_row() * it.g->num_col() == n &&
                    it.st->m.num_row() * it.st->m.num_col() == n && it.st->v.num_row() * it.st->v.num_col() == n &&
                    it.g->num_row() == it.w->num_row();
    }
    GraphRecording* rec = jzhip_graph_recording() ? current_recording() : nullptr;
    if (jzhip_graph_recording() && (!rec || !all_plain)) {
        std::cerr << "juzhen rocm: an optimiser step on transposed views, or outside a RocmStepGraph, cannot be recorded"
                  << std::endl;
        ERROR_OUT;
    }
    if (!all_plain) {
        for (const AdamItem& it : items) *it.w -= adam_update(std::move(*it.g), *it.st);
        return;
    }
    jzhip_adam_tensor t[16];
    int n = 0;
    for (const AdamItem& it : items) {
        t[n].w = p(*it.w); t[n].g = p(*it.g); t[n].m = p(it.st->m); t[n].v = p(it.st->v);
        t[n].count = it.w->num_row() * it.w->num_col();
        t[n].alpha = it.st->alpha; t[n].beta1 = it.st->beta1; t[n].beta2 = it.st->beta2; t[n].eps = it.st->eps;
        t[n].weight_decay = 0.0f;
        t[n].iteration = it.st->iteration;
        ++n;
    }
    if (rec) {
        // recorded: step number = iteration now + replays so far, formed on the device; the host-side
        // counts are advanced by RocmStepGraph::replay()
        must(jzhip_adamw_step_multi_counted(t, n, rec->replays_device), "adamw_step_multi_counted");
        for (const AdamItem& it : items) rec->states.push_back(it.st);
        return;
    }
    must(jzhip_adamw_step_multi(t, n), "adamw_step_multi");
    for (const AdamItem& it : items) it.st->iteration++;
}

}  // namespace rocm_detail

// A training step recorded once and replayed as one HIP graph launch, for models whose step
// is a few hundred small kernels and therefore bound by launch cost (no counterpart in the
// reference, which launches every kernel from the host each step).
//
//     RocmStepGraph graph;
//     graph.begin();                       // calls below are recorded, not run
//     forward(net, X); ... backprop(net, X);
//     graph.end();
//     for (...) graph.replay();            // each replay is the next optimiser step
//
// The recorded step works on the buffers it was recorded with (inputs, layer values,
// temporaries from the pool), so the batch is whatever X holds at replay time and results
// are read from the same matrices after any replay.  While recording: no host reads of
// device data (item(), to_host()), no host-to-device construction, no random draws (a
// replay would repeat them), and parameter updates only through the layers' backward().
// Run at least one ordinary step first so that the pool already holds every buffer size.
class RocmStepGraph {
    void* exec = nullptr;
    float* counter = nullptr;   // one int in device memory: replays so far
    rocm_detail::GraphRecording rec;
    // every buffer created while recording (layer values, temporaries): the replays write
    // them, so they stay out of the pool until the graph is destroyed
    std::vector<std::shared_ptr<ROCMfloat[]>> pinned;

   public:
    RocmStepGraph() = default;
    RocmStepGraph(const RocmStepGraph&) = delete;
    RocmStepGraph& operator=(const RocmStepGraph&) = delete;
    ~RocmStepGraph() {
        if (exec) jzhip_graph_destroy(exec);   // waits for the streams the replays were launched on
        if (counter) jzhip_free(counter);
        pinned.clear();                        // the buffers return to the pool
    }
    void begin() {
        using namespace rocm_detail;
        if (exec || current_recording()) {
            std::cerr << "juzhen rocm: RocmStepGraph::begin() on a graph that is recorded or recording" << std::endl;
            ERROR_OUT;
        }
        must(jzhip_malloc(&counter, 1), "malloc");
        must(jzhip_fill(counter, 1, 0.0f), "fill");   // all-zero bits: the int 0
        rec.replays_device = reinterpret_cast<int*>(counter);
        rec.states.clear();
        must(jzhip_graph_begin(), "graph_begin");
        (void)JzRocmFused::take_recording_pins();   // start from an empty list
        current_recording() = &rec;
    }
    void end() {
        using namespace rocm_detail;
        if (current_recording() != &rec) {
            std::cerr << "juzhen rocm: RocmStepGraph::end() without begin()" << std::endl;
            ERROR_OUT;
        }
        // the last recorded launch: every replay advances the optimiser step
        must(jzhip_counter_add(rec.replays_device, 1), "counter_add");
        current_recording() = nullptr;
        must(jzhip_graph_end(&exec), "graph_end");
        pinned = JzRocmFused::take_recording_pins();
    }
    void replay() {
        using namespace rocm_detail;
        if (!exec) {
            std::cerr << "juzhen rocm: RocmStepGraph::replay() before end()" << std::endl;
            ERROR_OUT;
        }
        must(jzhip_graph_launch(exec), "graph_launch");
        for (adam_state<ROCMfloat>* st : rec.states) st->iteration++;
    }
};

namespace rocm_detail {

// weights * input + bias * ones(1, n) (+ ReLU) in one launch: the chain every
// dense layer's eval() and grad() issues as a product, a rank-1 product, an
// addition and an activation (ml/layer.hpp:77-80, 118-121, 174-177, 189-195).
// Each step rounds as the separate kernels do.
inline Matrix<ROCMfloat> dense_affine(const Matrix<ROCMfloat>& W, const Matrix<ROCMfloat>& x,
                                      const Matrix<ROCMfloat>& b, int act) {
    const size_t m = W.num_row(), k = W.num_col(), n = x.num_col();
    if (k != x.num_row() || b.num_row() != m || b.num_col() != 1)
        throw std::invalid_argument("Matrix dimensions are not compatible");
    Matrix<ROCMfloat> out = JzRocmFused::make("affine", m, n, 0);
    if (m == 0 || n == 0) return out;
    if (k == 0) {   // empty contraction: the bias alone
        out.zeros();
        must(jzhip_add_bias(p(out), p(b), (int)m, (int)n), "add_bias");
        if (act == 1) must(jzhip_relu(p(out), p(out), m * n), "relu");
        return out;
    }
    must(jzhip_gemm_fused(p(W), p(x), p(out), (int)m, (int)n, (int)k, (int)W.get_transpose(), (int)x.get_transpose(),
                          (int)JzRocmFused::phys_rows(W), (int)JzRocmFused::phys_rows(x), (int)m, 1.0f, 0.0f, p(b), act,
                          nullptr, (int)m, nullptr, (int)m),
         "gemm_fused");
    return out;
}
}  // namespace rocm_detail

// ── dense layers (ml/layer.hpp:52-196) ───────────────────────────────────────

template <>
inline void Layer<ROCMfloat>::eval(const Matrix<ROCMfloat>& input) {
    val = tanh(rocm_detail::dense_affine(weights, input, bias, 0));
}
template <>
inline Matrix<ROCMfloat> Layer<ROCMfloat>::grad(const Matrix<ROCMfloat>& input) const {
    return d_tanh(rocm_detail::dense_affine(weights, input, bias, 0));
}
template <>
inline void LinearLayer<ROCMfloat>::eval(const Matrix<ROCMfloat>& input) {
    Layer<ROCMfloat>::val = rocm_detail::dense_affine(Layer<ROCMfloat>::weights, input, Layer<ROCMfloat>::bias, 0);
}
template <>
inline void ReluLayer<ROCMfloat>::eval(const Matrix<ROCMfloat>& input) {
    Layer<ROCMfloat>::val = rocm_detail::dense_affine(Layer<ROCMfloat>::weights, input, Layer<ROCMfloat>::bias, 1);
}
template <>
inline Matrix<ROCMfloat> ReluLayer<ROCMfloat>::grad(const Matrix<ROCMfloat>& input) const {
    return d_relu(rocm_detail::dense_affine(Layer<ROCMfloat>::weights, input, Layer<ROCMfloat>::bias, 0));
}

// Layer::backward (ml/layer.hpp:96-105) with the same statements in the same
// order; what changes is how many launches they take.  The activation
// derivative times the upstream gradient is one pass for the two layer kinds
// whose derivative is known here (all ones for LinearLayer: the product with
// ones is the upstream gradient itself; the ReLU mask for ReluLayer); any other
// subclass goes through its own grad().  Weights and bias take one optimiser
// launch together.  As in the reference, the returned input gradient is formed
// with the weights after their update.
template <>
inline Matrix<ROCMfloat> Layer<ROCMfloat>::backward(const Matrix<ROCMfloat>& input, Matrix<ROCMfloat>&& upstream_grad) {
    using namespace rocm_detail;
    using MD = Matrix<ROCMfloat>;
    MD t = [&]() -> MD {
        if (typeid(*this) == typeid(LinearLayer<ROCMfloat>)) return std::move(upstream_grad);
        if (typeid(*this) == typeid(ReluLayer<ROCMfloat>) && !upstream_grad.get_transpose()) {
            MD pre = dense_affine(weights, input, bias, 0);
            if (pre.num_row() != upstream_grad.num_row() || pre.num_col() != upstream_grad.num_col())
                throw std::invalid_argument("Matrix dimensions are not compatible");
            must(jzhip_drelu_mul(p(upstream_grad), p(pre), p(upstream_grad), pre.num_row() * pre.num_col()), "drelu_mul");
            return std::move(upstream_grad);
        }
        return hadmd(grad(input), std::move(upstream_grad));
    }();
    // the two parameter gradients from one pass over t where both operands are stored plainly
    MD gW = JzRocmFused::make("gW", 0, 0, 0), gb = JzRocmFused::make("gb", 0, 0, 0);
    if (!t.get_transpose() && !input.get_transpose() && t.num_col() == input.num_col() && t.num_row() > 0 &&
        input.num_row() > 0 && t.num_col() > 0) {
        const int m = (int)t.num_row(), n = (int)input.num_row(), k = (int)t.num_col();
        gW = JzRocmFused::make("gW", m, n, 0);
        gb = MD("gb", m, 1);
        must(jzhip_gemm_rowsum(p(t), p(input), p(gW), p(gb), m, n, k, 0, 1, m, n, m, 1.0f, 0.0f), "gemm_rowsum");
    } else {
        gW = t * input.T();
        gb = sum(t, 1);
    }
    // (Layer::update itself cannot be specialised here: the ROCm ConvLayer bodies earlier in
    // ml/layer.hpp have already instantiated it)
    if (need_update) fused_update({{&weights, &gW, &adamW}, {&bias, &gb, &adamb}});
    return W().T() * t;
}

// ── squared-error head (ml/layer.hpp:204-227) ────────────────────────────────
// eval() is five matrix operations and seven launches in the generic form, grad() three;
// with both operands stored the same way each is one launch over the flat buffers, every
// element rounded as the separate operations round it.
template <>
inline void LossLayer<ROCMfloat>::eval(const Matrix<ROCMfloat>& input) {
    using namespace rocm_detail;
    if (input.num_row() != output.num_row() || input.num_col() != output.num_col() ||
        input.get_transpose() != output.get_transpose()) {
        Layer<ROCMfloat>::val = sum(sum(square(output - input), 0), 1) / Layer<ROCMfloat>::nb;
        return;
    }
    Matrix<ROCMfloat> v = JzRocmFused::make("loss", 1, 1, 0);
    must(jzhip_mse_loss(p(v), p(output), p(input), input.num_row() * input.num_col(),
                        (float)(1.0 / Layer<ROCMfloat>::nb)),
         "mse_loss");
    Layer<ROCMfloat>::val = std::move(v);
}
template <>
inline Matrix<ROCMfloat> LossLayer<ROCMfloat>::grad(const Matrix<ROCMfloat>& input) const {
    using namespace rocm_detail;
    // (a difference is returned untransposed, cpp/core.hpp:414-449: transposed operands keep
    // the generic form, which turns them)
    if (input.num_row() != output.num_row() || input.num_col() != output.num_col() ||
        input.get_transpose() || output.get_transpose())
        return 2.0 * (input - output) / Layer<ROCMfloat>::nb;
    Matrix<ROCMfloat> g = JzRocmFused::make("loss_grad", input.num_row(), input.num_col(), 0);
    must(jzhip_mse_grad(p(g), p(input), p(output), input.num_row() * input.num_col(),
                        (float)(1.0 / Layer<ROCMfloat>::nb)),
         "mse_grad");
    return g;
}

// ── softmax cross-entropy head (ml/layer.hpp:232-284) ────────────────────────
// eval() and grad() are each a dozen matrix operations in the generic form (a functor
// reduction for the column maxima, two rank-1 products, exp, sums, log, a Hadamard product);
// here each is one pass over the logits with one wavefront per sample, plus the mean.
// Operands whose transpose flag is set are turned first, so the kernel sees K x N buffers.
namespace rocm_detail {
inline Matrix<ROCMfloat> xent_head(const Matrix<ROCMfloat>& input, const Matrix<ROCMfloat>& target, size_t nb,
                                   bool want_grad) {
    if (input.num_row() != target.num_row() || input.num_col() != target.num_col())
        throw std::invalid_argument("Matrix dimensions are not compatible");
    Matrix<ROCMfloat> turned_x = JzRocmFused::make("x", 0, 0, 0), turned_y = JzRocmFused::make("y", 0, 0, 0);
    if (input.get_transpose()) turned_x = JzRocmFused::materialise(input);
    if (target.get_transpose()) turned_y = JzRocmFused::materialise(target);
    const Matrix<ROCMfloat>& x = input.get_transpose() ? turned_x : input;
    const Matrix<ROCMfloat>& y = target.get_transpose() ? turned_y : target;
    const size_t K = x.num_row(), N = x.num_col();
    Matrix<ROCMfloat> out = want_grad ? JzRocmFused::make("xent_grad", K, N, 0) : JzRocmFused::make("xent", 1, 1, 0);
    if (K == 0 || N == 0) {
        out.zeros();
        return out;
    }
    must(jzhip_softmax_xent_dense(want_grad ? nullptr : p(out), want_grad ? p(out) : nullptr, p(x), p(y), (int)K,
                                  (int)N, (int)K, (float)(1.0 / nb)),
         "softmax_xent_dense");
    return out;
}
}  // namespace rocm_detail
template <>
inline void LogisticLayer<ROCMfloat>::eval(const Matrix<ROCMfloat>& input) {
    Layer<ROCMfloat>::val = rocm_detail::xent_head(input, output, Layer<ROCMfloat>::nb, false);
}
template <>
inline Matrix<ROCMfloat> LogisticLayer<ROCMfloat>::grad(const Matrix<ROCMfloat>& input) const {
    return rocm_detail::xent_head(input, output, Layer<ROCMfloat>::nb, true);
}

// ── LayerNorm ────────────────────────────────────────────────────────────────

template <>
inline Matrix<ROCMfloat> LayerNorm<ROCMfloat>::forward(const Matrix<ROCMfloat>& x) {
    using namespace rocm_detail;
    if (x.get_transpose()) return forward(JzRocmFused::materialise(x));
    const int N = (int)x.num_col();
    if ((int)cached_xhat.num_col() != N || cached_xhat.get_transpose()) {
        cached_xhat = Matrix<ROCMfloat>("ln_xhat", dim, N);
        cached_inv = Matrix<ROCMfloat>("ln_inv", 1, N);
    }
    Matrix<ROCMfloat> y("ln_y", dim, N);
    must(jzhip_layernorm_fwd(p(y), p(cached_xhat), p(cached_inv), p(x), p(gamma), p(beta), dim, N),
         "layernorm_fwd");
    return y;
}

template <>
inline Matrix<ROCMfloat> LayerNorm<ROCMfloat>::backward(Matrix<ROCMfloat>&& dy, bool update) {
    using namespace rocm_detail;
    if (dy.get_transpose()) return backward(JzRocmFused::materialise(dy), update);
    const int N = (int)dy.num_col();
    Matrix<ROCMfloat> dx("ln_dx", dim, N);
    // dx reads gamma, so the parameter step comes second (ml/layer.hpp:2682-2686)
    if (update) {
        // one sweep over dy and xhat for dx and the two parameter gradients
        Matrix<ROCMfloat> dg("ln_dgamma", dim, 1), db("ln_dbeta", dim, 1);
        must(jzhip_layernorm_bwd_residual_sums(p(dx), p(dy), p(gamma), p(cached_xhat), p(cached_inv), nullptr, p(dg),
                                               p(db), nullptr, nullptr, dim, N),
             "layernorm_bwd_residual_sums");
        fused_update({{&gamma, &dg, &adam_g}, {&beta, &db, &adam_b}});
        return dx;
    }
    must(jzhip_layernorm_bwd(p(dx), p(dy), p(gamma), p(cached_xhat), p(cached_inv), dim, N), "layernorm_bwd");
    return dx;
}

// Tangent through the normalisation at the point cached by forward()
// (ml/layer.hpp:2690-2702): one kernel instead of two sums, three rank-1
// products and four Hadamard products.
template <>
inline Matrix<ROCMfloat> LayerNorm<ROCMfloat>::jvp(const Matrix<ROCMfloat>& dx) const {
    using namespace rocm_detail;
    if (dx.get_transpose()) return jvp(JzRocmFused::materialise(dx));
    const int N = (int)dx.num_col();
    Matrix<ROCMfloat> out("ln_jvp", dim, N);
    must(jzhip_layernorm_jvp(p(out), p(dx), p(gamma), p(cached_xhat), p(cached_inv), dim, N), "layernorm_jvp");
    return out;
}

// ── TransformerLayer ─────────────────────────────────────────────────────────

template <>
inline void TransformerLayer<ROCMfloat>::add_bias(Matrix<ROCMfloat>& y, const Matrix<ROCMfloat>& b) {
    using namespace rocm_detail;
    if (!y.get_transpose() && !b.get_transpose()) {
        must(jzhip_add_bias(p(y), p(b), (int)y.num_row(), (int)y.num_col()), "add_bias");
        return;
    }
    y += b * ones_1N;
}

// op(W) * x with the rest of the statement it belongs to in the product's store:
//   out = act(op(W) x + bias) + residual,   act 0 none, 1 ReLU (pre-activation kept in *aux),
//                                           3 multiply by ReLU'(*aux) instead
// Every step rounds as the separate kernel it replaces (add_bias, relu / drelu_mul,
// operator+), so the block computes the same bits as the statement-by-statement form.
// x, aux and residual must be plain (callers materialise transposed views first).
namespace rocm_detail {
// *rowsum (optional) receives sum(out, 1), added up by the workgroups that store out.
inline Matrix<ROCMfloat> fused_product(const Matrix<ROCMfloat>& W, bool transpose_w, const Matrix<ROCMfloat>& x,
                                       const Matrix<ROCMfloat>* bias, int act, Matrix<ROCMfloat>* aux,
                                       const Matrix<ROCMfloat>* residual, Matrix<ROCMfloat>* rowsum = nullptr) {
    const bool tw = transpose_w != (bool)W.get_transpose();
    const size_t m = transpose_w ? W.num_col() : W.num_row(), k = transpose_w ? W.num_row() : W.num_col();
    const size_t n = x.num_col();
    if (k != x.num_row() || x.get_transpose() || (bias && (bias->num_row() * bias->num_col() != m)) ||
        (aux && (aux->get_transpose() || aux->num_row() != m || aux->num_col() != n)) ||
        (residual && (residual->get_transpose() || residual->num_row() != m || residual->num_col() != n)))
        throw std::invalid_argument("Matrix dimensions are not compatible");
    Matrix<ROCMfloat> out = JzRocmFused::make("fused_product", m, n, 0);
    if (rowsum) {
        *rowsum = Matrix<ROCMfloat>("fused_product_rowsum", m, 1);
        must(jzhip_gemm_fused_rowsum(p(W), p(x), p(out), p(*rowsum), (int)m, (int)n, (int)k, tw ? 1 : 0, 0,
                                     (int)JzRocmFused::phys_rows(W), (int)k, (int)m, 1.0f, 0.0f,
                                     bias ? p(*bias) : nullptr, act, aux ? p(*aux) : nullptr, (int)m,
                                     residual ? p(*residual) : nullptr, (int)m),
             "gemm_fused_rowsum");
        return out;
    }
    must(jzhip_gemm_fused(p(W), p(x), p(out), (int)m, (int)n, (int)k, tw ? 1 : 0, 0, (int)JzRocmFused::phys_rows(W),
                          (int)k, (int)m, 1.0f, 0.0f, bias ? p(*bias) : nullptr, act, aux ? p(*aux) : nullptr, (int)m,
                          residual ? p(*residual) : nullptr, (int)m),
         "gemm_fused");
    return out;
}
// LayerNorm::backward followed by `+ residual` (ml/layer.hpp:3309, 3371) as one pass over dy
// The three projections of a block can share a launch when their weights are stored alike
// (plain column-major, equal shapes) and the input is plain too.
inline bool qkv_as_one_launch(const Matrix<ROCMfloat>& Wq, const Matrix<ROCMfloat>& Wk, const Matrix<ROCMfloat>& Wv,
                              const Matrix<ROCMfloat>& x) {
    auto same = [&](const Matrix<ROCMfloat>& W) {
        return !W.get_transpose() && W.num_row() == Wq.num_row() && W.num_col() == Wq.num_col();
    };
    return same(Wq) && same(Wk) && same(Wv) && !x.get_transpose() && x.num_row() == Wq.num_col() &&
           Wq.num_row() > 0 && Wq.num_col() > 0 && x.num_col() > 0;
}
// a, b, c (equal shapes, plain) copied back to back into one buffer
inline Matrix<ROCMfloat> stacked_blocks(const char* name, const Matrix<ROCMfloat>& a, const Matrix<ROCMfloat>& b,
                                        const Matrix<ROCMfloat>& c) {
    const size_t n = a.num_row() * a.num_col();
    Matrix<ROCMfloat> out = JzRocmFused::make(name, a.num_row(), 3 * a.num_col(), 0);
    must(jzhip_copy(p(out), p(a), n), "copy");
    must(jzhip_copy(p(out) + n, p(b), n), "copy");
    must(jzhip_copy(p(out) + 2 * n, p(c), n), "copy");
    return out;
}

// sum_dx / sum_res (optional): the row sums of the result and of the residual, i.e. the bias
// gradients `sum(t, 1)` (ml/layer.hpp:100) of the dense layers those two matrices are the
// upstream gradients of, formed in the same sweep.
inline Matrix<ROCMfloat> ln_backward_plus(LayerNorm<ROCMfloat>& ln, Matrix<ROCMfloat>&& dy,
                                          const Matrix<ROCMfloat>& residual, bool update,
                                          Matrix<ROCMfloat>* sum_dx = nullptr, Matrix<ROCMfloat>* sum_res = nullptr) {
    if (dy.get_transpose() || residual.get_transpose()) {
        if (sum_res) *sum_res = sum(residual, 1);
        Matrix<ROCMfloat> dx = ln.backward(std::move(dy), update) + residual;
        if (sum_dx) *sum_dx = sum(dx, 1);
        return dx;
    }
    const int N = (int)dy.num_col();
    Matrix<ROCMfloat> dx("ln_dx", ln.dim, N);
    if (sum_dx) *sum_dx = Matrix<ROCMfloat>("ln_sum_dx", ln.dim, 1);
    if (sum_res) *sum_res = Matrix<ROCMfloat>("ln_sum_res", ln.dim, 1);
    if (update) {
        // one sweep: dx, the parameter gradients and the row sums; dx reads gamma, so the
        // parameter step comes after it (ml/layer.hpp:2682-2686)
        Matrix<ROCMfloat> dg("ln_dgamma", ln.dim, 1), db("ln_dbeta", ln.dim, 1);
        must(jzhip_layernorm_bwd_residual_sums(p(dx), p(dy), p(ln.gamma), p(ln.cached_xhat), p(ln.cached_inv), p(residual),
                                               p(dg), p(db), sum_dx ? p(*sum_dx) : nullptr,
                                               sum_res ? p(*sum_res) : nullptr, ln.dim, N),
             "layernorm_bwd_residual_sums");
        fused_update({{&ln.gamma, &dg, &ln.adam_g}, {&ln.beta, &db, &ln.adam_b}});
        return dx;
    }
    must(jzhip_layernorm_bwd_residual(p(dx), p(dy), p(ln.gamma), p(ln.cached_xhat), p(ln.cached_inv), p(residual),
                                      ln.dim, N),
         "layernorm_bwd_residual");
    if (sum_dx) must(jzhip_sum_rows(p(*sum_dx), p(dx), ln.dim, N, ln.dim), "sum_rows");
    if (sum_res) must(jzhip_sum_rows(p(*sum_res), p(residual), ln.dim, N, ln.dim), "sum_rows");
    return dx;
}
}  // namespace rocm_detail

namespace rocm_detail {
// Causal blocks of a supported shape run the attention pair that keeps no S x S matrix:
// eval() leaves two floats per query in the head of attn_scores_scratch instead of the
// probabilities in cached_A, backward() recomputes them tile by tile, and jvp(), which
// reads cached_A, fills it first.  (Without the mask the materialising pair is the faster
// one on MI355X and stays.)  JZ_MATERIALISE_ATTENTION=1 keeps the probabilities for every block.
inline bool attention_without_scores(bool causal, int d_k, int heads, int S, int B) {
    static const bool forced_off = [] {
        const char* e = std::getenv("JZ_MATERIALISE_ATTENTION");
        return e && e[0] == '1';
    }();
    return causal && !forced_off && jzhip_attention_flash_supported(d_k, heads, S, B) == 1;
}
}  // namespace rocm_detail

// TransformerLayer::eval (ml/layer.hpp:2946-3031) with the same statements in the same
// order; biases, ReLU and the two residual additions ride in the stores of the products
// they follow instead of being passes of their own over (d, N) and (d_ff, N) matrices.
template <>
inline void TransformerLayer<ROCMfloat>::eval(const Matrix<ROCMfloat>& input_in) {
    using namespace rocm_detail;
    using MD = Matrix<ROCMfloat>;
    MD held;
    if (input_in.get_transpose()) held = JzRocmFused::materialise(input_in);
    const MD& input = input_in.get_transpose() ? held : input_in;
    const int N = seq_len * batchN;
    // pre-norm attention
    cached_x1 = ln1.forward(input);
    if (qkv_as_one_launch(Wq, Wk, Wv, cached_x1)) {
        // Q, K, V = Wq x1, Wk x1, Wv x1 as one strided-batched launch: the weights copied into
        // three consecutive blocks, the results three consecutive blocks of one buffer (three
        // products of 512 tiles each fill half the chip; together they run as one and a half rounds)
        const size_t wsz = (size_t)d_k * d_model, qsz = (size_t)d_k * N;
        MD wblk = stacked_blocks("wqkv", Wq, Wk, Wv);
        MD qkv = JzRocmFused::make("qkv", d_k, 3 * (size_t)N, 0);
        must(jzhip_gemm_strided_batched(p(wblk), p(cached_x1), p(qkv), d_k, N, d_model, 0, 0, d_k, d_model, d_k,
                                        (long long)wsz, 0, (long long)qsz, 3, 1.0f, 0.0f),
             "gemm_strided_batched");
        cached_Q = JzRocmFused::block("tq", qkv, 0, d_k, N);
        cached_K = JzRocmFused::block("tk", qkv, qsz, d_k, N);
        cached_V = JzRocmFused::block("tv", qkv, 2 * qsz, d_k, N);
    } else {
        cached_Q = Wq * cached_x1;
        cached_K = Wk * cached_x1;
        cached_V = Wv * cached_x1;
    }
    if (attention_without_scores(causal, d_k, num_heads, seq_len, batchN)) {
        must(jzhip_attention_flash_fwd(p(cached_H), d_k, p(attn_scores_scratch), p(cached_Q), p(cached_K), p(cached_V), d_k,
                                       d_k, num_heads, seq_len, batchN, 1),
             "attention_flash_fwd");
    } else {
        must(jzhip_attention_fwd(p(cached_H), p(cached_A), p(cached_Q), p(cached_K), p(cached_V), d_k, num_heads,
                                 seq_len, batchN, causal ? 1 : 0),
             "attention_fwd");
    }
    // R = input + (Wo H + bo)
    cached_R = fused_product(Wo, false, cached_H, &bo, 0, nullptr, &input);
    // pre-norm feed-forward: F1 = W1 x2 + b1 kept beside relu(F1)
    cached_x2 = ln2.forward(cached_R);
    if (cached_F1.get_transpose() || (int)cached_F1.num_row() != d_ff || (int)cached_F1.num_col() != N)
        cached_F1 = MD("cached_F1", d_ff, N);
    cached_F1_relu = fused_product(W1, false, cached_x2, &b1, 1, &cached_F1, nullptr);
    // val = R + (W2 relu(F1) + b2)
    this->val = fused_product(W2, false, cached_F1_relu, &b2, 0, nullptr, &cached_R);
}

template <>
inline Matrix<ROCMfloat> TransformerLayer<ROCMfloat>::backward(const Matrix<ROCMfloat>& input,
                                                               Matrix<ROCMfloat>&& upstream_grad) {
    using namespace rocm_detail;
    using MD = Matrix<ROCMfloat>;
    const int N = seq_len * batchN;
    // read three times below; also the residual gradient
    MD dout = upstream_grad.get_transpose() ? JzRocmFused::materialise(upstream_grad) : std::move(upstream_grad);

    // feed-forward: F = W2 relu(W1 x2 + b1) + b2
    MD dW2 = dout * cached_F1_relu.T();
    MD db1 = JzRocmFused::make("db1", 0, 0, 0);
    MD dF1 = fused_product(W2, true, dout, nullptr, 3, &cached_F1, nullptr, &db1);   // (W2^T dout) .* relu'(F1); db1 = sum(dF1, 1)
    MD dW1 = dF1 * cached_x2.T();
    // the sweep that forms dR = LN2'(..) + dout also adds up the rows of dout and of dR: the
    // bias gradients db2 = sum(dout, 1) and dbo = sum(dR, 1)
    MD db2 = JzRocmFused::make("db2", 0, 0, 0), dbo = JzRocmFused::make("dbo", 0, 0, 0);
    MD dR = ln_backward_plus(ln2, W1.T() * dF1, dout, this->need_update, &dbo, &db2);

    // output projection: O = Wo H + bo
    MD dWo = dR * cached_H.T();
    MD dH = Wo.T() * dR;

    // attention core, all heads and sequences at once, then the three projections
    const size_t wsz = (size_t)d_k * d_model;
    MD dWq = JzRocmFused::make("dWq", 0, 0, 0), dWk = JzRocmFused::make("dWk", 0, 0, 0), dWv = JzRocmFused::make("dWv", 0, 0, 0);
    MD dx1 = JzRocmFused::make("dx1", 0, 0, 0);
    if (qkv_as_one_launch(Wq, Wk, Wv, cached_x1)) {
        // dQ, dK, dV as the row blocks of one (3 d_k x N) matrix.  The core is told when the forward
        // pass was causal: the probabilities above the diagonal are exact zeros and those key tiles
        // are skipped.
        MD dqkv = JzRocmFused::make("dqkv", 3 * (size_t)d_k, N, 0);
        if (attention_without_scores(causal, d_k, num_heads, seq_len, batchN)) {
            must(jzhip_attention_flash_bwd(p(dqkv), p(dqkv) + d_k, p(dqkv) + 2 * (size_t)d_k, 3 * d_k, p(dH), d_k, p(cached_Q),
                                           p(cached_K), p(cached_V), d_k, p(cached_H), d_k, p(attn_scores_scratch), d_k,
                                           num_heads, seq_len, batchN, 1),
                 "attention_flash_bwd");
        } else {
            must(jzhip_attention_bwd_ld(p(dqkv), p(dqkv) + d_k, p(dqkv) + 2 * (size_t)d_k, 3 * d_k, p(attn_dS_scratch), p(dH),
                                        d_k, p(cached_Q), p(cached_K), p(cached_V), d_k, p(cached_A), d_k, num_heads,
                                        seq_len, batchN, causal ? 1 : 0),
                 "attention_bwd");
        }
        // dW_i = dX_i x1^T for the three projections: one batched launch, K split over the tokens
        MD dw = JzRocmFused::make("dwqkv", d_k, 3 * (size_t)d_model, 0);
        must(jzhip_gemm_strided_batched(p(dqkv), p(cached_x1), p(dw), d_k, d_model, N, 0, 1, 3 * d_k, d_model, d_k,
                                        (long long)d_k, 0, (long long)wsz, 3, 1.0f, 0.0f),
             "gemm_strided_batched");
        dWq = JzRocmFused::block("dWq", dw, 0, d_k, d_model);
        dWk = JzRocmFused::block("dWk", dw, wsz, d_k, d_model);
        dWv = JzRocmFused::block("dWv", dw, 2 * wsz, d_k, d_model);
        // dx1 = Wq^T dQ + Wk^T dK + Wv^T dV = [Wq; Wk; Wv]^T [dQ; dK; dV]: one product over 3 d_k
        MD wrows = JzRocmFused::make("wqkv_rows", 3 * (size_t)d_k, d_model, 0);
        const MD* ws[3] = {&Wq, &Wk, &Wv};
        for (int i = 0; i < 3; ++i)
            must(jzhip_stack_copy_rows(p(wrows), 3 * (size_t)d_k, (size_t)i * d_k, p(*ws[i]), d_k, d_model, 0), "stack_copy_rows");
        dx1 = JzRocmFused::make("dx1", d_model, N, 0);
        must(jzhip_gemm(p(wrows), p(dqkv), p(dx1), d_model, N, 3 * d_k, 1, 0, 3 * d_k, 3 * d_k, d_model, 1.0f, 0.0f), "gemm");
    } else {
        MD dQ("dQ", d_k, N), dK("dK", d_k, N), dV("dV", d_k, N);
        if (attention_without_scores(causal, d_k, num_heads, seq_len, batchN)) {
            must(jzhip_attention_flash_bwd(p(dQ), p(dK), p(dV), d_k, p(dH), d_k, p(cached_Q), p(cached_K), p(cached_V), d_k,
                                           p(cached_H), d_k, p(attn_scores_scratch), d_k, num_heads, seq_len, batchN, 1),
                 "attention_flash_bwd");
        } else {
            must(jzhip_attention_bwd(p(dQ), p(dK), p(dV), p(attn_dS_scratch), p(dH), p(cached_Q), p(cached_K),
                                     p(cached_V), p(cached_A), d_k, num_heads, seq_len, batchN),
                 "attention_bwd");
        }
        dWq = dQ * cached_x1.T();
        dWk = dK * cached_x1.T();
        dWv = dV * cached_x1.T();
        // dx1 = Wq^T dQ + Wk^T dK + Wv^T dV: the second and third products add into the first
        dx1 = Wq.T() * dQ;
        auto add_product = [&](const MD& W, const MD& g) {
            must(jzhip_gemm(p(W), p(g), p(dx1), d_model, N, d_k, W.get_transpose() ? 0 : 1, 0, (int)JzRocmFused::phys_rows(W),
                            d_k, d_model, 1.0f, 1.0f),
                 "gemm");
        };
        add_product(Wk, dK);
        add_product(Wv, dV);
    }
    MD dx = ln_backward_plus(ln1, std::move(dx1), dR, this->need_update);

    if (this->need_update) {
        fused_update({{&Wq, &dWq, &adam_Wq}, {&Wk, &dWk, &adam_Wk}, {&Wv, &dWv, &adam_Wv}, {&Wo, &dWo, &adam_Wo},
                      {&bo, &dbo, &adam_bo}, {&W1, &dW1, &adam_W1}, {&b1, &db1, &adam_b1}, {&W2, &dW2, &adam_W2},
                      {&b2, &db2, &adam_b2}});
    }
    return dx;
}

// Tangent of the whole block at the point cached by eval() (ml/layer.hpp:3034-3178).
// The attention part follows the structure of the reference's batched CUDA
// branch (:3061-3142): per head two strided-batched products for the score
// tangent dS = dQ^T K + Q^T dK, one softmax-tangent kernel over all blocks
// (the softmax Jacobian is symmetric, so it is the backward kernel), two
// products for dH = dV A^T + V dA^T -- instead of about fifteen launches per
// (head, sequence) block of the generic slice loop.
template <>
inline Matrix<ROCMfloat> TransformerLayer<ROCMfloat>::jvp(const Matrix<ROCMfloat>&, const Matrix<ROCMfloat>& tangent_in) {
    using namespace rocm_detail;
    using MD = Matrix<ROCMfloat>;
    const int N = seq_len * batchN;
    const float scale = 1.0f / sqrtf((float)d_h);
    const MD tangent = plain(tangent_in);
    if (attention_without_scores(causal, d_k, num_heads, seq_len, batchN)) {
        // eval() kept no probabilities: form them now (H comes out the same)
        must(jzhip_attention_fwd(p(cached_H), p(cached_A), p(cached_Q), p(cached_K), p(cached_V), d_k, num_heads, seq_len,
                                 batchN, 1),
             "attention_fwd");
    }

    MD dx1 = ln1.jvp(tangent);
    MD dQ = Wq * dx1;
    MD dK = Wk * dx1;
    MD dV = Wv * dx1;

    const long long stride_qkv = (long long)d_k * seq_len;
    const long long stride_attn = (long long)seq_len * seq_len;
    const long long head_attn = stride_attn * batchN;
    float* ds = p(attn_dS_scratch);
    MD dH("jvp_dH", d_k, N);
    for (int hh = 0; hh < num_heads; ++hh) {
        // dS_h[query, key] = <dQ[:, query], K[:, key]> + <Q[:, query], dK[:, key]>, unscaled
        must(jzhip_gemm_strided_batched(p(dQ) + hh * d_h, p(cached_K) + hh * d_h, ds + hh * head_attn, seq_len, seq_len,
                                        d_h, 1, 0, d_k, d_k, seq_len, stride_qkv, stride_qkv, stride_attn, batchN,
                                        1.0f, 0.0f),
             "jvp scores (dQ)");
        must(jzhip_gemm_strided_batched(p(cached_Q) + hh * d_h, p(dK) + hh * d_h, ds + hh * head_attn, seq_len, seq_len,
                                        d_h, 1, 0, d_k, d_k, seq_len, stride_qkv, stride_qkv, stride_attn, batchN,
                                        1.0f, 1.0f),
             "jvp scores (dK)");
    }
    // dA = A .* (scale*dS - rowsum(A .* scale*dS)), in place
    must(jzhip_attn_softmax_bwd(ds, p(cached_A), ds, seq_len, batchN * num_heads, scale, 0), "jvp softmax");
    for (int hh = 0; hh < num_heads; ++hh) {
        // dH_h = dV_h A_h^T + V_h dA_h^T
        must(jzhip_gemm_strided_batched(p(dV) + hh * d_h, p(cached_A) + hh * head_attn, p(dH) + hh * d_h, d_h, seq_len,
                                        seq_len, 0, 1, d_k, seq_len, d_k, stride_qkv, stride_attn, stride_qkv, batchN,
                                        1.0f, 0.0f),
             "jvp dH (dV)");
        must(jzhip_gemm_strided_batched(p(cached_V) + hh * d_h, ds + hh * head_attn, p(dH) + hh * d_h, d_h, seq_len,
                                        seq_len, 0, 1, d_k, seq_len, d_k, stride_qkv, stride_attn, stride_qkv, batchN,
                                        1.0f, 1.0f),
             "jvp dH (dA)");
    }
    MD dR = tangent + Wo * dH;
    MD dx2 = ln2.jvp(dR);
    MD dF1 = W1 * dx2;
    must(jzhip_drelu_mul(p(dF1), p(cached_F1), p(dF1), (size_t)d_ff * N), "drelu_mul");
    return dR + W2 * dF1;
}

}  // namespace Juzhen

#endif
