// ref_shim.cpp — thin extern "C" window onto the reference's own CPU path.
//
// TEST INFRASTRUCTURE ONLY.  This translation unit contains no algorithm: each
// function builds Matrix<float> operands from caller buffers and calls the
// reference's templates (cpp/core.hpp, cpp/matrix.hpp, cpp/operators.hpp,
// ml/util.cuh, ml/layer.hpp) where they lie under the reference tree.  It is
// compiled by oracle/Makefile into oracle/_ref/libjzref.so, which is used to
// validate oracle/jz_oracle.c and the GPU kernels, and as the "reference" CPU
// baseline.  Nothing of the reference's source is copied here.
//
// Buffers are dense column-major (ld == physical row count).  A matrix is
// described by (pointer, physical rows, physical cols, transpose flag); results
// are written as dense column-major *logical* matrices.
#include <cstring>
#include <list>
#include <memory>
#include <vector>

#include "ml/layer.hpp"

using Juzhen::Layer;
typedef Matrix<float> MF;

namespace {

MF mk(const float* p, int pr, int pc, int trans) {
    MF m("shim", pr, pc);
    std::memcpy(const_cast<float*>(m.data()), p, sizeof(float) * (size_t)pr * pc);
    if (trans) return MF(m.T());  // deep copy keeps the flag (cpp/core.hpp:283-294)
    return m;
}

// write the logical content of m as dense column-major
void out_logical(float* dst, const MF& m) {
    const size_t R = m.num_row(), Cn = m.num_col();
    for (size_t j = 0; j < Cn; ++j)
        for (size_t i = 0; i < R; ++i) dst[j * R + i] = m.elem(i, j);
}

// write the physical buffer and report its flag
int out_physical(float* dst, const MF& m) {
    std::memcpy(dst, m.data(), sizeof(float) * m.num_row() * m.num_col());
    return m.get_transpose();
}

Memory<float>& pool_guard() {
    static Memory<float> guard;  // releases the pool at unload (cpp/launcher.cu:65-98)
    return guard;
}

}  // namespace

#define API extern "C" __attribute__((visibility("default")))

API void jzref_init() { (void)pool_guard(); }

API void jzref_dot(float* out, const float* A, int ar, int ac, int ta, const float* B, int br, int bc,
                   int tb) {
    out_logical(out, mk(A, ar, ac, ta) * mk(B, br, bc, tb));
}

// const add: returns a new matrix (cpp/core.hpp:414-431); flag of the result reported
API int jzref_add(float* out, const float* A, int ar, int ac, int ta, const float* B, int br, int bc,
                  int tb, float s1, float s2) {
    const MF a = mk(A, ar, ac, ta), b = mk(B, br, bc, tb);
    return out_physical(out, a.add(b, s1, s2));
}

// in-place add: A keeps its own layout (cpp/core.hpp:435-449)
API void jzref_add_inplace(float* A, int ar, int ac, int ta, const float* B, int br, int bc, int tb,
                           float s1, float s2) {
    MF a = mk(A, ar, ac, ta);
    a.add(mk(B, br, bc, tb), s1, s2);
    out_physical(A, a);
}

API int jzref_hadmd(float* out, const float* A, int ar, int ac, int ta, const float* B, int br, int bc,
                    int tb) {
    const MF a = mk(A, ar, ac, ta), b = mk(B, br, bc, tb);
    return out_physical(out, hadmd(a, b));
}

// op: 0 exp 1 log 2 tanh 3 d_tanh 4 square 5 add(a=p1, s1=p0) 6 eleminv(l=p0)
//     7 relu 8 d_relu 9 sqrt 10 clamp(lo=p0, hi=p1)
API int jzref_unary(int op, float* out, const float* in, int n, double p0, double p1) {
    const MF x = mk(in, n, 1, 0);
    MF y;
    switch (op) {
        case 0: y = exp(x); break;
        case 1: y = log(x); break;
        case 2: y = tanh(x); break;
        case 3: y = d_tanh(x); break;
        case 4: y = square(x); break;
        case 5: y = x.add((float)p1, (float)p0); break;
        case 6: y = x.eleminv(p0); break;
        case 7: y = relu(MF(x)); break;
        case 8: y = d_relu(MF(x)); break;
        case 9: y = sqrt(x); break;
        case 10: y = clamp(x, (float)p0, (float)p1); break;
        default: return -1;
    }
    out_physical(out, y);
    return 0;
}

// the operator chain of README.md:29-31 on an (m x k)*(k x n) product
API void jzref_chain(float* out, const float* A, int m, int k, const float* B, int n) {
    const MF a = mk(A, m, k, 0), b = mk(B, k, n, 0);
    out_logical(out, log(exp(a * b) + 1.0f) / 5.0f);
}

API void jzref_sum(float* out, const float* A, int ar, int ac, int ta, int dim) {
    out_logical(out, sum(mk(A, ar, ac, ta), dim));
}

API float jzref_norm(const float* A, int n) { return mk(A, n, 1, 0).norm(); }

API void jzref_slice(float* out, const float* A, int ar, int ac, int ta, int r0, int r1, int c0,
                     int c1) {
    out_logical(out, mk(A, ar, ac, ta).slice(r0, r1, c0, c1));
}

API void jzref_slice_assign(float* A, int ar, int ac, int ta, int r0, int r1, int c0, int c1,
                            const float* Mv, int mr, int mc, int tm) {
    MF a = mk(A, ar, ac, ta);
    a.slice(r0, r1, c0, c1, mk(Mv, mr, mc, tm));
    out_physical(A, a);
}

API void jzref_stack2(float* out, int horizontal, const float* A, int ar, int ac, int ta,
                      const float* B, int br, int bc, int tb) {
    const MF a = mk(A, ar, ac, ta), b = mk(B, br, bc, tb);
    std::vector<MatrixView<float>> v{a, b};
    out_logical(out, horizontal ? hstack<float>(v) : vstack<float>(v));
}

API void jzref_softmax(float* out, const float* A, int ar, int ac, int ta, int rowwise) {
    const MF a = mk(A, ar, ac, ta);
    out_logical(out, rowwise ? Juzhen::row_softmax(a) : Juzhen::col_softmax(a));
}

API void jzref_max_cols(float* out, const float* A, int ar, int ac) {
    // the functor of ml/layer.hpp:2346-2351
    out_logical(out, reduce(
                         [](float* v, float* vdes, int lenv, int) {
                             float m = -1e30f;
                             for (int i = 0; i < lenv; i++) m = m > v[i] ? m : v[i];
                             vdes[0] = m;
                         },
                         mk(A, ar, ac, 0), 0, 1));
}

API void jzref_adam_update(float* g, float* m, float* v, int n, float alpha, float beta1,
                           float beta2, float eps, int iteration) {
    adam_state<float> st(alpha, n, 1);
    st.beta1 = beta1;
    st.beta2 = beta2;
    st.eps = eps;
    st.iteration = iteration;
    st.m = mk(m, n, 1, 0);
    st.v = mk(v, n, 1, 0);
    MF upd = adam_update(mk(g, n, 1, 0), st);
    out_physical(g, upd);
    out_physical(m, st.m);
    out_physical(v, st.v);
}

API void jzref_layernorm_fwd(float* y, float* xhat, float* inv_std, const float* x,
                             const float* gamma, const float* beta, int dim, int N) {
    Juzhen::LayerNorm<float> ln(dim, N);
    ln.set_gamma(mk(gamma, dim, 1, 0));
    ln.set_beta(mk(beta, dim, 1, 0));
    out_logical(y, ln.forward(mk(x, dim, N, 0)));
    out_logical(xhat, ln.cached_xhat);
    out_logical(inv_std, ln.cached_inv);
}

API void jzref_layernorm_bwd(float* dx, float* dgamma, float* dbeta, const float* dy,
                             const float* x, const float* gamma, const float* beta, int dim,
                             int N) {
    Juzhen::LayerNorm<float> ln(dim, N);
    ln.set_gamma(mk(gamma, dim, 1, 0));
    ln.set_beta(mk(beta, dim, 1, 0));
    ln.forward(mk(x, dim, N, 0));
    const MF g = mk(dy, dim, N, 0);
    out_logical(dx, ln.backward(MF(g), false));
    // the parameter gradients of ml/layer.hpp:2683-2686
    out_logical(dgamma, sum(hadmd(g, ln.cached_xhat), 1));
    out_logical(dbeta, sum(g, 1));
}

// LayerNorm<float>::jvp at the point x (ml/layer.hpp:2690-2702)
API void jzref_layernorm_jvp(float* out, const float* dx, const float* x, const float* gamma,
                             const float* beta, int dim, int N) {
    Juzhen::LayerNorm<float> ln(dim, N);
    ln.set_gamma(mk(gamma, dim, 1, 0));
    ln.set_beta(mk(beta, dim, 1, 0));
    ln.forward(mk(x, dim, N, 0));
    out_logical(out, ln.jvp(mk(dx, dim, N, 0)));
}

// LogisticLayer value and gradient (ml/layer.hpp:232-284); targets one-hot K x N
API float jzref_logistic(float* grad, const float* logits, const float* onehot, int K, int N) {
    Juzhen::LogisticLayer<float> L(N, mk(onehot, K, N, 0));
    const MF x = mk(logits, K, N, 0);
    L.eval(x);
    const float loss = L.value().elem(0, 0);
    if (grad) out_logical(grad, L.grad(x));
    return loss;
}

// CPU ConvLayer forward / backward (ml/layer.hpp:2019-2090).  w is the stored
// (C_out*C_in*kH*kW, 1) weight column, b is (C_out, 1).
API void jzref_conv_eval(float* out, const float* x, const float* w, const float* b, int N, int C,
                         int H, int W, int Co, int kH, int kW, int pad, int stride, int relu) {
    Juzhen::ConvLayer L(N, C, H, W, Co, kH, kW, pad, stride, relu != 0);
    L.W() = mk(w, Co * C * kH * kW, 1, 0);
    L.b() = mk(b, Co, 1, 0);
    L.eval(mk(x, C * H * W, N, 0));
    out_logical(out, L.value());
}

API void jzref_conv_backward(float* dx, const float* x, const float* w, const float* b,
                             const float* upstream, int N, int C, int H, int W, int Co, int kH,
                             int kW, int pad, int stride, int relu) {
    Juzhen::ConvLayer L(N, C, H, W, Co, kH, kW, pad, stride, relu != 0);
    L.W() = mk(w, Co * C * kH * kW, 1, 0);
    L.b() = mk(b, Co, 1, 0);
    std::list<Layer<float>*> net{&L};
    Juzhen::freeze(net);
    const MF in = mk(x, C * H * W, N, 0);
    L.eval(in);
    const int Ho = (H + 2 * pad - kH) / stride + 1, Wo = (W + 2 * pad - kW) / stride + 1;
    out_logical(dx, L.backward(in, mk(upstream, Co * Ho * Wo, N, 0)));
}

API void jzref_convtrans_eval(float* out, const float* x, const float* w, const float* b, int N,
                              int C, int H, int W, int Co, int kH, int kW, int pad, int stride,
                              int relu) {
    Juzhen::convtransLayer L(N, C, H, W, Co, kH, kW, pad, stride, relu != 0);
    L.W() = mk(w, C * Co * kH * kW, 1, 0);
    L.b() = mk(b, Co, 1, 0);
    L.eval(mk(x, C * H * W, N, 0));
    out_logical(out, L.value());
}

API void jzref_convtrans_backward(float* dx, const float* x, const float* w, const float* b,
                                  const float* upstream, int N, int C, int H, int W, int Co,
                                  int kH, int kW, int pad, int stride, int relu) {
    Juzhen::convtransLayer L(N, C, H, W, Co, kH, kW, pad, stride, relu != 0);
    L.W() = mk(w, C * Co * kH * kW, 1, 0);
    L.b() = mk(b, Co, 1, 0);
    std::list<Layer<float>*> net{&L};
    Juzhen::freeze(net);
    const MF in = mk(x, C * H * W, N, 0);
    L.eval(in);
    const int Ho = (H - 1) * stride - 2 * pad + kH, Wo = (W - 1) * stride - 2 * pad + kW;
    out_logical(dx, L.backward(in, mk(upstream, Co * Ho * Wo, N, 0)));
}

// ── TransformerLayer<float> (ml/layer.hpp:2735-3447) ─────────────────────
struct RefBlock {
    std::unique_ptr<Juzhen::TransformerLayer<float>> layer;
    int d_model, d_k, d_ff, S, B;
};

API void* jzref_block_create(int d_model, int d_k, int d_ff, int S, int B, int heads, int causal) {
    auto* blk = new RefBlock;
    blk->layer = std::make_unique<Juzhen::TransformerLayer<float>>(d_model, d_k, d_ff, S, B, heads,
                                                                  causal != 0);
    blk->d_model = d_model; blk->d_k = d_k; blk->d_ff = d_ff; blk->S = S; blk->B = B;
    return blk;
}
API void jzref_block_destroy(void* h) { delete static_cast<RefBlock*>(h); }

// which: 0 Wq 1 Wk 2 Wv 3 Wo 4 bo 5 W1 6 b1 7 W2 8 b2 9 ln1g 10 ln1b 11 ln2g 12 ln2b
API int jzref_block_param(void* h, int which, float* buf, int set) {
    auto& L = *static_cast<RefBlock*>(h)->layer;
    auto* b = static_cast<RefBlock*>(h);
    const int dm = b->d_model, dk = b->d_k, df = b->d_ff;
    const int rows[] = {dk, dk, dk, dm, dm, df, df, dm, dm, dm, dm, dm, dm};
    const int cols[] = {dm, dm, dm, dk, 1, dm, 1, df, 1, 1, 1, 1, 1};
    if (which < 0 || which > 12) return -1;
    if (set) {
        const MF m = mk(buf, rows[which], cols[which], 0);
        switch (which) {
            case 0: L.set_Wq(m); break;   case 1: L.set_Wk(m); break;
            case 2: L.set_Wv(m); break;   case 3: L.set_Wo(m); break;
            case 4: L.set_bo(m); break;   case 5: L.set_W1(m); break;
            case 6: L.set_b1(m); break;   case 7: L.set_W2(m); break;
            case 8: L.set_b2(m); break;   case 9: L.set_ln1_gamma(m); break;
            case 10: L.set_ln1_beta(m); break; case 11: L.set_ln2_gamma(m); break;
            case 12: L.set_ln2_beta(m); break;
        }
    } else {
        const MF* m = nullptr;
        switch (which) {
            case 0: m = &L.get_Wq(); break;  case 1: m = &L.get_Wk(); break;
            case 2: m = &L.get_Wv(); break;  case 3: m = &L.get_Wo(); break;
            case 4: m = &L.get_bo(); break;  case 5: m = &L.get_W1(); break;
            case 6: m = &L.get_b1(); break;  case 7: m = &L.get_W2(); break;
            case 8: m = &L.get_b2(); break;  case 9: m = &L.get_ln1_gamma(); break;
            case 10: m = &L.get_ln1_beta(); break; case 11: m = &L.get_ln2_gamma(); break;
            case 12: m = &L.get_ln2_beta(); break;
        }
        out_logical(buf, *m);
    }
    return 0;
}

API void jzref_block_set_lr(void* h, float lr) { static_cast<RefBlock*>(h)->layer->set_lr(lr); }

API void jzref_block_eval(void* h, float* out, const float* x) {
    auto* b = static_cast<RefBlock*>(h);
    b->layer->eval(mk(x, b->d_model, b->S * b->B, 0));
    out_logical(out, b->layer->value());
}

// backward at the point cached by the last eval; update != 0 applies Adam
API void jzref_block_backward(void* h, float* dx, const float* x, const float* upstream, int update) {
    auto* b = static_cast<RefBlock*>(h);
    std::list<Layer<float>*> net{b->layer.get()};
    if (update) Juzhen::unfreeze(net); else Juzhen::freeze(net);
    out_logical(dx, b->layer->backward(mk(x, b->d_model, b->S * b->B, 0),
                                       mk(upstream, b->d_model, b->S * b->B, 0)));
}

// ── dense MLP of Layer/LinearLayer/ReluLayer + LossLayer ─────────────────
// One Adam training step of a stack of fully connected layers with MSE loss
// (examples/helloworld_nn.cu:72-99).  kinds[l]: 0 linear, 1 relu, 2 tanh.
// W/b buffers are read and written back so the caller owns the state; Adam
// moments likewise (mW, vW, mb, vb), `iteration` is shared.
API float jzref_mlp_step(int nlayers, const int* kinds, const int* dims, float** W, float** b,
                         float** mW, float** vW, float** mb, float** vb, const float* X,
                         const float* Y, int nb, float alpha, int iteration) {
    using namespace Juzhen;
    std::vector<std::unique_ptr<Layer<float>>> own;
    std::list<Layer<float>*> net;
    for (int l = 0; l < nlayers; ++l) {
        const int in = dims[l], out = dims[l + 1];
        Layer<float>* L = nullptr;
        if (kinds[l] == 0) L = new LinearLayer<float>(out, in, nb);
        else if (kinds[l] == 1) L = new ReluLayer<float>(out, in, nb);
        else L = new Layer<float>(out, in, nb);
        own.emplace_back(L);
        L->W() = mk(W[l], out, in, 0);
        L->b() = mk(b[l], out, 1, 0);
        auto& aw = L->adamWstate();
        auto& ab = L->adambstate();
        aw.alpha = alpha; ab.alpha = alpha;
        aw.iteration = iteration; ab.iteration = iteration;
        aw.m = mk(mW[l], out, in, 0); aw.v = mk(vW[l], out, in, 0);
        ab.m = mk(mb[l], out, 1, 0);  ab.v = mk(vb[l], out, 1, 0);
        net.push_front(L);  // forward() evaluates from the back of the list
    }
    const MF x = mk(X, dims[0], nb, 0);
    LossLayer<float> loss(nb, mk(Y, dims[nlayers], nb, 0));
    net.push_front(&loss);
    const float value = forward(net, x).elem(0, 0);
    backprop(net, x);
    net.pop_front();
    int l = nlayers - 1;
    for (auto* L : net) {  // list order is last layer first
        out_logical(W[l], L->W());
        out_logical(b[l], L->b());
        out_physical(mW[l], L->adamWstate().m); out_physical(vW[l], L->adamWstate().v);
        out_physical(mb[l], L->adambstate().m); out_physical(vb[l], L->adambstate().v);
        --l;
    }
    return value;
}

// ── character LM built from the reference's own classes ──────────────────
// embed LinearLayer(d, V+S) on the stacked one-hot [token; position] input,
// `layers` TransformerLayer<float> blocks, proj LinearLayer(V, d), LogisticLayer
// loss, Adam — the wiring of examples/demo_transformer.cu:285-340.
struct RefLM {
    int V, d, heads, ff, layers, S, B, N;
    std::unique_ptr<Juzhen::LinearLayer<float>> embed, proj;
    std::vector<std::unique_ptr<Juzhen::TransformerLayer<float>>> blocks;
    std::list<Layer<float>*> net;
};

API void* jzref_lm_create(int V, int d, int heads, int ff, int layers, int S, int B) {
    using namespace Juzhen;
    auto* m = new RefLM{V, d, heads, ff, layers, S, B, S * B};
    m->embed = std::make_unique<LinearLayer<float>>(d, V + S, m->N);
    m->proj = std::make_unique<LinearLayer<float>>(V, d, m->N);
    for (int i = 0; i < layers; ++i)
        m->blocks.push_back(std::make_unique<TransformerLayer<float>>(d, d, ff, S, B, heads));
    m->net.push_back(m->proj.get());
    for (int i = layers - 1; i >= 0; --i) m->net.push_back(m->blocks[i].get());
    m->net.push_back(m->embed.get());
    return m;
}
API void jzref_lm_destroy(void* h) { delete static_cast<RefLM*>(h); }

// kind 0 embed.W (d x (V+S)), 1 embed.b, 2 proj.W (V x d), 3 proj.b, 4 block parameter `which` of block `layer`
API int jzref_lm_param(void* h, int kind, int layer, int which, float* buf, int set) {
    auto* m = static_cast<RefLM*>(h);
    if (kind == 4) {
        RefBlock tmp;  // reuse the block accessor through a non-owning view
        tmp.layer.reset(m->blocks[layer].get());
        tmp.d_model = m->d; tmp.d_k = m->d; tmp.d_ff = m->ff; tmp.S = m->S; tmp.B = m->B;
        const int rc = jzref_block_param(&tmp, which, buf, set);
        tmp.layer.release();
        return rc;
    }
    Layer<float>* L = kind < 2 ? static_cast<Layer<float>*>(m->embed.get()) : m->proj.get();
    MF& dst = (kind % 2 == 0) ? L->W() : L->b();
    if (set) dst = mk(buf, (int)dst.num_row(), (int)dst.num_col(), 0);
    else out_logical(buf, dst);
    return 0;
}

API void jzref_lm_set_lr(void* h, float lr) {
    auto* m = static_cast<RefLM*>(h);
    for (auto* L : {static_cast<Layer<float>*>(m->embed.get()), static_cast<Layer<float>*>(m->proj.get())}) {
        L->adamWstate().alpha = lr;
        L->adambstate().alpha = lr;
    }
    for (auto& b : m->blocks) b->set_lr(lr);
}

// One training step (forward, loss, backprop with Adam).  X is the stacked
// one-hot input ((V+S) x N), Y the one-hot targets (V x N).  Returns the loss
// of the forward pass.
API float jzref_lm_step(void* h, const float* X, const float* Y) {
    using namespace Juzhen;
    auto* m = static_cast<RefLM*>(h);
    const MF x = mk(X, m->V + m->S, m->N, 0);
    LogisticLayer<float> loss(m->N, mk(Y, m->V, m->N, 0));
    m->net.push_front(&loss);
    const float value = forward(m->net, x).elem(0, 0);
    backprop(m->net, x);
    m->net.pop_front();
    return value;
}
