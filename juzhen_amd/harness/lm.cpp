// Character-level transformer language model trained on one MI355X through the
// C ABI of libjzhip.so: the train-step harness of the benchmark configuration
// (6 pre-LayerNorm decoder blocks, d_model 512, 8 heads, FFN 2048 with GELU,
// tied embeddings, learned positional table, cross-entropy, AdamW).
//
// The block is the reference's TransformerLayer (ml/layer.hpp:2735-3447): same
// tensors, same layouts (activations are (features, tokens) column-major with
// token n = b*S + s), same forward/backward algebra, so with relu/adam/untied
// options it reproduces a stack built from the reference's own classes
// (examples/demo_transformer.cu:214-383: one-hot token+position input into a
// LinearLayer, TransformerLayers, a LinearLayer head, LogisticLayer loss).
// The reference feeds one-hot token and position matrices through a dense layer
// (demo_transformer.cu:133-149).  A product with a one-hot matrix copies one
// column per token, so the forward embedding is a lookup with the same bits,
// and the position-table gradient is a sum over sequences; the token-table
// gradient and the head stay products (against the one-hot matrix and the
// logits gradient), deterministic and checkable against the CPU path.
//
// Everything is preallocated at creation; a step issues only library calls
// (no allocation, no host synchronisation).  The loss stays on the device until
// jzlm_loss() is called.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "jzhip.h"

#define JZLM_API extern "C" __attribute__((visibility("default")))

namespace {

struct Config {
    int vocab, d_model, heads, d_ff, layers, seq, batch;
    int gelu;        // 1: exact-erf GELU FFN, 0: ReLU (the reference block)
    int tied;        // 1: head = embedding^T, no biases on embedding/head; 0: separate head with biases
    int adamw;       // 1: decoupled weight decay on matrices
    float lr, weight_decay, beta1, beta2, eps;
};

// Parameters live in a few arenas (one per optimiser group) that hold weights,
// gradients and both Adam moments at equal offsets, so the optimiser is one
// fused AdamW launch per group instead of one per tensor.  A tensor is a
// (rows x cols) view with leading dimension ld: Wq, Wk, Wv are the three row
// blocks of one stacked (3d x d) projection matrix (ld = 3d).
enum Group { kDecay = 0, kPlain = 1, kHeadDecay = 2, kHeadPlain = 3, kGroups = 4 };

struct Tensor {
    std::string name;
    int rows = 0, cols = 0, ld = 0;
    int group = kPlain;
    size_t offset = 0;    // floats from the arena start
    float* w = nullptr;   // parameter
    float* g = nullptr;   // gradient
    float* m = nullptr;   // Adam first moment
    float* v = nullptr;   // Adam second moment
    size_t count() const { return static_cast<size_t>(rows) * cols; }
};

struct Arena {
    size_t used = 0;
    float *w = nullptr, *g = nullptr, *m = nullptr, *v = nullptr;
};

struct Block {
    int Wq, Wk, Wv, Wo, bo, W1, b1, W2, b2, g1, be1, g2, be2;           // tensor indices
    float *x1, *xhat1, *inv1, *QKV, *A, *H, *R, *x2, *xhat2, *inv2, *F1, *F1a, *out;  // cached activations
    float* stats = nullptr;       // per query: score maximum and reciprocal sum (the attention that keeps no S x S matrix)
    bool A_masked_zero = false;   // A's entries above the diagonal already hold the zeros of a first forward call
};

struct Model {
    Config c;
    int N = 0;  // tokens per step
    std::vector<Tensor> t;
    std::vector<Block> blocks;
    std::vector<float*> owned;
    Arena arena[kGroups];
    int E = -1, P = -1, be = -1, Wp = -1, bp = -1;
    float *oh_tok = nullptr, *x0 = nullptr, *logits = nullptr, *dlogits = nullptr;
    int32_t *tokens = nullptr, *targets = nullptr;
    float* loss = nullptr;
    // backward scratch shared by all blocks
    // (the ones the weight-gradient products read exist twice, alternating by
    // block, and the block-output gradient three times: see backward())
    float *dx[3] = {}, *dR[2] = {}, *dtmp[2] = {}, *dtmp1[2] = {}, *dQKV[2] = {}, *dF1[2] = {};
    float *dH = nullptr, *dA = nullptr;
    bool dA_masked_zero = false;   // dA's entries above the diagonal already hold the zeros of a first backward call
    // Attention without the S x S probabilities (jzhip_attention_flash_*): two floats per query are
    // kept instead of A, and the backward pass needs no score-gradient scratch.  Taken whenever the
    // shape qualifies; JZLM_MATERIALISE_ATTENTION=1 keeps the buffers of the reference's layout.
    bool flash = false;
    // Weight, bias and LayerNorm-parameter gradients are leaves of the backward
    // graph: with `overlap` they go to a second stream and fill the gaps the
    // gradient chain leaves (tile prologues and tails, bandwidth-bound kernels).
    // Off by default: since the tiled products keep two stages of loads in flight
    // they leave little to fill, and two of them sharing the CUs measured 2 % slower
    // per step than one after the other (with the earlier single-stage products the
    // second stream gained 2 %).
    bool overlap = false;
    void* side = nullptr;
    static constexpr int kEvents = 8, kDone = 4;
    void* ev[kEvents] = {};
    void* done[kDone] = {};   // side stream finished a block's weight gradients
    int ev_next = 0;
    // Batches are staged in two page-locked host buffers (ids, then targets) and
    // copied asynchronously, so handing over the next batch does not wait for the
    // step in flight; staged[k] marks the stream position after buffer k's copies.
    int32_t* stage[2] = {};
    void* staged[2] = {};
    unsigned batches = 0;
    float* io = nullptr;  // dense staging for get/set of strided views
    size_t io_floats = 0;
    int iteration = 1;
    int rc = 0;  // first failing return code, sticky

    float* alloc(size_t n) {
        float* p = nullptr;
        int r = jzhip_malloc(&p, n);
        if (r != 0 && rc == 0) rc = r;
        owned.push_back(p);
        return p;
    }
    // Reserve rows x cols (contiguous) in a group's arena; pointers are bound by finish().
    int add(const std::string& name, int rows, int cols, int group) {
        Tensor x;
        x.name = name; x.rows = rows; x.cols = cols; x.ld = rows; x.group = group;
        x.offset = arena[group].used;
        arena[group].used += (x.count() + 3) / 4 * 4;   // keep every tensor 16-byte aligned
        t.push_back(x);
        return static_cast<int>(t.size()) - 1;
    }
    // Three row blocks of one stacked (3*rows x cols) matrix.
    void add_stacked3(const std::string& n0, const std::string& n1, const std::string& n2, int rows, int cols,
                      int group, int& i0, int& i1, int& i2) {
        const size_t base = arena[group].used;
        arena[group].used += (static_cast<size_t>(3) * rows * cols + 3) / 4 * 4;
        const std::string* names[3] = {&n0, &n1, &n2};
        int* idx[3] = {&i0, &i1, &i2};
        for (int k = 0; k < 3; ++k) {
            Tensor x;
            x.name = *names[k]; x.rows = rows; x.cols = cols; x.ld = 3 * rows; x.group = group;
            x.offset = base + static_cast<size_t>(k) * rows;
            t.push_back(x);
            *idx[k] = static_cast<int>(t.size()) - 1;
        }
    }
    void finish() {
        for (Arena& a : arena) {
            if (a.used == 0) continue;
            a.w = alloc(a.used); a.g = alloc(a.used); a.m = alloc(a.used); a.v = alloc(a.used);
            if (rc != 0) return;
            ck(jzhip_fill(a.w, a.used, 0.f)); ck(jzhip_fill(a.g, a.used, 0.f));
            ck(jzhip_fill(a.m, a.used, 0.f)); ck(jzhip_fill(a.v, a.used, 0.f));
        }
        for (Tensor& x : t) {
            Arena& a = arena[x.group];
            x.w = a.w + x.offset; x.g = a.g + x.offset; x.m = a.m + x.offset; x.v = a.v + x.offset;
            if (x.count() > io_floats) io_floats = x.count();
        }
        io = alloc(io_floats);
    }
    void ck(int r) { if (r != 0 && rc == 0) rc = r; }
};

// C(m x n) = alpha*op(A)op(B) + beta*C, dense operands unless ld is given
inline void gemm(Model& M, const float* A, bool ta, const float* B, bool tb, float* C, int m, int n, int k,
                 float beta = 0.f, int lda = 0, int ldb = 0, int ldc = 0) {
    M.ck(jzhip_gemm(A, B, C, m, n, k, ta, tb, lda ? lda : (ta ? k : m), ldb ? ldb : (tb ? n : k),
                    ldc ? ldc : m, 1.0f, beta));
}
// C = act(A*B + bias) + residual with the elementwise tail fused into the store
// (act codes of jzhip_gemm_fused); operands dense, A possibly transposed
inline void gemm_tail(Model& M, const float* A, bool ta, const float* B, float* C, int m, int n, int k,
                      const float* bias, int act, float* aux, const float* residual, float beta = 0.f) {
    M.ck(jzhip_gemm_fused(A, B, C, m, n, k, ta, 0, ta ? k : m, k, m, 1.0f, beta, bias, act, aux, m, residual, m));
}

void forward(Model& M) {
    const Config& c = M.c;
    const int d = c.d_model, N = M.N, ff = c.d_ff;
    // x0 = E * onehot(tokens) + P * onehot(positions) [+ embedding bias], as a lookup
    M.ck(jzhip_embedding_fwd(M.x0, M.t[M.E].w, M.t[M.P].w, M.be >= 0 ? M.t[M.be].w : nullptr, M.tokens, d, c.vocab,
                             c.seq, N));
    const float* x = M.x0;
    for (Block& b : M.blocks) {
        M.ck(jzhip_layernorm_fwd(b.x1, b.xhat1, b.inv1, x, M.t[b.g1].w, M.t[b.be1].w, d, N));
        // Q, K, V in one product against the stacked projection
        gemm(M, M.t[b.Wq].w, false, b.x1, false, b.QKV, 3 * d, N, d);
        // the weights above the diagonal are zeros written by the first call; later
        // calls leave them alone (a third of the kernel's stores)
        if (M.flash) {
            M.ck(jzhip_attention_flash_fwd(b.H, d, b.stats, b.QKV, b.QKV + d, b.QKV + 2 * d, 3 * d, d, c.heads, c.seq,
                                           c.batch, 1));
        } else {
            M.ck(jzhip_attention_fwd_ld(b.H, d, b.A, b.QKV, b.QKV + d, b.QKV + 2 * d, 3 * d, d, c.heads, c.seq,
                                        c.batch, b.A_masked_zero ? 2 : 1));
            b.A_masked_zero = true;
        }
        // R = x + (Wo*H + bo)
        gemm_tail(M, M.t[b.Wo].w, false, b.H, b.R, d, N, d, M.t[b.bo].w, 0, nullptr, x);
        M.ck(jzhip_layernorm_fwd(b.x2, b.xhat2, b.inv2, b.R, M.t[b.g2].w, M.t[b.be2].w, d, N));
        // F1 = W1*x2 + b1 (kept for the backward pass), F1a = act(F1)
        gemm_tail(M, M.t[b.W1].w, false, b.x2, b.F1a, ff, N, d, M.t[b.b1].w, c.gelu ? 2 : 1, b.F1, nullptr);
        // out = R + (W2*F1a + b2)
        gemm_tail(M, M.t[b.W2].w, false, b.F1a, b.out, d, N, ff, M.t[b.b2].w, 0, nullptr, b.R);
        x = b.out;
    }
    if (c.tied) {
        gemm(M, M.t[M.E].w, true, x, false, M.logits, c.vocab, N, d);    // E^T x
    } else {
        gemm_tail(M, M.t[M.Wp].w, false, x, M.logits, c.vocab, N, d, M.t[M.bp].w, 0, nullptr, nullptr);
    }
}

void step_group(Model& M, int group) {
    const Config& c = M.c;
    Arena& a = M.arena[group];
    if (a.used == 0) return;
    const bool decay = group == kDecay || group == kHeadDecay;
    const float wd = (c.adamw && decay) ? c.weight_decay : 0.0f;
    M.ck(jzhip_adamw_step(a.w, a.g, a.m, a.v, a.used, c.lr, c.beta1, c.beta2, c.eps, wd, M.iteration));
}

// The backward pass on two streams.  `fork()` makes the side stream wait for
// everything issued so far on the main stream and routes the next calls to it;
// `back()` returns to the main stream without waiting; `mark(i)` records the
// side stream's position in done[i % kDone] and `await(i)` makes the main
// stream wait for that mark; `join()` makes the main stream wait for
// everything issued so far on the side stream.
struct Lanes {
    Model& M;
    void* main_stream;
    bool on;
    explicit Lanes(Model& m) : M(m), main_stream(jzhip_get_stream()), on(m.overlap && m.side != nullptr) {}
    void* next_event() { void* e = M.ev[M.ev_next]; M.ev_next = (M.ev_next + 1) % Model::kEvents; return e; }
    void fork() {
        if (!on) return;
        void* e = next_event();
        M.ck(jzhip_event_record(e));
        M.ck(jzhip_set_stream(M.side));
        M.ck(jzhip_stream_wait_event(e));
    }
    void back() {
        if (on) M.ck(jzhip_set_stream(main_stream));
    }
    void mark(int i) {
        if (!on) return;
        M.ck(jzhip_set_stream(M.side));
        M.ck(jzhip_event_record(M.done[i % Model::kDone]));
        M.ck(jzhip_set_stream(main_stream));
    }
    void await(int i) {
        if (on) M.ck(jzhip_stream_wait_event(M.done[i % Model::kDone]));
    }
    void join() {
        if (!on) return;
        void* e = next_event();
        M.ck(jzhip_set_stream(M.side));
        M.ck(jzhip_event_record(e));
        M.ck(jzhip_set_stream(main_stream));
        M.ck(jzhip_stream_wait_event(e));
    }
};

void backward(Model& M, bool update) {
    const Config& c = M.c;
    const int d = c.d_model, N = M.N, ff = c.d_ff, V = c.vocab;
    const float* xL = M.blocks.empty() ? M.x0 : M.blocks.back().out;
    Lanes lanes(M);
    M.ck(jzhip_softmax_xent(M.loss, M.dlogits, M.logits, M.targets, V, N, V));
    float* dy = M.dx[0];  // gradient w.r.t. the current block's output
    if (c.tied) {
        gemm(M, M.t[M.E].w, false, M.dlogits, false, dy, d, N, V);       // E * dlogits
        lanes.fork();
        gemm(M, xL, false, M.dlogits, true, M.t[M.E].g, d, V, N);        // head part of dE
        lanes.back();
    } else {
        gemm(M, M.dlogits, false, xL, true, M.t[M.Wp].g, V, d, N);
        M.ck(jzhip_sum_rows(M.t[M.bp].g, M.dlogits, V, N, V));
        // The reference's dense layers step their weights before forming the
        // gradient they hand down (Layer::backward, ml/layer.hpp:96-105: update(),
        // then `return W().T() * t`); the untied head reproduces that order.
        if (update) { step_group(M, kHeadDecay); step_group(M, kHeadPlain); }
        gemm(M, M.t[M.Wp].w, true, M.dlogits, false, dy, d, N, V);
    }
    const int L = static_cast<int>(M.blocks.size());
    for (int i = 0; i < L; ++i) {   // i-th block from the top
        Block& b = M.blocks[L - 1 - i];
        // Scratch gradients alternate between two sets by block (three for the
        // block-output gradient, which is written one block before it is read by
        // the side stream): set i % 2 is rewritten here, so the side stream must
        // have finished the weight gradients of block i - 2, and may still be
        // working on those of block i - 1.
        if (i >= 2) lanes.await(i - 2);
        float* dF1 = M.dF1[i % 2];
        float* dx2 = M.dtmp[i % 2];
        float* dx1 = M.dtmp1[i % 2];
        float* dR = M.dR[i % 2];
        float* dQKV = M.dQKV[i % 2];
        float* dy_next = M.dx[(i + 1) % 3];
        // feed-forward
        lanes.fork();
        gemm(M, dy, false, b.F1a, true, M.t[b.W2].g, d, ff, N);   // (db2 = row sums of dy: with the LayerNorm sweep below)
        lanes.back();
        // dF1 = (W2^T dy) .* act'(F1)
        // (with db1 = row sums of dF1, added up by the workgroups that store it)
        M.ck(jzhip_gemm_fused_rowsum(M.t[b.W2].w, dy, dF1, M.t[b.b1].g, ff, N, d, 1, 0, d, d, ff, 1.0f, 0.0f, nullptr,
                                     c.gelu ? 4 : 3, b.F1, ff, nullptr, ff));
        lanes.fork();
        gemm(M, dF1, false, b.x2, true, M.t[b.W1].g, ff, d, N);
        lanes.back();
        gemm(M, M.t[b.W1].w, true, dF1, false, dx2, d, N, ff);
        // dR = LN2'(dx2) + dy, and in the same sweep the LayerNorm's parameter gradients and the
        // two bias gradients that are row sums of its operands: dbo of dR, db2 of dy
        M.ck(jzhip_layernorm_bwd_residual_sums(dR, dx2, M.t[b.g2].w, b.xhat2, b.inv2, dy, M.t[b.g2].g, M.t[b.be2].g,
                                               M.t[b.bo].g, M.t[b.b2].g, d, N));
        // output projection
        lanes.fork();
        gemm(M, dR, false, b.H, true, M.t[b.Wo].g, d, d, N);
        lanes.back();
        gemm(M, M.t[b.Wo].w, true, dR, false, M.dH, d, N, d);
        // attention core, gradients into the stacked (3d x N) buffer
        if (M.flash) {
            M.ck(jzhip_attention_flash_bwd(dQKV, dQKV + d, dQKV + 2 * d, 3 * d, M.dH, d, b.QKV, b.QKV + d, b.QKV + 2 * d,
                                           3 * d, b.H, d, b.stats, d, c.heads, c.seq, c.batch, 1));
        } else {
            M.ck(jzhip_attention_bwd_ld(dQKV, dQKV + d, dQKV + 2 * d, 3 * d, M.dA, M.dH, d, b.QKV, b.QKV + d,
                                        b.QKV + 2 * d, 3 * d, b.A, d, c.heads, c.seq, c.batch,
                                        M.dA_masked_zero ? 2 : 1));
            M.dA_masked_zero = true;   // the score-gradient scratch is shared by all blocks and only ever used here
        }
        lanes.fork();
        gemm(M, dQKV, false, b.x1, true, M.t[b.Wq].g, 3 * d, d, N);          // stacked dWq, dWk, dWv
        lanes.back();
        gemm(M, M.t[b.Wq].w, true, dQKV, false, dx1, d, N, 3 * d);
        lanes.mark(i);
        // dx = LN1'(dx1) + dR with the LayerNorm's parameter gradients (and, under the lowest block,
        // the row sums of dx for the embedding bias)
        float* sum_dx = (i == L - 1 && M.be >= 0) ? M.t[M.be].g : nullptr;
        M.ck(jzhip_layernorm_bwd_residual_sums(dy_next, dx1, M.t[b.g1].w, b.xhat1, b.inv1, dR, M.t[b.g1].g,
                                               M.t[b.be1].g, sum_dx, nullptr, d, N));
        dy = dy_next;
    }
    lanes.join();
    // embedding tables: dE (+)= dx0 * onehot_tok^T, dP = dx0 * onehot_pos^T
    gemm(M, dy, false, M.oh_tok, true, M.t[M.E].g, d, V, N, c.tied ? 1.0f : 0.0f);
    // (token n = b*S + s: the (d, N) gradient is a (d*S) x B matrix whose row sums are dP)
    M.ck(jzhip_sum_rows(M.t[M.P].g, dy, d * c.seq, c.batch, d * c.seq));
    if (M.be >= 0 && L == 0) M.ck(jzhip_sum_rows(M.t[M.be].g, dy, d, N, d));
    if (update) {
        step_group(M, kDecay);
        step_group(M, kPlain);
        M.iteration++;
    }
}

}  // namespace

struct jzlm_config {
    int vocab, d_model, heads, d_ff, layers, seq, batch, gelu, tied, adamw;
    float lr, weight_decay, beta1, beta2, eps;
};

JZLM_API void* jzlm_create(const jzlm_config* cfg) {
    if (!cfg || cfg->vocab <= 0 || cfg->d_model <= 0 || cfg->heads <= 0 || cfg->d_model % cfg->heads != 0 ||
        cfg->d_ff <= 0 || cfg->layers < 0 || cfg->seq <= 0 || cfg->batch <= 0)
        return nullptr;
    Model* M = new Model;
    Config& c = M->c;
    c.vocab = cfg->vocab; c.d_model = cfg->d_model; c.heads = cfg->heads; c.d_ff = cfg->d_ff;
    c.layers = cfg->layers; c.seq = cfg->seq; c.batch = cfg->batch; c.gelu = cfg->gelu; c.tied = cfg->tied;
    c.adamw = cfg->adamw; c.lr = cfg->lr; c.weight_decay = cfg->weight_decay; c.beta1 = cfg->beta1;
    c.beta2 = cfg->beta2; c.eps = cfg->eps;
    const int d = c.d_model, ff = c.d_ff, V = c.vocab, S = c.seq;
    const int N = M->N = c.seq * c.batch;
    const size_t dN = static_cast<size_t>(d) * N, fN = static_cast<size_t>(ff) * N;
    const size_t aN = static_cast<size_t>(S) * S * c.batch * c.heads;
    {
        const char* keep = std::getenv("JZLM_MATERIALISE_ATTENTION");
        // the stacked (3d x N) projection and d-row outputs are 16-byte aligned when d % 4 == 0
        M->flash = !(keep && std::atoi(keep) != 0) && d % 4 == 0 &&
                   jzhip_attention_flash_supported(d, c.heads, S, c.batch) == 1;
    }

    M->E = M->add("embed", d, V, kDecay);
    M->P = M->add("pos", d, S, kDecay);
    if (!c.tied) {
        M->be = M->add("embed_bias", d, 1, kPlain);
        M->Wp = M->add("head", V, d, kHeadDecay);
        M->bp = M->add("head_bias", V, 1, kHeadPlain);
    }
    M->blocks.resize(c.layers);
    for (int l = 0; l < c.layers; ++l) {
        Block& b = M->blocks[l];
        const std::string p = "block" + std::to_string(l) + ".";
        M->add_stacked3(p + "Wq", p + "Wk", p + "Wv", d, d, kDecay, b.Wq, b.Wk, b.Wv);
        b.Wo = M->add(p + "Wo", d, d, kDecay);
        b.bo = M->add(p + "bo", d, 1, kPlain);
        b.W1 = M->add(p + "W1", ff, d, kDecay); b.b1 = M->add(p + "b1", ff, 1, kPlain);
        b.W2 = M->add(p + "W2", d, ff, kDecay); b.b2 = M->add(p + "b2", d, 1, kPlain);
        b.g1 = M->add(p + "ln1_gamma", d, 1, kPlain); b.be1 = M->add(p + "ln1_beta", d, 1, kPlain);
        b.g2 = M->add(p + "ln2_gamma", d, 1, kPlain); b.be2 = M->add(p + "ln2_beta", d, 1, kPlain);
    }
    M->finish();
    for (int l = 0; l < c.layers && M->rc == 0; ++l) {
        Block& b = M->blocks[l];
        M->ck(jzhip_fill(M->t[b.g1].w, d, 1.0f));
        M->ck(jzhip_fill(M->t[b.g2].w, d, 1.0f));
        b.x1 = M->alloc(dN); b.xhat1 = M->alloc(dN); b.inv1 = M->alloc(N);
        b.QKV = M->alloc(3 * dN); b.H = M->alloc(dN);
        if (M->flash) b.stats = M->alloc(2 * static_cast<size_t>(S) * c.batch * c.heads);
        else b.A = M->alloc(aN);
        b.R = M->alloc(dN); b.x2 = M->alloc(dN); b.xhat2 = M->alloc(dN); b.inv2 = M->alloc(N);
        b.F1 = M->alloc(fN); b.F1a = M->alloc(fN); b.out = M->alloc(dN);
    }
    M->oh_tok = M->alloc(static_cast<size_t>(V) * N);
    M->tokens = reinterpret_cast<int32_t*>(M->alloc(2 * static_cast<size_t>(N)));   // ids, then targets: one upload
    M->targets = M->tokens + N;
    M->x0 = M->alloc(dN);
    M->logits = M->alloc(static_cast<size_t>(V) * N);
    M->dlogits = M->alloc(static_cast<size_t>(V) * N);
    M->loss = M->alloc(1);
    for (float*& p : M->dx) p = M->alloc(dN);
    for (int k = 0; k < 2; ++k) {
        M->dR[k] = M->alloc(dN); M->dtmp[k] = M->alloc(dN); M->dtmp1[k] = M->alloc(dN);
        M->dQKV[k] = M->alloc(3 * dN); M->dF1[k] = M->alloc(fN);
    }
    M->dH = M->alloc(dN);
    if (!M->flash) M->dA = M->alloc(aN);
    if (M->rc != 0) {
        std::fprintf(stderr, "jzlm_create: device allocation failed (%s)\n", jzhip_error_string(M->rc));
        return M;
    }
    M->ck(jzhip_stream_create(&M->side));
    for (void*& e : M->ev) M->ck(jzhip_event_create(&e));
    for (void*& e : M->done) M->ck(jzhip_event_create(&e));
    for (int k = 0; k < 2; ++k) {
        void* p = nullptr;
        M->ck(jzhip_host_alloc(&p, sizeof(int32_t) * 2 * static_cast<size_t>(N)));
        M->stage[k] = static_cast<int32_t*>(p);
        M->ck(jzhip_event_create(&M->staged[k]));
    }
    if (const char* env = std::getenv("JZLM_OVERLAP")) M->overlap = std::atoi(env) != 0;
    return M;
}

JZLM_API void jzlm_destroy(void* h) {
    Model* M = static_cast<Model*>(h);
    if (!M) return;
    jzhip_synchronize();
    for (void* e : M->ev) jzhip_event_destroy(e);
    for (void* e : M->done) jzhip_event_destroy(e);
    jzhip_stream_destroy(M->side);
    for (int k = 0; k < 2; ++k) {
        jzhip_event_destroy(M->staged[k]);
        jzhip_host_free(M->stage[k]);
    }
    for (float* p : M->owned) jzhip_free(p);
    delete M;
}

// 1: weight-gradient work of the backward pass on a second stream (default);
// 0: everything on the library's current stream in program order.
JZLM_API void jzlm_set_overlap(void* h, int on) { static_cast<Model*>(h)->overlap = on != 0; }
// 1 when the model runs the attention that keeps no S x S matrix, 0 when it keeps the probabilities
JZLM_API int jzlm_flash_attention(void* h) { return static_cast<Model*>(h)->flash ? 1 : 0; }

JZLM_API int jzlm_status(void* h) { return static_cast<Model*>(h)->rc; }
JZLM_API int jzlm_num_tensors(void* h) { return static_cast<int>(static_cast<Model*>(h)->t.size()); }
JZLM_API size_t jzlm_param_count(void* h) {
    size_t n = 0;
    for (const Tensor& x : static_cast<Model*>(h)->t) n += x.count();
    return n;
}
JZLM_API const char* jzlm_tensor_name(void* h, int i) { return static_cast<Model*>(h)->t[i].name.c_str(); }
JZLM_API int jzlm_tensor_rows(void* h, int i) { return static_cast<Model*>(h)->t[i].rows; }
JZLM_API int jzlm_tensor_cols(void* h, int i) { return static_cast<Model*>(h)->t[i].cols; }

// which: 0 parameter, 1 gradient, 2 Adam m, 3 Adam v.  Column-major host buffers.
JZLM_API int jzlm_get(void* h, int i, int which, float* host) {
    Model* M = static_cast<Model*>(h);
    Tensor& x = M->t[i];
    float* src = which == 0 ? x.w : which == 1 ? x.g : which == 2 ? x.m : x.v;
    if (x.ld == x.rows) return jzhip_memcpy_d2h(host, src, x.count());
    int rc = jzhip_copy2d(M->io, x.rows, 0, 0, 0, src, x.ld, 0, 0, 0, x.rows, x.cols);
    return rc ? rc : jzhip_memcpy_d2h(host, M->io, x.count());
}
JZLM_API int jzlm_set(void* h, int i, int which, const float* host) {
    Model* M = static_cast<Model*>(h);
    Tensor& x = M->t[i];
    float* dst = which == 0 ? x.w : which == 1 ? x.g : which == 2 ? x.m : x.v;
    if (x.ld == x.rows) return jzhip_memcpy_h2d(dst, host, x.count());
    int rc = jzhip_memcpy_h2d(M->io, host, x.count());
    return rc ? rc : jzhip_copy2d(dst, x.ld, 0, 0, 0, M->io, x.rows, 0, 0, 0, x.rows, x.cols);
}

// tokens: batch windows of seq+1 ids each (window b = tokens[b*(seq+1) ...]);
// inputs are ids 0..seq-1 of a window, targets ids 1..seq.
JZLM_API int jzlm_set_batch(void* h, const int32_t* tokens) {
    Model* M = static_cast<Model*>(h);
    const Config& c = M->c;
    const int N = M->N;
    const int slot = static_cast<int>(M->batches & 1u);
    if (!M->stage[slot]) return -1;
    // the copies issued from this buffer two batches ago must have run
    if (M->batches >= 2) {
        const int rc0 = jzhip_event_synchronize(M->staged[slot]);
        if (rc0 != 0) return rc0;
    }
    int32_t* tk = M->stage[slot];
    int32_t* tg = tk + N;
    for (int b = 0; b < c.batch; ++b)
        for (int s = 0; s < c.seq; ++s) {
            const int n = b * c.seq + s;
            const int32_t tok = tokens[static_cast<size_t>(b) * (c.seq + 1) + s];
            const int32_t nxt = tokens[static_cast<size_t>(b) * (c.seq + 1) + s + 1];
            if (tok < 0 || tok >= c.vocab || nxt < 0 || nxt >= c.vocab) return -1;
            tk[n] = tok;
            tg[n] = nxt;
        }
    // only the ids cross PCIe (2 x 4 bytes per token); the one-hot matrix the
    // embedding gradient multiplies by is built on the device
    int rc = jzhip_memcpy_h2d_async(M->tokens, tk, sizeof(int32_t) * 2 * static_cast<size_t>(N));
    if (rc == 0) rc = jzhip_event_record(M->staged[slot]);
    if (rc == 0) rc = jzhip_one_hot(M->oh_tok, M->tokens, c.vocab, static_cast<size_t>(N));
    ++M->batches;
    return rc;
}

JZLM_API int jzlm_forward(void* h) {
    Model* M = static_cast<Model*>(h);
    forward(*M);
    return M->rc;
}
// forward must have run; computes the loss and all gradients, applies the
// optimiser when update != 0
JZLM_API int jzlm_backward(void* h, int update) {
    Model* M = static_cast<Model*>(h);
    backward(*M, update != 0);
    return M->rc;
}
// one training step: forward, loss, backward, optimiser
JZLM_API int jzlm_step(void* h) {
    Model* M = static_cast<Model*>(h);
    forward(*M);
    backward(*M, true);
    return M->rc;
}
// loss of the last backward()/step(); synchronises
JZLM_API float jzlm_loss(void* h) {
    Model* M = static_cast<Model*>(h);
    float v = NAN;
    if (jzhip_memcpy_d2h(&v, M->loss, 1) != 0) return NAN;
    return v;
}
JZLM_API int jzlm_logits(void* h, float* host) {
    Model* M = static_cast<Model*>(h);
    return jzhip_memcpy_d2h(host, M->logits, static_cast<size_t>(M->c.vocab) * M->N);
}
JZLM_API int jzlm_tokens_per_step(void* h) { return static_cast<Model*>(h)->N; }
JZLM_API void jzlm_set_iteration(void* h, int it) { static_cast<Model*>(h)->iteration = it; }
