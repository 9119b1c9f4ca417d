// Fused Adam / AdamW: one pass over (g, m, v[, w]) instead of the ~12 generic
// matrix ops and temporaries of adam_update's generic formulation
// (ml/util.cuh:247-255).  24 bytes per parameter for the update-only form,
// 28 for the form with the weight update fused (g is not rewritten).
//
// The expression is the CPU oracle's fused loop (ml/util.cuh:223-245), which
// is itself bit-identical to the generic op chain: every product and sum is
// rounded separately (this file is built with -ffp-contract=off), the "+0.0f"
// terms come from scale() being add(0, s), the bias corrections are narrowed
// from double, and the final division is a double reciprocal narrowed to float
// followed by a float multiply.
#include "common.hpp"

#include <cmath>

namespace jz {
namespace {

struct AdamConst {
    float alpha, beta1, beta2, omb1, omb2, eps, r1, r2, decay;  // decay = 1 - alpha*wd
    int use_decay;
};

__device__ __forceinline__ float adam_one(float gi, float& mi_io, float& vi_io, const AdamConst& c) {
    const float mi = (c.beta1 * mi_io + 0.0f) + (c.omb1 * gi + 0.0f);
    const float vi = (c.beta2 * vi_io + 0.0f) + (c.omb2 * (gi * gi) + 0.0f);
    mi_io = mi;
    vi_io = vi;
    const float mh = c.r1 * mi + 0.0f;
    const float vh = c.r2 * vi + 0.0f;
    const float den = 1.0f * sqrtf(vh) + c.eps;
    return (c.alpha * mh + 0.0f) * static_cast<float>(1.0 / static_cast<double>(den));
}

// FUSE_W = false: g <- step.  FUSE_W = true: w <- decay*w - step, g untouched.
// NT: non-temporal loads and stores (a launch that streams past the cache).
template <bool FUSE_W, bool VEC, bool NT>
__global__ __launch_bounds__(kBlock) void adam_kernel(float* w, float* g, float* m, float* v,
                                                      size_t n, AdamConst c) {
    // one float4 per thread, grid covers the data once (see elementwise.hip)
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    const size_t tid = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if constexpr (VEC) {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride) {
            float4 gv = load4<NT>(g + 4 * i);
            float4 mv = load4<NT>(m + 4 * i);
            float4 vv = load4<NT>(v + 4 * i);
            float4 st;
            st.x = adam_one(gv.x, mv.x, vv.x, c);
            st.y = adam_one(gv.y, mv.y, vv.y, c);
            st.z = adam_one(gv.z, mv.z, vv.z, c);
            st.w = adam_one(gv.w, mv.w, vv.w, c);
            store4<NT>(m + 4 * i, mv);
            store4<NT>(v + 4 * i, vv);
            if constexpr (FUSE_W) {
                float4 wv = load4<NT>(w + 4 * i);
                if (c.use_decay) {
                    wv.x *= c.decay; wv.y *= c.decay; wv.z *= c.decay; wv.w *= c.decay;
                }
                wv.x = 1.0f * wv.x + -1.0f * st.x;
                wv.y = 1.0f * wv.y + -1.0f * st.y;
                wv.z = 1.0f * wv.z + -1.0f * st.z;
                wv.w = 1.0f * wv.w + -1.0f * st.w;
                store4<NT>(w + 4 * i, wv);
            } else {
                store4<NT>(g + 4 * i, st);
            }
        }
        for (size_t j = n4 * 4 + tid; j < n; j += stride) {
            float mi = m[j], vi = v[j];
            const float st = adam_one(g[j], mi, vi, c);
            m[j] = mi;
            v[j] = vi;
            if constexpr (FUSE_W) {
                float wj = w[j];
                if (c.use_decay) wj *= c.decay;
                w[j] = 1.0f * wj + -1.0f * st;
            } else {
                g[j] = st;
            }
        }
    } else {
        for (size_t j = tid; j < n; j += stride) {
            float mi = m[j], vi = v[j];
            const float st = adam_one(g[j], mi, vi, c);
            m[j] = mi;
            v[j] = vi;
            if constexpr (FUSE_W) {
                float wj = w[j];
                if (c.use_decay) wj *= c.decay;
                w[j] = 1.0f * wj + -1.0f * st;
            } else {
                g[j] = st;
            }
        }
    }
}

AdamConst make_const(float alpha, float beta1, float beta2, float eps, float wd, int iteration) {
    AdamConst c;
    c.alpha = alpha;
    c.beta1 = beta1;
    c.beta2 = beta2;
    c.omb1 = 1 - beta1;
    c.omb2 = 1 - beta2;
    c.eps = eps;
    // ml/util.cuh:226-227
    c.r1 = static_cast<float>(1.0 / (1.0 - std::pow(static_cast<double>(beta1), static_cast<double>(iteration))));
    c.r2 = static_cast<float>(1.0 / (1.0 - std::pow(static_cast<double>(beta2), static_cast<double>(iteration))));
    c.use_decay = wd != 0.0f;
    c.decay = 1.0f - alpha * wd;
    return c;
}

template <bool FUSE_W>
int launch_adam(float* w, float* g, float* m, float* v, size_t n, const AdamConst& c) {
    if (n == 0) return 0;
    const bool vec = aligned16(g) && aligned16(m) && aligned16(v) && (!FUSE_W || aligned16(w));
    const size_t items = vec ? (n + 3) / 4 : n;
    const size_t blocks = (items + kBlock - 1) / kBlock;
    if (blocks > 0x7fffffffull) return -1;
    const unsigned grid = static_cast<unsigned>(blocks);
    // (the moments and weights of a 19 M parameter model, 0.5 GB per step, are partly still in
    // the last-level cache from the step before: 82 us plain, 95 us hinted; at 3.2 GB the hint wins)
    if (vec && streams_past_cache((FUSE_W ? 7 : 6) * n * sizeof(float) / 2))
        adam_kernel<FUSE_W, true, true><<<grid, kBlock, 0, stream()>>>(w, g, m, v, n, c);
    else if (vec)
        adam_kernel<FUSE_W, true, false><<<grid, kBlock, 0, stream()>>>(w, g, m, v, n, c);
    else
        adam_kernel<FUSE_W, false, false><<<grid, kBlock, 0, stream()>>>(w, g, m, v, n, c);
    return launch_rc();
}

// Several tensors in one launch (a layer's weights and bias, or every tensor
// of a small model): a workgroup owns 1024 consecutive elements of one tensor
// and finds its tensor by walking the table of first-block indices.
constexpr int kMultiMax = 16;
constexpr int kMultiPerBlock = kBlock * 4;
struct AdamMulti {
    float* w[kMultiMax];
    const float* g[kMultiMax];
    float* m[kMultiMax];
    float* v[kMultiMax];
    unsigned long long n[kMultiMax];
    unsigned first_block[kMultiMax + 1];
    AdamConst c[kMultiMax];
    int vec[kMultiMax];
    int base_iteration[kMultiMax];
    int count;
};

// COUNTED: the step number of a tensor is its `iteration` plus a counter read from device
// memory, and the two bias corrections (ml/util.cuh:226-227) are formed here, in double as
// on the host; with it a recorded launch can be replayed for successive steps.
template <bool COUNTED>
__global__ __launch_bounds__(kBlock) void adam_multi_kernel(AdamMulti p, const int* __restrict__ replays) {
    int t = 0;
    while (t + 1 < p.count && blockIdx.x >= p.first_block[t + 1]) ++t;
    AdamConst c = p.c[t];
    if constexpr (COUNTED) {
        __shared__ float corr[2];
        if (threadIdx.x == 0) {
            const double it = static_cast<double>(p.base_iteration[t] + *replays);
            corr[0] = static_cast<float>(1.0 / (1.0 - pow(static_cast<double>(c.beta1), it)));
            corr[1] = static_cast<float>(1.0 / (1.0 - pow(static_cast<double>(c.beta2), it)));
        }
        __syncthreads();
        c.r1 = corr[0];
        c.r2 = corr[1];
    }
    float* w = p.w[t];
    const float* g = p.g[t];
    float* m = p.m[t];
    float* v = p.v[t];
    const size_t n = p.n[t];
    const size_t base = (static_cast<size_t>(blockIdx.x - p.first_block[t]) * kBlock + threadIdx.x) * 4;
    if (base >= n) return;
    if (p.vec[t] && base + 3 < n) {
        const float4 gv = *reinterpret_cast<const float4*>(g + base);
        float4 mv = *reinterpret_cast<float4*>(m + base);
        float4 vv = *reinterpret_cast<float4*>(v + base);
        float4 st;
        st.x = adam_one(gv.x, mv.x, vv.x, c);
        st.y = adam_one(gv.y, mv.y, vv.y, c);
        st.z = adam_one(gv.z, mv.z, vv.z, c);
        st.w = adam_one(gv.w, mv.w, vv.w, c);
        *reinterpret_cast<float4*>(m + base) = mv;
        *reinterpret_cast<float4*>(v + base) = vv;
        float4 wv = *reinterpret_cast<float4*>(w + base);
        if (c.use_decay) {
            wv.x *= c.decay; wv.y *= c.decay; wv.z *= c.decay; wv.w *= c.decay;
        }
        wv.x = 1.0f * wv.x + -1.0f * st.x;
        wv.y = 1.0f * wv.y + -1.0f * st.y;
        wv.z = 1.0f * wv.z + -1.0f * st.z;
        wv.w = 1.0f * wv.w + -1.0f * st.w;
        *reinterpret_cast<float4*>(w + base) = wv;
        return;
    }
    for (size_t j = base; j < n && j < base + 4; ++j) {
        float mi = m[j], vi = v[j];
        const float st = adam_one(g[j], mi, vi, c);
        m[j] = mi;
        v[j] = vi;
        float wj = w[j];
        if (c.use_decay) wj *= c.decay;
        w[j] = 1.0f * wj + -1.0f * st;
    }
}

}  // namespace
}  // namespace jz

using namespace jz;

namespace {
int adam_multi(const jzhip_adam_tensor* tensors, int n_tensors, const int* replays) {
    if (n_tensors < 0 || (n_tensors > 0 && !tensors)) return -1;
    for (int i = 0; i < n_tensors; ++i) {
        const jzhip_adam_tensor& t = tensors[i];
        if (t.count && (!t.w || !t.g || !t.m || !t.v)) return -1;
        if (t.iteration < 1) return -1;
    }
    hipStream_t s = jz::stream();
    for (int at = 0; at < n_tensors;) {
        jz::AdamMulti p;
        p.count = 0;
        unsigned blocks = 0;
        for (; at < n_tensors && p.count < jz::kMultiMax; ++at) {
            const jzhip_adam_tensor& t = tensors[at];
            if (t.count == 0) continue;
            const size_t nb = (t.count + jz::kMultiPerBlock - 1) / jz::kMultiPerBlock;
            if (nb > 0x7fffffffull - blocks) {   // a tensor this large goes alone
                if (p.count > 0) break;
            }
            const int k = p.count++;
            p.w[k] = t.w; p.g[k] = t.g; p.m[k] = t.m; p.v[k] = t.v;
            p.n[k] = t.count;
            p.first_block[k] = blocks;
            p.c[k] = jz::make_const(t.alpha, t.beta1, t.beta2, t.eps, t.weight_decay, t.iteration);
            p.base_iteration[k] = t.iteration;
            p.vec[k] = jz::aligned16(t.w) && jz::aligned16(t.g) && jz::aligned16(t.m) && jz::aligned16(t.v);
            if (nb > 0x7fffffffull) return -1;
            blocks += static_cast<unsigned>(nb);
        }
        if (p.count == 0) continue;
        p.first_block[p.count] = blocks;
        if (replays) jz::adam_multi_kernel<true><<<blocks, jz::kBlock, 0, s>>>(p, replays);
        else jz::adam_multi_kernel<false><<<blocks, jz::kBlock, 0, s>>>(p, nullptr);
        const int rc = jz::launch_rc();
        if (rc) return rc;
    }
    return 0;
}

__global__ void counter_add_kernel(int* counter, int delta) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *counter += delta;
}
}  // namespace

JZ_API int jzhip_adamw_step_multi(const jzhip_adam_tensor* tensors, int n_tensors) {
    return adam_multi(tensors, n_tensors, nullptr);
}

JZ_API int jzhip_adamw_step_multi_counted(const jzhip_adam_tensor* tensors, int n_tensors, const int* replays_device) {
    if (!replays_device) return -1;
    return adam_multi(tensors, n_tensors, replays_device);
}

JZ_API int jzhip_counter_add(int* counter_device, int delta) {
    if (!counter_device) return -1;
    counter_add_kernel<<<1, 64, 0, jz::stream()>>>(counter_device, delta);
    return jz::launch_rc();
}

JZ_API int jzhip_adam_update(float* g, float* m, float* v, size_t count, float alpha, float beta1,
                             float beta2, float eps, int iteration) {
    if (count && (!g || !m || !v)) return -1;
    if (iteration < 1) return -1;
    return launch_adam<false>(nullptr, g, m, v, count, make_const(alpha, beta1, beta2, eps, 0.f, iteration));
}

JZ_API int jzhip_adamw_step(float* w, const float* g, float* m, float* v, size_t count, float alpha,
                            float beta1, float beta2, float eps, float weight_decay, int iteration) {
    if (count && (!w || !g || !m || !v)) return -1;
    if (iteration < 1) return -1;
    return launch_adam<true>(w, const_cast<float*>(g), m, v, count,
                             make_const(alpha, beta1, beta2, eps, weight_decay, iteration));
}
