// Attention backward that never holds an S x S matrix: the probabilities are
// recomputed tile by tile from Q, K and the per-query (max, 1/sum) pair the
// forward pass kept, the score gradients are formed in registers, and dQ, dK
// and dV come out of one kernel.  Stands for the same mathematics as
// jzhip_attention_bwd (ml/layer.hpp:3214-3283, 3329-3363), which reads the
// cached probabilities A and writes dS through a scratch buffer:
//     P  = exp(scale*K^T Q - m) * inv            (masked keys: 0)
//     dA = V^T dH,   D = sum_keys P .* dA = sum_d dH .* H   (H = V P, the forward output)
//     dS = P .* (dA - D) * scale
//     dV = dH P^T,   dK = Q dS^T,   dQ = K dS
// Layouts as in attention.hip: Q, K, V, H, dH, dQ, dK, dV are (d_k, S*B)
// column-major, head hh owns rows [hh*d_h, (hh+1)*d_h), sequence b the columns
// [b*S, (b+1)*S); stats holds, per block hh*B + b, S maxima then S reciprocals.
//
// One workgroup per (head, sequence) block.  The S/16 key tiles are dealt to
// S/32 waves: wave o owns key tiles o and S/16-1-o, which under the causal mask
// is the same number of (query tile, key tile) cells for every wave.  A wave
// keeps its key tile's K and V fragments and the dK, dV accumulators in
// registers and visits that tile's query tiles one cell per step.  In a cell:
//   S^T, dA^T   (queries x keys) by v_mfma_f32_16x16x4_f32 with both operands in
//               registers: the query tile's Q and dH fragments come straight from
//               global memory, requested one step ahead;
//   P^T, dS^T   in registers (register v of a lane is query 4*kq+v, the lane's l16
//               the key), which is the B-operand layout of the next two products;
//   dV += dH P^T, dK += Q dS^T   with dH and Q read as A operands from a copy of the
//               query tile that the wave keeps in LDS ([query][d], its own region);
//   dQ contribution K dS: dS^T goes through a 16 x 16 LDS patch of the wave to
//               become a B operand, the result is added to the block's dQ
//               accumulator in LDS.
// Every query tile receives contributions from several waves.  The cells are
// ordered by a table (flash_schedule) in which the waves of a step work on
// distinct query tiles, and steps are separated by a barrier, so each element of
// dQ is summed in one fixed order: results are the same bits from run to run.
#include "common.hpp"

#include <cmath>
#include <cstring>
#include <mutex>

namespace jz {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kMaxTiles = 16;              // S <= 256
constexpr int kMaxOwners = kMaxTiles / 2;
constexpr int kMaxSteps = 2 * kMaxTiles;   // without a mask every wave visits 2 * S/16 cells

// row[j][o]: query tile of wave o's cell in step j.  Steps [0, first[o]) of wave o
// belong to key tile o, the others to key tile tiles-1-o.  packed[o] holds wave o's
// column of row[][] as 4-bit fields, step j in bits 4*(j%16) of word j/16: two scalar
// loads give a wave its whole visiting order.
// Everything the kernel reads is a 4-byte or 8-byte field at an aligned offset: the
// compiler folds a wave-uniform byte index into the base of a scalar load, and scalar
// loads drop the two low address bits (a byte-sized `first` made waves 1, 2, 3 of
// every four read another wave's order).
struct FlashSchedule {
    uint64_t packed[kMaxOwners][2];
    int32_t first[kMaxOwners];
    int32_t steps;
    int32_t tiles;
    uint8_t row[kMaxSteps][kMaxOwners];   // host side only: the table the packed form is made from
};

// Cells (query tile t, key tile k), t >= k under the causal mask.  Every wave walks
// its first key tile's cells, then its second's; within a step all waves must be on
// distinct query tiles.  A query tile that still has as many cells left as there
// are steps left must be visited in every one of them, which prunes the search to
// nothing: the tables for S = 32 ... 256 are found without backtracking far.
struct ScheduleSearch {
    int tiles, owners, steps;
    bool causal;
    uint16_t left[kMaxOwners][2];   // bit t set: cell (t, key tile) not yet visited
    FlashSchedule* out;

    int key_tile(int o, int half) const { return half ? tiles - 1 - o : o; }
    bool place(int j, int i, const int* order, int half_of[], uint16_t used, uint16_t must, int assign[]) {
        if (i == owners) {
            if ((must & ~used) != 0) return false;
            for (int o = 0; o < owners; ++o) {
                left[o][half_of[o]] &= static_cast<uint16_t>(~(1u << assign[o]));
                out->row[j][o] = static_cast<uint8_t>(assign[o]);
            }
            if (step(j + 1)) return true;
            for (int o = 0; o < owners; ++o) left[o][half_of[o]] |= static_cast<uint16_t>(1u << assign[o]);
            return false;
        }
        const int o = order[i];
        // most demanded query tiles first
        int demand[kMaxTiles] = {};
        for (int p = 0; p < owners; ++p)
            for (int h = 0; h < 2; ++h)
                for (int t = 0; t < tiles; ++t) demand[t] += (left[p][h] >> t) & 1;
        bool tried[kMaxTiles] = {};
        for (int n = 0; n < tiles; ++n) {
            int best = -1;
            for (int t = 0; t < tiles; ++t)
                if (!tried[t] && ((left[o][half_of[o]] >> t) & 1) && !((used >> t) & 1) &&
                    (best < 0 || demand[t] > demand[best]))
                    best = t;
            if (best < 0) break;
            tried[best] = true;
            assign[o] = best;
            if (place(j, i + 1, order, half_of, static_cast<uint16_t>(used | (1u << best)), must, assign)) return true;
        }
        return false;
    }
    bool step(int j) {
        if (j == steps) return true;
        int half_of[kMaxOwners], order[kMaxOwners], count[kMaxOwners], assign[kMaxOwners];
        for (int o = 0; o < owners; ++o) {
            half_of[o] = j < out->first[o] ? 0 : 1;
            count[o] = __builtin_popcount(left[o][half_of[o]]);
            order[o] = o;
        }
        for (int a = 1; a < owners; ++a)   // fewest candidates first
            for (int b = a; b > 0 && count[order[b]] < count[order[b - 1]]; --b) std::swap(order[b], order[b - 1]);
        uint16_t must = 0;
        for (int t = 0; t < tiles; ++t) {
            int d = 0;
            for (int p = 0; p < owners; ++p)
                for (int h = 0; h < 2; ++h) d += (left[p][h] >> t) & 1;
            if (d == steps - j) must |= static_cast<uint16_t>(1u << t);
        }
        return place(j, 0, order, half_of, 0, must, assign);
    }
};

bool build_schedule(int tiles, bool causal, FlashSchedule* s) {
    std::memset(s, 0, sizeof(*s));
    ScheduleSearch q;
    q.tiles = tiles;
    q.owners = tiles / 2;
    q.causal = causal;
    q.steps = causal ? tiles + 1 : 2 * tiles;
    q.out = s;
    s->steps = q.steps;
    s->tiles = tiles;
    const uint16_t all = static_cast<uint16_t>((1u << tiles) - 1u);
    for (int o = 0; o < q.owners; ++o)
        for (int h = 0; h < 2; ++h) {
            const int k = q.key_tile(o, h);
            q.left[o][h] = causal ? static_cast<uint16_t>(all & ~((1u << k) - 1u)) : all;
            if (h == 0) s->first[o] = __builtin_popcount(q.left[o][0]);
        }
    if (!q.step(0)) return false;
    for (int o = 0; o < q.owners; ++o)
        for (int j = 0; j < q.steps; ++j) s->packed[o][j / 16] |= static_cast<uint64_t>(s->row[j][o]) << (4 * (j % 16));
    return true;
}

// One table per (S/32, causal) in device memory, built and uploaded on first use
// and kept until the process ends (6.5 KB in all).
constexpr int kScheduleSlots = kMaxOwners * 2;
struct ScheduleStore {
    std::mutex mutex;
    FlashSchedule* device = nullptr;
    bool ready[kScheduleSlots] = {};
};
ScheduleStore g_sched;

int device_schedule(int tiles, bool causal, const FlashSchedule** out) {
    const int slot = (tiles / 2 - 1) * 2 + (causal ? 1 : 0);
    std::lock_guard<std::mutex> lock(g_sched.mutex);
    if (!g_sched.device) {
        void* p = nullptr;
        const int rc = rc_of(hipMalloc(&p, sizeof(FlashSchedule) * kScheduleSlots));
        if (rc) return rc;
        g_sched.device = static_cast<FlashSchedule*>(p);
    }
    if (!g_sched.ready[slot]) {
        FlashSchedule host;
        if (!build_schedule(tiles, causal, &host)) return -1;
        // a blocking copy on the library's stream: the table is read by the launch that follows
        int rc = rc_of(hipMemcpyAsync(g_sched.device + slot, &host, sizeof(host), hipMemcpyHostToDevice, stream()));
        if (!rc) rc = rc_of(hipStreamSynchronize(stream()));
        if (rc) return rc;
        g_sched.ready[slot] = true;
    }
    *out = g_sched.device + slot;
    return 0;
}

template <int DH>
struct FlashLds {
    static constexpr int LDP = DH + 4;            // pitch of every [token][d] array: b128 rows hit all banks
    static constexpr int kPatch = 16 * 20;        // 16 x 16 transposition patch, pitch 20
    static size_t floats(int S) {
        const int owners = S / 32;
        return static_cast<size_t>(owners) * 2 * 16 * LDP      // per wave: Q and dH of its query tile
               + static_cast<size_t>(S) * LDP                  // dQ accumulator
               + static_cast<size_t>(owners) * kPatch          // per wave: dS patch
               + 3 * static_cast<size_t>(S);                   // max, 1/sum, D per query
    }
};

template <int DH>
__global__ __launch_bounds__(512) void attn_flash_bwd_kernel(
    float* __restrict__ dQ, float* __restrict__ dK, float* __restrict__ dV, int ld_d, const float* __restrict__ dH,
    int ld_dh, const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ V, int ld_qkv,
    const float* __restrict__ H, int ld_h, const float* __restrict__ stats, const FlashSchedule* __restrict__ sched,
    int S, int B, float scale, int causal) {
    constexpr int HD4 = DH / 4;     // contraction steps over d; a lane's share of a column
    constexpr int NDT = DH / 16;    // 16-row tiles along d
    constexpr int LDP = FlashLds<DH>::LDP;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int owners = S / 32;
    float* stage_all = lds;
    float* dq_acc = stage_all + static_cast<size_t>(owners) * 2 * 16 * LDP;
    float* patch_all = dq_acc + static_cast<size_t>(S) * LDP;
    float* st_m = patch_all + static_cast<size_t>(owners) * FlashLds<DH>::kPatch;
    float* st_inv = st_m + S;
    float* st_D = st_inv + S;

    const int blk = blockIdx.x;            // hh*B + b
    const int hh = blk / B, b = blk % B;
    const size_t col0 = static_cast<size_t>(b) * S;
    const float* q_blk = Q + col0 * ld_qkv + hh * DH;
    const float* k_blk = K + col0 * ld_qkv + hh * DH;
    const float* v_blk = V + col0 * ld_qkv + hh * DH;
    const float* dh_blk = dH + col0 * ld_dh + hh * DH;
    const float* h_blk = H + col0 * ld_h + hh * DH;
    float* dq_blk = dQ + col0 * ld_d + hh * DH;
    float* dk_blk = dK + col0 * ld_d + hh * DH;
    float* dv_blk = dV + col0 * ld_d + hh * DH;
    const float* st_blk = stats + static_cast<size_t>(blk) * 2 * S;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int o = __builtin_amdgcn_readfirstlane(tid / kWave);     // this wave's slot in the schedule
    const int l16 = lane & 15, kq = lane >> 4;
    const int tiles = S / 16;


    float* stage_q = stage_all + static_cast<size_t>(o) * 2 * 16 * LDP;   // [16 queries][LDP]
    float* stage_dh = stage_q + 16 * LDP;
    float* patch = patch_all + static_cast<size_t>(o) * FlashLds<DH>::kPatch;

    // fragments of a 16-token tile as the operand whose free index is the token: lane (l16, kq)
    // holds d = HD4*kq .. HD4*kq + HD4-1 of token 16*tile + l16 (one contiguous run)
    auto load_rows = [&](const float* base, int ld, int tile, float (&f)[HD4]) {
        const float* src = base + static_cast<size_t>(16 * tile + l16) * ld + HD4 * kq;
#pragma unroll
        for (int i = 0; i < HD4 / 4; ++i) {
            const floatx4 t4 = *reinterpret_cast<const floatx4*>(src + 4 * i);
            f[4 * i] = t4.x; f[4 * i + 1] = t4.y; f[4 * i + 2] = t4.z; f[4 * i + 3] = t4.w;
        }
    };

    // K, V of a key tile as B operands of S^T and dA^T (kb, vb) and K as the A operand of the dQ
    // product (ka: d = 16u + l16, key 4kq + s).  Both key tiles of the wave are fetched before the
    // loop: a fetch in the step where a wave changes tiles would hold every wave at that step's
    // barrier, and the eight waves change at eight different steps.
    auto load_key_tile = [&](int kt, float (&kb)[HD4], float (&vb)[HD4], float (&ka)[NDT][4]) {
        load_rows(k_blk, ld_qkv, kt, kb);
        load_rows(v_blk, ld_qkv, kt, vb);
#pragma unroll
        for (int u = 0; u < NDT; ++u)
#pragma unroll
            for (int s = 0; s < 4; ++s)
                ka[u][s] = k_blk[static_cast<size_t>(16 * kt + 4 * kq + s) * ld_qkv + 16 * u + l16];
    };
    // register v of accumulator tile u is d = 16u + 4kq + v of key 16*kt + l16
    auto store_key_tile = [&](int kt, const floatx4 (&dv_acc)[NDT], const floatx4 (&dk_acc)[NDT]) {
        float* pv = dv_blk + static_cast<size_t>(16 * kt + l16) * ld_d + 4 * kq;
        float* pk = dk_blk + static_cast<size_t>(16 * kt + l16) * ld_d + 4 * kq;
#pragma unroll
        for (int u = 0; u < NDT; ++u) {
            *reinterpret_cast<floatx4*>(pv + 16 * u) = dv_acc[u];
            *reinterpret_cast<floatx4*>(pk + 16 * u) = dk_acc[u];
        }
    };
    float kb0[HD4], vb0[HD4], ka0[NDT][4], kb1[HD4], vb1[HD4], ka1[NDT][4];
    load_key_tile(o, kb0, vb0, ka0);
    load_key_tile(tiles - 1 - o, kb1, vb1, ka1);

    const int steps = sched->steps;
    const int first = sched->first[o];
    const uint64_t order_lo = sched->packed[o][0], order_hi = sched->packed[o][1];
    auto row_of = [&](int j) { return static_cast<int>(((j < 16 ? order_lo : order_hi) >> (4 * (j & 15))) & 15u); };
    float qf[HD4], hf[HD4];          // the step's query tile: Q and dH, token-major fragments
    int t = row_of(0);
    load_rows(q_blk, ld_qkv, t, qf);
    load_rows(dh_blk, ld_dh, t, hf);

    // ── prologue: clear the dQ accumulator, fetch the row statistics, form D.  It comes after the
    // requests for the key tiles and the first query tile, so that all of the block's first
    // reads are in flight together instead of one latency after another ──
    for (int i = tid; i < S * LDP / 4; i += blockDim.x)
        reinterpret_cast<floatx4*>(dq_acc)[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    {
        // two threads per query (blockDim.x == 2*S): each half of the d range
        const int q = tid >> 1, half = tid & 1;
        const float* a = dh_blk + static_cast<size_t>(q) * ld_dh + half * (DH / 2);
        const float* c = h_blk + static_cast<size_t>(q) * ld_h + half * (DH / 2);
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < DH / 8; ++i) {
            const floatx4 x = *reinterpret_cast<const floatx4*>(a + 4 * i);
            const floatx4 y = *reinterpret_cast<const floatx4*>(c + 4 * i);
            dot += (x.x * y.x + x.y * y.y) + (x.z * y.z + x.w * y.w);
        }
        dot += __shfl_xor(dot, 1, kWave);
        if (half == 0) {
            st_D[q] = dot;
            st_m[q] = st_blk[q];
            st_inv[q] = st_blk[S + q];
        }
    }
    __syncthreads();

    // one cell: query tile t against key tile kt
    auto cell = [&](int j, int kt, const float (&kb)[HD4], const float (&vb)[HD4], const float (&ka)[NDT][4],
                    floatx4 (&dv_acc)[NDT], floatx4 (&dk_acc)[NDT]) {
        // the wave's copy of the query tile, [query][d]; the tile's slice of the dQ accumulator
        // (nobody else touches query tile t in this step) is requested now and used last
        {
            float* dq_ = stage_q + l16 * LDP + HD4 * kq;
            float* dh_ = stage_dh + l16 * LDP + HD4 * kq;
#pragma unroll
            for (int i = 0; i < HD4 / 4; ++i) {
                *reinterpret_cast<floatx4*>(dq_ + 4 * i) = floatx4{qf[4 * i], qf[4 * i + 1], qf[4 * i + 2], qf[4 * i + 3]};
                *reinterpret_cast<floatx4*>(dh_ + 4 * i) = floatx4{hf[4 * i], hf[4 * i + 1], hf[4 * i + 2], hf[4 * i + 3]};
            }
        }
        float* acc = dq_acc + static_cast<size_t>(16 * t + l16) * LDP + 4 * kq;
        floatx4 cur[NDT];
#pragma unroll
        for (int u = 0; u < NDT; ++u) cur[u] = *reinterpret_cast<floatx4*>(acc + 16 * u);
        const floatx4 m4 = *reinterpret_cast<const floatx4*>(st_m + 16 * t + 4 * kq);
        const floatx4 i4 = *reinterpret_cast<const floatx4*>(st_inv + 16 * t + 4 * kq);
        const floatx4 d4 = *reinterpret_cast<const floatx4*>(st_D + 16 * t + 4 * kq);
        // S^T and dA^T: rows = queries of tile t, columns = keys of tile kt
        floatx4 sc = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < HD4; ++kk) {
            sc = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[kk], kb[kk], sc, 0, 0, 0);
            da = __builtin_amdgcn_mfma_f32_16x16x4f32(hf[kk], vb[kk], da, 0, 0, 0);
        }
        // the next step's query tile leaves now: its registers are free
        const int t_next = j + 1 < steps ? row_of(j + 1) : t;
        load_rows(q_blk, ld_qkv, t_next, qf);
        load_rows(dh_blk, ld_dh, t_next, hf);

        // P^T and dS^T: register v is query 16t + 4kq + v, the lane's key is 16kt + l16
        floatx4 p, ds;
        const int key = 16 * kt + l16;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int query = 16 * t + 4 * kq + v;
            float pv = exp_neg(sc[v] * scale - m4[v]) * i4[v];
            if (causal && key > query) pv = 0.f;       // ml/layer.hpp:2979-2994
            p[v] = pv;
            ds[v] = (pv * (da[v] - d4[v])) * scale;
        }
        // dS^T into the patch as [query][key], read back as the B operand of the dQ product
        // (query l16, key 4kq + s); the wave's LDS accesses run in program order
#pragma unroll
        for (int v = 0; v < 4; ++v) patch[(4 * kq + v) * 20 + l16] = ds[v];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const floatx4 dst = *reinterpret_cast<const floatx4*>(patch + l16 * 20 + 4 * kq);

        // dV += dH P^T, dK += Q dS^T: A operand d = 16u + l16, query 4kq + s from the wave's copy;
        // the fragments of step s + 1 are requested before the MFMAs of step s are issued
        float av[NDT], ak[NDT], avn[NDT], akn[NDT];
        const float* rq = stage_q + (4 * kq) * LDP + l16;
        const float* rh = stage_dh + (4 * kq) * LDP + l16;
#pragma unroll
        for (int u = 0; u < NDT; ++u) {
            av[u] = rh[16 * u];
            ak[u] = rq[16 * u];
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            if (s + 1 < 4) {
#pragma unroll
                for (int u = 0; u < NDT; ++u) {
                    avn[u] = rh[(s + 1) * LDP + 16 * u];
                    akn[u] = rq[(s + 1) * LDP + 16 * u];
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < NDT; ++u) {
                dv_acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[u], p[s], dv_acc[u], 0, 0, 0);
                dk_acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(ak[u], ds[s], dk_acc[u], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < NDT; ++u) {
                av[u] = avn[u];
                ak[u] = akn[u];
            }
        }
        // dQ contribution of this cell, added to the accumulator slice read above:
        // register v of tile u is d = 16u + 4kq + v of query 16t + l16
        floatx4 dqc[NDT];
#pragma unroll
        for (int u = 0; u < NDT; ++u) dqc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int u = 0; u < NDT; ++u) dqc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[u][s], dst[s], dqc[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NDT; ++u) *reinterpret_cast<floatx4*>(acc + 16 * u) = cur[u] + dqc[u];
        t = t_next;
        __syncthreads();   // the next step's cells touch other query tiles of the accumulator
    };

    floatx4 dv_acc[NDT], dk_acc[NDT];
    auto clear_acc = [&]() {
#pragma unroll
        for (int u = 0; u < NDT; ++u) {
            dv_acc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
            dk_acc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
    };
    clear_acc();
    for (int j = 0; j < first; ++j) cell(j, o, kb0, vb0, ka0, dv_acc, dk_acc);
    store_key_tile(o, dv_acc, dk_acc);
    clear_acc();
    for (int j = first; j < steps; ++j) cell(j, tiles - 1 - o, kb1, vb1, ka1, dv_acc, dk_acc);
    store_key_tile(tiles - 1 - o, dv_acc, dk_acc);
    __syncthreads();
    // dQ of the block: S columns of DH contiguous floats
    for (int i = tid; i < S * (DH / 4); i += blockDim.x) {
        const int q = i / (DH / 4), c4 = i % (DH / 4);
        *reinterpret_cast<floatx4*>(dq_blk + static_cast<size_t>(q) * ld_d + 4 * c4) =
            *reinterpret_cast<const floatx4*>(dq_acc + static_cast<size_t>(q) * LDP + 4 * c4);
    }
}

template <int DH>
int launch_flash_bwd(float* dQ, float* dK, float* dV, int ld_d, const float* dH, int ld_dh, const float* Q,
                     const float* K, const float* V, int ld_qkv, const float* H, int ld_h, const float* stats,
                     const FlashSchedule* sched, int heads, int S, int B, float scale, int causal) {
    static std::once_flag once;   // per instantiation
    static int configure_rc = 0;
    std::call_once(once, [] {
        configure_rc = rc_of(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_flash_bwd_kernel<DH>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    });
    if (configure_rc) return configure_rc;
    const size_t lds = FlashLds<DH>::floats(S) * sizeof(float);
    attn_flash_bwd_kernel<DH><<<heads * B, 2 * S, lds, stream()>>>(dQ, dK, dV, ld_d, dH, ld_dh, Q, K, V, ld_qkv, H, ld_h,
                                                                  stats, sched, S, B, scale, causal);
    return launch_rc();
}

bool flash_shape_ok(int d_k, int heads, int S, int B) {
    if (d_k <= 0 || heads <= 0 || S <= 0 || B <= 0 || d_k % heads != 0) return false;
    const int d_h = d_k / heads;
    if (!(d_h == 32 || d_h == 64)) return false;
    if (S % 32 != 0 || S > 16 * kMaxTiles) return false;
    return static_cast<long long>(heads) * B <= 0x7fffffffLL;
}

}  // namespace
}  // namespace jz

JZ_API int jzhip_attention_flash_order(int S, int causal, int* cells, int capacity) {
    if (S <= 0 || S % 32 != 0 || S > 16 * jz::kMaxTiles || !cells || causal < 0 || causal > 1) return -1;
    jz::FlashSchedule s;
    if (!jz::build_schedule(S / 16, causal != 0, &s)) return -1;
    const int owners = S / 32;
    if (capacity < 2 * s.steps * owners) return -1;
    for (int j = 0; j < s.steps; ++j)
        for (int o = 0; o < owners; ++o) {
            // decoded the way the kernel decodes it
            const uint64_t word = j < 16 ? s.packed[o][0] : s.packed[o][1];
            cells[2 * (j * owners + o)] = static_cast<int>((word >> (4 * (j & 15))) & 15u);
            cells[2 * (j * owners + o) + 1] = j < s.first[o] ? o : s.tiles - 1 - o;
        }
    return s.steps;
}

JZ_API int jzhip_attention_flash_supported(int d_k, int heads, int S, int B) {
    return jz::flash_shape_ok(d_k, heads, S, B) ? 1 : 0;
}

JZ_API int jzhip_attention_flash_bwd(float* dQ, float* dK, float* dV, int ld_dqkv, const float* dH, int ld_dh,
                                     const float* Q, const float* K, const float* V, int ld_qkv, const float* H,
                                     int ld_h, const float* stats, int d_k, int heads, int S, int B, int causal) {
    if (!dQ || !dK || !dV || !dH || !Q || !K || !V || !H || !stats) return -1;
    if (!jz::flash_shape_ok(d_k, heads, S, B)) return -1;
    if (ld_dqkv < d_k || ld_dh < d_k || ld_qkv < d_k || ld_h < d_k) return -1;
    if (ld_dqkv % 4 || ld_dh % 4 || ld_qkv % 4 || ld_h % 4) return -1;
    if (!jz::aligned16(dQ) || !jz::aligned16(dK) || !jz::aligned16(dV) || !jz::aligned16(dH) || !jz::aligned16(Q) ||
        !jz::aligned16(K) || !jz::aligned16(V) || !jz::aligned16(H))
        return -1;
    if (causal < 0 || causal > 1) return -1;
    const int d_h = d_k / heads;
    const jz::FlashSchedule* sched = nullptr;
    int rc = jz::device_schedule(S / 16, causal != 0, &sched);
    if (rc) return rc;
    const float scale = 1.0f / sqrtf(static_cast<float>(d_h));
    if (d_h == 64)
        return jz::launch_flash_bwd<64>(dQ, dK, dV, ld_dqkv, dH, ld_dh, Q, K, V, ld_qkv, H, ld_h, stats, sched, heads, S,
                                        B, scale, causal);
    return jz::launch_flash_bwd<32>(dQ, dK, dV, ld_dqkv, dH, ld_dh, Q, K, V, ld_qkv, H, ld_h, stats, sched, heads, S, B,
                                    scale, causal);
}
