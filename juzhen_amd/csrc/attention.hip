// Batched causal self-attention core for TransformerLayer<ROCMfloat>: replaces
// the reference's per-(head, sequence) slice loop with its host-side mask
// writes (ml/layer.hpp:2967-3006, 3329-3363) by five batched launches forward
// and backward.  Same mathematics and the same buffer layouts as the
// reference's CUDA path (ml/layer.hpp:2880-2927, 3214-3283):
//   Q, K, V, H, dQ, dK, dV, dH : (d_k, S*B) column-major, head hh owns rows
//                                [hh*d_h, (hh+1)*d_h), sequence b columns [b*S, (b+1)*S)
//   A, dA                      : (S, S*B*heads), block hh*B + b is the S x S
//                                matrix A[query, key] of that head and sequence.
#include "common.hpp"

#include <cmath>

namespace jz {
int gemm_batched2(const float* A, const float* B, float* C, int m, int n, int k, bool ta, bool tb,
                  int lda, int ldb, int ldc, long long sA, long long sB, long long sC, int batch,
                  long long sA2, long long sB2, long long sC2, int batch2, float alpha, float beta);
}

JZ_API int jzhip_attention_fwd_ld(float* H, int ld_h, float* A, const float* Q, const float* K,
                                  const float* V, int ld_qkv, int d_k, int heads, int S, int B,
                                  int causal) {
    if (d_k <= 0 || heads <= 0 || S <= 0 || B <= 0 || d_k % heads != 0) return -1;
    if (!H || !A || !Q || !K || !V || ld_h < d_k || ld_qkv < d_k) return -1;
    const int d_h = d_k / heads;
    const long long seq = static_cast<long long>(S) * ld_qkv;  // next sequence in Q/K/V
    const long long seq_h = static_cast<long long>(S) * ld_h;  // next sequence in H
    const long long blk = static_cast<long long>(S) * S;       // next score block
    const float scale = 1.0f / sqrtf(static_cast<float>(d_h));
    // scores[q, k] = <Q_i[:, q], K_i[:, k]>
    int rc = jz::gemm_batched2(Q, K, A, S, S, d_h, true, false, ld_qkv, ld_qkv, S, seq, seq, blk, B, d_h, d_h,
                               blk * B, heads, 1.0f, 0.0f);
    if (rc) return rc;
    // A = softmax over keys of (scores*scale, masked)
    rc = jzhip_attn_softmax(A, A, S, B * heads, scale, causal, 0);
    if (rc) return rc;
    // H_i = V_i * A_i^T
    return jz::gemm_batched2(V, A, H, d_h, S, S, false, true, ld_qkv, S, ld_h, seq, blk, seq_h, B, d_h,
                             blk * B, d_h, heads, 1.0f, 0.0f);
}

JZ_API int jzhip_attention_fwd(float* H, float* A, const float* Q, const float* K, const float* V,
                               int d_k, int heads, int S, int B, int causal) {
    return jzhip_attention_fwd_ld(H, d_k, A, Q, K, V, d_k, d_k, heads, S, B, causal);
}

JZ_API int jzhip_attention_bwd_ld(float* dQ, float* dK, float* dV, int ld_dqkv, float* dA_scratch,
                                  const float* dH, int ld_dh, const float* Q, const float* K,
                                  const float* V, int ld_qkv, const float* A, int d_k, int heads,
                                  int S, int B) {
    if (d_k <= 0 || heads <= 0 || S <= 0 || B <= 0 || d_k % heads != 0) return -1;
    if (!dQ || !dK || !dV || !dA_scratch || !dH || !Q || !K || !V || !A) return -1;
    if (ld_dqkv < d_k || ld_dh < d_k || ld_qkv < d_k) return -1;
    const int d_h = d_k / heads;
    const long long seq = static_cast<long long>(S) * ld_qkv;
    const long long seq_d = static_cast<long long>(S) * ld_dqkv;
    const long long seq_h = static_cast<long long>(S) * ld_dh;
    const long long blk = static_cast<long long>(S) * S;
    const float scale = 1.0f / sqrtf(static_cast<float>(d_h));
    // dV_i = dH_i * A_i
    int rc = jz::gemm_batched2(dH, A, dV, d_h, S, S, false, false, ld_dh, S, ld_dqkv, seq_h, blk, seq_d, B, d_h,
                               blk * B, d_h, heads, 1.0f, 0.0f);
    if (rc) return rc;
    // dA_i[q, k] = <dH_i[:, q], V_i[:, k]>
    rc = jz::gemm_batched2(dH, V, dA_scratch, S, S, d_h, true, false, ld_dh, ld_qkv, S, seq_h, seq, blk, B, d_h,
                           d_h, blk * B, heads, 1.0f, 0.0f);
    if (rc) return rc;
    // dS = A .* (dA - rowsum(A .* dA)) * scale, in place
    rc = jzhip_attn_softmax_bwd(dA_scratch, A, dA_scratch, S, B * heads, scale, 0);
    if (rc) return rc;
    // dQ_i = K_i * dS_i^T
    rc = jz::gemm_batched2(K, dA_scratch, dQ, d_h, S, S, false, true, ld_qkv, S, ld_dqkv, seq, blk, seq_d, B, d_h,
                           blk * B, d_h, heads, 1.0f, 0.0f);
    if (rc) return rc;
    // dK_i = Q_i * dS_i
    return jz::gemm_batched2(Q, dA_scratch, dK, d_h, S, S, false, false, ld_qkv, S, ld_dqkv, seq, blk, seq_d, B,
                             d_h, blk * B, d_h, heads, 1.0f, 0.0f);
}

JZ_API int jzhip_attention_bwd(float* dQ, float* dK, float* dV, float* dA_scratch, const float* dH,
                               const float* Q, const float* K, const float* V, const float* A,
                               int d_k, int heads, int S, int B) {
    return jzhip_attention_bwd_ld(dQ, dK, dV, d_k, dA_scratch, dH, d_k, Q, K, V, d_k, A, d_k, heads, S, B);
}
