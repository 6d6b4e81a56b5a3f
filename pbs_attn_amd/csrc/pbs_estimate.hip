// Block-importance estimation: softmax over strictly-earlier-segment key blocks of
// the pooled-Q x pooled-K logits.
//
//   logit[qb, kb] = bf16( bf16(<Pq[qb], Pk[kb]>) / sqrt(D) )      kb < first block of qb's segment
//   P[qb, :]      = softmax_fp32(logit[qb, :])                     (0 outside the candidates)
// Rows with no candidate (query blocks of segment 0) are NaN, as a softmax over an
// all -inf row is.  One workgroup owns 32 query blocks of one head; its four
// waves split the key-block tiles, first to find each row's (max, sum), then to
// recompute the logits and write P with 128-byte row segments per store.
#include "pbs_common.h"
#include "pbs_div.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations

namespace {

constexpr int D = 128;

__device__ __forceinline__ bf16x8 load_frag(const uint16_t* row_ptr, int t, int half) {
  return *reinterpret_cast<const bf16x8*>(row_ptr + 16 * t + 8 * half);
}
// two accumulators -> the logits a bf16 matmul followed by a bf16 division by sqrt(D) yields: round to bf16, divide
// (the exact quotient, see pbs_div.h), round to bf16
struct Divisor {
  float b, y;   // sqrt(D) and its correctly rounded reciprocal
};
__device__ __forceinline__ f32x2 logit_round2(float acc0, float acc1, Divisor d) {
  const f32x2 r = hw_round_bf16x2((f32x2){acc0, acc1});
  return hw_round_bf16x2((f32x2){pbs_div_by_const(r.x, d.b, d.y), pbs_div_by_const(r.y, d.b, d.y)});
}

// number of candidate key blocks of query block qb (its candidates are key blocks 0 .. count - 1): the blocks
// of strictly earlier segments, or -- CAUSAL, the rule of the reference's un-permuted MeanPooling baseline --
// every block up to and including the diagonal one
template <bool CAUSAL>
__device__ __forceinline__ int candidate_count(int qb, int bps) {
  return CAUSAL ? qb + 1 : (qb / bps) * bps;
}

// CANDIDATES_ONLY: only the candidate entries of a row are written (the selection that follows on the single-call path
// reads no others); otherwise all nb columns, zeros outside the candidates and NaN rows where there are none.
template <bool CAUSAL, bool CANDIDATES_ONLY>
__global__ __launch_bounds__(256) void block_logits_softmax_kernel(const uint16_t* pooled_q, const uint16_t* pooled_k,
                                                                   float* P, int nb, int bps, Divisor sqrt_d) {
  __shared__ float s_m[4][32], s_l[4][32];
  __shared__ float s_max[32], s_inv[32];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 31, half = lane >> 5;
  const int qt = (int)gridDim.x - 1 - (int)blockIdx.x, bh = blockIdx.y;   // the tiles with the most candidates start first
  const uint16_t* pq = pooled_q + (int64_t)bh * nb * D;
  const uint16_t* pk = pooled_k + (int64_t)bh * nb * D;
  float* out = P + (int64_t)bh * nb * nb;

  const int q_last = min(32 * qt + 31, nb - 1);
  const int cand_max = candidate_count<CAUSAL>(q_last, bps);   // candidates of the tile's last row
  const int n_kt_cand = (cand_max + 31) / 32;
  const int n_kt_all = (nb + 31) / 32;

  bf16x8 qf[8];
  {
    const uint16_t* row = pq + (int64_t)min(32 * qt + j, nb - 1) * D;
#pragma unroll
    for (int t = 0; t < 8; ++t) qf[t] = load_frag(row, t, half);
  }

  // ---- pass A: per query block (column j) running max / sum over its candidates
  const int qb_col = 32 * qt + j;
  const int cand_col = qb_col < nb ? candidate_count<CAUSAL>(qb_col, bps) : 0;
  float m_run = -INFINITY, l_run = 0.f;
  for (int kt = wave; kt < n_kt_cand; kt += 4) {
    const uint16_t* row = pk + (int64_t)min(32 * kt + j, nb - 1) * D;
    f32x16 acc = {0};
#pragma unroll
    for (int t = 0; t < 8; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load_frag(row, t, half), qf[t], acc, 0, 0, 0);
    float v[16], mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const int kb = 32 * kt + 8 * (r >> 2) + 4 * half + (r & 3);
      const f32x2 l2 = logit_round2(acc[r], acc[r + 1], sqrt_d);
      v[r] = kb < cand_col ? l2.x : -INFINITY;
      v[r + 1] = kb + 1 < cand_col ? l2.y : -INFINITY;
      mx = fmaxf(mx, fmaxf(v[r], v[r + 1]));
    }
    if (mx > -INFINITY) {
      const float m_new = fmaxf(m_run, mx);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += __expf(v[r] - m_new);
      l_run = l_run * __expf(m_run - m_new) + sum;
      m_run = m_new;
    }
  }
  {
    const float m_o = xhalf_f32(m_run), l_o = xhalf_f32(l_run);
    const float m_new = fmaxf(m_run, m_o);
    float l_new = 0.f;
    if (m_new > -INFINITY) l_new = l_run * __expf(m_run - m_new) + l_o * __expf(m_o - m_new);
    if (half == 0) {
      s_m[wave][j] = m_new;
      s_l[wave][j] = l_new;
    }
  }
  __syncthreads();
  if (threadIdx.x < 32) {
    float m = -INFINITY, l = 0.f;
    for (int w = 0; w < 4; ++w) m = fmaxf(m, s_m[w][threadIdx.x]);
    if (m > -INFINITY)
      for (int w = 0; w < 4; ++w) l += s_l[w][threadIdx.x] * __expf(s_m[w][threadIdx.x] - m);
    s_max[threadIdx.x] = m;
    s_inv[threadIdx.x] = 1.0f / l;
  }
  __syncthreads();

  // ---- pass B: rows = query blocks, column = key block j of tile kt
  bf16x8 qa[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) qa[t] = qf[t];
  for (int kt = wave; kt < (CANDIDATES_ONLY ? n_kt_cand : n_kt_all); kt += 4) {
    const int kb = 32 * kt + j;
    f32x16 acc = {0};
    if (kt < n_kt_cand) {
      const uint16_t* row = pk + (int64_t)min(kb, nb - 1) * D;
#pragma unroll
      for (int t = 0; t < 8; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[t], load_frag(row, t, half), acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const f32x2 l2 = logit_round2(acc[r], acc[r + 1], sqrt_d);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int ql = 8 * (r >> 2) + 4 * half + (r & 3) + u;
        const int qb = 32 * qt + ql;
        if (qb < nb && kb < nb) {
          const int cand = candidate_count<CAUSAL>(qb, bps);
          float p;
          if (cand == 0) p = __uint_as_float(0x7fc00000u);
          else if (kb < cand) p = __expf((u ? l2.y : l2.x) - s_max[ql]) * s_inv[ql];
          else p = 0.f;
          if (!CANDIDATES_ONLY || kb < cand) out[(int64_t)qb * nb + kb] = p;
        }
      }
    }
  }
}

}  // namespace

namespace {
int launch_block_logits(const char* who, bool causal, bool candidates_only, const void* pooled_q, const void* pooled_k, float* block_attn_scores,
                        int rows, int nb, int head_dim, int blocks_per_segment, void* stream) {
  PBS_REQUIRE(pooled_q && pooled_k && block_attn_scores, "%s: null tensor pointer", who);
  PBS_REQUIRE(head_dim == D, "%s: head_dim must be 128, got %d", who, head_dim);
  PBS_REQUIRE(rows > 0 && rows <= 65535 && nb > 0 && blocks_per_segment > 0, "%s: bad shape", who);
  const dim3 grid((nb + 31) / 32, rows);
  Divisor sqrt_d;
  sqrt_d.b = (float)sqrt((double)head_dim);
  sqrt_d.y = (float)(1.0 / (double)sqrt_d.b);   // the correctly rounded reciprocal for head_dim 128 (tests/c_abi/div_check.c)
  if (candidates_only)
    hipLaunchKernelGGL((block_logits_softmax_kernel<false, true>), grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)pooled_q,
                       (const uint16_t*)pooled_k, block_attn_scores, nb, blocks_per_segment, sqrt_d);
  else if (causal)
    hipLaunchKernelGGL((block_logits_softmax_kernel<true, false>), grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)pooled_q,
                       (const uint16_t*)pooled_k, block_attn_scores, nb, blocks_per_segment, sqrt_d);
  else
    hipLaunchKernelGGL((block_logits_softmax_kernel<false, false>), grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)pooled_q,
                       (const uint16_t*)pooled_k, block_attn_scores, nb, blocks_per_segment, sqrt_d);
  return pbs_check_launch(who);
}
}  // namespace

extern "C" int pbs_block_logits_softmax(const void* pooled_q, const void* pooled_k, float* block_attn_scores, int rows,
                                        int nb, int head_dim, int blocks_per_segment, void* stream) {
  return launch_block_logits("pbs_block_logits_softmax", false, false, pooled_q, pooled_k, block_attn_scores, rows, nb, head_dim,
                             blocks_per_segment, stream);
}

extern "C" int pbs_block_logits_softmax_causal(const void* pooled_q, const void* pooled_k, float* block_attn_scores,
                                               int rows, int nb, int head_dim, void* stream) {
  return launch_block_logits("pbs_block_logits_softmax_causal", true, false, pooled_q, pooled_k, block_attn_scores, rows, nb,
                             head_dim, 1, stream);
}

extern "C" int pbs_block_logits_softmax_candidates_only(const void* pooled_q, const void* pooled_k, float* block_attn_scores, int rows,
                                             int nb, int head_dim, int blocks_per_segment, void* stream) {
  return launch_block_logits("pbs_block_logits_softmax", false, true, pooled_q, pooled_k, block_attn_scores, rows, nb, head_dim,
                             blocks_per_segment, stream);
}
