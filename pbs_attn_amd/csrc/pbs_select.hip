// Cumulative-threshold block selection and CSR emission.
//
// One workgroup per (head, query block) row of the block-probability matrix:
//   * NaN -> 0, stable descending sort of the row in LDS (64-bit composite keys),
//   * running sum in the order torch's CPU cumsum uses: sequential, accumulated in
//     float64, every prefix rounded to float32 and compared with float32(threshold),
//   * keep ranks <= the first prefix that reaches the threshold (none if never),
//   * OR in the block holding original key 0 (optional) and the row's own segment,
//   * emit the dense byte masks and the visit list: the ascending selected key blocks of
//     strictly earlier segments (the attention kernel adds the causal part of the row's
//     own segment itself, in original key order).
// Rows of up to 1024 blocks take the wave-level variant further down (one wave per row,
// the row in registers).
#include "pbs_common.h"
#include <utility>
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations
#include <float.h>

namespace {

struct SelectArgs {
  const float* P;          // (rows, nb, nb) or null when threshold_is_int_one
  const float* thr_rows;   // per-head thresholds (rows) or null
  float thr;
  int thr_is_int_one;
  int force_first;
  const int32_t* idx;      // (rows, nb*bs)
  int32_t* first_blk;      // (rows) workspace
  int nb, bs, bps, S, n_pow2;
  uint8_t* sel_mask;       // (rows, nb, nb) or null: selected | first-token
  uint8_t* final_mask;     // (rows, nb, nb) or null: sel | own segment
  int32_t* csr_cols;       // (rows, nb, nb) or null
  int32_t* csr_cnt;        // (rows, nb)
  uint8_t* needed;         // (rows, nb) or null: set to 1 for every key block on some query block's visit list
  int cand_rule;           // which entries of a row can be non-zero: 0 any, 1 kb < first block of qb's segment, 2 kb <= qb
  int qb_lo, qb_hi;        // wave kernel: the query blocks this launch covers
};

// Block that holds original key 0.  A segment-wise permutation keeps it inside the first segment, so that
// part of the row is searched first; the rest only if it is not there (any index layout stays correct).
__global__ __launch_bounds__(1024) void first_token_block_kernel(const int32_t* idx, int32_t* first_blk, int S_pad, int bs,
                                                                 int first_span) {
  __shared__ int found;
  if (threadIdx.x == 0) found = -1;
  __syncthreads();
  const int32_t* row = idx + (int64_t)blockIdx.x * S_pad;
  for (int i = threadIdx.x; i < first_span; i += blockDim.x)
    if (row[i] == 0) atomicMax(&found, i / bs);
  __syncthreads();
  if (found < 0) {
    for (int i = first_span + threadIdx.x; i < S_pad; i += blockDim.x)
      if (row[i] == 0) atomicMax(&found, i / bs);
  }
  __syncthreads();
  if (threadIdx.x == 0) first_blk[blockIdx.x] = found;
}

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int lane_mask) {
  const uint32_t lo = __shfl_xor((uint32_t)v, lane_mask, 64), hi = __shfl_xor((uint32_t)(v >> 32), lane_mask, 64);
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ double shfl_up_f64(double v, int delta) {
  const uint64_t u = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = __shfl_up((uint32_t)u, delta, 64), hi = __shfl_up((uint32_t)(u >> 32), delta, 64);
  return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ double readlane_f64(double v, int lane) {
  const uint64_t u = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)u, lane), hi = __builtin_amdgcn_readlane((int)(uint32_t)(u >> 32), lane);
  return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

__global__ __launch_bounds__(256) void select_blocks_kernel(SelectArgs a) {
  extern __shared__ uint64_t keys[];
  uint8_t* flag = reinterpret_cast<uint8_t*>(keys + a.n_pow2);
  __shared__ int s_first;
  __shared__ int s_scan[256];
  const int qb = blockIdx.x, row = blockIdx.y;
  const int nb = a.nb;
  const int seg_first = (qb / a.bps) * a.bps;
  const int seg_end = min(seg_first + a.bps, nb);
  const int64_t row_off = ((int64_t)row * nb + qb) * nb;

  for (int kb = threadIdx.x; kb < nb; kb += blockDim.x) flag[kb] = 0;

  if (a.thr_is_int_one) {
    __syncthreads();
    for (int kb = threadIdx.x; kb < seg_first; kb += blockDim.x) flag[kb] = 1;
  } else {
    const float* p = a.P + row_off;
    for (int i = threadIdx.x; i < a.n_pow2; i += blockDim.x) {
      uint64_t key = ~0ull;
      if (i < nb) {
        float v = p[i];
        if (v != v) v = 0.f;
        else if (v == INFINITY) v = FLT_MAX;
        else if (v == -INFINITY) v = -FLT_MAX;
        key = desc_stable_key(v, (uint32_t)i);
      }
      keys[i] = key;
    }
    bitonic_sort_lds(keys, a.n_pow2);
    if (threadIdx.x < 64) {
      // Running sum of the sorted row by ONE wave: lane l owns the `per` consecutive ranks from l * per.  The
      // sum is first taken as a parallel float64 prefix (local sums + wave scan), which differs from the
      // sequential float64 sum torch's CPU cumsum forms by < 1e-12; "float32(prefix) >= threshold" is decided
      // from it unless a prefix up to the first hit lies within 1e-11 of the float32 rounding boundary of the
      // threshold -- only then the exact sequential sum is evaluated, lane after lane.  Either way the decision
      // is the sequential sum's.
      const int lane = threadIdx.x;
      const int per = a.n_pow2 / 64;   // n_pow2 >= 2048 here
      const float thr = a.thr_rows ? a.thr_rows[row] : a.thr;
      const int r_lo = lane * per;
      double c = 0.0;
      for (int u = 0; u < per; ++u) {
        const int r = r_lo + u;
        c += r < nb ? (double)desc_key_value(keys[r]) : 0.0;
      }
      double incl = c;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const double t = shfl_up_f64(incl, d);
        if (lane >= d) incl += t;
      }
      double excl = shfl_up_f64(incl, 1);
      if (lane == 0) excl = 0.0;
      const double mid = 0.5 * ((double)thr + (double)nextafterf(thr, -INFINITY));
      const double tol = 1e-11 * fmax(1.0, fabs(mid));
      int my_first = INT_MAX, my_amb = INT_MAX;   // first reaching rank / first ambiguous rank of this lane
      {
        double cp = excl;
        for (int u = 0; u < per; ++u) {
          const int r = r_lo + u;
          if (r >= nb) break;
          cp += (double)desc_key_value(keys[r]);
          if (my_first == INT_MAX && (float)cp >= thr) my_first = r;
          if (my_amb == INT_MAX && fabs(cp - mid) <= tol) my_amb = r;
        }
      }
      int first = my_first, amb = my_amb;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        first = min(first, __shfl_xor(first, off, 64));
        amb = min(amb, __shfl_xor(amb, off, 64));
      }
      if (amb <= first && amb != INT_MAX) {
        // exact sequential sum: lane after lane, each continuing from the lane before
        double carry = 0.0;
        first = INT_MAX;
        for (int L = 0; L < 64 && first == INT_MAX; ++L) {
          double cs = carry;
          int hit = INT_MAX;
          if (lane == L) {
            for (int u = 0; u < per; ++u) {
              const int r = r_lo + u;
              if (r >= nb) break;
              cs += (double)desc_key_value(keys[r]);
              if (hit == INT_MAX && (float)cs >= thr) hit = r;
            }
          }
          carry = readlane_f64(cs, L);
          first = __builtin_amdgcn_readlane(hit, L);
        }
      }
      if (lane == 0) s_first = (first == INT_MAX || first >= nb) ? -1 : first;
    }
    __syncthreads();
    const int first = s_first;
    for (int r = threadIdx.x; r <= first; r += blockDim.x) flag[(uint32_t)keys[r]] = 1;
  }
  __syncthreads();
  if (a.force_first && threadIdx.x == 0) {
    const int fb = a.first_blk[row];
    if (fb >= 0 && fb < nb) flag[fb] = 1;
  }
  __syncthreads();

  // visit list: the selected blocks of strictly earlier segments (the attention kernel adds the query
  // block's own segment itself)
  const int per = (nb + 255) / 256;
  const int k0 = threadIdx.x * per, k1 = min(k0 + per, nb);
  int cnt = 0;
  for (int kb = k0; kb < k1; ++kb) {
    const bool own = kb >= seg_first && kb < seg_end;
    const uint8_t s = flag[kb];
    if (a.sel_mask) a.sel_mask[row_off + kb] = s;
    if (a.final_mask) a.final_mask[row_off + kb] = s | (own ? 1 : 0);
    cnt += (s && kb < seg_first) ? 1 : 0;
  }
  s_scan[threadIdx.x] = cnt;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    int v = 0;
    if ((int)threadIdx.x >= off) v = s_scan[threadIdx.x - off];
    __syncthreads();
    s_scan[threadIdx.x] += v;
    __syncthreads();
  }
  int w = s_scan[threadIdx.x] - cnt;
  if (a.csr_cols) {
    for (int kb = k0; kb < k1; ++kb) {
      if (flag[kb] && kb < seg_first) a.csr_cols[row_off + w++] = kb;
    }
  }
  if (a.needed) {
    for (int kb = k0; kb < k1; ++kb)
      if (flag[kb] && kb < seg_first) a.needed[(int64_t)row * nb + kb] = 1;   // every writer stores the same value
  }
  if (threadIdx.x == 255) a.csr_cnt[(int64_t)row * nb + qb] = s_scan[255];
}


// ---------------------------------------------------------------------------------------------
// Wave-level variant (rows of up to 1024 blocks): ONE wave per row, the row lives in registers.
//   * bitonic network on the 32-bit value keys, NPL keys per lane: strides below NPL are register
//     compare-exchanges, larger strides exchange with lane ^ (stride / NPL); no barriers; the stable order's
//     tie-break by index is applied only where it matters, at the value where the threshold is reached;
//   * the running sum is first taken as a parallel float64 prefix (local prefixes + wave scan).  It
//     differs from the sequential sum by < 1e-12, so "float32(prefix) >= threshold" is decided from it
//     unless some prefix up to the first hit lies within 1e-11 of the float32 rounding boundary of the
//     threshold; only then the exact sequential sum is evaluated (lane after lane).  Either way the
//     decision is the one the sequential float64 sum gives;
//   * flags, own-segment minima, masks and the compacted visit list as in the block-level kernel.
// ---------------------------------------------------------------------------------------------
// The bitonic network on 32-bit keys, NPL per lane: a compare-exchange is a minimum and a maximum.
template <int NPL>
__device__ __forceinline__ void wave_bitonic_sort_u32(uint32_t (&k)[NPL], int lane) {
  constexpr int N = 64 * NPL;
#pragma unroll
  for (int size = 2; size <= N; size <<= 1) {
#pragma unroll
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (stride >= NPL) {
        const int lstride = stride / NPL;
        const bool keep_min = ((lane & lstride) == 0) == ((lane & (size / NPL)) == 0);
#pragma unroll
        for (int r = 0; r < NPL; ++r) {
          const uint32_t o = (uint32_t)__shfl_xor((int)k[r], lstride, 64);
          k[r] = keep_min ? min(k[r], o) : max(k[r], o);
        }
      } else {
#pragma unroll
        for (int r = 0; r < NPL; ++r) {
          if ((r & stride) == 0) {
            const int p = r | stride;
            const bool up = (size >= NPL) ? ((lane & (size / NPL)) == 0) : ((r & size) == 0);
            const uint32_t lo = min(k[r], k[p]), hi = max(k[r], k[p]);
            k[r] = up ? lo : hi;
            k[p] = up ? hi : lo;
          }
        }
      }
    }
  }
}

// one wave decides row `rq` ((row, qb - qb_lo) flattened) of the group of rows [qb_lo, qb_hi) x all heads
template <int NPL>
__device__ __forceinline__ void select_row_by_wave(const SelectArgs& a, int64_t rq, int total_rows, uint8_t* smem_w) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nb = a.nb;
  const int nb_pad = (nb + 15) & ~15;
  uint8_t* flag = smem_w + wave * nb_pad;
  if (rq >= total_rows) return;
  const int nqb = a.qb_hi - a.qb_lo;
  const int row = (int)(rq / nqb), qb = a.qb_lo + (int)(rq % nqb);
  const int seg_first = (qb / a.bps) * a.bps;
  const int seg_end = min(seg_first + a.bps, nb);
  const int64_t row_off = ((int64_t)row * nb + qb) * nb;

  for (int kb = lane; kb < nb; kb += 64) flag[kb] = 0;

  if (a.thr_is_int_one) {
    for (int kb = lane; kb < seg_first; kb += 64) flag[kb] = 1;
  } else {
    const float* p = a.P + row_off;
    // entries that are zero by construction sort behind every candidate (ties keep index order) and add nothing
    // to the running sum: the row is sorted up to its last candidate only (the launch is sized for that)
    const int count = a.cand_rule == 1 ? seg_first : a.cand_rule == 2 ? min(qb + 1, nb) : nb;
    uint64_t k[NPL];
#pragma unroll
    for (int r = 0; r < NPL; ++r) {
      const int i = lane * NPL + r;
      uint64_t key = ~0ull;
      if (i < count) {
        float v = p[i];
        if (v != v) v = 0.f;
        else if (v == INFINITY) v = FLT_MAX;
        else if (v == -INFINITY) v = -FLT_MAX;
        key = desc_stable_key(v, (uint32_t)i);
      }
      k[r] = key;
    }
    const float thr = a.thr_rows ? a.thr_rows[row] : a.thr;

    // Rows whose mass sits in a few blocks need no sort: the largest remaining entry is taken out of the row
    // (smallest composite key: value descending, ties by index -- the order of the sort) and added to the
    // sequential float64 sum until float32(sum) reaches the threshold: the reference's decision, term by term.
    // Tried only when EXTRACT_MAX times the row's largest value can reach the threshold; a row that does not
    // get there in EXTRACT_MAX steps is sorted whole like any other.
    bool decided = false;
    if (NPL > 1) {
      constexpr int EXTRACT_MAX = 16;
      uint64_t best = k[0];
#pragma unroll
      for (int r = 1; r < NPL; ++r) best = k[r] < best ? k[r] : best;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const uint64_t o = shfl_xor_u64(best, off);
        best = o < best ? o : best;
      }
      if (best != ~0ull && (float)((double)desc_key_value(best) * EXTRACT_MAX) >= thr) {
        uint64_t w[NPL];
#pragma unroll
        for (int r = 0; r < NPL; ++r) w[r] = k[r];
        double cum = 0.0;
        uint32_t my_idx = 0;
        int taken = 0;
        for (int it = 0; it < EXTRACT_MAX; ++it) {
          if (it > 0) {
            best = w[0];
#pragma unroll
            for (int r = 1; r < NPL; ++r) best = w[r] < best ? w[r] : best;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
              const uint64_t o = shfl_xor_u64(best, off);
              best = o < best ? o : best;
            }
            if (best == ~0ull) break;   // the row has no further entry: not reached, let the sort path say so
          }
          if (lane == it) my_idx = (uint32_t)best;
#pragma unroll
          for (int r = 0; r < NPL; ++r) w[r] = (w[r] == best) ? ~0ull : w[r];
          cum += (double)desc_key_value(best);
          taken = it + 1;
          if ((float)cum >= thr) {
            decided = true;
            break;
          }
        }
        if (decided && lane < taken) flag[my_idx] = 1;
      }
    }
    if (!decided) {
    // The sort runs on the 32-bit value keys alone (ascending key = descending value).  Entries of equal value are
    // interchangeable in the running sum; which of them the stable order takes first matters only for the value at
    // which the threshold is reached, and is settled there by index (below).
    uint32_t kv[NPL], k0v[NPL];
#pragma unroll
    for (int r = 0; r < NPL; ++r) kv[r] = k0v[r] = (uint32_t)(k[r] >> 32);
    wave_bitonic_sort_u32<NPL>(kv, lane);

    float v[NPL];
#pragma unroll
    for (int r = 0; r < NPL; ++r) v[r] = (lane * NPL + r < count) ? f32_from_orderable(~kv[r]) : 0.f;
    // parallel float64 prefix
    double loc[NPL];
    double c = 0.0;
#pragma unroll
    for (int r = 0; r < NPL; ++r) {
      c += (double)v[r];
      loc[r] = c;
    }
    double incl = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const double t = shfl_up_f64(incl, d);
      if (lane >= d) incl += t;
    }
    double excl = shfl_up_f64(incl, 1);
    if (lane == 0) excl = 0.0;
    // float32 rounding boundary of the threshold (midpoint to its predecessor), as a double
    const double mid = 0.5 * ((double)thr + (double)nextafterf(thr, -INFINITY));
    uint32_t reach = 0, amb = 0;
#pragma unroll
    for (int r = 0; r < NPL; ++r) {
      const double cp = excl + loc[r];
      reach |= ((float)cp >= thr ? 1u : 0u) << r;
      amb |= (fabs(cp - mid) <= 1e-11 * fmax(1.0, fabs(mid)) ? 1u : 0u) << r;
    }
    int first = reach ? lane * NPL + __builtin_ctz(reach) : INT_MAX;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) first = min(first, __shfl_xor(first, off, 64));
    // ambiguous prefixes at or before the first hit?
    bool my_amb = false;
#pragma unroll
    for (int r = 0; r < NPL; ++r) my_amb |= ((amb >> r) & 1u) && (lane * NPL + r <= first) && (lane * NPL + r < nb);
    if (__any(my_amb)) {
      // exact sequential sum, lane after lane
      double carry = 0.0;
      first = INT_MAX;
      for (int L = 0; L < 64; ++L) {
        double cs = carry;
        uint32_t rch = 0;
#pragma unroll
        for (int r = 0; r < NPL; ++r) {
          cs += (double)v[r];
          rch |= ((float)cs >= thr ? 1u : 0u) << r;
        }
        const uint32_t rl = (uint32_t)__builtin_amdgcn_readlane((int)rch, L);
        carry = readlane_f64(cs, L);
        if (rl) {
          first = L * NPL + __builtin_ctz(rl);
          break;
        }
      }
    }
    if (first >= count) first = -1;   // never reached (padding ranks cannot qualify: they add zero)
    if (first >= 0) {
      // the selection is ranks 0 .. first of the stable order: every entry above the value at rank `first`, and of
      // the entries equal to it the m lowest indices, m = first + 1 - (number of entries above it)
      uint32_t mine = 0;
#pragma unroll
      for (int r = 0; r < NPL; ++r) mine = (r == first % NPL) ? kv[r] : mine;
      const uint32_t kstar = (uint32_t)__builtin_amdgcn_readlane((int)mine, first / NPL);
      int above = 0, ties = 0;
#pragma unroll
      for (int r = 0; r < NPL; ++r) {
        above += k0v[r] < kstar ? 1 : 0;
        ties += k0v[r] == kstar ? 1 : 0;
      }
      int ties_incl = ties;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int t = __shfl_up(ties_incl, d, 64);
        if (lane >= d) ties_incl += t;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) above += __shfl_xor(above, off, 64);
      const int m = first + 1 - above;
      int tie_rank = ties_incl - ties;   // ties at lower indices
#pragma unroll
      for (int r = 0; r < NPL; ++r) {
        const bool tie = k0v[r] == kstar;
        if (k0v[r] < kstar || (tie && tie_rank < m)) flag[lane * NPL + r] = 1;
        tie_rank += tie ? 1 : 0;
      }
    }
    }   // !decided
    // a row without candidates is all zeros: sorted whole, its first entry is block 0 and the running sum is 0
    if (count == 0 && 0.0f >= thr && lane == 0) flag[0] = 1;
  }
  __builtin_amdgcn_wave_barrier();
  if (a.force_first && lane == 0) {
    const int fb = a.first_blk[row];
    if (fb >= 0 && fb < nb) flag[fb] = 1;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  int base = 0;
  // without mask outputs only the blocks of earlier segments matter: they are what the visit list and the gather's
  // filter hold
  const int kb_end = (a.sel_mask || a.final_mask) ? nb : seg_first;
  for (int kb0 = 0; kb0 < kb_end; kb0 += 64) {
    const int kb = kb0 + lane;
    bool visit = false;
    if (kb < kb_end) {
      const bool own = kb >= seg_first && kb < seg_end;
      const uint8_t sf = flag[kb];
      if (a.sel_mask) a.sel_mask[row_off + kb] = sf;
      if (a.final_mask) a.final_mask[row_off + kb] = sf | (own ? 1 : 0);
      visit = sf && kb < seg_first;   // own-segment blocks are the attention kernel's business
    }
    const uint64_t ballot = __ballot(visit);
    if (visit && a.csr_cols) a.csr_cols[row_off + base + __popcll(ballot & ((1ull << lane) - 1ull))] = kb;
    if (visit && a.needed) a.needed[(int64_t)row * nb + kb] = 1;   // every writer stores the same value
    base += __popcll(ballot);
  }
  if (lane == 0) a.csr_cnt[(int64_t)row * nb + qb] = base;
}

template <int NPL>
__global__ __launch_bounds__(256) void select_blocks_wave_kernel(SelectArgs a, int total_rows) {
  extern __shared__ uint8_t smem_w[];
  select_row_by_wave<NPL>(a, (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), total_rows, smem_w);
}

// Up to five groups of rows of like length (see pbs_select_blocks) in ONE launch, the longest rows first: as launches
// of their own the groups run one after the other and each ends with a tail of idle CUs.
struct SelectGroups {
  int n;
  int npl[5], qb_lo[5], qb_hi[5];
  int wg_end[5];   // workgroups of groups 0 .. g
};
__global__ __launch_bounds__(256) void select_blocks_groups_kernel(SelectArgs a, SelectGroups gr, int rows) {
  extern __shared__ uint8_t smem_w[];
  int g = 0;
  while (g + 1 < gr.n && (int)blockIdx.x >= gr.wg_end[g]) ++g;
  const int wg0 = g == 0 ? 0 : gr.wg_end[g - 1];
  a.qb_lo = gr.qb_lo[g];
  a.qb_hi = gr.qb_hi[g];
  const int total = rows * (a.qb_hi - a.qb_lo);
  const int64_t rq = (int64_t)((int)blockIdx.x - wg0) * 4 + (threadIdx.x >> 6);
  switch (gr.npl[g]) {
    case 1: select_row_by_wave<1>(a, rq, total, smem_w); break;
    case 2: select_row_by_wave<2>(a, rq, total, smem_w); break;
    case 4: select_row_by_wave<4>(a, rq, total, smem_w); break;
    case 8: select_row_by_wave<8>(a, rq, total, smem_w); break;
    default: select_row_by_wave<16>(a, rq, total, smem_w); break;
  }
}

// Visit lists from a given block mask: one wave per (row, query block), the set bits of strictly earlier segments
// compacted in ascending order; own_missing counts the blocks of the query block's own segment the mask leaves out
// (in permuted order any of them can hold keys the query may see).
__global__ __launch_bounds__(256) void mask_to_csr_kernel(const uint8_t* __restrict__ mask, int32_t* __restrict__ cols,
                                                          int32_t* __restrict__ cnt, int32_t* __restrict__ own_missing, int nb,
                                                          int bps, int total_rows) {
  const int lane = threadIdx.x & 63;
  const int64_t rq = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (rq >= total_rows) return;
  const int qb = (int)(rq % nb);
  const int seg_first = (qb / bps) * bps, seg_end = min(seg_first + bps, nb);
  const uint8_t* m = mask + rq * nb;
  int base = 0, missing = 0;
  for (int kb0 = 0; kb0 < seg_end; kb0 += 64) {
    const int kb = kb0 + lane;
    const bool on = kb < seg_end && m[kb] != 0;
    const bool visit = on && kb < seg_first;
    const uint64_t ballot = __ballot(visit);
    if (visit) cols[rq * nb + base + __popcll(ballot & ((1ull << lane) - 1ull))] = kb;
    base += __popcll(ballot);
    missing += __popcll(__ballot(kb >= seg_first && kb < seg_end && !on));
  }
  if (lane == 0) {
    cnt[rq] = base;
    if (missing) atomicAdd(own_missing, missing);
  }
}

}  // namespace

extern "C" int pbs_block_mask_to_csr(const uint8_t* block_mask, int32_t* csr_cols, int32_t* csr_cnt, int32_t* own_missing,
                                     int rows, int nb, int blocks_per_segment, void* stream) {
  PBS_REQUIRE(block_mask && csr_cols && csr_cnt && own_missing, "pbs_block_mask_to_csr: null pointer");
  PBS_REQUIRE(rows > 0 && nb > 0 && nb <= 4096 && blocks_per_segment > 0 && (int64_t)rows * nb < (1ll << 31),
              "pbs_block_mask_to_csr: bad shape");
  const int total = rows * nb;
  hipLaunchKernelGGL(mask_to_csr_kernel, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, (hipStream_t)stream, block_mask,
                     csr_cols, csr_cnt, own_missing, nb, blocks_per_segment, total);
  return pbs_check_launch("pbs_block_mask_to_csr");
}

extern "C" size_t pbs_select_blocks_workspace_bytes(int rows) { return (size_t)rows * sizeof(int32_t); }

extern "C" int pbs_select_blocks(const float* block_attn_scores, const float* threshold_per_row, float threshold,
                                 int threshold_is_int_one, int force_select_first_block, int candidate_rule,
                                 const int32_t* key_indices, int rows, int S, int block_size, int segment_size, uint8_t* sel_mask,
                                 uint8_t* final_mask, int32_t* csr_cols, int32_t* csr_cnt, uint8_t* block_needed,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  PBS_REQUIRE(key_indices && csr_cnt, "pbs_select_blocks: null index / count pointer");
  PBS_REQUIRE(threshold_is_int_one || block_attn_scores, "pbs_select_blocks: null score pointer");
  PBS_REQUIRE(rows > 0 && rows <= 65535 && S > 0, "pbs_select_blocks: bad shape");
  PBS_REQUIRE(candidate_rule >= 0 && candidate_rule <= 2, "pbs_select_blocks: candidate_rule must be 0, 1 or 2");
  PBS_REQUIRE(block_size > 0 && block_size <= 256, "pbs_select_blocks: block_size %d outside (0, 256]", block_size);
  PBS_REQUIRE(segment_size > 0 && segment_size % block_size == 0, "pbs_select_blocks: segment_size must be a multiple of block_size");
  const int nb = (S + block_size - 1) / block_size;
  const int bps = segment_size / block_size;
  PBS_REQUIRE(nb <= 4096, "pbs_select_blocks: more than 4096 blocks per sequence (%d)", nb);
  PBS_REQUIRE(workspace && workspace_bytes >= pbs_select_blocks_workspace_bytes(rows), "pbs_select_blocks: workspace too small");
  SelectArgs a;
  a.P = block_attn_scores; a.thr_rows = threshold_per_row; a.thr = threshold;
  a.thr_is_int_one = threshold_is_int_one; a.force_first = force_select_first_block;
  a.idx = key_indices; a.first_blk = (int32_t*)workspace;
  a.nb = nb; a.bs = block_size; a.bps = bps; a.S = S; a.n_pow2 = next_pow2_int(nb);
  a.sel_mask = sel_mask; a.final_mask = final_mask; a.csr_cols = csr_cols; a.csr_cnt = csr_cnt;
  a.needed = block_needed;
  a.cand_rule = candidate_rule; a.qb_lo = 0; a.qb_hi = nb;
  hipStream_t st = (hipStream_t)stream;
  if (force_select_first_block)
    hipLaunchKernelGGL(first_token_block_kernel, dim3(rows), dim3(1024), 0, st, key_indices, a.first_blk, nb * block_size, block_size,
                       min(segment_size, nb * block_size));
  if (nb <= 1024) {
    // one wave per row, four rows per workgroup.  The sort network is sized for the longest row of a launch;
    // where the number of candidates grows with the query block, the rows are launched in groups of like length
    const size_t lds_w = (size_t)4 * ((nb + 15) & ~15);
    auto launch = [&](int npl, int qb_lo, int qb_hi) {
      SelectArgs g = a;
      g.qb_lo = qb_lo; g.qb_hi = qb_hi;
      const int total = rows * (qb_hi - qb_lo);
      const dim3 grid((unsigned)((total + 3) / 4));
      switch (npl) {
        case 1: hipLaunchKernelGGL(select_blocks_wave_kernel<1>, grid, dim3(256), lds_w, st, g, total); break;
        case 2: hipLaunchKernelGGL(select_blocks_wave_kernel<2>, grid, dim3(256), lds_w, st, g, total); break;
        case 4: hipLaunchKernelGGL(select_blocks_wave_kernel<4>, grid, dim3(256), lds_w, st, g, total); break;
        case 8: hipLaunchKernelGGL(select_blocks_wave_kernel<8>, grid, dim3(256), lds_w, st, g, total); break;
        default: hipLaunchKernelGGL(select_blocks_wave_kernel<16>, grid, dim3(256), lds_w, st, g, total); break;
      }
    };
    if (candidate_rule == 0 || threshold_is_int_one) {
      launch(threshold_is_int_one || nb <= 64 ? 1 : nb <= 128 ? 2 : nb <= 256 ? 4 : nb <= 512 ? 8 : 16, 0, nb);
    } else {
      SelectGroups gr;
      gr.n = 0;
      int qb_lo = 0;
      for (int npl = 1; npl <= 16 && qb_lo < nb; npl *= 2) {
        // query blocks whose candidate count fits 64 * npl sorted entries
        const int64_t lim = 64 * npl;
        int64_t hi = candidate_rule == 1 ? (lim / bps + 1) * (int64_t)bps : lim;
        if (npl == 16 || hi > nb) hi = nb;
        if (hi > qb_lo) {
          gr.npl[gr.n] = npl; gr.qb_lo[gr.n] = qb_lo; gr.qb_hi[gr.n] = (int)hi;
          ++gr.n;
          qb_lo = (int)hi;
        }
      }
      if (gr.n == 1) {
        launch(gr.npl[0], gr.qb_lo[0], gr.qb_hi[0]);
      } else {
        // longest rows first
        for (int x = 0; x < gr.n / 2; ++x) {
          std::swap(gr.npl[x], gr.npl[gr.n - 1 - x]);
          std::swap(gr.qb_lo[x], gr.qb_lo[gr.n - 1 - x]);
          std::swap(gr.qb_hi[x], gr.qb_hi[gr.n - 1 - x]);
        }
        int wgs = 0;
        for (int x = 0; x < gr.n; ++x) {
          wgs += (rows * (gr.qb_hi[x] - gr.qb_lo[x]) + 3) / 4;
          gr.wg_end[x] = wgs;
        }
        hipLaunchKernelGGL(select_blocks_groups_kernel, dim3((unsigned)wgs), dim3(256), lds_w, st, a, gr, rows);
      }
    }
    return pbs_check_launch("pbs_select_blocks");
  }
  const size_t lds = (size_t)a.n_pow2 * sizeof(uint64_t) + (size_t)((nb + 15) / 16) * 16;
  hipLaunchKernelGGL(select_blocks_kernel, dim3(nb, rows), dim3(256), lds, st, a);
  return pbs_check_launch("pbs_select_blocks");
}
