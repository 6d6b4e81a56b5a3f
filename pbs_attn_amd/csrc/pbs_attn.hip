// Block-sparse flash-attention forward over permuted keys (bf16, head_dim 128).
//
// One workgroup = one 128-query block of one head; its four waves own 32 queries
// each and walk the row's list of selected key blocks.  Per key block the K tile
// (128 keys x 128 d, row-major) and the V tile (stored transposed, 128 d x 128
// keys) are copied asynchronously straight into LDS (no registers) with a 16-byte
// XOR swizzle -- the next K tile while softmax and P.V run, the next V tile while
// the next S is computed -- and consumed by
// v_mfma_f32_32x32x16_bf16 in the transposed formulation
//     S^T = K Q^T            (rows = keys,  columns = queries)
//     O^T += V^T P^T         (rows = d,     columns = queries)
// so that every lane owns ONE query column: row max / row sum are in-lane
// reductions plus one exchange with lane^32, and the S^T accumulator registers
// are, after conversion to bf16, exactly the B operand of the second product
// (the key rows of each 32-row MFMA tile are fed in the order that makes this so).
// Softmax runs in the exp2 domain in fp32; P is rounded to bf16 before P.V and
// the row sum uses the unrounded values; the output is normalised at the end.
// Key blocks of the query block's own segment take the element mask
// "original key position > query position"; earlier segments need no mask.
#include "pbs_common.h"

namespace {

constexpr int D = 128;
constexpr int BS = 128;

struct AttnArgs {
  const uint16_t* q;
  const uint16_t* pk;    // (B*Hq, nb*128, 128)
  const uint16_t* pvt;   // (B*Hq, nb, 128, 128)
  const int32_t* idx;    // (B*Hq, nb*128)
  const int32_t* cols;   // (B*Hq, nb, nb)
  const int32_t* cnt;    // (B*Hq, nb)
  uint16_t* o;
  int BH, Hq, S, nb, bps;
  int64_t q_sb, q_sh, q_ss, o_sb, o_sh, o_ss;
  float scale_log2;
};

// row of the 32-row MFMA tile -> key of the 32-key sub-tile, chosen so that the
// accumulator registers 8u..8u+7 of lane-half g hold keys 16u + 8g + 0..7
__device__ __forceinline__ int mfma_row_to_key(int i) {
  const int a = i >> 3, g = (i >> 2) & 1, c = i & 3;
  return 16 * (a >> 1) + 8 * g + 4 * (a & 1) + c;
}

// ---- asynchronous global -> LDS copy of one 32 KB tile ------------------------------------
// LDS keeps a tile as 128 rows x 16 chunks of 16 bytes; physical chunk p of row r holds logical
// chunk p ^ (r & 15) (bank-conflict-free fragment reads).  global_load_lds_dwordx4 writes lane l
// at M0 + 16 l, so one wave instruction fills 4 consecutive rows and the swizzle is applied on
// the GLOBAL side: lane l of wave w fetches chunk (l & 15) ^ (row & 15) of row 4 w + 16 n + (l >> 4).
// That chunk does not depend on n: one per-lane byte offset serves the eight loads of a tile,
// the tile base and the LDS base advance by 4096 bytes per load in scalar registers.
// The copy is issued from inline assembly so that the compiler does not order later LDS reads
// of OTHER buffers behind it; completion is awaited with explicit s_waitcnt vmcnt(N).
__device__ __forceinline__ uint32_t async_lane_offset(int wave, int lane) {
  const int row = 4 * wave + (lane >> 4);
  const int c = (lane & 15) ^ (row & 15);
  return (uint32_t)((row * D + c * 8) * 2);
}

__device__ __forceinline__ void stage_tile_async(const uint16_t* src, const uint16_t* lds, int wave, uint32_t lane_off) {
  const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane(
      (int)((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)lds + wave * 1024));
  // readfirstlane returns int: widen through uint32_t or the low half would be sign-extended
  const uint64_t src0 = (uint64_t)(uintptr_t)src;
  const uint32_t src_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src0);
  const uint32_t src_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(src0 >> 32));
  const uint64_t srcu = ((uint64_t)src_hi << 32) | (uint64_t)src_lo;
#pragma unroll
  for (int n = 0; n < 8; ++n) {
    const uint64_t base = srcu + n * 4096;
    const uint32_t m0v = lds0 + n * 4096;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(lane_off), "s"(base)
                 : "memory");
  }
}

#define PBS_WAIT_VMCNT_8() __builtin_amdgcn_s_waitcnt(0x0f78)   // at most the 8 newest loads outstanding
#define PBS_WAIT_VMCNT_0() __builtin_amdgcn_s_waitcnt(0x0f70)

__device__ __forceinline__ bf16x8 lds_frag(const uint16_t* lds, int row, int chunk) {
  return *reinterpret_cast<const bf16x8*>(lds + row * D + ((chunk ^ (row & 15)) * 8));
}

__global__ __launch_bounds__(256, 2) void sparse_attn_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t lds_k[BS * D];
  __shared__ __attribute__((aligned(16))) uint16_t lds_v[BS * D];

  // workgroup -> (head, query block): heads stay on one XCD (blockIdx % 8), long rows first
  const int w_id = blockIdx.x;
  const int xcd = w_id & 7, slot = w_id >> 3;
  const int heads_per_xcd = (a.BH + 7) >> 3;
  const int bh = (slot % heads_per_xcd) * 8 + xcd;
  const int qb = a.nb - 1 - slot / heads_per_xcd;
  if (bh >= a.BH) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, gh = lane >> 5;
  const int b = bh / a.Hq, h = bh % a.Hq;
  const int qpos = qb * BS + 32 * wave + j;

  // Q^T fragments (B operand): query column j, d = 16 t + 8 gh + 0..7
  bf16x8 qf[8];
  {
    const uint16_t* qrow = a.q + b * a.q_sb + h * a.q_sh + (int64_t)min(qpos, a.S - 1) * a.q_ss;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      qf[t] = *reinterpret_cast<const bf16x8*>(qrow + 16 * t + 8 * gh);
      if (qpos >= a.S) qf[t] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  const int n_tiles = a.cnt[(int64_t)bh * a.nb + qb];
  const int32_t* cols = a.cols + ((int64_t)bh * a.nb + qb) * a.nb;
  const int own_first = (qb / a.bps) * a.bps;
  const uint16_t* pk = a.pk + (int64_t)bh * a.nb * BS * D;
  const uint16_t* pvt = a.pvt + (int64_t)bh * a.nb * BS * D;
  const int32_t* idx = a.idx + (int64_t)bh * a.nb * BS;

  f32x16 o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) o[dt] = (f32x16){0};
  float m_run = -INFINITY, l_run = 0.f;

  const int krow_in_tile = mfma_row_to_key(j);
  const uint32_t lane_off = async_lane_offset(wave, lane);

  // the visit list is read 64 entries at a time, one per lane, and handed out with readlane:
  // no vector-memory wait sits between the asynchronous copies and their consumers
  int col_cache = (lane < n_tiles) ? cols[lane] : 0;
  int col_cache_next = 0;
  if (n_tiles > 0) {
    PBS_WAIT_VMCNT_0();
    const int kb0 = __builtin_amdgcn_readlane(col_cache, 0);
    stage_tile_async(pk + (int64_t)kb0 * BS * D, lds_k, wave, lane_off);
    stage_tile_async(pvt + (int64_t)kb0 * BS * D, lds_v, wave, lane_off);
  }

  for (int it = 0; it < n_tiles; ++it) {
    if ((it & 63) == 0) col_cache_next = (it + 64 + lane < n_tiles) ? cols[it + 64 + lane] : 0;
    const int kb = __builtin_amdgcn_readlane(col_cache, it & 63);
    const bool has_next = it + 1 < n_tiles;
    if ((it & 63) == 63) col_cache = col_cache_next;
    const int kb_next = has_next ? __builtin_amdgcn_readlane(col_cache, (it + 1) & 63) : 0;

    PBS_WAIT_VMCNT_8();   // K(it) has landed; V(it) may still be in flight
    __syncthreads();

    // ---- S^T = K Q^T
    f32x16 s[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      s[ks] = (f32x16){0};
      const int row = 32 * ks + krow_in_tile;
#pragma unroll
      for (int t = 0; t < 8; ++t) s[ks] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(lds_k, row, 2 * t + gh), qf[t], s[ks], 0, 0, 0);
    }
    __syncthreads();      // every wave is done with K(it): the next K tile may overwrite it
    if (has_next) stage_tile_async(pk + (int64_t)kb_next * BS * D, lds_k, wave, lane_off);

    // ---- element mask inside the query block's own segment
    if (kb >= own_first) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        __builtin_amdgcn_sched_barrier(0);   // keep the index loads of one sub-tile at a time in flight
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          const int p = kb * BS + 32 * ks + 16 * (a4 >> 1) + 8 * gh + 4 * (a4 & 1);
          const int4 ki = *reinterpret_cast<const int4*>(idx + p);
          if (ki.x > qpos) s[ks][4 * a4 + 0] = -INFINITY;
          if (ki.y > qpos) s[ks][4 * a4 + 1] = -INFINITY;
          if (ki.z > qpos) s[ks][4 * a4 + 2] = -INFINITY;
          if (ki.w > qpos) s[ks][4 * a4 + 3] = -INFINITY;
        }
      }
    }

    // ---- online softmax (exp2 domain), one query per lane pair (lane, lane^32)
    float mx = -INFINITY;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[ks][r]);
    mx = fmaxf(mx, xhalf_f32(mx));
    const float m_new = fmaxf(m_run, mx * a.scale_log2);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float rs = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = __builtin_amdgcn_exp2f(s[ks][r] * a.scale_log2 - m_use);
        s[ks][r] = p;
        rs += p;
      }
    rs += xhalf_f32(rs);
    l_run = l_run * alpha + rs;
    m_run = m_new;
    if (__any(alpha != 1.0f)) {   // the running maximum settles after a few tiles
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
    }

    if (has_next) PBS_WAIT_VMCNT_8();   // V(it) has landed (K(it+1) may be in flight)
    else PBS_WAIT_VMCNT_0();
    __syncthreads();

    // ---- O^T += V^T P^T
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        bf16x8 pf;
#pragma unroll
        for (int e = 0; e < 8; ++e) pf[e] = (__bf16)s[ks][8 * u + e];
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(lds_v, 32 * dt + j, 4 * ks + 2 * u + gh), pf, o[dt], 0, 0, 0);
      }
    __syncthreads();      // every wave is done with V(it)
    if (has_next) stage_tile_async(pvt + (int64_t)kb_next * BS * D, lds_v, wave, lane_off);
  }

  // ---- epilogue: normalise, transpose through LDS (same swizzle), coalesced 16-byte stores
  __syncthreads();
  const float inv = 1.0f / l_run;
  uint16_t* os = lds_k;
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int a4 = 0; a4 < 4; ++a4) {
      const int row = 32 * wave + j;
      const int c = 4 * dt + a4;   // 16-byte chunk of d = 32 dt + 8 a4 + 4 gh + 0..3
      bf16x4 v4;
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) v4[cc] = (__bf16)(o[dt][4 * a4 + cc] * inv);
      *reinterpret_cast<bf16x4*>(os + row * D + ((c ^ (row & 15)) * 8) + 4 * gh) = v4;
    }
  __syncthreads();
  uint16_t* obase = a.o + b * a.o_sb + h * a.o_sh;
#pragma unroll
  for (int n = 0; n < 8; ++n) {
    const int ci = tid + 256 * n;
    const int row = ci >> 4, c = ci & 15;
    const int pos = qb * BS + row;
    if (pos < a.S)
      *reinterpret_cast<u32x4*>(obase + (int64_t)pos * a.o_ss + c * 8) =
          *reinterpret_cast<const u32x4*>(os + row * D + ((c ^ (row & 15)) * 8));
  }
}

}  // namespace

extern "C" int pbs_sparse_attn_fwd(const void* q, const void* perm_k, const void* perm_vt, const int32_t* key_indices,
                                   const int32_t* csr_cols, const int32_t* csr_cnt, void* out, int B, int Hq, int S,
                                   int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh,
                                   int64_t q_ss, int64_t o_sb, int64_t o_sh, int64_t o_ss, float softmax_scale,
                                   void* stream) {
  PBS_REQUIRE(q && perm_k && perm_vt && key_indices && csr_cols && csr_cnt && out, "pbs_sparse_attn_fwd: null tensor pointer");
  PBS_REQUIRE(head_dim == D && block_size == BS, "pbs_sparse_attn_fwd: head_dim and block_size must be 128 (got %d, %d)", head_dim, block_size);
  PBS_REQUIRE(B > 0 && Hq > 0 && S > 0, "pbs_sparse_attn_fwd: empty shape");
  PBS_REQUIRE(segment_size > 0 && segment_size % block_size == 0, "pbs_sparse_attn_fwd: segment_size must be a multiple of block_size");
  PBS_REQUIRE(q_sb % 8 == 0 && q_sh % 8 == 0 && q_ss % 8 == 0 && o_sb % 8 == 0 && o_sh % 8 == 0 && o_ss % 8 == 0,
              "pbs_sparse_attn_fwd: strides must keep rows 16-byte aligned");
  PBS_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)perm_k % 16) == 0 && ((uintptr_t)perm_vt % 16) == 0,
              "pbs_sparse_attn_fwd: pointers must be 16-byte aligned");
  AttnArgs a;
  a.q = (const uint16_t*)q; a.pk = (const uint16_t*)perm_k; a.pvt = (const uint16_t*)perm_vt;
  a.idx = key_indices; a.cols = csr_cols; a.cnt = csr_cnt; a.o = (uint16_t*)out;
  a.BH = B * Hq; a.Hq = Hq; a.S = S; a.nb = (S + BS - 1) / BS; a.bps = segment_size / block_size;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_ss = q_ss; a.o_sb = o_sb; a.o_sh = o_sh; a.o_ss = o_ss;
  a.scale_log2 = softmax_scale * 1.4426950408889634f;
  const int heads_per_xcd = (a.BH + 7) / 8;
  const int64_t n_wg = (int64_t)8 * heads_per_xcd * a.nb;
  PBS_REQUIRE(n_wg < (1ll << 31), "pbs_sparse_attn_fwd: launch too large");
  hipLaunchKernelGGL(sparse_attn_kernel, dim3((unsigned)n_wg), dim3(256), 0, (hipStream_t)stream, a);
  return pbs_check_launch("pbs_sparse_attn_fwd");
}
