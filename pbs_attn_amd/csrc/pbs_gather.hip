// Gather of K and V into permuted order, fused with the key-block pooling.
//
// One workgroup moves one block of 128 permuted keys of one head:
//   perm_k  (B, Hq, nb*128, 128)   row-major, rows past S are zero
//   perm_vt (B, Hq, nb, 128, 128)  V block TRANSPOSED: [d][key in block] -- the
//                                  layout the attention kernel feeds to MFMA
//   pooled_k(B, Hq, nb, 128)       bf16 mean (fp32 accumulate / 128) or max
// A 256-byte source row is read by 16 lanes x 16 bytes; K/V may be stored at
// the KV-head count (query head h reads KV head h / G).
// The same kernel runs in two reduced forms so that a caller can gather only what the attention will read:
//   * pooling only (POOL_ONLY): pooled_k of every permuted block straight from K through the indices, nothing
//     else read or written -- the block estimate needs no more -- and the per-block "needed" flags cleared;
//   * filtered: the permuted blocks whose "needed" flag (set by the block selection for every block some query
//     block visits) is zero are skipped; their perm_k / perm_vt tiles stay unwritten.
// The pooled values of the two forms are the same bits: same loads, same order of additions.
#include "pbs_common.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations

namespace {

constexpr int D = 128;
constexpr int BS = 128;
constexpr int VT_PITCH = 130;  // bf16 elements per staged V row (padded: bank spread)

struct GatherArgs {
  const uint16_t* k;
  const uint16_t* v;
  const int32_t* idx;  // (B*Hq, S_pad)
  uint16_t* perm_k;
  uint16_t* perm_vt;
  uint16_t* pooled_k;
  uint8_t* needed;     // (B*Hq, nb) or null: filter (full form), cleared (pooling-only form)
  int B, Hq, Hkv, S, nb;
  int64_t k_sb, k_sh, k_ss, v_sb, v_sh, v_ss;
  int pool_max;
};

template <bool POOL_ONLY>
__device__ __forceinline__ void gather_block(GatherArgs& a, uint16_t* vt, float (&pool)[16][D], int kb, int grid_row) {
  const int bh = grid_row;
  if (POOL_ONLY) {
    if (a.needed && threadIdx.x == 0) a.needed[(int64_t)bh * a.nb + kb] = 0;
  } else if (a.needed && a.needed[(int64_t)bh * a.nb + kb] == 0) {
    return;
  }
  const int b = bh / a.Hq, h = bh % a.Hq, kvh = h / (a.Hq / a.Hkv);
  const int rg = threadIdx.x >> 4, c = threadIdx.x & 15;  // row group, 16-byte chunk
  const uint16_t* ksrc = a.k + b * a.k_sb + kvh * a.k_sh;
  const uint16_t* vsrc = a.v + b * a.v_sb + kvh * a.v_sh;
  const int32_t* idx = a.idx + (int64_t)bh * a.nb * BS + kb * BS;
  uint16_t* kdst = a.perm_k + ((int64_t)bh * a.nb + kb) * BS * D;

  // Every load of the block is requested before the first is used: a workgroup's rows are then in flight together
  // (one pass at a time, a workgroup waits eight times for 4 or 8 KB).  Rows past the end of the sequence read
  // row 0 and are zeroed afterwards, so that no load sits behind a branch.
  int src[8];
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) src[pass] = idx[pass * 16 + rg];
  u32x4 kv[8], vv[8];
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const bool live = kb * BS + pass * 16 + rg < a.S;
    const int row = live ? src[pass] : 0;
    kv[pass] = *reinterpret_cast<const u32x4*>(ksrc + (int64_t)row * a.k_ss + c * 8);
    if (!POOL_ONLY) vv[pass] = *reinterpret_cast<const u32x4*>(vsrc + (int64_t)row * a.v_ss + c * 8);
  }
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const bool live = kb * BS + pass * 16 + rg < a.S;
    if (!live) {
      kv[pass] = (u32x4){0, 0, 0, 0};
      if (!POOL_ONLY) vv[pass] = (u32x4){0, 0, 0, 0};
    }
  }

  float acc[8];
  if (a.pool_max) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = -INFINITY;
#pragma unroll
    for (int pass = 0; pass < 8; ++pass)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] = fmaxf(acc[2 * e], bf16_bits_to_f32(kv[pass][e] & 0xffffu));
        acc[2 * e + 1] = fmaxf(acc[2 * e + 1], bf16_bits_to_f32(kv[pass][e] >> 16));
      }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
    for (int pass = 0; pass < 8; ++pass)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] += bf16_bits_to_f32(kv[pass][e] & 0xffffu);
        acc[2 * e + 1] += bf16_bits_to_f32(kv[pass][e] >> 16);
      }
  }
  if (!POOL_ONLY) {
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
      const int i = pass * 16 + rg;
      __builtin_nontemporal_store(kv[pass], reinterpret_cast<u32x4*>(kdst + i * D + c * 8));
      // stage V row-major (4-byte stores: the padded pitch keeps them aligned)
#pragma unroll
      for (int e = 0; e < 4; ++e) *reinterpret_cast<uint32_t*>(&vt[i * VT_PITCH + c * 8 + 2 * e]) = vv[pass][e];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) pool[rg][c * 8 + e] = acc[e];
  __syncthreads();

  if (threadIdx.x < D && a.pooled_k) {
    float s = pool[0][threadIdx.x];
    for (int r = 1; r < 16; ++r) s = a.pool_max ? fmaxf(s, pool[r][threadIdx.x]) : s + pool[r][threadIdx.x];
    if (!a.pool_max) s = s / (float)BS;
    a.pooled_k[((int64_t)bh * a.nb + kb) * D + threadIdx.x] = (uint16_t)f32_to_bf16_bits(s);
  }

  if (POOL_ONLY) return;
  // transposed write-out: thread (d, key group of 8) -> 16 bytes of row d
  uint16_t* vdst = a.perm_vt + ((int64_t)bh * a.nb + kb) * D * BS;
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int d = pass * 16 + rg;
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t lo = vt[(c * 8 + 2 * e) * VT_PITCH + d], hi = vt[(c * 8 + 2 * e + 1) * VT_PITCH + d];
      o[e] = lo | (hi << 16);
    }
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(vdst + d * BS + c * 8));
  }
}

// Launch order.  The query heads of a KV group read the same keys (and values) in different orders, and a permuted
// block only holds rows of its own segment.  Workgroups are handed to the XCDs round-robin in launch order (x
// fastest), so the grid is (8, members of a task group, groups / 8): the workgroups of one task group -- CHUNK
// consecutive blocks of every query head of one KV head -- have the same blockIdx.x, run on one XCD at about the same
// time, and the chunk's rows come from HBM once for the whole group (for segments up to the chunk: 256 KB of K per
// group at 128 keys a block).  Decoding costs one division: most workgroups of a filtered gather leave at once, and
// what they run before that is the launch's time.
constexpr int CHUNK = 8;

struct TaskGroups {
  int n_chunks;    // chunks of CHUNK blocks per head
  int n_groups;    // B * Hkv * n_chunks; group = blockIdx.z * 8 + blockIdx.x
  int G;           // query heads per KV head
  dim3 grid;
};

__host__ inline TaskGroups task_groups(int B, int Hq, int Hkv, int nb, int kinds) {
  TaskGroups t;
  t.n_chunks = (nb + CHUNK - 1) / CHUNK;
  t.n_groups = B * Hkv * t.n_chunks;
  t.G = Hq / Hkv;
  t.grid = dim3(8, (unsigned)(kinds * t.G * CHUNK), (unsigned)((t.n_groups + 7) / 8));
  return t;
}

// (kind, head, block) of this workgroup; false if it has none (the last groups of a launch, the tail of a head's blocks)
__device__ __forceinline__ bool my_task(const TaskGroups& t, int nb, int& kind, int& bh, int& blk) {
  const int m = blockIdx.y, per_kind = t.G * CHUNK;
  kind = m >= per_kind;
  const int mm = m - (kind ? per_kind : 0);
  const int tg = blockIdx.z * 8 + blockIdx.x;
  const int bkv = tg / t.n_chunks, chunk = tg - bkv * t.n_chunks;
  blk = chunk * CHUNK + (mm & (CHUNK - 1));
  bh = bkv * t.G + mm / CHUNK;   // (b * Hkv + kvh) * G + head in group == b * Hq + h
  return tg < t.n_groups && blk < nb;
}

template <bool POOL_ONLY>
__global__ __launch_bounds__(256) void gather_kv_kernel(GatherArgs a, TaskGroups t) {
  __shared__ uint16_t vt[POOL_ONLY ? 2 : BS * VT_PITCH];
  __shared__ float pool[16][D];
  int kind, bh, blk;
  if (!my_task(t, a.nb, kind, bh, blk)) return;
  gather_block<POOL_ONLY>(a, vt, pool, blk, bh);
}


// Mean / max pooling of Q blocks (rows past S count as zeros, the divisor stays 128).
__device__ __forceinline__ void pool_q_block(float (&pool)[16][D], const uint16_t* q, uint16_t* pooled, int Hq, int S, int nb,
                                             int64_t q_sb, int64_t q_sh, int64_t q_ss, int pool_max, int qb, int bh) {
  const int b = bh / Hq, h = bh % Hq;
  const int rg = threadIdx.x >> 4, c = threadIdx.x & 15;
  const uint16_t* src = q + b * q_sb + h * q_sh;
  // all eight loads in flight before the first is used; rows past the end read the last row and count as zeros
  u32x4 x[8];
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int pos = qb * BS + pass * 16 + rg;
    x[pass] = *reinterpret_cast<const u32x4*>(src + (int64_t)min(pos, S - 1) * q_ss + c * 8);
  }
#pragma unroll
  for (int pass = 0; pass < 8; ++pass)
    if (qb * BS + pass * 16 + rg >= S) x[pass] = (u32x4){0, 0, 0, 0};
  float acc[8];
  if (pool_max) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = -INFINITY;
#pragma unroll
    for (int pass = 0; pass < 8; ++pass)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] = fmaxf(acc[2 * e], bf16_bits_to_f32(x[pass][e] & 0xffffu));
        acc[2 * e + 1] = fmaxf(acc[2 * e + 1], bf16_bits_to_f32(x[pass][e] >> 16));
      }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
    for (int pass = 0; pass < 8; ++pass)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] += bf16_bits_to_f32(x[pass][e] & 0xffffu);
        acc[2 * e + 1] += bf16_bits_to_f32(x[pass][e] >> 16);
      }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) pool[rg][c * 8 + e] = acc[e];
  __syncthreads();
  if (threadIdx.x < D) {
    float s = pool[0][threadIdx.x];
    for (int r = 1; r < 16; ++r) s = pool_max ? fmaxf(s, pool[r][threadIdx.x]) : s + pool[r][threadIdx.x];
    if (!pool_max) s = s / (float)BS;
    pooled[((int64_t)bh * nb + qb) * D + threadIdx.x] = (uint16_t)f32_to_bf16_bits(s);
  }
}

__global__ __launch_bounds__(256) void pool_q_kernel(const uint16_t* q, uint16_t* pooled, int Hq, int S, int nb,
                                                     int64_t q_sb, int64_t q_sh, int64_t q_ss, int pool_max) {
  __shared__ float pool[16][D];
  pool_q_block(pool, q, pooled, Hq, S, nb, q_sb, q_sh, q_ss, pool_max, blockIdx.x, blockIdx.y);
}

// Both poolings of the block estimate in one launch: the pooling of permuted key blocks waits on scattered 256-byte
// rows, the pooling of query blocks streams Q from HBM; side by side each fills what the other leaves idle.  A task
// group's key poolings come first, then the query poolings of the same heads and blocks.
struct PoolQArgs {
  const uint16_t* q;
  uint16_t* pooled_q;
  int64_t q_sb, q_sh, q_ss;
  int pool_max;
};

__global__ __launch_bounds__(256) void pool_qk_kernel(GatherArgs a, PoolQArgs p, TaskGroups t) {
  __shared__ uint16_t vt[2];
  __shared__ float pool[16][D];
  int kind, bh, blk;
  if (!my_task(t, a.nb, kind, bh, blk)) return;
  if (kind) pool_q_block(pool, p.q, p.pooled_q, a.Hq, a.S, a.nb, p.q_sb, p.q_sh, p.q_ss, p.pool_max, blk, bh);
  else gather_block<true>(a, vt, pool, blk, bh);
}

}  // namespace

extern "C" int pbs_gather_kv(const void* k, const void* v, const int32_t* key_indices, void* perm_k, void* perm_vt,
                             void* pooled_k, int B, int Hq, int Hkv, int S, int head_dim, int block_size, int64_t k_sb,
                             int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss, int key_pool_max,
                             const uint8_t* block_needed, void* stream) {
  PBS_REQUIRE(k && v && key_indices && perm_k && perm_vt, "pbs_gather_kv: null tensor pointer");
  PBS_REQUIRE(head_dim == D && block_size == BS, "pbs_gather_kv: head_dim and block_size must be 128 (got %d, %d)", head_dim, block_size);
  PBS_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && S > 0, "pbs_gather_kv: bad shape");
  PBS_REQUIRE(k_sb % 8 == 0 && k_sh % 8 == 0 && k_ss % 8 == 0 && v_sb % 8 == 0 && v_sh % 8 == 0 && v_ss % 8 == 0,
              "pbs_gather_kv: strides must keep rows 16-byte aligned");
  PBS_REQUIRE(((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0, "pbs_gather_kv: pointers must be 16-byte aligned");
  GatherArgs a;
  a.k = (const uint16_t*)k; a.v = (const uint16_t*)v; a.idx = key_indices;
  a.perm_k = (uint16_t*)perm_k; a.perm_vt = (uint16_t*)perm_vt; a.pooled_k = (uint16_t*)pooled_k;
  a.needed = const_cast<uint8_t*>(block_needed);
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.S = S; a.nb = (S + BS - 1) / BS;
  a.k_sb = k_sb; a.k_sh = k_sh; a.k_ss = k_ss; a.v_sb = v_sb; a.v_sh = v_sh; a.v_ss = v_ss;
  a.pool_max = key_pool_max;
  const TaskGroups t = task_groups(B, Hq, Hkv, a.nb, 1);
  PBS_REQUIRE(t.grid.y <= 65535 && t.grid.z <= 65535, "pbs_gather_kv: too many heads or blocks");
  hipLaunchKernelGGL(gather_kv_kernel<false>, t.grid, dim3(256), 0, (hipStream_t)stream, a, t);
  return pbs_check_launch("pbs_gather_kv");
}

extern "C" int pbs_pool_k_permuted(const void* k, const int32_t* key_indices, void* pooled_k, uint8_t* block_needed, int B,
                                   int Hq, int Hkv, int S, int head_dim, int block_size, int64_t k_sb, int64_t k_sh,
                                   int64_t k_ss, int key_pool_max, void* stream) {
  PBS_REQUIRE(k && key_indices && pooled_k, "pbs_pool_k_permuted: null tensor pointer");
  PBS_REQUIRE(head_dim == D && block_size == BS, "pbs_pool_k_permuted: head_dim and block_size must be 128 (got %d, %d)", head_dim, block_size);
  PBS_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && S > 0, "pbs_pool_k_permuted: bad shape");
  PBS_REQUIRE(k_sb % 8 == 0 && k_sh % 8 == 0 && k_ss % 8 == 0 && ((uintptr_t)k % 16) == 0,
              "pbs_pool_k_permuted: rows must be 16-byte aligned");
  GatherArgs a = {};
  a.k = (const uint16_t*)k; a.idx = key_indices; a.pooled_k = (uint16_t*)pooled_k; a.needed = block_needed;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.S = S; a.nb = (S + BS - 1) / BS;
  a.k_sb = k_sb; a.k_sh = k_sh; a.k_ss = k_ss;
  a.pool_max = key_pool_max;
  const TaskGroups t = task_groups(B, Hq, Hkv, a.nb, 1);
  PBS_REQUIRE(t.grid.y <= 65535 && t.grid.z <= 65535, "pbs_pool_k_permuted: too many heads or blocks");
  hipLaunchKernelGGL(gather_kv_kernel<true>, t.grid, dim3(256), 0, (hipStream_t)stream, a, t);
  return pbs_check_launch("pbs_pool_k_permuted");
}

extern "C" int pbs_pool_blocks(const void* q, const void* k, const int32_t* key_indices, void* pooled_q, void* pooled_k,
                               uint8_t* block_needed, int B, int Hq, int Hkv, int S, int head_dim, int block_size,
                               int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss,
                               int query_pool_max, int key_pool_max, void* stream) {
  PBS_REQUIRE(q && k && key_indices && pooled_q && pooled_k, "pbs_pool_blocks: null tensor pointer");
  PBS_REQUIRE(head_dim == D && block_size == BS, "pbs_pool_blocks: head_dim and block_size must be 128 (got %d, %d)", head_dim, block_size);
  PBS_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && S > 0, "pbs_pool_blocks: bad shape");
  PBS_REQUIRE(q_sb % 8 == 0 && q_sh % 8 == 0 && q_ss % 8 == 0 && k_sb % 8 == 0 && k_sh % 8 == 0 && k_ss % 8 == 0 &&
                  ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0,
              "pbs_pool_blocks: rows must be 16-byte aligned");
  GatherArgs a = {};
  a.k = (const uint16_t*)k; a.idx = key_indices; a.pooled_k = (uint16_t*)pooled_k; a.needed = block_needed;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.S = S; a.nb = (S + BS - 1) / BS;
  a.k_sb = k_sb; a.k_sh = k_sh; a.k_ss = k_ss;
  a.pool_max = key_pool_max;
  PoolQArgs p;
  p.q = (const uint16_t*)q; p.pooled_q = (uint16_t*)pooled_q; p.q_sb = q_sb; p.q_sh = q_sh; p.q_ss = q_ss;
  p.pool_max = query_pool_max;
  const TaskGroups t = task_groups(B, Hq, Hkv, a.nb, 2);
  PBS_REQUIRE(t.grid.y <= 65535 && t.grid.z <= 65535, "pbs_pool_blocks: too many heads or blocks");
  hipLaunchKernelGGL(pool_qk_kernel, t.grid, dim3(256), 0, (hipStream_t)stream, a, p, t);
  return pbs_check_launch("pbs_pool_blocks");
}

extern "C" int pbs_pool_q(const void* q, void* pooled_q, int B, int Hq, int S, int head_dim, int block_size,
                          int64_t q_sb, int64_t q_sh, int64_t q_ss, int query_pool_max, void* stream) {
  PBS_REQUIRE(q && pooled_q, "pbs_pool_q: null tensor pointer");
  PBS_REQUIRE(head_dim == D && block_size == BS, "pbs_pool_q: head_dim and block_size must be 128 (got %d, %d)", head_dim, block_size);
  PBS_REQUIRE(B > 0 && Hq > 0 && S > 0 && B * Hq <= 65535, "pbs_pool_q: bad shape");
  PBS_REQUIRE(q_sb % 8 == 0 && q_sh % 8 == 0 && q_ss % 8 == 0 && ((uintptr_t)q % 16) == 0,
              "pbs_pool_q: rows must be 16-byte aligned");
  const int nb = (S + BS - 1) / BS;
  hipLaunchKernelGGL(pool_q_kernel, dim3(nb, B * Hq), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)q,
                     (uint16_t*)pooled_q, Hq, S, nb, q_sb, q_sh, q_ss, query_pool_max);
  return pbs_check_launch("pbs_pool_q");
}
