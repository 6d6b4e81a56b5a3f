// Key scoring: mean over the last 128 queries of softmax(Q_last K^T / sqrt(D))
// over all keys of the complete segments (no causal mask).
//
// Three launches, K is read twice (each time once per workgroup, through LDS) and never re-materialised:
//   (all exponentials are base 2 on logits pre-multiplied by log2(e))
//   1. score_partial : per (head, key chunk) online (max, sum-exp) of every query row
//   2. score_reduce  : fold the chunk partials into row max + log2(row sum)
//   3. score_final   : recompute the logits and emit the per-key mean probability
// Logits reproduce the rounding points of a bf16 matmul followed by a bf16
// divide: fp32 accumulate -> bf16 -> / sqrt(D) -> bf16.
#include "pbs_common.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations
#include <atomic>
#include <mutex>

namespace {

constexpr int D = 128;             // head dim
constexpr int NQ = 128;            // scoring queries (= block size)
constexpr int KEYS_PER_WAVE_STEP = 32;
constexpr int KEYS_PER_WG = 1024;  // keys one 4-wave workgroup walks through (256 for 1-wave groups)

struct ScoreArgs {
  const uint16_t* q;
  const uint16_t* k;
  int B, Hq, Hkv, S, Sc;
  int64_t q_sb, q_sh, q_ss;
  int64_t k_sb, k_sh, k_ss;
  float inv_sqrt_d;
  float* part;    // (B*Hq, nchunk, NQ, 2)
  float* stats;   // (B*Hq, NQ)  row max + log2(row sum)
  float* scores;  // (B*Hq, Sc)
  int nchunk;
  int chunk_keys;
};

__device__ __forceinline__ bf16x8 load_frag(const uint16_t* row_ptr, int t, int half) {
  return *reinterpret_cast<const bf16x8*>(row_ptr + 16 * t + 8 * half);
}

// fp32 accumulator -> the bf16 logit a bf16 matmul followed by a bf16 divide by sqrt(D) yields: round to
// bf16, scale (multiplication by the reciprocal; it differs from the true quotient by at most one fp32 ulp,
// which survives the second bf16 rounding only for values within 2^-16 of a tie), round to bf16.
// Hardware conversions (round to nearest even), two values per conversion instruction.
__device__ __forceinline__ f32x2 logit2(float acc0, float acc1, float inv_sqrt_d) {
  const f32x2 r = hw_round_bf16x2((f32x2){acc0, acc1});
  return hw_round_bf16x2((f32x2){r.x * inv_sqrt_d, r.y * inv_sqrt_d});
}
constexpr float LOG2E = 1.4426950408889634f;

// ---- key rows through LDS: the waves of a workgroup (one per query head of the KV group) walk the same keys,
// so a stage of 64 key rows is copied once per workgroup with asynchronous global -> LDS copies (no registers),
// double-buffered, and every wave reads its MFMA fragments from there.  Rows are 16 chunks of 16 bytes with the
// chunk index XORed with (row & 15): fragment reads (row = lane % 32, one chunk) are bank-conflict free.  The copy
// instruction writes lane l at M0 + 16 l, so the swizzle is applied on the global side: lane l of copy i fetches
// chunk (l & 15) ^ (row & 15) of row 4 i + (l >> 4).
constexpr int STAGE_KEYS = 64;
constexpr uint32_t STAGE_BYTES = STAGE_KEYS * D * 2;      // 16 KB
constexpr uint32_t LDS_STATS = 2 * STAGE_BYTES;           // per wave: NQ floats (row max + log2 row sum)
constexpr uint32_t LDS_SCORE_TOTAL = LDS_STATS + 4 * NQ * 4;

typedef __attribute__((address_space(3))) uint8_t lds_u8;

__device__ __forceinline__ bf16x8 lds_frag(uint32_t byte_addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>((const lds_u8*)(uintptr_t)byte_addr);
}

// copies of rows [0, STAGE_KEYS) starting at `rows` (row stride k_ss elements) into the stage buffer at LDS byte
// offset `lds_byte`; wave w of nwaves issues copies w, w + nwaves, ...
__device__ __forceinline__ void stage_keys_async(const uint16_t* rows, int64_t k_ss, uint32_t lds_byte, int wave, int nwaves, int lane) {
  const uint64_t src0 = (uint64_t)(uintptr_t)rows;
  const uint32_t src_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src0);
  const uint32_t src_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(src0 >> 32));
  const uint64_t srcu = ((uint64_t)src_hi << 32) | (uint64_t)src_lo;
  const uint32_t row_bytes = (uint32_t)k_ss * 2u;   // < 2^29 (checked on the host)
  for (int i = wave; i < STAGE_KEYS / 4; i += nwaves) {
    const uint32_t r = (uint32_t)(lane >> 4);
    const uint32_t c = (uint32_t)(lane & 15) ^ ((4u * (uint32_t)(i & 3) + r) & 15u);
    const uint32_t voff = r * row_bytes + c * 16u;
    const uint64_t base = srcu + (uint64_t)(4 * i) * row_bytes;
    register uint32_t m0v asm("m0") = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_byte + (uint32_t)i * 1024u));
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(voff), "s"(base) : "memory");
  }
}

// One wave per query head of the KV group; the waves of a workgroup share the staged key rows.
template <bool FINAL>
__global__ __launch_bounds__(256, 2) void score_kernel(ScoreArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // starts at LDS offset 0: this kernel has no static LDS
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int j = lane & 31, half = lane >> 5;
  const int G = a.Hq / a.Hkv;
  const int b = blockIdx.y / a.Hkv, kvh = blockIdx.y % a.Hkv;
  const int chunk = blockIdx.x;
  const int key_lo = chunk * a.chunk_keys;
  const int key_hi = min(key_lo + a.chunk_keys, a.Sc);   // chunk_keys and Sc are multiples of STAGE_KEYS
  const int nwaves = (int)blockDim.x >> 6;
  const uint16_t* kbase = a.k + b * a.k_sb + kvh * a.k_sh;
  float* s_stats = reinterpret_cast<float*>(smem + LDS_STATS) + wave * NQ;   // p = exp2(logit - stat)
  // LDS byte offset of fragment 0 of key row j inside a stage buffer; fragment t lies at frag0 ^ (t << 5),
  // rows 32 .. 63 of the stage 8 KB further on
  const uint32_t frag0 = (uint32_t)(j * 256 + ((half ^ (j & 15)) * 16));
  const int n_stages = (key_hi - key_lo) / STAGE_KEYS;

  for (int g0 = 0; g0 < G; g0 += nwaves) {
    const int g = g0 + wave;
    const bool active = g < G;
    const int h = kvh * G + (active ? g : 0);
    const int bh = b * a.Hq + h;
    const uint16_t* qbase = a.q + b * a.q_sb + h * a.q_sh + (int64_t)(a.S - NQ) * a.q_ss;

    __syncthreads();   // every wave is done with the stage buffers (and the statistics) of the previous group of heads
    stage_keys_async(kbase + (int64_t)key_lo * a.k_ss, a.k_ss, 0u, wave, nwaves, lane);

    // the head's 128 scoring queries, resident for the whole chunk
    bf16x8 qf[4][8];
#pragma unroll
    for (int qt = 0; qt < 4; ++qt)
#pragma unroll
      for (int t = 0; t < 8; ++t) qf[qt][t] = load_frag(qbase + (int64_t)(32 * qt + j) * a.q_ss, t, half);

    if (FINAL && active)
      for (int i = lane; i < NQ; i += 64) s_stats[i] = a.stats[(int64_t)bh * NQ + i];

    float m_run[4], l_run[4];
#pragma unroll
    for (int qt = 0; qt < 4; ++qt) {
      m_run[qt] = -INFINITY;
      l_run[qt] = 0.f;
    }

    for (int st = 0; st < n_stages; ++st) {
      const uint32_t buf = (uint32_t)(st & 1) * STAGE_BYTES;
      __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): this wave's copies of stage st have landed
      __syncthreads();                      // every wave's have; everyone is done with the other buffer
      if (st + 1 < n_stages)
        stage_keys_async(kbase + (int64_t)(key_lo + (st + 1) * STAGE_KEYS) * a.k_ss, a.k_ss, buf ^ STAGE_BYTES, wave, nwaves, lane);
      if (!active) continue;
#pragma unroll
      for (int sub = 0; sub < STAGE_KEYS / KEYS_PER_WAVE_STEP; ++sub) {
        const int key = key_lo + st * STAGE_KEYS + sub * KEYS_PER_WAVE_STEP + j;   // always < Sc
        bf16x8 kf[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) kf[t] = lds_frag(buf + (uint32_t)sub * 8192u + (frag0 ^ (uint32_t)(t << 5)));

        if (!FINAL) {
          // S^T tile: rows = keys, column = query j of sub-tile qt
#pragma unroll
          for (int qt = 0; qt < 4; ++qt) {
            f32x16 acc = {0};
#pragma unroll
            for (int t = 0; t < 8; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[t], qf[qt][t], acc, 0, 0, 0);
            float v[16], mx = -INFINITY;   // logits before the log2(e) factor
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
              const f32x2 l2 = logit2(acc[r], acc[r + 1], a.inv_sqrt_d);
              v[r] = l2.x;
              v[r + 1] = l2.y;
              mx = fmaxf(fmaxf(mx, l2.x), l2.y);
            }
            const float m_new = fmaxf(m_run[qt], mx * LOG2E);
            float sum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) sum += __builtin_amdgcn_exp2f(__builtin_fmaf(v[r], LOG2E, -m_new));
            l_run[qt] = l_run[qt] * __builtin_amdgcn_exp2f(m_run[qt] - m_new) + sum;
            m_run[qt] = m_new;
          }
        } else {
          // S tile: rows = queries of sub-tile qt, column = key j
          float accp = 0.f;
#pragma unroll
          for (int qt = 0; qt < 4; ++qt) {
            f32x16 acc = {0};
#pragma unroll
            for (int t = 0; t < 8; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[qt][t], kf[t], acc, 0, 0, 0);
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
              const float4 st4 = *reinterpret_cast<const float4*>(&s_stats[32 * qt + 8 * r4 + 4 * half]);
              const f32x2 la = logit2(acc[4 * r4 + 0], acc[4 * r4 + 1], a.inv_sqrt_d);
              const f32x2 lb = logit2(acc[4 * r4 + 2], acc[4 * r4 + 3], a.inv_sqrt_d);
              accp += __builtin_amdgcn_exp2f(__builtin_fmaf(la.x, LOG2E, -st4.x));
              accp += __builtin_amdgcn_exp2f(__builtin_fmaf(la.y, LOG2E, -st4.y));
              accp += __builtin_amdgcn_exp2f(__builtin_fmaf(lb.x, LOG2E, -st4.z));
              accp += __builtin_amdgcn_exp2f(__builtin_fmaf(lb.y, LOG2E, -st4.w));
            }
          }
          accp += xhalf_f32(accp);
          if (half == 0) a.scores[(int64_t)bh * a.Sc + key] = accp * (1.0f / NQ);
        }
      }
    }
    if (!FINAL && active) {
#pragma unroll
      for (int qt = 0; qt < 4; ++qt) {
        const float m_o = xhalf_f32(m_run[qt]), l_o = xhalf_f32(l_run[qt]);
        const float m_new = fmaxf(m_run[qt], m_o);
        const float l_new = l_run[qt] * __builtin_amdgcn_exp2f(m_run[qt] - m_new) + l_o * __builtin_amdgcn_exp2f(m_o - m_new);
        if (half == 0) {
          float* p = a.part + (((int64_t)bh * a.nchunk + chunk) * NQ + 32 * qt + j) * 2;
          p[0] = m_new;
          p[1] = l_new;
        }
      }
    }
  }
}

// Folds the chunk partials of one head into row max + log2(row sum).  A row's chunks are spread over REDUCE_LANES
// threads and taken in two passes -- the maximum over all chunks, then the sum of the chunk sums scaled to it -- so
// that no term waits for the one before it: folded one after the other with a running maximum, a row is a chain of
// `nchunk` dependent loads and exponentials (19 us for 64 chunks, as long as the two scoring passes of a short
// sequence together).  The order of the additions is fixed: per thread ascending chunks, then ascending threads.
constexpr int REDUCE_LANES = 8;

__global__ __launch_bounds__(NQ * REDUCE_LANES) void score_reduce_kernel(ScoreArgs a) {
  __shared__ float part[REDUCE_LANES][NQ];
  const int bh = blockIdx.x, qrow = threadIdx.x % NQ, cl = threadIdx.x / NQ;
  const float* p = a.part + (int64_t)bh * a.nchunk * NQ * 2 + qrow * 2;
  float m = -INFINITY;
#pragma unroll 8
  for (int c = cl; c < a.nchunk; c += REDUCE_LANES) m = fmaxf(m, p[(int64_t)c * NQ * 2]);
  part[cl][qrow] = m;
  __syncthreads();
#pragma unroll
  for (int x = 0; x < REDUCE_LANES; ++x) m = fmaxf(m, part[x][qrow]);
  __syncthreads();
  float l = 0.f;
#pragma unroll 8
  for (int c = cl; c < a.nchunk; c += REDUCE_LANES) {
    const float2 ml = *reinterpret_cast<const float2*>(p + (int64_t)c * NQ * 2);
    l += ml.y * __builtin_amdgcn_exp2f(ml.x - m);
  }
  part[cl][qrow] = l;
  __syncthreads();
  if (cl == 0) {
    l = 0.f;
#pragma unroll
    for (int x = 0; x < REDUCE_LANES; ++x) l += part[x][qrow];
    a.stats[(int64_t)bh * NQ + qrow] = m + __builtin_amdgcn_logf(l);   // log base 2
  }
}

int chunks_for(int Sc, int chunk_keys) { return (Sc + chunk_keys - 1) / chunk_keys; }

// Keys per workgroup.  With one query head per KV head a workgroup is a single wave and starts from a
// quarter of the keys; short sequences get shorter chunks until the launch has enough workgroups to
// fill the chip (each workgroup re-reads its heads' 128 queries, so chunks stay >= 64 keys).
int chunk_keys_for(int B, int Hq, int Hkv, int Sc) {
  const bool grouped = Hq / Hkv > 1;
  int chunk = grouped ? KEYS_PER_WG : KEYS_PER_WG / 4;
  const int64_t want = grouped ? 512 : 2048;
  while (chunk > 64 && (int64_t)chunks_for(Sc, chunk) * B * Hkv < want) chunk /= 2;
  return chunk;
}

}  // namespace

extern "C" size_t pbs_score_keys_workspace_bytes(int B, int Hq, int Hkv, int S, int segment_size) {
  if (segment_size <= 0 || B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv) return 0;
  const int Sc = (S / segment_size) * segment_size;
  if (Sc == 0) return 0;
  return (size_t)B * Hq * ((size_t)chunks_for(Sc, chunk_keys_for(B, Hq, Hkv, Sc)) + 1) * NQ * 2 * sizeof(float);
}

namespace {

// Argument checks and the three launches shared by the two entry points; `workspace` holds the chunk
// partials and the folded row statistics.
int score_keys_launch(const char* who, const void* q, const void* k, float* scores, int B, int Hq, int Hkv, int S,
                      int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                      int64_t k_sb, int64_t k_sh, int64_t k_ss, void* workspace, size_t workspace_bytes, void* stream) {
  PBS_REQUIRE(q && k && scores, "%s: null tensor pointer", who);
  PBS_REQUIRE(head_dim == D, "%s: head_dim must be 128, got %d", who, head_dim);
  PBS_REQUIRE(block_size == NQ, "%s: block_size must be 128, got %d", who, block_size);
  PBS_REQUIRE(B > 0 && Hkv > 0 && Hq > 0 && Hq % Hkv == 0, "%s: bad head counts Hq=%d Hkv=%d", who, Hq, Hkv);
  PBS_REQUIRE(segment_size > 0 && segment_size % block_size == 0, "%s: segment_size %d not a multiple of block_size", who, segment_size);
  PBS_REQUIRE(S >= NQ, "%s: sequence shorter than one block", who);
  PBS_REQUIRE(q_ss % 8 == 0 && k_ss % 8 == 0 && q_sh % 8 == 0 && k_sh % 8 == 0 && q_sb % 8 == 0 && k_sb % 8 == 0,
              "%s: strides must keep rows 16-byte aligned", who);
  PBS_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0, "%s: pointers must be 16-byte aligned", who);
  PBS_REQUIRE(k_ss >= D && k_ss < (1 << 28), "%s: key row stride %lld outside [128, 2^28)", who, (long long)k_ss);
  PBS_REQUIRE((int64_t)B * Hkv <= 65535, "%s: too many KV heads (%lld)", who, (long long)B * Hkv);
  const int Sc = (S / segment_size) * segment_size;
  if (Sc == 0) return 0;
  PBS_REQUIRE(workspace && workspace_bytes >= pbs_score_keys_workspace_bytes(B, Hq, Hkv, S, segment_size),
              "%s: workspace too small (%zu < %zu bytes)", who, workspace_bytes,
              pbs_score_keys_workspace_bytes(B, Hq, Hkv, S, segment_size));
  ScoreArgs a;
  a.q = (const uint16_t*)q;
  a.k = (const uint16_t*)k;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.S = S; a.Sc = Sc;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_ss = q_ss;
  a.k_sb = k_sb; a.k_sh = k_sh; a.k_ss = k_ss;
  a.inv_sqrt_d = (float)(1.0 / sqrt((double)head_dim));
  a.chunk_keys = chunk_keys_for(B, Hq, Hkv, Sc);
  a.nchunk = chunks_for(Sc, a.chunk_keys);
  a.part = (float*)workspace;
  a.stats = a.part + (size_t)B * Hq * a.nchunk * NQ * 2;
  a.scores = scores;
  static std::atomic<bool> lds_checked{false};   // once per process: a property of the code object
  if (!lds_checked.load(std::memory_order_acquire)) {
    if (const int rc = pbs_require_no_static_lds((const void*)score_kernel<false>, who)) return rc;
    if (const int rc = pbs_require_no_static_lds((const void*)score_kernel<true>, who)) return rc;
    lds_checked.store(true, std::memory_order_release);
  }
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(a.nchunk, B * Hkv);
  const dim3 block(Hq / Hkv > 1 ? 256 : 64);
  hipLaunchKernelGGL(score_kernel<false>, grid, block, LDS_SCORE_TOTAL, st, a);
  hipLaunchKernelGGL(score_reduce_kernel, dim3(B * Hq), dim3(NQ * REDUCE_LANES), 0, st, a);
  hipLaunchKernelGGL(score_kernel<true>, grid, block, LDS_SCORE_TOTAL, st, a);
  return pbs_check_launch(who);
}

}  // namespace

extern "C" int pbs_score_keys(const void* q, const void* k, float* scores, int B, int Hq, int Hkv, int S, int head_dim,
                              int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb,
                              int64_t k_sh, int64_t k_ss, void* workspace, size_t workspace_bytes, void* stream) {
  return score_keys_launch("pbs_score_keys", q, k, scores, B, Hq, Hkv, S, head_dim, block_size, segment_size, q_sb, q_sh,
                           q_ss, k_sb, k_sh, k_ss, workspace, workspace_bytes, stream);
}

// ---- the variant that allocates nothing: chunk partials and row statistics live in a library-owned
// device array.  Every GPU holds its own copy of the array at its own address; the address is looked up
// once per device, on that device's first call, and only that pointer is ever handed to kernels.
namespace {

constexpr size_t SCRATCH_BYTES = PBS_SCORE_KEYS_STATIC_SCRATCH_BYTES;   // 8 MiB per GPU, held until the process ends
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_lock;
void* g_scratch_ptr[MAX_DEVICES] = {};

// device pointer of `scratch` on the current device (null + error message on failure)
void* scratch_on_current_device(const char* who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    pbs_set_error("%s: cannot identify the current device (%s, device %d)", who, hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      pbs_set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}

}  // namespace

extern "C" int pbs_score_keys_static(const void* q, const void* k, float* scores, int B, int Hq, int Hkv, int S,
                                     int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh,
                                     int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss, void* stream) {
  PBS_REQUIRE(B > 0 && Hkv > 0 && Hq > 0 && Hq % Hkv == 0 && S > 0 && segment_size > 0,
              "pbs_score_keys_static: bad shape B=%d Hq=%d Hkv=%d S=%d segment_size=%d", B, Hq, Hkv, S, segment_size);
  const size_t need = pbs_score_keys_workspace_bytes(B, Hq, Hkv, S, segment_size);
  PBS_REQUIRE(need <= SCRATCH_BYTES,
              "pbs_score_keys_static: this shape needs %zu bytes of scratch memory, the library-owned buffer holds %zu; "
              "use pbs_score_keys with a caller-provided workspace", need, SCRATCH_BYTES);
  void* ws = scratch_on_current_device("pbs_score_keys_static");
  if (!ws) return -2;
  // every partial and statistic the later launches read is written by the earlier ones of this call:
  // nothing needs clearing between calls
  return score_keys_launch("pbs_score_keys_static", q, k, scores, B, Hq, Hkv, S, head_dim, block_size, segment_size,
                           q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, ws, SCRATCH_BYTES, stream);
}
