// Measurement aid, not part of the attention path: a loop of nothing but matrix instructions -- the attention
// kernel's v_mfma_f32_16x16x32_bf16 or, for comparison, v_mfma_f32_32x32x16_bf16 (the same FLOP per launch) -- on
// operands the caller provides.  On MI355X the rate this loop sustains depends on the operand VALUES
// (zeros run at the full clock, normally distributed values make the chip lower its clock to stay inside
// its power limit), so the benchmark reports it next to the attention kernel's rate as the MFMA ceiling
// for data like the attention kernel's.
#include "pbs_attn_tile.h"
#include "pbs_probe.h"   // the definitions below are checked against these declarations

namespace {

constexpr int PROBE_WGS = 256, PROBE_THREADS = 512, PROBE_OPERANDS = 65536;

template <bool SHAPE_32X32X16>
__global__ __launch_bounds__(PROBE_THREADS, 2) void mfma_probe_kernel(const uint16_t* operands, int iters, float* sink,
                                                                        unsigned long long* clocks) {
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  bf16x8 a[8], b[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    a[t] = *reinterpret_cast<const bf16x8*>(operands + ((threadIdx.x * 128 + t * 16) & (PROBE_OPERANDS - 1)));
    b[t] = *reinterpret_cast<const bf16x8*>(operands + ((threadIdx.x * 128 + t * 16 + 8) & (PROBE_OPERANDS - 1)));
  }
  float s = 0.f;
  if (SHAPE_32X32X16) {
    f32x16 c[4] = {{0}, {0}, {0}, {0}};
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int t = 0; t < 8; ++t) c[t & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t], b[t], c[t & 3], 0, 0, 0);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) s += (c[0][e] + c[1][e]) + (c[2][e] + c[3][e]);
  } else {
    f32x4 c[8] = {{0}, {0}, {0}, {0}, {0}, {0}, {0}, {0}};
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int t = 0; t < 8; ++t) c[t] = PBS_MFMA(a[t], b[(t + u) & 7], c[t]);
    }
#pragma unroll
    for (int t = 0; t < 8; ++t) s += (c[t][0] + c[t][1]) + (c[t][2] + c[t][3]);
  }
  sink[blockIdx.x * PROBE_THREADS + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    atomicAdd(&clocks[0], __builtin_amdgcn_s_memtime() - c0);       // shader clock ticks
    atomicAdd(&clocks[1], __builtin_amdgcn_s_memrealtime() - r0);   // 100 MHz ticks
  }
}

}  // namespace

extern "C" int pbs_mfma_probe(const void* operands, int iters, int shape_32x32x16, float* sink, unsigned long long* clocks,
                              void* stream) {
  PBS_REQUIRE(operands && sink && clocks && iters > 0, "pbs_mfma_probe: bad arguments");
  PBS_REQUIRE(((uintptr_t)operands % 16) == 0, "pbs_mfma_probe: operands must be 16-byte aligned");
  if (shape_32x32x16)
    hipLaunchKernelGGL(mfma_probe_kernel<true>, dim3(PROBE_WGS), dim3(PROBE_THREADS), 0, (hipStream_t)stream,
                       (const uint16_t*)operands, iters, sink, clocks);
  else
    hipLaunchKernelGGL(mfma_probe_kernel<false>, dim3(PROBE_WGS), dim3(PROBE_THREADS), 0, (hipStream_t)stream,
                       (const uint16_t*)operands, iters, sink, clocks);
  return pbs_check_launch("pbs_mfma_probe");
}

extern "C" double pbs_mfma_probe_flop(int iters) {
  return (double)PROBE_WGS * (PROBE_THREADS / 64) * (double)iters * 8.0 * (2.0 * 32 * 32 * 16);
}

namespace {

// ---- measurement aid: the tile pipeline alone.  Every workgroup runs `iters` unmasked fast tiles out of its two
// LDS buffer pairs with the kernel's per-tile barrier and, if asked, the kernel's 64 KB of copies per tile (from a
// ring of `n_src` K / V^T tile pairs), without lists, items, write-out or rare paths: what the schedule of
// fast_tile sustains by itself.  V_ROWS: the tiles are handled as the kernel handles a tile of the query block's own
// segment (K and V copied row by row, V fragments by transposing reads).  Workgroup 0 reports its shader-clock and
// 100 MHz ticks.
template <bool V_ROWS>
__global__ __launch_bounds__(512, 2) void tile_probe_kernel(const uint16_t* __restrict__ tiles, int n_src, int iters, int with_copies,
                                                            float* __restrict__ sink, unsigned long long* __restrict__ clocks) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  for (int i = threadIdx.x; i < (int)(4 * TILE_BYTES / 16); i += 512)   // both buffer pairs start as copies of the first tiles
    reinterpret_cast<u32x4*>(smem)[i] = reinterpret_cast<const u32x4*>(tiles)[i % (2 * TILE_BYTES / 16)];
  __syncthreads();
  const int lane = lane_id_here();
  const int i16 = lane & 15, g4 = lane >> 4;
  const int krow = 8 * (i16 >> 2) + (i16 & 3);
  const uint32_t koff0 = (uint32_t)(krow * 256 + ((g4 ^ i16) * 16));
  const uint32_t voff0 = LDS_V0 + (uint32_t)(i16 * 256 + ((g4 ^ i16) * 16));
  const uint32_t lane_off = async_lane_offset(wave, lane);
  bf16x8 qf[2][4];
#pragma unroll
  for (int qg = 0; qg < 2; ++qg)
#pragma unroll
    for (int kd = 0; kd < 4; ++kd)
      qf[qg][kd] = *reinterpret_cast<const bf16x8*>(tiles + (wave * 32 + 16 * qg + i16) * D + 32 * kd + 8 * g4);
  f32x4 o[8][2];
  float zero = 0.f;
  asm volatile("" : "+v"(zero));
#pragma unroll
  for (int dt = 0; dt < 8; ++dt)
#pragma unroll
    for (int qg = 0; qg < 2; ++qg)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][qg][r] = zero;
  float m_ref[2] = {8.f, 8.f}, l_part[2] = {0.f, 0.f}, c_log2 = 0.12751743f;   // exp2(s / sqrt(128) * log2 e - 8): no rescale on N(0, 1) data
  asm volatile("" : "+s"(c_log2));
  bool poisoned = false;
  uint32_t bufx = 0;
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it, bufx ^= 0x8000u) {
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    if (with_copies) {
      // the 32 workgroups of an XCD (blockIdx % 8) copy the same tile at the same step, as the kernel's workgroups
      // of an XCD walk one head's K / V stream together and share it in that XCD's L2
      const uint16_t* src = tiles + (size_t)((it * 7 + (int)(blockIdx.x & 7) * 29) % n_src) * (2 * BS * D);
      if (V_ROWS) {
        stage_krows_async(src, D, BS, bufx ^ 0x8000u, wave, lane_id_here());
        stage_vrows_async(src + BS * D, D, BS, LDS_V0 + (bufx ^ 0x8000u), wave, lane_id_here());
      } else {
        if (wave < 4) {   // as the kernel does: the first wave of every SIMD issues the second wave's share too
          stage_tile_async(src, bufx ^ 0x8000u, wave, lane_off ^ k_copy_xor(wave));
          stage_tile_async(src, bufx ^ 0x8000u, wave + 4, (lane_off + 4096u) ^ k_copy_xor(wave + 4));
          stage_tile_async(src + BS * D, LDS_V0 + (bufx ^ 0x8000u), wave, lane_off);
          stage_tile_async(src + BS * D, LDS_V0 + (bufx ^ 0x8000u), wave + 4, lane_off + 4096u);
        }
      }
    }
    uint32_t ka[4], va[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      ka[n] = koff0 ^ (uint32_t)(n << 6) ^ bufx;
      va[n] = voff0 ^ (uint32_t)(n << 6) ^ bufx;
    }
    fast_tile<false, PREFETCH_SLOTS, V_ROWS>(o, qf, ka, va, c_log2, m_ref, l_part, poisoned, wave & 3);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);
  const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = l_part[0] + l_part[1] + m_ref[0] + m_ref[1] + (poisoned ? 1.f : 0.f);
#pragma unroll
  for (int dt = 0; dt < 8; ++dt)
#pragma unroll
    for (int qg = 0; qg < 2; ++qg)
#pragma unroll
      for (int r = 0; r < 4; ++r) s += o[dt][qg][r];
  sink[blockIdx.x * 512 + threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = c1 - c0;
    clocks[1] = r1 - r0;
  }
}

}  // namespace

extern "C" int pbs_attn_tile_probe(const void* tiles, int n_src_tiles, int iters, int with_copies, float* sink,
                                   unsigned long long* clocks, void* stream) {
  PBS_REQUIRE(tiles && sink && clocks && iters > 0 && n_src_tiles >= 2, "pbs_attn_tile_probe: bad arguments");
  PBS_REQUIRE(((uintptr_t)tiles % 16) == 0, "pbs_attn_tile_probe: tiles must be 16-byte aligned");
  const bool v_rows = (with_copies & 2) != 0;
  const void* kernel = v_rows ? (const void*)tile_probe_kernel<true> : (const void*)tile_probe_kernel<false>;
  hipError_t attr = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_TOTAL);
  if (attr != hipSuccess) {
    pbs_set_error("pbs_attn_tile_probe: cannot reserve %u bytes of LDS: %s", LDS_TOTAL, hipGetErrorString(attr));
    return (int)attr;
  }
  if (v_rows)
    hipLaunchKernelGGL(tile_probe_kernel<true>, dim3(256), dim3(512), LDS_TOTAL, (hipStream_t)stream, (const uint16_t*)tiles,
                       n_src_tiles, iters, with_copies & 1, sink, clocks);
  else
    hipLaunchKernelGGL(tile_probe_kernel<false>, dim3(256), dim3(512), LDS_TOTAL, (hipStream_t)stream, (const uint16_t*)tiles,
                       n_src_tiles, iters, with_copies & 1, sink, clocks);
  return pbs_check_launch("pbs_attn_tile_probe");
}
