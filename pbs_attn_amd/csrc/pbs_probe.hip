// Measurement aid, not part of the attention path: a loop of nothing but v_mfma_f32_32x32x16_bf16 on
// operands the caller provides.  On MI355X the rate this loop sustains depends on the operand VALUES
// (zeros run at the full clock, normally distributed values make the chip lower its clock to stay inside
// its power limit), so the benchmark reports it next to the attention kernel's rate as the MFMA ceiling
// for data like the attention kernel's.
#include "pbs_common.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations

namespace {

constexpr int PROBE_WGS = 256, PROBE_THREADS = 512, PROBE_OPERANDS = 65536;

__global__ __launch_bounds__(PROBE_THREADS, 2) void mfma_probe_kernel(const uint16_t* operands, int iters, float* sink,
                                                                        unsigned long long* clocks) {
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  bf16x8 a[8], b[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    a[t] = *reinterpret_cast<const bf16x8*>(operands + ((threadIdx.x * 128 + t * 16) & (PROBE_OPERANDS - 1)));
    b[t] = *reinterpret_cast<const bf16x8*>(operands + ((threadIdx.x * 128 + t * 16 + 8) & (PROBE_OPERANDS - 1)));
  }
  f32x16 c[4] = {{0}, {0}, {0}, {0}};
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int t = 0; t < 8; ++t) c[t & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t], b[t], c[t & 3], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 16; ++e) s += (c[0][e] + c[1][e]) + (c[2][e] + c[3][e]);
  sink[blockIdx.x * PROBE_THREADS + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    atomicAdd(&clocks[0], __builtin_amdgcn_s_memtime() - c0);       // shader clock ticks
    atomicAdd(&clocks[1], __builtin_amdgcn_s_memrealtime() - r0);   // 100 MHz ticks
  }
}

}  // namespace

extern "C" int pbs_mfma_probe(const void* operands, int iters, float* sink, unsigned long long* clocks, void* stream) {
  PBS_REQUIRE(operands && sink && clocks && iters > 0, "pbs_mfma_probe: bad arguments");
  PBS_REQUIRE(((uintptr_t)operands % 16) == 0, "pbs_mfma_probe: operands must be 16-byte aligned");
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(PROBE_WGS), dim3(PROBE_THREADS), 0, (hipStream_t)stream,
                     (const uint16_t*)operands, iters, sink, clocks);
  return pbs_check_launch("pbs_mfma_probe");
}

extern "C" double pbs_mfma_probe_flop(int iters) {
  return (double)PROBE_WGS * (PROBE_THREADS / 64) * (double)iters * 8.0 * (2.0 * 32 * 32 * 16);
}
