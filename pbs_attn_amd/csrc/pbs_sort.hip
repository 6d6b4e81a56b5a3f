// Per-segment stable descending argsort of the key scores.
//
// One workgroup sorts one segment in LDS with a bitonic network over 64-bit
// composite keys (inverted order-preserving score bits << 32 | local index), so
// equal scores keep ascending index order whatever the network does.  The
// trailing partial segment and the padding up to a whole block keep identity order.
#include "pbs_common.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations

namespace {

__global__ __launch_bounds__(256) void segment_argsort_kernel(const float* scores, int32_t* idx, int S, int Sc,
                                                              int S_pad, int seg, int n_pow2) {
  extern __shared__ uint64_t keys[];
  const int row = blockIdx.y;
  const int nseg = Sc / seg;
  int32_t* out = idx + (int64_t)row * S_pad;
  if ((int)blockIdx.x >= nseg) {
    // identity tail: remainder of the sequence and the block padding
    for (int i = Sc + (blockIdx.x - nseg) * seg + threadIdx.x; i < min(S_pad, Sc + ((int)blockIdx.x - nseg + 1) * seg); i += blockDim.x)
      out[i] = i;
    return;
  }
  const int base = blockIdx.x * seg;
  const float* src = scores + (int64_t)row * Sc + base;
  for (int i = threadIdx.x; i < n_pow2; i += blockDim.x)
    keys[i] = i < seg ? desc_stable_key(src[i], (uint32_t)i) : ~0ull;
  bitonic_sort_lds(keys, n_pow2);
  for (int i = threadIdx.x; i < seg; i += blockDim.x) out[base + i] = base + (int32_t)(uint32_t)keys[i];
}

}  // namespace

extern "C" int pbs_segment_argsort(const float* scores, int32_t* key_indices, int rows, int S, int S_pad,
                                   int segment_size, void* stream) {
  PBS_REQUIRE(key_indices, "pbs_segment_argsort: null index pointer");
  PBS_REQUIRE(rows > 0 && S > 0 && S_pad >= S, "pbs_segment_argsort: bad shape rows=%d S=%d S_pad=%d", rows, S, S_pad);
  PBS_REQUIRE(segment_size > 0 && segment_size <= 8192, "pbs_segment_argsort: segment_size %d outside (0, 8192]", segment_size);
  const int Sc = (S / segment_size) * segment_size;
  PBS_REQUIRE(Sc == 0 || scores, "pbs_segment_argsort: null score pointer");
  const int nseg = Sc / segment_size;
  const int tail_blocks = (S_pad - Sc + segment_size - 1) / segment_size;
  const int n_pow2 = next_pow2_int(segment_size);
  PBS_REQUIRE(rows <= 65535, "pbs_segment_argsort: too many rows (%d)", rows);
  hipLaunchKernelGGL(segment_argsort_kernel, dim3(nseg + tail_blocks, rows), dim3(256), (size_t)n_pow2 * sizeof(uint64_t),
                     (hipStream_t)stream, scores, key_indices, S, Sc, S_pad, segment_size, n_pow2);
  return pbs_check_launch("pbs_segment_argsort");
}
