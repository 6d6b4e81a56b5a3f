// Shared device/host helpers for the PBS-Attn gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#define PBS_WAVE 64

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// ---- error reporting across the C ABI (thread-local message) --------------
extern "C" const char* pbs_last_error(void);
void pbs_set_error(const char* fmt, ...);
int pbs_arg_error(const char* fmt, ...);        // sets message, returns -1
int pbs_check_launch(const char* what);         // hipGetLastError -> positive code
// Kernels that address LDS by absolute byte offsets (M0 of global_load_lds, integer-to-LDS-pointer casts) rely on
// their dynamic LDS starting at offset 0, i.e. on having no static LDS: 0 if `kernel` has none, else an error code
// with the message set.
int pbs_require_no_static_lds(const void* kernel, const char* what);

#define PBS_REQUIRE(cond, ...)                      \
  do {                                              \
    if (!(cond)) return pbs_arg_error(__VA_ARGS__); \
  } while (0)

// ---- bf16 <-> f32 ------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// two values rounded to bf16 (nearest even) by one hardware conversion, returned as floats
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
__device__ __forceinline__ f32x2 hw_round_bf16x2(f32x2 x) {
  const uint32_t packed = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
  return (f32x2){__builtin_bit_cast(float, packed << 16), __builtin_bit_cast(float, packed & 0xffff0000u)};
}

// ---- order-preserving float key ---------------------------------------------
// ascending unsigned order == ascending float order; -0 == +0; NaN greatest.
__device__ __forceinline__ uint32_t f32_orderable(float f) {
  uint32_t u = __float_as_uint(f);
  if (u == 0x80000000u) u = 0;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float f32_from_orderable(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}
// composite key: ascending sort == descending value, ties by ascending index
__device__ __forceinline__ uint64_t desc_stable_key(float v, uint32_t index) {
  return ((uint64_t)(~f32_orderable(v)) << 32) | index;
}
__device__ __forceinline__ float desc_key_value(uint64_t key) { return f32_from_orderable(~(uint32_t)(key >> 32)); }

// In-place ascending bitonic sort of n_pow2 uint64 keys held in LDS by one workgroup (whole waves, any number).
// Thread t of a stage exchanges elements lo(t) and lo(t) + stride.  The 64 threads t = 64 c .. 64 c + 63 belong to
// one wave in every stage, and for strides up to 64 their pairs are exactly elements 128 c .. 128 c + 127: those
// stages need no workgroup barrier between them (a wave's LDS accesses complete in order), only the stages with
// longer strides and the first short one after them do -- 9 barriers instead of 55 for 1024 keys.
__device__ __forceinline__ void bitonic_sort_lds(uint64_t* keys, int n_pow2) {
  __syncthreads();
  for (int size = 2; size <= n_pow2; size <<= 1) {
    for (int stride = size >> 1, sh = __builtin_ctz(size) - 1; stride > 0; stride >>= 1, --sh) {
      if (stride >= 64) __syncthreads();            // stride 64: the data may come from a longer stride's stage
      else __builtin_amdgcn_wave_barrier();
      for (int t = threadIdx.x; t < (n_pow2 >> 1); t += blockDim.x) {
        const int lo = ((t >> sh) << (sh + 1)) | (t & (stride - 1));
        const int hi = lo + stride;
        const bool up = ((lo & size) == 0);
        const uint64_t a = keys[lo], b = keys[hi];
        if ((a > b) == up) {
          keys[lo] = b;
          keys[hi] = a;
        }
      }
    }
  }
  __syncthreads();
}

static inline int next_pow2_int(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

// cross-half exchange inside a 64-wide wavefront (lane ^ 32)
__device__ __forceinline__ float xhalf_f32(float v) { return __shfl_xor(v, 32, 64); }
