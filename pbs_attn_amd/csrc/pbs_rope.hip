// Rotary position embedding of Q and K in one pass, written head-major and contiguous.
// The glue around the attention call applies RoPE with five elementwise torch kernels per tensor
// (q * cos, rotate_half, * sin, +, and a concatenation); this kernel produces the same bits in one read
// and one write: out = bf16(bf16(x * cos) + bf16(rotate_half(x) * sin)), every product and the sum
// computed in fp32 and rounded to bf16 exactly where the bf16 tensor expression rounds.
#include "pbs_common.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations

namespace {

constexpr int D = 128;

struct RopeArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* cos;
  const uint16_t* sin;
  uint16_t* q_out;   // (B, Hq, S, 128) contiguous
  uint16_t* k_out;   // (B, Hkv, S, 128) contiguous
  int B, Hq, Hkv, S;
  int64_t q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, c_sb, c_ss;
};

__device__ __forceinline__ uint32_t round_pair(float lo, float hi) {
  return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// 16 lanes x 16 bytes per 256-byte row, 16 rows per workgroup
__global__ __launch_bounds__(256) void rope_qk_kernel(RopeArgs a) {
  const int c = threadIdx.x & 15, s = blockIdx.x * 16 + (threadIdx.x >> 4);
  if (s >= a.S) return;
  const int heads = a.Hq + a.Hkv;
  const int b = blockIdx.y / heads, hh = blockIdx.y % heads;
  const bool is_k = hh >= a.Hq;
  const int h = is_k ? hh - a.Hq : hh;
  const uint16_t* src = is_k ? a.k + b * a.k_sb + h * a.k_sh + (int64_t)s * a.k_ss
                             : a.q + b * a.q_sb + h * a.q_sh + (int64_t)s * a.q_ss;
  uint16_t* dst = is_k ? a.k_out + (((int64_t)b * a.Hkv + h) * a.S + s) * D : a.q_out + (((int64_t)b * a.Hq + h) * a.S + s) * D;
  const u32x4 x = *reinterpret_cast<const u32x4*>(src + c * 8);
  const u32x4 xp = *reinterpret_cast<const u32x4*>(src + ((c + 8) & 15) * 8);   // the other half of the row
  const u32x4 cs = *reinterpret_cast<const u32x4*>(a.cos + b * a.c_sb + (int64_t)s * a.c_ss + c * 8);
  const u32x4 sn = *reinterpret_cast<const u32x4*>(a.sin + b * a.c_sb + (int64_t)s * a.c_ss + c * 8);
  const float sign = c < 8 ? -1.0f : 1.0f;   // rotate_half = (-second half, first half)
  u32x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int sh = 16 * p;
      const float xv = bf16_bits_to_f32((x[e] >> sh) & 0xffffu), pv = sign * bf16_bits_to_f32((xp[e] >> sh) & 0xffffu);
      const float cv = bf16_bits_to_f32((cs[e] >> sh) & 0xffffu), sv = bf16_bits_to_f32((sn[e] >> sh) & 0xffffu);
      const float t0 = bf16_bits_to_f32(f32_to_bf16_bits(xv * cv));
      const float t1 = bf16_bits_to_f32(f32_to_bf16_bits(pv * sv));
      r[p] = t0 + t1;
    }
    o[e] = round_pair(r[0], r[1]);
  }
  *reinterpret_cast<u32x4*>(dst + c * 8) = o;
}

}  // namespace

extern "C" int pbs_rope_qk(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int B,
                           int Hq, int Hkv, int S, int head_dim, int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb,
                           int64_t k_sh, int64_t k_ss, int64_t c_sb, int64_t c_ss, void* stream) {
  PBS_REQUIRE(q && k && cos && sin && q_out && k_out, "pbs_rope_qk: null tensor pointer");
  PBS_REQUIRE(head_dim == D, "pbs_rope_qk: head_dim must be 128, got %d", head_dim);
  PBS_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && S > 0 && (int64_t)B * (Hq + Hkv) <= 65535, "pbs_rope_qk: bad shape");
  PBS_REQUIRE(q_sb % 8 == 0 && q_sh % 8 == 0 && q_ss % 8 == 0 && k_sb % 8 == 0 && k_sh % 8 == 0 && k_ss % 8 == 0 &&
                  c_sb % 8 == 0 && c_ss % 8 == 0,
              "pbs_rope_qk: strides must keep rows 16-byte aligned");
  PBS_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)cos % 16) == 0 &&
                  ((uintptr_t)sin % 16) == 0 && ((uintptr_t)q_out % 16) == 0 && ((uintptr_t)k_out % 16) == 0,
              "pbs_rope_qk: pointers must be 16-byte aligned");
  RopeArgs a;
  a.q = (const uint16_t*)q; a.k = (const uint16_t*)k; a.cos = (const uint16_t*)cos; a.sin = (const uint16_t*)sin;
  a.q_out = (uint16_t*)q_out; a.k_out = (uint16_t*)k_out;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.S = S;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_ss = q_ss; a.k_sb = k_sb; a.k_sh = k_sh; a.k_ss = k_ss; a.c_sb = c_sb; a.c_ss = c_ss;
  hipLaunchKernelGGL(rope_qk_kernel, dim3((S + 15) / 16, B * (Hq + Hkv)), dim3(256), 0, (hipStream_t)stream, a);
  return pbs_check_launch("pbs_rope_qk");
}
