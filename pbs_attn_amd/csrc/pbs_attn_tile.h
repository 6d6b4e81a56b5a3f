// The tile pipeline of the PBS block-sparse attention kernel: LDS layout constants, the asynchronous global -> LDS
// tile copies, MFMA fragment reads and the 48-slot software pipeline over one 128 x 128 tile (fast_tile).  Shared by
// the attention kernel and by the bench-only probe that times this pipeline by itself.
#pragma once
#include "pbs_common.h"

namespace {


constexpr int D = 128;
constexpr int BS = 128;
constexpr int TILE_BYTES = BS * D * 2;            // 32 KB
constexpr uint32_t LDS_V0 = 2 * TILE_BYTES;       // K buffers at 0 / 32 KB, V buffers at 64 / 96 KB
constexpr uint32_t LDS_LIST = 4 * TILE_BYTES;     // two merged visit lists (current item, next item), uint16 entries
constexpr uint32_t LIST_BYTES = 9728;             // count + at most 4096 + 511 + 1 entries, rounded up
constexpr uint32_t LDS_MISC = LDS_LIST + 2 * LIST_BYTES;   // ints: [1] redo flag, [2] first work item, [4] next work item
constexpr uint32_t LDS_DUMP = LDS_MISC + 1024;    // 1 KB per wave: landing area of copies issued only to bring lines into L2
constexpr uint32_t LDS_TOTAL = LDS_DUMP + 8192;   // 159 744 bytes of the CU's 160 KB
constexpr uint32_t ENT_KB = 0x1fffu;              // visit-list entry: key block ...
constexpr uint32_t ENT_ORIG = 0x2000u;            // ... | tile of the un-permuted K / V (own segment) | use bits 14, 15
constexpr int PREFETCH_SLOTS = 2;                 // LDS fragment reads run this many slots ahead

typedef __attribute__((address_space(3))) uint8_t lds_u8;

// lane id formed where it is asked for: as a plain intrinsic it is computed once at the top of the kernel and
// everything derived from it holds registers from there on
__device__ __forceinline__ int lane_id_here() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
}

// row of the 32-row MFMA tile -> key of the 32-key sub-tile, chosen so that the accumulator
// registers 8u..8u+7 of lane-half g hold keys 16u + 8g + 0..7
__device__ __forceinline__ int mfma_row_to_key(int i) {
  const int a = i >> 3, g = (i >> 2) & 1, c = i & 3;
  return 16 * (a >> 1) + 8 * g + 4 * (a & 1) + c;
}

// ---- asynchronous global -> LDS copy of one 32 KB tile by 512 threads ----------------------
// global_load_lds_dwordx4 writes lane l at M0 + 16 l, so one wave instruction fills 4 consecutive
// LDS rows and the chunk swizzle is applied on the GLOBAL side: lane l of wave w fetches chunk
// (l & 15) ^ (row & 15) of row 4 w + 32 n + (l >> 4).  That chunk does not depend on n: one
// per-lane byte offset serves the four loads, tile base and LDS base advance by 8192 bytes in
// scalar registers.  The copy is issued from inline assembly so that the compiler does not order
// later LDS reads of the OTHER buffer behind it; M0 is handed over as a register operand (the compiler
// writes it and knows it is in use; the s_nop is the wait state between that write and the copy);
// completion is awaited with s_waitcnt vmcnt(0) before the barrier that publishes the tile.
__device__ __forceinline__ uint32_t async_lane_offset(int wave, int lane) {
  const int row = 4 * wave + (lane >> 4);
  const int c = (lane & 15) ^ (row & 15);
  return (uint32_t)((row * D + c * 8) * 2);
}

__device__ __forceinline__ void stage_tile_async(const uint16_t* src, uint32_t lds_byte, int wave, uint32_t lane_off) {
  const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_byte + wave * 1024));
  // readfirstlane returns int: widen through uint32_t or the low half would be sign-extended
  const uint64_t src0 = (uint64_t)(uintptr_t)src;
  const uint32_t src_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src0);
  const uint32_t src_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(src0 >> 32));
  const uint64_t srcu = ((uint64_t)src_hi << 32) | (uint64_t)src_lo;
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    const uint64_t base = srcu + n * 8192;
    register uint32_t m0v asm("m0") = lds0 + n * 8192;
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(lane_off), "s"(base) : "memory");
  }
}

// K tile of the ORIGINAL tensor: 128 rows at the caller's row stride (same LDS layout and swizzle).  Rows
// past the end of the sequence re-read the last valid row: their keys lie after every query and are masked.
__device__ __forceinline__ void stage_krows_async(const uint16_t* src, uint32_t row_stride, int rows_valid, uint32_t lds_byte,
                                                  int wave, int lane) {
  const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_byte + wave * 1024));
  const uint64_t src0 = (uint64_t)(uintptr_t)src;
  const uint32_t src_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src0);
  const uint32_t src_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(src0 >> 32));
  const uint64_t srcu = ((uint64_t)src_hi << 32) | (uint64_t)src_lo;
  // lane l of wave w fetches chunk (l & 15) ^ (row & 15) of row 4 w + 32 n + (l >> 4); offsets fit 32 bits
  // (row stride < 2^22 elements, checked on the host)
  const uint32_t r0 = (uint32_t)(4 * wave + (lane >> 4));
  const uint32_t c16 = (uint32_t)(((lane & 15) ^ (r0 & 15)) * 16);
  if (rows_valid >= BS) {
    const uint32_t voff = r0 * row_stride * 2u + c16;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const uint64_t base = srcu + (uint64_t)n * (64u * row_stride);
      register uint32_t m0v asm("m0") = lds0 + n * 8192;
      asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(voff), "s"(base) : "memory");
    }
  } else {
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const uint32_t row = min(r0 + 32u * n, (uint32_t)(rows_valid - 1));
      const uint32_t voff = row * row_stride * 2u + c16;
      register uint32_t m0v asm("m0") = lds0 + n * 8192;
      asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(voff), "s"(srcu) : "memory");
    }
  }
}

__device__ __forceinline__ bf16x8 ldsf(uint32_t byte_addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>((const lds_u8*)(uintptr_t)byte_addr);
}

#define PBS_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)


// ---- fast tile: 48 slots = 6 steps x 8.  Step s issues, interleaved, S of sub-tile s (s <= 3),
// exponentials of sub-tile s - 1 (1 <= s <= 4), P.V of sub-tile s - 2 (s >= 2); S and P are
// double-buffered by sub-tile parity; one scheduling barrier per slot keeps the order.  The MASKED tile
// (the diagonal block, read in original key order) zeroes the exponentials of keys that lie after the
// query: key-in-tile > query-in-block, an arithmetic test.
template <bool MASKED, int PF>
__device__ __forceinline__ void fast_tile(f32x16 (&o)[4], const bf16x8 (&qf)[8], const uint32_t koff0,
                                          const uint32_t voff0, const uint32_t (&bx)[8], float c_log2, float& m_ref,
                                          float& l_part, bool& poisoned, int wq) {
  // query-in-block minus the lane half's key offset; made opaque per call: the 128 mask compares of a
  // diagonal tile depend only on the lane, and hoisted out of the tile loop they would each pin a 64-bit
  // scalar mask
  int qrel8 = 0;
  if (MASKED) {
    const int ln = lane_id_here();          // nothing below may be formed outside the tile
    qrel8 = 32 * wq + (ln & 31) - 8 * (ln >> 5);
  }
  const float negm = -m_ref;
  float rsum[4] = {0.f, 0.f, 0.f, 0.f};
  f32x16 sbuf[2];
  bf16x8 pbuf[2][2];
  constexpr int R = PF + 1;
  bf16x8 frk[R], frv[R];
#pragma unroll
  for (int n = 0; n < PF; ++n) frk[n % R] = ldsf((koff0 ^ bx[n & 7]) + (n >> 3) * 8192);
#pragma clang loop unroll(full)
  for (int n = 0; n < 48; ++n) {
    const int step = n >> 3, t = n & 7;
    {   // fragment reads for slot n + PF
      const int m = n + PF, mstep = m >> 3, mt = m & 7;
      if (m < 48 && mstep <= 3) frk[m % R] = ldsf((koff0 ^ bx[mt]) + mstep * 8192);
      if (m < 48 && mstep >= 2) frv[m % R] = ldsf((voff0 ^ bx[2 * (mstep - 2) + (mt >> 2)]) + (mt & 3) * 8192);
    }
    // the reads go out before this slot's matrix instructions: left to the scheduler they sink behind them
    // (their address is formed in the slot) and the fragments arrive a slot late
    __builtin_amdgcn_sched_barrier(0);
    if (step <= 3) {
      const f32x16 acc = (t == 0) ? (f32x16){0} : sbuf[step & 1];
      sbuf[step & 1] = PBS_MFMA(frk[n % R], qf[t], acc);
    }
    if (step >= 2) o[t & 3] = PBS_MFMA(frv[n % R], pbuf[step & 1][t >> 2], o[t & 3]);
    if (step >= 1 && step <= 4) {
      const int sb = (step - 1) & 1, r = 2 * t;
      float x0 = sbuf[sb][r], x1 = sbuf[sb][r + 1];
      if (MASKED) {
        // registers r, r + 1 of sub-tile ks hold keys 32 ks + 16 (a4 >> 1) + 8 gh + 4 (a4 & 1) + (r & 3), a4 = r >> 2
        const int ks = step - 1, a4 = r >> 2;
        const int key = 32 * ks + 16 * (a4 >> 1) + 4 * (a4 & 1) + (r & 3);
        if (key > qrel8) x0 = -INFINITY;
        if (key + 1 > qrel8) x1 = -INFINITY;
      }
      const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(x0, c_log2, negm));
      const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(x1, c_log2, negm));
      rsum[t & 3] += e0;
      rsum[(t + 2) & 3] += e1;
      pbuf[sb][r >> 3][r & 7] = (__bf16)e0;
      pbuf[sb][r >> 3][(r & 7) + 1] = (__bf16)e1;
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  const float rs = (rsum[0] + rsum[1]) + (rsum[2] + rsum[3]);
  l_part += rs;
  // lazy reference maximum without tracking maxima: a row sum of this tile above 2^14 says some
  // exponential was large; any reference >= the old one is valid, so move it up by log2(sum)
  if (__any(rs > 16384.0f)) {
    const float big = fmaxf(rs, xhalf_f32(rs));
    if (__any(!(big < 1e30f))) poisoned = true;   // overflow (inf / nan): redo the row without speculation
    const float m_new = (big > 16384.0f) ? m_ref + __builtin_amdgcn_logf(big) : m_ref;
    const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
    m_ref = m_new;
    l_part *= alpha;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
  }
}

}  // namespace
