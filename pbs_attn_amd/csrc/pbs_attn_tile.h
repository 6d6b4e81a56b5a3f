// The tile pipeline of the PBS block-sparse attention kernel: LDS layout constants, the asynchronous global -> LDS
// tile copies, MFMA fragment reads and the 48-slot software pipeline over one 128 x 128 tile (fast_tile).  Shared by
// the attention kernel and by the bench-only probe that times this pipeline by itself.
#pragma once
#include "pbs_common.h"

// branch hints: they decide which side of a branch is laid out as the fall-through.  A taken branch refills the
// wave's instruction buffer, and in the tile loop all eight waves of a workgroup take it at about the same time with
// the matrix pipes idle, so the common path of that loop has to be the straight one.
#define PBS_LIKELY(x) __builtin_expect(!!(x), 1)
#define PBS_UNLIKELY(x) __builtin_expect(!!(x), 0)

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

// ---- operand geometry of a wave (32 queries = two column groups qg of 16; lane l: i = l % 16, g = l / 16)
//   S^T = K Q^T per 32-key sub-tile ks: two 16-key row tiles T, four d-steps kd of 32:
//       A = K[key(T, i)][32 kd + 8 g + 0..7],  key(T, i) = 32 ks + 8 (i / 4) + 4 T + i % 4
//       B = Q[16 qg + i][32 kd + 8 g + 0..7]
//       D: lane holds query 16 qg + i, keys 32 ks + 8 g + 4 T + 0..3
//     so the eight values of (T = 0, T = 1) are keys 32 ks + 8 g + 0..7: converted to bf16 they ARE the B operand of
//   O^T += V^T P^T per sub-tile: eight 16-row d tiles dt:
//       A = V^T[16 dt + i][32 ks + 8 g + 0..7],  B = P[keys 32 ks + 8 g + 0..7][16 qg + i]
//       D: lane holds query 16 qg + i, d = 16 dt + 4 g + 0..3
// LDS tiles are 128 rows x 16 chunks of 16 bytes, chunk index XOR hash(row): rows of a K tile are keys and the 16
// lanes of a fragment read take keys 8 (i / 4) + i % 4 (+ 4 T), so the hash is (row & 3) | ((row >> 3) & 3) << 2
// (= i: sixteen chunks, no bank conflict); rows of a V^T tile are d and the lanes take consecutive rows: row & 15.
__device__ __forceinline__ int k_row_hash(int row) { return (row & 3) | (((row >> 3) & 3) << 2); }

// A tile of V rows taken from the caller's tensor (a query block's own segment) is not transposed on the way in.  Its
// fragments are read with the transposing LDS read (ds_read_b64_tr_b16: lane l of a group of 16 hands in the address of
// four consecutive d of key (l / 4), and receives, for d = l, the four keys), two reads per fragment.  Four rows (keys
// 4 m + 0..3) share 1024 bytes of LDS, 32-byte piece p (d = 16 p .. 16 p + 15) of row 4 m + e at m * 1024 + p * 128 +
// e * 32: a group's four keys x 32 bytes are 128 consecutive bytes (no bank conflict), the d tile, the sub-tile and the
// key half of a read are constant offsets from one address per lane, and one copy instruction (1024 bytes of LDS)
// reads four whole rows.
// the copy of a K tile fetches chunk (l & 15) ^ k_row_hash(row) where async_lane_offset has (l & 15) ^ (row & 15), row =
// 4 wave + (l >> 4) + 32 n: the two differ by a wave-uniform XOR of the byte offset
__device__ __forceinline__ uint32_t k_copy_xor(int wave) { return (uint32_t)(((wave & 3) ^ ((wave >> 1) & 3)) << 6); }

// ---- asynchronous global -> LDS copy of one 32 KB tile by 512 threads ----------------------
// global_load_lds_dwordx4 writes lane l at M0 + 16 l, so one wave instruction fills 4 consecutive
// LDS rows and the chunk swizzle is applied on the GLOBAL side: lane l of wave w fetches chunk
// (l & 15) ^ (row & 15) of row 4 w + 32 n + (l >> 4) (a V^T tile; for a K tile the offset is XORed with k_copy_xor).  That chunk does not depend on n: one
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

// K tile of the ORIGINAL tensor: 128 rows at the caller's row stride, chunk index XOR k_row_hash of the row.  Rows
// past the end of the sequence re-read the last valid row: their keys lie after every query and are masked.
__device__ __forceinline__ void stage_krows_async(const uint16_t* src, uint32_t row_stride, int rows_valid, uint32_t lds_byte,
                                                  int wave, int lane) {
  const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_byte + wave * 1024));
  const uint64_t src0 = (uint64_t)(uintptr_t)src;
  const uint32_t src_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src0);
  const uint32_t src_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(src0 >> 32));
  const uint64_t srcu = ((uint64_t)src_hi << 32) | (uint64_t)src_lo;
  // lane l of wave w fetches chunk (l & 15) ^ hash(row) of row 4 w + 32 n + (l >> 4) (the hash does not depend on n);
  // offsets fit 32 bits (row stride < 2^22 elements, checked on the host)
  const uint32_t r0 = (uint32_t)(4 * wave + (lane >> 4));
  const uint32_t c16 = (uint32_t)(((lane & 15) ^ k_row_hash((int)r0)) * 16);
  if (PBS_LIKELY(rows_valid >= BS)) {
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

// V tile of the ORIGINAL tensor in the layout above: wave w, instruction n copy rows 4 w + 32 n + 0..3 like the K copy;
// lane l takes row (l >> 1) & 3 of them and the 16-byte chunk 2 (l >> 3) + (l & 1).  Rows past the end of the sequence
// re-read the last valid row.
__device__ __forceinline__ void stage_vrows_async(const uint16_t* src, uint32_t row_stride, int rows_valid, uint32_t lds_byte,
                                                  int wave, int lane) {
  const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_byte + wave * 1024));
  const uint64_t src0 = (uint64_t)(uintptr_t)src;
  const uint32_t src_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src0);
  const uint32_t src_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(src0 >> 32));
  const uint64_t srcu = ((uint64_t)src_hi << 32) | (uint64_t)src_lo;
  const uint32_t r0 = (uint32_t)(4 * wave + ((lane >> 1) & 3));
  const uint32_t c16 = (uint32_t)((2 * (lane >> 3) + (lane & 1)) * 16);
  if (PBS_LIKELY(rows_valid >= BS)) {
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

// v_mfma_f32_16x16x32_bf16: D (16 x 16) += A (16 x 32) B (32 x 16).  Lane l holds row l % 16 of A and column l % 16 of
// B, each with k = 8 (l / 16) + 0..7, and of D column l % 16, rows 4 (l / 16) + 0..3.  On normally distributed
// operands the chip sustains about 11 % more FLOP/s with this shape than with 32x32x16 (it moves half the
// accumulator registers per FLOP and holds a higher clock inside its power limit).
// V^T fragment (16 d x 32 keys of a sub-tile) out of a tile copied by stage_vrows_async: addr = this lane's address
// for the fragment's d tile and sub-tile; keys 8 g + 0..3 at addr, 8 g + 4..7 in the next four rows (1024 bytes further)
typedef __attribute__((ext_vector_type(4))) short s16x4;
__device__ __forceinline__ bf16x8 ldsf_transposed(uint32_t addr) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(lds_u8*)(uintptr_t)addr);
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(lds_u8*)(uintptr_t)(addr + 1024));
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, both);
}
// this lane's address of the fragment of sub-tile 0, d tile 0 in the tile whose buffer starts at LDS byte offset
// v_buf; d tile dt: + dt * 128, sub-tile ks: + ks * 8192
__device__ __forceinline__ uint32_t vrow_lane_addr(uint32_t v_buf, int lane) {
  const int l16 = lane & 15, g = lane >> 4;
  return v_buf + (uint32_t)(g * 2048 + (l16 >> 2) * 32 + (l16 & 3) * 8);
}

#define PBS_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0)

// lane ^ 16: with xhalf_f32 (lane ^ 32) it reaches the four lanes that share a query column
__device__ __forceinline__ float xq16_f32(float v) { return __shfl_xor(v, 16, 64); }
__device__ __forceinline__ float max_over_lane_groups(float v) {
  v = fmaxf(v, xq16_f32(v));
  return fmaxf(v, xhalf_f32(v));
}
__device__ __forceinline__ float sum_over_lane_groups(float v) {
  v += xq16_f32(v);
  return v + xhalf_f32(v);
}

// ---- fast tile: 48 slots = 6 steps x 8.  Step s issues, interleaved, S of sub-tile s (s <= 3),
// exponentials of sub-tile s - 1 (1 <= s <= 4), P.V of sub-tile s - 2 (s >= 2); S and P are
// double-buffered by sub-tile parity; one scheduling barrier per slot keeps the order.  A slot reads one K and one
// V^T fragment (two slots ahead) and feeds each to two matrix instructions, one per query column group.  The MASKED
// tile (the diagonal block, read in original key order) zeroes the exponentials of keys that lie after the
// query: key-in-tile > query-in-block, an arithmetic test.
// ka[kd] / va[ks]: this lane's byte addresses of the K fragments of d-step kd (row tile 0, sub-tile 0) and of the V^T
// fragments of sub-tile ks (d tile 0) in the tile's buffers: held in registers and switched between the two buffers
// once per tile, so that a fragment read needs no address arithmetic (a vector instruction per read is a tenth of
// the pipeline's vector work, and vector work overlaps only a third of a matrix instruction's time).
// V_ROWS: the tile's V is a tile of the caller's tensor, copied by stage_vrows_async, and its fragments come from
// transposing reads; otherwise it is a transposed (V^T) tile and they are plain 16-byte reads.
template <bool MASKED, int PF, bool V_ROWS>
__device__ __forceinline__ void fast_tile(f32x4 (&o)[8][2], const bf16x8 (&qf)[2][4], const uint32_t (&ka)[4],
                                          const uint32_t (&va)[4], float c_log2, float (&m_ref)[2],
                                          float (&l_row)[2], bool& poisoned, int wq) {
  // query-in-block minus the lane group's key offset; made opaque per call: the mask compares of a
  // diagonal tile depend only on the lane, and hoisted out of the tile loop they would each pin a 64-bit
  // scalar mask
  int qrel8 = 0;
  if (MASKED) {
    const int ln = lane_id_here();          // nothing below may be formed outside the tile
    qrel8 = 32 * wq + (ln & 15) - 8 * (ln >> 4);
  }
  const float negm[2] = {-m_ref[0], -m_ref[1]};
  uint32_t vr = 0;
  if (V_ROWS) vr = vrow_lane_addr(LDS_V0 + (va[0] & 0x8000u), lane_id_here());   // va[] carries the buffer switch in bit 15
  // row sums: one more matrix instruction per sub-tile and column group, ones x P, whose every output row is the sum
  // over the sub-tile's 32 keys of the probabilities as the P.V product sees them (rounded to bf16).  Summing them
  // with vector adds instead costs 64 vector instructions per tile, and the vector unit is as busy as the matrix
  // unit here.
  f32x4 lsum[2];
  u32x4 one_bits = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  asm volatile("" : "+v"(one_bits));
  const bf16x8 ones = __builtin_bit_cast(bf16x8, one_bits);
  f32x4 sacc[2][2][2];     // [sub-tile parity][T][qg]
  bf16x8 pbuf[2][2];       // [sub-tile parity][qg]
  constexpr int R = PF + 1;
  bf16x8 frk[R], frv[R];
#pragma unroll
  for (int n = 0; n < PF; ++n) frk[n % R] = ldsf(ka[n & 3] + ((n >> 2) & 1) * 1024 + (n >> 3) * 8192);
#pragma clang loop unroll(full)
  for (int n = 0; n < 48; ++n) {
    const int step = n >> 3, t = n & 7;
    {   // fragment reads for slot n + PF
      const int m = n + PF, mstep = m >> 3, mt = m & 7;
      if (m < 48 && mstep <= 3) frk[m % R] = ldsf(ka[mt & 3] + (mt >> 2) * 1024 + mstep * 8192);
      if (m < 48 && mstep >= 2) {
        if (V_ROWS) {
          frv[m % R] = ldsf_transposed(vr + mt * 128 + (mstep - 2) * 8192);
        } else {
          frv[m % R] = ldsf(va[mstep - 2] + mt * 4096);
        }
      }
    }
    // the reads go out before this slot's matrix instructions: left to the scheduler they sink behind them
    // (their address is formed in the slot) and the fragments arrive a slot late
    __builtin_amdgcn_sched_barrier(0);
    if (step <= 3) {
      const int T = t >> 2, kd = t & 3;
#pragma unroll
      for (int qg = 0; qg < 2; ++qg) {
        const f32x4 acc = (kd == 0) ? (f32x4){0} : sacc[step & 1][T][qg];
        sacc[step & 1][T][qg] = PBS_MFMA(frk[n % R], qf[qg][kd], acc);
      }
    }
    if (step >= 2) {
#pragma unroll
      for (int qg = 0; qg < 2; ++qg) o[t][qg] = PBS_MFMA(frv[n % R], pbuf[step & 1][qg], o[t][qg]);
      if (t == 1 || t == 5) {
        const int qg = t >> 2;
        lsum[qg] = PBS_MFMA(ones, pbuf[step & 1][qg], step == 2 ? (f32x4){0} : lsum[qg]);
      }
    }
    if (step >= 1 && step <= 4) {
      const int sb = (step - 1) & 1, qg = t >> 2, T = (t >> 1) & 1, c0 = 2 * (t & 1);
      float x0 = sacc[sb][T][qg][c0], x1 = sacc[sb][T][qg][c0 + 1];
      if (MASKED) {
        // the two values are keys 32 ks + 8 g + 4 T + c0 (+ 1) of query 32 wq + 16 qg + i
        const int key = 32 * (step - 1) + 4 * T + c0 - 16 * qg;
        if (key > qrel8) x0 = -INFINITY;
        if (key + 1 > qrel8) x1 = -INFINITY;
      }
      const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(x0, c_log2, negm[qg]));
      const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(x1, c_log2, negm[qg]));
      pbuf[sb][qg][4 * T + c0] = (__bf16)e0;
      pbuf[sb][qg][4 * T + c0 + 1] = (__bf16)e1;
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  const float rs[2] = {lsum[0][0], lsum[1][0]};   // the whole row of this tile, the same in the four lanes of a query
  l_row[0] += rs[0];
  l_row[1] += rs[1];
  // lazy reference maximum without tracking maxima: a row sum of this tile above 2^14 says some
  // exponential was large; any reference >= the old one is valid, so move it up by log2(sum)
  if (PBS_UNLIKELY(__any(rs[0] > 16384.0f || rs[1] > 16384.0f))) {
#pragma unroll
    for (int qg = 0; qg < 2; ++qg) {
      const float big = max_over_lane_groups(rs[qg]);
      if (__any(!(big < 1e30f))) poisoned = true;   // overflow (inf / nan): redo the row without speculation
      const float m_new = (big > 16384.0f) ? m_ref[qg] + __builtin_amdgcn_logf(big) : m_ref[qg];
      const float alpha = __builtin_amdgcn_exp2f(m_ref[qg] - m_new);
      m_ref[qg] = m_new;
      l_row[qg] *= alpha;
#pragma unroll
      for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[dt][qg][r] *= alpha;
    }
  }
}

}  // namespace
