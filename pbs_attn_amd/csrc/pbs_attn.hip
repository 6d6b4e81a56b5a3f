// Block-sparse flash-attention forward of PBS-Attn (bf16, head_dim 128).
//
// What a query block attends to
//   * the permuted K / V tiles of the selected key blocks of EARLIER segments (the visit list), no mask;
//   * its own segment, read from the ORIGINAL K and V (the caller's tensors, in place): blocks
//     first-of-segment .. query block, with the plain causal triangle on the last one (the diagonal block).
//     A segment's permuted blocks hold the same keys as its original blocks and attention does not depend
//     on key order, so this is the reference's "every block of the own segment, element mask original key
//     position > query position" with half the tiles and one masked tile instead of all.
// Work decomposition
//   A work item is TWO adjacent 128-query blocks of one head, served by one workgroup (8 waves, two per
//   SIMD): waves 0-3 take the first block, waves 4-7 the second, 32 queries per wave.  A small kernel
//   first merges the two visit lists of every item (ascending key-block indices, own-segment blocks
//   appended) into one list in HBM; every merged tile is copied ONCE into LDS for both query blocks, which
//   halves the L2 -> LDS traffic and doubles the time a tile stays in flight.  K and V tiles are
//   double-buffered (2 x 64 KB) and fetched one tile ahead with asynchronous global -> LDS copies (no
//   registers), one workgroup barrier per tile.
//   The attention kernel is PERSISTENT: one workgroup per CU takes item after item from a counter (one per
//   XCD, over that XCD's share of the items; when it runs dry, the other XCDs' counters).  The tile pipeline
//   runs across items: the next item is claimed three tiles before the end of the current one, its list and
//   its queries (into L2) are requested one tile later, its first K / V tiles at the last tile, so that an
//   item's fixed costs (list, first tile, write-out of the previous item) overlap attention work.  With short
//   visit lists (a few tiles per item) that is the difference between waiting for HBM three times per item
//   and once.
// Data layout
//   K tile: 128 keys x 128 d row-major; permuted V tile: stored TRANSPOSED in HBM by the gather kernel,
//   128 d x 128 keys; V tile of an own segment: 128 keys x 128 d as in the caller's tensor, its MFMA fragments
//   read with the transposing LDS read.  K and V^T tiles sit in LDS as 128 rows x 16 chunks of 16 bytes with the
//   chunk index XORed with a hash of the row (pbs_attn_tile.h), so that fragment reads are bank-conflict free.
// Math (transposed formulation, v_mfma_f32_16x16x32_bf16)
//     S^T = K Q^T   (rows = keys, columns = queries)      O^T += V^T P^T   (rows = d, columns = queries)
//   Every lane owns query columns (one per column group of 16 queries), so the softmax reference values are
//   per-lane, and the S^T accumulator registers are, after conversion to bf16, exactly the B operand of the
//   second product (the key rows of each 16-row MFMA tile are fed in the order that makes this so).
//   Softmax runs in the exp2 domain in fp32; P is rounded to bf16 before P.V, and a pipelined tile takes its row
//   sums from one more matrix product, ones x P, i.e. of the rounded values; the output is normalised once at
//   the end.
// Tile kinds
//   * fast tiles: a software pipeline over the four 32-key sub-tiles -- S of sub-tile k+1, exponentials
//     of sub-tile k and P.V of sub-tile k-1 are issued interleaved, LDS fragments are read two slots
//     ahead.  Exponentials are taken against a LAZY reference maximum: it is not updated per tile; a row
//     sum of one tile above 2^14 triggers a uniform rescale (exact, all terms share the reference); an
//     overflow marks the row and the whole workgroup redoes it without speculation.  The first tile of a
//     row takes its reference from the exact maximum over its first 32 keys.  The diagonal tile runs the
//     same pipeline and zeroes the exponentials of keys after the query (key-in-tile > query-in-block).
//   * careful tiles (a row whose first tile is the diagonal one, and the redo pass): one 32-key sub-tile at a
//     time, exact running maximum, classic online softmax.
//   An item's tiles come in the order permuted tiles, own-segment tiles before the diagonal, diagonal tile, and
//   each kind has a loop of its own (see the loops): one tile body per loop keeps the accumulators in place.
#include "pbs_attn_tile.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations
#include <atomic>
#include <type_traits>

namespace {

struct AttnArgs {
  const uint16_t* q;
  const uint16_t* pk;    // (B*Hq, nb*128, 128)  permuted K
  const uint16_t* pvt;   // (B*Hq, nb, 128, 128) permuted V blocks, transposed
  const uint16_t* k;     // original K at the KV heads, caller's strides
  const uint16_t* v;     // original V at the KV heads, caller's strides
  const uint16_t* plist; // (B*Hq * npair, cap) merged visit lists
  int* queue;            // 8 work counters, one per XCD
  int cap;               // entries per list row (multiple of 8)
  uint16_t* o;
  int BH, Hq, Hkv, S, nb, bps;
  uint32_t k_ss, v_ss;   // key / value row strides in elements (< 2^22)
  int xcd_start[9];   // work items (head-major, long rows first) of XCD x: [xcd_start[x], xcd_start[x + 1])
  int interleave;     // 0, or 1 + log2(whole heads per XCD range) of a small launch whose tickets go pair-major (see ticket_item)
  int64_t q_sb, q_sh, q_ss, k_sb, k_sh, v_sb, v_sh, o_sb, o_sh, o_ss;
  float scale_log2;
};

typedef const __attribute__((address_space(4))) struct AttnArgs* ArgsPtr;

// ---- merged visit list of a pair of query blocks, built once per pass by its own kernel:
// row (bh * npair + pair) of `plist`: [0] = number of tiles, [1 ..] = entries kb | ENT_ORIG? | use_first << 14 |
// use_second << 15: the union of the two visit lists (ascending), then the own segments in ORIGINAL key order
// (blocks first-of-segment .. query block, shared where the two blocks share a segment).  Block 0 also clears
// the work counters of the attention kernel that follows on the stream.
constexpr int MERGE_THREADS = 256;
__global__ __launch_bounds__(MERGE_THREADS) void merge_pair_lists_kernel(const int32_t* __restrict__ cols, const int32_t* __restrict__ cnt,
                                                               uint16_t* __restrict__ plist, int* __restrict__ queue, int nb,
                                                               int bps, int cap, const uint8_t* __restrict__ own_needed) {
  __shared__ uint8_t flags0[4096], flags1[4096];
  __shared__ int wsum[MERGE_THREADS / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int npair = (nb + 1) >> 1;
  const int bh = blockIdx.x / npair, pair = blockIdx.x % npair;
  if (blockIdx.x == 0 && tid < 8) queue[tid] = 0;
  const bool second = 2 * pair + 1 < nb;
  const int32_t* l0 = cols + ((int64_t)bh * nb + 2 * pair) * nb;
  const int32_t* l1 = l0 + (second ? nb : 0);
  const int n0 = cnt[(int64_t)bh * nb + 2 * pair];
  const int n1 = second ? cnt[(int64_t)bh * nb + 2 * pair + 1] : 0;
  constexpr int MAX_PER = 4096 / MERGE_THREADS;
  int c0[MAX_PER], c1[MAX_PER];
#pragma unroll
  for (int u = 0; u < MAX_PER; ++u) {
    const int i = tid + MERGE_THREADS * u;
    c0[u] = i < n0 ? l0[i] : 0;
    c1[u] = i < n1 ? l1[i] : 0;
  }
  for (int i = tid; i < nb; i += MERGE_THREADS) {
    flags0[i] = 0;
    flags1[i] = 0;
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < MAX_PER; ++u) {
    const int i = tid + MERGE_THREADS * u;
    if (i < n0) flags0[c0[u]] = 1;
    if (i < n1) flags1[c1[u]] = 2;
  }
  __syncthreads();
  // compaction: thread t owns `per` consecutive key blocks; wave-level prefix, then wave totals
  const int per = (nb + MERGE_THREADS - 1) / MERGE_THREADS;
  const int k0 = tid * per, k1 = min(k0 + per, nb);
  int c = 0;
  for (int kb = k0; kb < k1; ++kb) c += (flags0[kb] | flags1[kb]) ? 1 : 0;
  int incl = c;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63) wsum[wave] = incl;
  __syncthreads();
  int w = incl - c, total = 0;
#pragma unroll
  for (int x = 0; x < MERGE_THREADS / 64; ++x) {
    const int ws = wsum[x];
    if (x < wave) w += ws;
    total += ws;
  }
  uint16_t* out = plist + (int64_t)blockIdx.x * cap;
  for (int kb = k0; kb < k1; ++kb) {
    const int f = flags0[kb] | flags1[kb];
    if (f) out[1 + w++] = (uint16_t)(kb | (f << 14));
  }
  const int qb0 = 2 * pair, qb1 = second ? qb0 + 1 : qb0;
  const int sf0 = (qb0 / bps) * bps, sf1 = (qb1 / bps) * bps;
  const int n_own = qb1 - sf0 + 1;
  if (own_needed) {
    // one-block segments with an optional diagonal: a query block's own block is listed only where its flag is set
    if (tid == 0) {
      int n = total;
      if (own_needed[(int64_t)bh * nb + qb0]) out[1 + n++] = (uint16_t)(qb0 | ENT_ORIG | (1u << 14));
      if (second && own_needed[(int64_t)bh * nb + qb1]) out[1 + n++] = (uint16_t)(qb1 | ENT_ORIG | (2u << 14));
      // every list ends with an own-segment entry: a pair with neither own block listed gets the first one's, used by
      // neither query block.  The attention kernel's item protocol -- first tile in flight, claim and hand-over of the
      // next item at the last tiles -- then needs no empty case and none where a permuted tile ends the item; a query
      // block that used no tile writes zeros
      if (n == total) out[1 + n++] = (uint16_t)(qb0 | ENT_ORIG);
      out[0] = (uint16_t)n;
    }
    return;
  }
  for (int t = tid; t < n_own; t += MERGE_THREADS) {
    const int kb = sf0 + t;
    const int f = (kb <= qb0 ? 1 : 0) | ((second && kb >= sf1) ? 2 : 0);
    out[1 + total + t] = (uint16_t)(kb | ENT_ORIG | (f << 14));
  }
  if (tid == 0) out[0] = (uint16_t)(total + n_own);
}

// Ticket t of the counter of a range of `count` items starting at `begin` -> work item.  Items are numbered head by
// head, long rows first, and normally handed out in that order (an XCD walks one head at a time: its workgroups
// share that head's K / V stream in L2).  A launch with only a few items per workgroup cannot balance that way: a
// workgroup that starts with a short item of one head is handed a long item of the next and finishes last.  There
// (`il` = 1 + log2 of the whole heads per range, a power of two) the same row pair of every head of the range goes
// out before the next shorter pair: longest items first across the range.
// Takes and returns begin + ticket (wave-uniform values: scalar arithmetic only); a ticket past the range is left alone.
__device__ __forceinline__ int ticket_item(int begin, int end, int item, int il, int npair) {
  if (il > 0 && item < end) {
    const int t = item - begin;
    item = begin + (t & ((1 << (il - 1)) - 1)) * npair + (t >> (il - 1));
  }
  return item;
}

// asynchronous copy of one list row (`chunks` 16-byte pieces) into LDS at byte offset `lds_byte`
__device__ __forceinline__ void stage_list_async(const uint16_t* src, int chunks, uint32_t lds_byte, int wave, int tid) {
  const uint64_t src0 = (uint64_t)(uintptr_t)src;
  const uint32_t src_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src0);
  const uint32_t src_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(src0 >> 32));
  const uint64_t srcu = ((uint64_t)src_hi << 32) | (uint64_t)src_lo;
  for (int p = 0; p * 512 < chunks; ++p) {
    const int chunk = p * 512 + tid;
    const uint32_t voff = (uint32_t)chunk * 16u;
    if (chunk < chunks) {
      register uint32_t m0v asm("m0") = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_byte + p * 8192 + wave * 1024));
      asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(voff), "s"(srcu) : "memory");
    }
  }
}

__global__ __launch_bounds__(512, 2) void sparse_attn_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // starts at LDS offset 0
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int grp = wave >> 2, wq = wave & 3;

  // Work items = (head, pair of query blocks), ordered head by head with the long rows of a head first and cut
  // into eight contiguous ranges of about equal work, one per XCD (blockIdx % 8): an XCD works through one
  // head at a time, so its resident workgroups walk the same permuted K/V stream at about the same pace and
  // share its tiles in that XCD's L2.  The launch holds one workgroup per CU; each takes the next item of its
  // XCD's range from a counter until the range is used up, so that the copies of an item's first tiles, the
  // fetch of its list and of its queries overlap the previous item's last tile and epilogue.
  // The arguments are read through the kernel-argument pointer where they are needed, and that pointer is made
  // opaque once per item: scalar loads from it stay next to their use instead of pinning some fifty scalar
  // registers for the whole kernel.
#define PBS_ARGS() ({ ArgsPtr p_ = (ArgsPtr)__builtin_amdgcn_kernarg_segment_ptr(); asm volatile("" : "+s"(p_)); p_; })
  ArgsPtr a0 = PBS_ARGS();
  const int npair = (a0->nb + 1) >> 1;
  const int xcd = blockIdx.x & 7;
  int q_begin = a0->xcd_start[xcd], q_end = a0->xcd_start[xcd + 1];   // the range being served: this XCD's, later others'
  int vic = xcd, vic_tried = 0;
  int* misc = reinterpret_cast<int*>(smem + LDS_MISC);   // [1] redo flag, [2] first item, [4] next item
  // the first item: from this XCD's range, or, when that one is empty or already handed out, from the next XCD's
  // range that still has items
  int cur;
  for (;;) {
    if (threadIdx.x == 0) {
      misc[2] = q_begin + atomicAdd(a0->queue + vic, 1);
      misc[1] = 0;
    }
    __syncthreads();
    cur = ticket_item(q_begin, q_end, __builtin_amdgcn_readfirstlane(misc[2]), a0->interleave, npair);
    if (cur < q_end) break;
    if (++vic_tried > 7) return;
    vic = (xcd + vic_tried) & 7;
    q_begin = a0->xcd_start[vic];
    q_end = a0->xcd_start[vic + 1];
    __syncthreads();   // everyone has read the ticket before the next one is written
  }
  int nxt = q_end;   // the next item is claimed late in the current one: an item claimed early waits for this
                     // workgroup while others may be idle
  bool has_nxt = false;
  const uint32_t use_bit = 1u << (14 + grp);

  // base pointers of one head's tiles: permuted K, permuted V^T, original K rows, original-order V^T
  struct HeadBase {
    const uint16_t *pk, *pvt, *korig, *vorig;
    uint32_t k_ss, v_ss;
    int S;
  };
  auto head_base = [&](ArgsPtr ap, int bh_e) __attribute__((always_inline)) {
    HeadBase hb;
    const int Hq_e = ap->Hq, Hkv_e = ap->Hkv, nb_e = ap->nb;
    const int b_e = bh_e / Hq_e, kvh = (bh_e % Hq_e) / (Hq_e / Hkv_e);
    hb.pk = ap->pk + (int64_t)bh_e * nb_e * BS * D;
    hb.pvt = ap->pvt + (int64_t)bh_e * nb_e * BS * D;
    hb.korig = ap->k + b_e * ap->k_sb + kvh * ap->k_sh;
    hb.vorig = ap->v + b_e * ap->v_sb + kvh * ap->v_sh;
    hb.k_ss = ap->k_ss;
    hb.v_ss = ap->v_ss;
    hb.S = ap->S;
    return hb;
  };
  // copy of one visit-list entry's K and V^T tiles into the buffers at LDS byte offset `buf`
  auto stage_entry = [&](const HeadBase& hb, uint32_t e, uint32_t buf, int lane, uint32_t lane_off) __attribute__((always_inline)) {
    const int kb_e = (int)(e & ENT_KB);
    if (PBS_UNLIKELY(e & ENT_ORIG)) {
      // the lane id is formed afresh: offsets derived from the item's one are loop invariants that get hoisted out of
      // the tile loop and, when registers run out there, spilled and reloaded per tile
      stage_krows_async(hb.korig + (int64_t)kb_e * BS * hb.k_ss, hb.k_ss, hb.S - kb_e * BS, buf, wave, lane_id_here());
      stage_vrows_async(hb.vorig + (int64_t)kb_e * BS * hb.v_ss, hb.v_ss, hb.S - kb_e * BS, LDS_V0 + buf, wave, lane_id_here());
    } else {
      // the first wave of every SIMD issues its own share and that of the SIMD's second wave (rows 16 further: the
      // same chunk, 4096 bytes on), which goes straight on to the matrix instructions of the current tile: the copy
      // instructions of a tile then queue behind the barrier in four waves instead of eight
      if (wave < 4) {
        const uint16_t* ks = hb.pk + (int64_t)kb_e * BS * D;
        const uint16_t* vs = hb.pvt + (int64_t)kb_e * BS * D;
        stage_tile_async(ks, buf, wave, lane_off ^ k_copy_xor(wave));
        stage_tile_async(ks, buf, wave + 4, (lane_off + 4096u) ^ k_copy_xor(wave + 4));
        stage_tile_async(vs, LDS_V0 + buf, wave, lane_off);
        stage_tile_async(vs, LDS_V0 + buf, wave + 4, lane_off + 4096u);
      }
    }
  };
  auto list_row = [&](ArgsPtr ap, int item) __attribute__((always_inline)) {
    const int bh_i = item / npair, pair_i = npair - 1 - item % npair;
    return ap->plist + ((int64_t)bh_i * npair + pair_i) * ap->cap;
  };

  // the first item's list, then its first tile
  stage_list_async(list_row(a0, cur), a0->cap >> 3, LDS_LIST, wave, (int)threadIdx.x);
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();
  uint32_t li = 0;        // which list buffer holds the current item's list
  uint32_t par = 0;       // which tile buffers hold the current item's first tile (0 or 0x8000)
  {
    stage_entry(head_base(a0, cur / npair), (uint32_t)__builtin_amdgcn_readfirstlane((int)reinterpret_cast<const uint16_t*>(smem + LDS_LIST)[1]), 0u,
                (int)threadIdx.x & 63, async_lane_offset(wave, (int)threadIdx.x & 63));
  }

  bool careful_only = false;   // the current pass repeats an item without speculation
  for (;;) {
    const uint16_t* mlist = reinterpret_cast<const uint16_t*>(smem + LDS_LIST + li * LIST_BYTES);
    const uint16_t* nlist = reinterpret_cast<const uint16_t*>(smem + LDS_LIST + (li ^ 1u) * LIST_BYTES);
    ArgsPtr ap = PBS_ARGS();
    // everything per lane is derived afresh from the lane id in every item: nothing but scalars lives across items
    const int lane = lane_id_here();
    const int tid = wave * 64 + lane;
    const int i16 = lane & 15, g4 = lane >> 4;
    // per-lane LDS byte offsets of the fragments inside buffer 0; XOR 0x8000 switches buffer.
    //   K fragment (sub-tile ks, row tile T, d-step kd) : (koff0 ^ kd << 6) + T * 1024 + ks * 8192
    //   V^T fragment (sub-tile ks, d tile dt)           : (voff0 ^ ks << 6) + dt * 4096
    // The 16-byte chunk index is XORed with a hash of the row, so the fragments of a row lie at (offset of the
    // first) ^ (n << 6).
    const int krow = 8 * (i16 >> 2) + (i16 & 3);   // k_row_hash(krow) == i16
    const uint32_t koff0 = (uint32_t)(krow * 256 + ((g4 ^ i16) * 16));
    const uint32_t voff0 = LDS_V0 + (uint32_t)(i16 * 256 + ((g4 ^ i16) * 16));
    // the addresses in the buffers of the item's first tile; switched to the other buffers after every tile
    uint32_t ka[4], va[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      ka[n] = koff0 ^ (uint32_t)(n << 6) ^ par;
      va[n] = voff0 ^ (uint32_t)(n << 6) ^ par;
    }
    const uint32_t lane_off = async_lane_offset(wave, lane);
    int claim = 0;   // ticket of the next item: in flight during one tile

    const int bh = cur / npair;
    const int pair = npair - 1 - cur % npair;
    const HeadBase hb = head_base(ap, bh);
    const int b = bh / ap->Hq, h = bh % ap->Hq;
    const int qb = 2 * pair + grp;
    const bool qb_valid = qb < ap->nb;
    const float c_log2 = ap->scale_log2;
    const int qpos = qb * BS + 32 * wq + i16;

    // Q^T fragments (B operand): query column 16 qg + i16, d = 32 kd + 8 g4 + 0..7.  Rows past the end of the
    // sequence compute on the last row's values and are never stored.
    bf16x8 qf[2][4];
#pragma unroll
    for (int qg = 0; qg < 2; ++qg) {
      const uint16_t* qrow = ap->q + b * ap->q_sb + h * ap->q_sh + (int64_t)min(qpos + 16 * qg, ap->S - 1) * ap->q_ss;
#pragma unroll
      for (int kd = 0; kd < 4; ++kd) qf[qg][kd] = *reinterpret_cast<const bf16x8*>(qrow + 32 * kd + 8 * g4);
    }
    const int n_tiles = __builtin_amdgcn_readfirstlane((int)mlist[0]);
    // the next item: claimed three tiles before the end of this one (the counter's latency passes under a
    // tile), published and its list and queries requested one tile later, its first tile requested at the last
    // tile.  Items of fewer than three tiles finish these steps after their loop.
    const int claim_it = careful_only ? -8 : max(n_tiles - 3, 0);
    auto publish_and_fetch = [&]() __attribute__((always_inline)) {   // between the wait for this thread's loads and the barrier ...
      if (wave == 0 && lane_id_here() == 0) misc[4] = q_begin + claim;
    };
    auto adopt_next = [&]() __attribute__((always_inline)) {          // ... and after the barrier
      nxt = ticket_item(q_begin, q_end, __builtin_amdgcn_readfirstlane(misc[4]), PBS_ARGS()->interleave, npair);
      has_nxt = nxt < q_end;
      if (has_nxt) {
        ArgsPtr an = PBS_ARGS();
        const int ln = lane_id_here();
        stage_list_async(list_row(an, nxt), an->cap >> 3, LDS_LIST + (li ^ 1u) * LIST_BYTES, wave, wave * 64 + ln);
        // the next item's queries are read once, from HBM: bring this wave's 32 rows into L2 now (copies into a
        // landing area nobody reads), so that the loads at the top of the item find them there
        const int bh_n = nxt / npair, qb_n = 2 * (npair - 1 - nxt % npair) + grp;
        const int pos0 = qb_n * BS + 32 * wq;
        if (pos0 + 32 <= an->S) {
          const int64_t q_ss = an->q_ss;
          const uint16_t* qn = an->q + (bh_n / an->Hq) * an->q_sb + (bh_n % an->Hq) * an->q_sh + (int64_t)pos0 * q_ss;
          const uint32_t voff = (uint32_t)((ln >> 4) * (uint32_t)q_ss * 2u + (ln & 15) * 16u);
#pragma unroll
          for (int n = 0; n < 8; ++n) {
            const uint64_t base = (uint64_t)(uintptr_t)(qn + 4 * n * q_ss);
            const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)base);
            const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(base >> 32));
            const uint64_t bu = ((uint64_t)b_hi << 32) | b_lo;
            register uint32_t m0v asm("m0") = (uint32_t)__builtin_amdgcn_readfirstlane((int)(LDS_DUMP + wave * 1024));
            asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(voff), "s"(bu) : "memory");
          }
        }
      }
    };

    {
      f32x4 o[8][2];   // [d tile][query column group]
      {
        float zero = 0.f;   // opaque: a constant zero vector would be kept (and spilled) as registers of its own
        asm volatile("" : "+v"(zero));
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
#pragma unroll
          for (int qg = 0; qg < 2; ++qg)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[dt][qg][r] = zero;
      }
      float m_ref[2] = {-INFINITY, -INFINITY};   // reference maxima of queries i16 and 16 + i16, identical in the four lanes i16 + 16 g
      float l_row[2] = {0.f, 0.f};               // row sums of queries i16 and 16 + i16, identical in the four lanes too
      bool first = true, poisoned = false;
      bool all_seen = false;     // every query of this wave has a finite reference maximum (wave-uniform)

      if (careful_only) {
        // the redo pass starts the item over: its first tile goes back into the buffers it had (the next
        // item's first tile, if it was on its way there, is fetched again at the end of this pass)
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        stage_entry(hb, (uint32_t)__builtin_amdgcn_readfirstlane((int)mlist[1]), par, lane, lane_off);
      }
      uint32_t bufx = par;
      auto next_buffers = [&]() __attribute__((always_inline)) {
        bufx ^= 0x8000u;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
          ka[n] ^= 0x8000u;
          va[n] ^= 0x8000u;
        }
      };
      // what every tile starts with: wait for its copies, hand over the buffers of the tile before, and request the
      // copies of the tile after it (or, at the last tile, of the next item's first tile)
      uint32_t e_cur = (uint32_t)__builtin_amdgcn_readfirstlane((int)mlist[1]);   // the entry of the current tile
      uint32_t e_nxt = 0;                                                        // of the next one, set by tile_head
      uint16_t e_ahead = mlist[2];                                               // per lane, not yet made uniform
      // `may_be_last`: the item's last tile is an own-segment tile (merge_pair_lists_kernel ends every list with one),
      // so the loop over the permuted tiles always has a next entry to request and carries no code for the next item's
      // first tile
      auto tile_head = [&](int it, auto may_be_last) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): this thread's share of tile `it` (and of the next list) has landed
        if (PBS_UNLIKELY(it == claim_it + 1)) publish_and_fetch();
        __syncthreads();                      // every share has; every wave is done with tile it - 1
        if (PBS_UNLIKELY(it == claim_it + 1)) adopt_next();
        if (PBS_UNLIKELY(it == claim_it) && wave == 0 && lane_id_here() == 0) claim = atomicAdd(PBS_ARGS()->queue + vic, 1);
        // the list entries are read from LDS one tile ahead of their use (the read's latency would otherwise sit in
        // front of the copy requests of every tile): `e_ahead` holds entry it + 1, requested at the tile before
        e_nxt = (uint32_t)__builtin_amdgcn_readfirstlane((int)e_ahead);
        e_ahead = mlist[3 + it];
        if (!decltype(may_be_last)::value || PBS_LIKELY(it + 1 < n_tiles))
          stage_entry(hb, e_nxt, bufx ^ 0x8000u, lane, lane_off);
        else if (has_nxt && (careful_only || n_tiles >= 3))   // shorter items: after the loop, once the list has landed
          stage_entry(head_base(PBS_ARGS(), nxt / npair), (uint32_t)__builtin_amdgcn_readfirstlane((int)nlist[1]), bufx ^ 0x8000u, lane, lane_off);
      };
      constexpr std::integral_constant<bool, true> any_tile{};
      constexpr std::integral_constant<bool, false> not_the_last{};
      // first tile of a row, every key visible: the exact maximum over its first 32 keys is a good enough reference
      // to start the pipelined path (later keys move it up lazily)
      auto first_reference = [&]() __attribute__((always_inline)) {
        first = false;
        float mx[2] = {-INFINITY, -INFINITY};
#pragma unroll
        for (int T = 0; T < 2; ++T) {
          f32x4 s0[2] = {(f32x4){0}, (f32x4){0}};
#pragma unroll
          for (int kd = 0; kd < 4; ++kd) {
            const bf16x8 fk = ldsf(ka[kd] + T * 1024);
#pragma unroll
            for (int qg = 0; qg < 2; ++qg) s0[qg] = PBS_MFMA(fk, qf[qg][kd], s0[qg]);
          }
#pragma unroll
          for (int qg = 0; qg < 2; ++qg)
#pragma unroll
            for (int r = 0; r < 4; ++r) mx[qg] = fmaxf(mx[qg], s0[qg][r]);
        }
#pragma unroll
        for (int qg = 0; qg < 2; ++qg) m_ref[qg] = max_over_lane_groups(mx[qg]) * c_log2;
        all_seen = true;
      };
      // careful tile: classic online softmax, one 32-key sub-tile at a time.  The redo pass, and a diagonal tile
      // while some query has not seen a single key yet (its reference maximum is still -inf)
      auto careful_tile = [&](uint32_t ent, bool masked) __attribute__((always_inline)) {
        first = false;
#pragma nounroll
        for (int ks = 0; ks < 4; ++ks) {   // a real loop: the rare path stays small, in code and in registers
          f32x4 s[2][2];   // [T][qg]
#pragma unroll
          for (int T = 0; T < 2; ++T) {
            s[T][0] = (f32x4){0};
            s[T][1] = (f32x4){0};
#pragma unroll
            for (int kd = 0; kd < 4; ++kd) {
              const bf16x8 fk = ldsf(ka[kd] + T * 1024 + ks * 8192);
#pragma unroll
              for (int qg = 0; qg < 2; ++qg) s[T][qg] = PBS_MFMA(fk, qf[qg][kd], s[T][qg]);
            }
          }
          if (masked) {
            const int ln = lane_id_here();   // keep the compares inside the tile (see fast_tile)
            const int qrel8 = 32 * wq + (ln & 15) - 8 * (ln >> 4);
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
              for (int qg = 0; qg < 2; ++qg)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  if (32 * ks + 4 * T + r - 16 * qg > qrel8) s[T][qg][r] = -INFINITY;
          }
          float alpha[2];
          bf16x8 pf[2];
#pragma unroll
          for (int qg = 0; qg < 2; ++qg) {
            float mx = fmaxf(fmaxf(s[0][qg][0], s[0][qg][1]), fmaxf(s[0][qg][2], s[0][qg][3]));
            mx = fmaxf(mx, fmaxf(fmaxf(s[1][qg][0], s[1][qg][1]), fmaxf(s[1][qg][2], s[1][qg][3])));
            mx = max_over_lane_groups(mx);
            const float m_new = fmaxf(m_ref[qg], mx * c_log2);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            alpha[qg] = __builtin_amdgcn_exp2f(m_ref[qg] - m_use);
            m_ref[qg] = m_new;
            float rs = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float pe = __builtin_amdgcn_exp2f(s[e >> 2][qg][e & 3] * c_log2 - m_use);
              rs += pe;
              pf[qg][e] = (__bf16)pe;
            }
            l_row[qg] = l_row[qg] * alpha[qg] + sum_over_lane_groups(rs);
          }
          if (__any(alpha[0] != 1.0f || alpha[1] != 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
#pragma unroll
              for (int qg = 0; qg < 2; ++qg)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[dt][qg][r] *= alpha[qg];
          }
#pragma unroll
          for (int dt = 0; dt < 8; ++dt) {
            const bf16x8 fv = (ent & ENT_ORIG)
                                  ? ldsf_transposed(vrow_lane_addr(LDS_V0 + (va[0] & 0x8000u), lane_id_here()) + dt * 128 + ks * 8192)
                                  : ldsf((va[0] ^ (uint32_t)(ks << 6)) + dt * 4096);
#pragma unroll
            for (int qg = 0; qg < 2; ++qg) o[dt][qg] = PBS_MFMA(fv, pf[qg], o[dt][qg]);
          }
        }
        all_seen = !__any(m_ref[0] == -INFINITY || m_ref[1] == -INFINITY);
      };
      // The merged list holds the permuted tiles of earlier segments first, then the tiles of the own segments in
      // ascending order: for a query block those before its own block, its own (diagonal) block, and -- for the first
      // block of a pair -- the second block's, which it skips.  Each kind has a loop of its own, and so has the redo
      // pass: a loop whose body updates the 64 accumulator registers on one path only keeps them in place, where
      // alternative tile bodies inside one loop cost a copy of all of them per tile (and the registers for it).
      int it = 0;
      if (PBS_UNLIKELY(careful_only)) {
        for (; it < n_tiles; ++it, next_buffers(), e_cur = e_nxt) {
          tile_head(it, any_tile);
          if (!(e_cur & use_bit) || !qb_valid) continue;
          careful_tile(e_cur, (e_cur & ENT_ORIG) && (int)(e_cur & ENT_KB) == qb);
        }
      } else {
        for (; it < n_tiles; ++it, next_buffers(), e_cur = e_nxt) {          // permuted tiles
          if (PBS_UNLIKELY(e_cur & ENT_ORIG)) break;
          tile_head(it, not_the_last);
          if (PBS_UNLIKELY(!(e_cur & use_bit) || !qb_valid)) continue;
          if (PBS_UNLIKELY(first)) first_reference();
          fast_tile<false, PREFETCH_SLOTS, false>(o, qf, ka, va, c_log2, m_ref, l_row, poisoned, wq);
        }
        for (; it < n_tiles; ++it, next_buffers(), e_cur = e_nxt) {          // own-segment tiles before the diagonal: every key visible
          if ((int)(e_cur & ENT_KB) >= qb) break;
          tile_head(it, any_tile);
          if (!(e_cur & use_bit) || !qb_valid) continue;
          if (first) first_reference();
          fast_tile<false, PREFETCH_SLOTS, true>(o, qf, ka, va, c_log2, m_ref, l_row, poisoned, wq);
        }
        if (it < n_tiles && (int)(e_cur & ENT_KB) == qb) {   // the diagonal tile
          tile_head(it, any_tile);
          if ((e_cur & use_bit) && qb_valid) {
            if (first || !all_seen) careful_tile(e_cur, true);
            else fast_tile<true, PREFETCH_SLOTS, true>(o, qf, ka, va, c_log2, m_ref, l_row, poisoned, wq);
          }
          ++it;
          next_buffers();
          e_cur = e_nxt;
        }
        for (; it < n_tiles; ++it, next_buffers(), e_cur = e_nxt) tile_head(it, any_tile);   // tiles of the pair's other block only
      }
      if (!careful_only && n_tiles < 3) {
        if (n_tiles < 2) {
          __builtin_amdgcn_s_waitcnt(0x0f70);
          publish_and_fetch();
          __syncthreads();
          adopt_next();
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        if (has_nxt)
          stage_entry(head_base(PBS_ARGS(), nxt / npair), (uint32_t)__builtin_amdgcn_readfirstlane((int)nlist[1]), bufx, lane, lane_off);
      }
      if (poisoned) misc[1] = 1;
      __syncthreads();   // every wave is done with the last tile
      if (!careful_only && misc[1] != 0) {   // the whole workgroup redoes both rows without speculation
        careful_only = true;
        continue;
      }

      // ---- epilogue: normalise, transpose through LDS (same swizzle), coalesced 16-byte stores.  The staging
      // area is the pair of buffers the last tile sat in (the other pair is receiving the next item's first
      // tile): its K buffer for the first query block, its V buffer for the second.
      // a query block that used no tile (no selected block and no own block: possible only with an optional diagonal)
      // has a zero sum and writes zeros, as the reference does for a row without selected blocks
      float inv[2];
#pragma unroll
      for (int qg = 0; qg < 2; ++qg) {
        const float l_all = l_row[qg];
        inv[qg] = l_all == 0.f ? 0.f : 1.0f / l_all;
      }
      // lane-dependent addresses of the epilogue come from a fresh opaque lane id: derived from the item's one
      // they would be computed at the top of the item and held across the tile loop
      const int lane_e = lane_id_here();
      const int i_e = lane_e & 15, g_e = lane_e >> 4;
      const uint32_t last_buf = par ^ (((n_tiles - 1) & 1) ? 0x8000u : 0u);
      uint16_t* os = reinterpret_cast<uint16_t*>(smem + last_buf + (grp ? LDS_V0 : 0u));
#pragma unroll
      for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int qg = 0; qg < 2; ++qg) {
          const int row = 32 * wq + 16 * qg + i_e;
          const int c = 2 * dt + (g_e >> 1);   // 16-byte chunk of d = 16 dt + 4 g + 0..3
          bf16x4 v4;
#pragma unroll
          for (int cc = 0; cc < 4; ++cc) v4[cc] = (__bf16)(o[dt][qg][cc] * inv[qg]);
          *reinterpret_cast<bf16x4*>(os + row * D + ((c ^ (row & 15)) * 8) + 4 * (g_e & 1)) = v4;
        }
      __syncthreads();
      if (qb_valid) {
        ArgsPtr ae = PBS_ARGS();
        const int bh_e = cur / npair;
        uint16_t* obase = ae->o + (bh_e / ae->Hq) * ae->o_sb + (bh_e % ae->Hq) * ae->o_sh;
        const int S_e = ae->S;
        const int64_t o_ss = ae->o_ss;
        // the query block index is rebuilt from the thread id here: keeping it alive across the tile loop
        // costs a register the loop does not have
        const int tid_e = wave * 64 + lane_e;
        const int qb_e = 2 * (npair - 1 - cur % npair) + (tid_e >> 8);
        const int t256 = tid_e & 255;
        const uint16_t* os_e = reinterpret_cast<const uint16_t*>(smem + last_buf + ((tid_e >> 8) ? LDS_V0 : 0u));
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          const int ci = t256 + 256 * n;
          const int row = ci >> 4, c = ci & 15;
          const int pos = qb_e * BS + row;
          if (pos < S_e)
            *reinterpret_cast<u32x4*>(obase + (int64_t)pos * o_ss + c * 8) =
                *reinterpret_cast<const u32x4*>(os_e + row * D + ((c ^ (row & 15)) * 8));
        }
      }
    }
    if (!has_nxt) {
      // the range is used up: serve the other XCDs' ranges, one after the other.  No look-ahead on this path:
      // claim, fetch the list, request the first tile, each after the other
      ArgsPtr as = PBS_ARGS();
      while (vic_tried < 7) {
        ++vic_tried;
        vic = (xcd + vic_tried) & 7;
        q_begin = as->xcd_start[vic];
        q_end = as->xcd_start[vic + 1];
        __syncthreads();   // everyone has read the previous ticket
        if (wave == 0 && lane_id_here() == 0) misc[4] = q_begin + atomicAdd(as->queue + vic, 1);
        __syncthreads();
        nxt = ticket_item(q_begin, q_end, __builtin_amdgcn_readfirstlane(misc[4]), as->interleave, npair);
        if (nxt < q_end) {
          has_nxt = true;
          break;
        }
      }
      if (has_nxt) {
        stage_list_async(list_row(as, nxt), as->cap >> 3, LDS_LIST + (li ^ 1u) * LIST_BYTES, wave, wave * 64 + lane_id_here());
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        stage_entry(head_base(as, nxt / npair), (uint32_t)__builtin_amdgcn_readfirstlane((int)nlist[1]),
                    par ^ ((n_tiles & 1) ? 0x8000u : 0u), lane, lane_off);
      }
    }
    if (!has_nxt) break;
    careful_only = false;
    par ^= (n_tiles & 1) ? 0x8000u : 0u;
    li ^= 1u;
    cur = nxt;
    nxt = q_end;
    has_nxt = false;
    if (wave == 0 && lane_id_here() == 0) misc[1] = 0;   // read by everyone before the epilogue's barrier, set again only after the next item's barriers
  }
}

std::atomic<uint64_t> g_lds_reserved{0};   // bit d: the kernel's LDS size has been raised on device d
std::atomic<int> g_cu_count[64];           // CUs of device d (0: not looked up yet)

}  // namespace

// entries per merged list row (a multiple of 8: rows stay 16-byte aligned): the count, at most nb blocks of
// earlier segments, at most bps + 1 own-segment blocks
static int list_cap(int nb, int bps) { return (1 + nb + std::min(bps, nb) + 1 + 7) / 8 * 8; }

// workspace: 256 bytes of work counters, then one merged visit list per pair of query blocks

extern "C" size_t pbs_sparse_attn_workspace_bytes(int B, int Hq, int S, int segment_size) {
  const int64_t nb = (S + BS - 1) / BS, npair = (nb + 1) / 2, cap = list_cap((int)nb, segment_size / BS);
  return 256 + (size_t)B * Hq * npair * cap * 2;
}

static int sparse_attn_launch(const void* q, const void* perm_k, const void* perm_vt, const void* k, const void* v,
                              const int32_t* csr_cols, const int32_t* csr_cnt, void* out, int B, int Hq, int Hkv, int S,
                              int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                              int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss, int64_t o_sb,
                              int64_t o_sh, int64_t o_ss, float softmax_scale, const uint8_t* own_block_needed, void* workspace,
                              void* stream);

extern "C" int pbs_sparse_attn_fwd(const void* q, const void* perm_k, const void* perm_vt, const void* k, const void* v,
                                   const int32_t* csr_cols, const int32_t* csr_cnt, void* out, int B, int Hq, int Hkv, int S,
                                   int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                   int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                   int64_t o_sb, int64_t o_sh, int64_t o_ss, float softmax_scale, void* workspace, void* stream) {
  return sparse_attn_launch(q, perm_k, perm_vt, k, v, csr_cols, csr_cnt, out, B, Hq, Hkv, S, head_dim, block_size, segment_size,
                            q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss, softmax_scale, nullptr,
                            workspace, stream);
}

extern "C" int pbs_sparse_attn_fwd_optional_diagonal(const void* q, const void* perm_k, const void* perm_vt, const void* k,
                                                     const void* v, const int32_t* csr_cols, const int32_t* csr_cnt,
                                                     const uint8_t* own_block_needed, void* out, int B, int Hq, int Hkv, int S,
                                                     int head_dim, int block_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                                     int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh,
                                                     int64_t v_ss, int64_t o_sb, int64_t o_sh, int64_t o_ss, float softmax_scale,
                                                     void* workspace, void* stream) {
  PBS_REQUIRE(own_block_needed, "pbs_sparse_attn_fwd_optional_diagonal: null own_block_needed");
  return sparse_attn_launch(q, perm_k, perm_vt, k, v, csr_cols, csr_cnt, out, B, Hq, Hkv, S, head_dim, block_size, block_size,
                            q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss, softmax_scale,
                            own_block_needed, workspace, stream);
}

static int sparse_attn_launch(const void* q, const void* perm_k, const void* perm_vt, const void* k, const void* v,
                              const int32_t* csr_cols, const int32_t* csr_cnt, void* out, int B, int Hq, int Hkv, int S,
                              int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                              int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss, int64_t o_sb,
                              int64_t o_sh, int64_t o_ss, float softmax_scale, const uint8_t* own_block_needed, void* workspace,
                              void* stream) {
  PBS_REQUIRE(q && perm_k && perm_vt && k && v && csr_cols && csr_cnt && out, "pbs_sparse_attn_fwd: null tensor pointer");
  PBS_REQUIRE(workspace && ((uintptr_t)workspace % 256) == 0, "pbs_sparse_attn_fwd: workspace must be a 256-byte aligned device buffer of pbs_sparse_attn_workspace_bytes()");
  PBS_REQUIRE(head_dim == D && block_size == BS, "pbs_sparse_attn_fwd: head_dim and block_size must be 128 (got %d, %d)", head_dim, block_size);
  PBS_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && S > 0, "pbs_sparse_attn_fwd: bad shape");
  PBS_REQUIRE(segment_size > 0 && segment_size % block_size == 0, "pbs_sparse_attn_fwd: segment_size must be a multiple of block_size");
  PBS_REQUIRE(segment_size / block_size <= 511, "pbs_sparse_attn_fwd: more than 511 blocks per segment");
  PBS_REQUIRE(q_sb % 8 == 0 && q_sh % 8 == 0 && q_ss % 8 == 0 && o_sb % 8 == 0 && o_sh % 8 == 0 && o_ss % 8 == 0 &&
                  k_sb % 8 == 0 && k_sh % 8 == 0 && k_ss % 8 == 0 && v_sb % 8 == 0 && v_sh % 8 == 0 && v_ss % 8 == 0,
              "pbs_sparse_attn_fwd: strides must keep rows 16-byte aligned");
  PBS_REQUIRE(k_ss >= D && k_ss < (1 << 22), "pbs_sparse_attn_fwd: key row stride %lld outside [128, 2^22)", (long long)k_ss);
  PBS_REQUIRE(v_ss >= D && v_ss < (1 << 22), "pbs_sparse_attn_fwd: value row stride %lld outside [128, 2^22)", (long long)v_ss);
  PBS_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)perm_k % 16) == 0 &&
                  ((uintptr_t)perm_vt % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0,
              "pbs_sparse_attn_fwd: pointers must be 16-byte aligned");
  AttnArgs a;
  a.q = (const uint16_t*)q; a.pk = (const uint16_t*)perm_k; a.pvt = (const uint16_t*)perm_vt;
  a.k = (const uint16_t*)k; a.v = (const uint16_t*)v;
  a.o = (uint16_t*)out;
  a.BH = B * Hq; a.Hq = Hq; a.Hkv = Hkv; a.S = S; a.nb = (S + BS - 1) / BS; a.bps = segment_size / block_size;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_ss = q_ss; a.k_sb = k_sb; a.k_sh = k_sh; a.k_ss = (uint32_t)k_ss; a.v_sb = v_sb; a.v_sh = v_sh; a.v_ss = (uint32_t)v_ss; a.o_sb = o_sb; a.o_sh = o_sh; a.o_ss = o_ss;
  a.scale_log2 = softmax_scale * 1.4426950408889634f;
  PBS_REQUIRE(a.nb <= 4096, "pbs_sparse_attn_fwd: more than 4096 blocks per sequence (%d)", a.nb);
  // eight ranges of equal estimated work: the row pair p of a head costs about p + 1 (causal length)
  const int64_t npair = (a.nb + 1) / 2;
  PBS_REQUIRE((int64_t)a.BH * npair < (1ll << 28), "pbs_sparse_attn_fwd: launch too large");
  const double head_work = 0.5 * (double)npair * (double)(npair + 1);
  int max_items = 0;
  for (int x = 0; x <= 8; ++x) {
    const double target = head_work * a.BH * x / 8.0;
    int64_t head = (int64_t)(target / head_work);
    if (head > a.BH) head = a.BH;
    const double rem = target - head * head_work;
    // items of a head in launch order are pairs npair - 1, npair - 2, ...: the first i of them cost
    // i * npair - i (i - 1) / 2
    int64_t lo = 0, hi = npair;
    while (lo < hi) {
      const int64_t mid = (lo + hi) / 2;
      if ((double)mid * npair - 0.5 * (double)mid * (mid - 1) >= rem - 1e-6) hi = mid; else lo = mid + 1;
    }
    int64_t start = head * npair + (head < a.BH ? lo : 0);
    if (x == 8) start = (int64_t)a.BH * npair;
    a.xcd_start[x] = (int)start;
    if (x > 0) max_items = std::max(max_items, a.xcd_start[x] - a.xcd_start[x - 1]);
  }
  // at most two items per workgroup and ranges of whole heads: hand the tickets out pair-major (see ticket_item;
  // with four and more items per workgroup the head-by-head order balances well enough and is 1-3 % faster)
  a.interleave = 0;
  const int nh = a.BH / 8;
  if (a.BH % 8 == 0 && (nh & (nh - 1)) == 0 && (int64_t)a.BH * npair <= (int64_t)2 * 256) {
    for (a.interleave = 1; (1 << (a.interleave - 1)) < nh; ++a.interleave) {}
    for (int x = 0; x <= 8; ++x) a.xcd_start[x] = (int)(x * (int64_t)nh * npair);
  }
  a.cap = list_cap(a.nb, a.bps);
  PBS_REQUIRE((uint32_t)a.cap * 2 <= LIST_BYTES, "pbs_sparse_attn_fwd: visit list too long");
  a.queue = (int*)workspace;
  a.plist = (const uint16_t*)((char*)workspace + 256);
  // the kernel's dynamic LDS size is raised once per device, not per call; the CU count is looked up once too
  int dev = 0;
  hipError_t attr = hipGetDevice(&dev);
  const bool tracked = attr == hipSuccess && dev >= 0 && dev < 64;
  int n_cu = tracked ? g_cu_count[dev].load(std::memory_order_relaxed) : 0;
  if (n_cu <= 0) {
    if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0) n_cu = 256;
    if (tracked) g_cu_count[dev].store(n_cu, std::memory_order_relaxed);
  }
  // one workgroup per CU (the kernel's LDS leaves room for one), a multiple of 8 so that every XCD gets its share;
  // fewer when there are fewer items
  const int64_t n_wg = std::min<int64_t>((int64_t)8 * max_items, (int64_t)(n_cu + 7) / 8 * 8);
  if (attr == hipSuccess && !(tracked && (g_lds_reserved.load(std::memory_order_acquire) >> dev & 1))) {
    if (const int rc = pbs_require_no_static_lds((const void*)sparse_attn_kernel, "pbs_sparse_attn_fwd")) return rc;
    attr = hipFuncSetAttribute((const void*)sparse_attn_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_TOTAL);
    if (attr == hipSuccess && tracked) g_lds_reserved.fetch_or(1ull << dev, std::memory_order_release);
  }
  if (attr != hipSuccess) {
    pbs_set_error("pbs_sparse_attn_fwd: cannot reserve %u bytes of LDS: %s", LDS_TOTAL, hipGetErrorString(attr));
    return (int)attr;
  }
  hipLaunchKernelGGL(merge_pair_lists_kernel, dim3((unsigned)(a.BH * npair)), dim3(MERGE_THREADS), 0, (hipStream_t)stream, csr_cols, csr_cnt,
                     (uint16_t*)((char*)workspace + 256), a.queue, a.nb, a.bps, a.cap, own_block_needed);
  hipLaunchKernelGGL(sparse_attn_kernel, dim3((unsigned)n_wg), dim3(512), LDS_TOTAL, (hipStream_t)stream, a);
  return pbs_check_launch("pbs_sparse_attn_fwd");
}
