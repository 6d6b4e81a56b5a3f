/* Declarations of the bench-only probe library (libpbs_probe.so).  It is not part of the operator's ABI: bench.py
 * loads it to report what the matrix pipe and the attention kernel's tile pipeline sustain by themselves. */
#pragma once
#ifdef __cplusplus
extern "C" {
#endif

/* A loop of matrix instructions only: per wave `iters` x 16 v_mfma_f32_16x16x32_bf16 (the attention kernel's) or,
 * shape_32x32x16 != 0, `iters` x 8 v_mfma_f32_32x32x16_bf16 (the same FLOP), on
 * 256 workgroups of 8 waves, operands taken from `operands` (65536 bf16 values of the caller's choice: the
 * sustained rate depends on the values).  `sink` takes 256 * 512 floats, `clocks` (two 64-bit counters the
 * caller zeroes) accumulates shader-clock and 100 MHz ticks over the workgroups; time the launch with
 * events.  pbs_mfma_probe_flop gives the FLOP count of one launch. */
int pbs_mfma_probe(const void* operands, int iters, int shape_32x32x16, float* sink, unsigned long long* clocks, void* stream);
double pbs_mfma_probe_flop(int iters);

/* the attention kernel's tile pipeline alone.  256
 * workgroups of 8 waves each run `iters` unmasked 128-key tiles for their 256 queries (2 x 128 x 128 block pairs
 * per workgroup and tile, 8.389 MFLOP each) out of LDS, with the kernel's barrier per tile and, if `with_copies`,
 * its asynchronous copies of the next tile (64 KB from a ring of `n_src_tiles` >= 2 K / V^T tile pairs of 65536
 * bytes each at `tiles`, whose first 32 KB also serve as the queries; the workgroups of an XCD copy the same tile at
 * the same step, as the kernel's share a head's stream in their L2) -- no visit lists, no write-out.  `sink`
 * takes 256 * 512 floats; `clocks` receives workgroup 0's shader-clock ticks and 100 MHz ticks.  `with_copies`
 * bit 1 handles the tiles as a tile of the query block's own segment is handled: K and V copied row by row, the V
 * fragments formed by transposing reads.  Time the launch
 * with events: the same cycles per tile on every input, but on data the clock drops with the power limit. */
int pbs_attn_tile_probe(const void* tiles, int n_src_tiles, int iters, int with_copies, float* sink,
                        unsigned long long* clocks, void* stream);

#ifdef __cplusplus
}
#endif
