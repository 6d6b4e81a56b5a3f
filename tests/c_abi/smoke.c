/* The library used from plain C, without Python or torch: one whole PBS prefill pass through
 * pbs_prefill_attn_fwd on device buffers from hipMalloc, checked against a float attention computed on
 * the host.  With every candidate block selected (threshold_is_int_one) the result must be plain causal
 * attention whatever the key permutation; with threshold 0.9 it must at least be finite and change
 * nothing else.  Also checks that argument errors come back as codes with a message. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "pbs_hip.h"

#define CHECK_HIP(x)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (x);                                                               \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "%s failed: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__); \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)

static uint16_t f2bf(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float bf2f(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t rng_state = 12345u;
static float rnd(void) { /* roughly N(0,1): sum of 4 uniforms */
  float s = 0.f;
  for (int i = 0; i < 4; ++i) {
    rng_state = rng_state * 1664525u + 1013904223u;
    s += (float)(rng_state >> 8) / 16777216.0f;
  }
  return (s - 2.0f) * 1.7320508f;
}

int main(void) {
  const int B = 1, Hq = 2, Hkv = 1, S = 700, D = 128, BS = 128, SEG = 256;
  const size_t nq = (size_t)B * Hq * S * D, nk = (size_t)B * Hkv * S * D;
  uint16_t *hq = malloc(nq * 2), *hk = malloc(nk * 2), *hv = malloc(nk * 2), *ho = malloc(nq * 2);
  for (size_t i = 0; i < nq; ++i) hq[i] = f2bf(rnd());
  for (size_t i = 0; i < nk; ++i) hk[i] = f2bf(rnd());
  for (size_t i = 0; i < nk; ++i) hv[i] = f2bf(rnd());

  if (pbs_abi_version() != 1) { fprintf(stderr, "unexpected ABI version\n"); return 1; }
  /* argument errors: a code and a message, no launch */
  if (pbs_prefill_attn_fwd(NULL, NULL, NULL, NULL, B, Hq, Hkv, S, D, BS, SEG, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0.9f, NULL,
                           0, 1, 0, 0, 0.0883883f, NULL, 0, NULL) >= 0 || strlen(pbs_last_error()) == 0) {
    fprintf(stderr, "null pointers were not rejected\n");
    return 1;
  }

  void *dq, *dk, *dv, *dout, *ws;
  CHECK_HIP(hipMalloc(&dq, nq * 2));
  CHECK_HIP(hipMalloc(&dk, nk * 2));
  CHECK_HIP(hipMalloc(&dv, nk * 2));
  CHECK_HIP(hipMalloc(&dout, nq * 2));
  CHECK_HIP(hipMemcpy(dq, hq, nq * 2, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dk, hk, nk * 2, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dv, hv, nk * 2, hipMemcpyHostToDevice));
  const size_t ws_bytes = pbs_prefill_attn_workspace_bytes(B, Hq, Hkv, S, D, BS, SEG);
  if (ws_bytes == 0) { fprintf(stderr, "workspace query failed\n"); return 1; }
  CHECK_HIP(hipMalloc(&ws, ws_bytes));
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  const int64_t sb_q = (int64_t)Hq * S * D, sb_k = (int64_t)Hkv * S * D, sh = (int64_t)S * D, ss = D;
  const float scale = 1.0f / sqrtf((float)D);

  for (int pass = 0; pass < 2; ++pass) {
    const int int_one = pass == 0;
    int rc = pbs_prefill_attn_fwd(dq, dk, dv, dout, B, Hq, Hkv, S, D, BS, SEG, sb_q, sh, ss, sb_k, sh, ss, sb_k, sh, ss, sb_q,
                                  sh, ss, 0.9f, NULL, int_one, 1, 0, 0, scale, ws, ws_bytes, stream);
    if (rc != 0) { fprintf(stderr, "pbs_prefill_attn_fwd: %d %s\n", rc, pbs_last_error()); return 1; }
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipMemcpy(ho, dout, nq * 2, hipMemcpyDeviceToHost));
    double max_err = 0.0, sum_err = 0.0;
    float *p = malloc((size_t)S * sizeof(float));
    for (int h = 0; h < Hq; ++h)
      for (int i = 0; i < S; ++i) {
        const uint16_t* qi = hq + ((size_t)h * S + i) * D;
        float mx = -INFINITY, l = 0.f;
        for (int j = 0; j <= i; ++j) {
          const uint16_t* kj = hk + (size_t)j * D; /* Hkv = 1 */
          float s = 0.f;
          for (int d = 0; d < D; ++d) s += bf2f(qi[d]) * bf2f(kj[d]);
          p[j] = s * scale;
          if (p[j] > mx) mx = p[j];
        }
        for (int j = 0; j <= i; ++j) { p[j] = expf(p[j] - mx); l += p[j]; }
        for (int d = 0; d < D; ++d) {
          float o = 0.f;
          for (int j = 0; j <= i; ++j) o += p[j] * bf2f(hv[(size_t)j * D + d]);
          o /= l;
          const float got = bf2f(ho[((size_t)h * S + i) * D + d]);
          if (!isfinite(got)) { fprintf(stderr, "non-finite output\n"); return 1; }
          if (int_one) {
            const double e = fabs((double)got - (double)o);
            if (e > max_err) max_err = e;
            sum_err += e;
          }
        }
      }
    free(p);
    if (int_one) {
      const double mean_err = sum_err / (double)nq;
      printf("every block selected vs host causal attention: max-abs %.4g mean-abs %.4g\n", max_err, mean_err);
      if (max_err > 2e-2 || mean_err > 2e-3) { fprintf(stderr, "outside the tolerance\n"); return 1; }
    }
  }
  printf("c_abi_smoke ok\n");
  return 0;
}
