/* Host check of pbs_attn_amd/csrc/pbs_div.h: for the divisor the block estimate uses, sqrt(128) rounded to float,
 * the three-instruction quotient equals the `/` operator for every bf16-representable dividend (all 65 536 bit
 * patterns, infinities included; NaN must stay NaN) of magnitude 2^-100 and more.  Below that the remainder step
 * underflows (it is 2^-23 of the quotient): there the two may differ by one unit in the last place of the quotient,
 * and zero quotients may differ in sign.
 * Exit status 0 and "ok <count>" on success, otherwise the first mismatches. */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <stdio.h>
#include <string.h>
#include "../../pbs_attn_amd/csrc/pbs_div.h"

int main(int argc, char** argv) {
  const int head_dim = argc > 1 ? atoi(argv[1]) : 128;
  const float b = (float)sqrt((double)head_dim);
  const float y = (float)(1.0 / (double)b);
  /* the reciprocal must be the correctly rounded one: its two float neighbours are further from 1 / b */
  const long double exact = 1.0L / (long double)b;
  const long double err = fabsl((long double)y - exact);
  if (fabsl((long double)nextafterf(y, 0.f) - exact) < err || fabsl((long double)nextafterf(y, 1.f) - exact) < err) {
    printf("reciprocal of %a is not correctly rounded\n", b);
    return 2;
  }
  int bad = 0, checked = 0;
  for (uint32_t hi = 0; hi < 65536u; ++hi) {
    const uint32_t bits = hi << 16;
    float x;
    memcpy(&x, &bits, 4);
    volatile float want = x / b;
    const float got = pbs_div_by_const(x, b, y);
    ++checked;
    if (isnan(want)) {
      if (!isnan(got)) ++bad;
      continue;
    }
    if (want == 0.f && got == 0.f) continue;
    if (fabsf(x) < 0x1p-100f) {
      if (got != want && got != nextafterf(want, INFINITY) && got != nextafterf(want, -INFINITY) && bad++ < 10)
        printf("x = %a: %a / b = %a, got %a (tiny)\n", x, x, want, got);
      continue;
    }
    if (memcmp((const void*)&want, &got, 4) != 0 && bad++ < 10) printf("x = %a: %a / b = %a, got %a\n", x, x, want, got);
  }
  if (bad) {
    printf("%d mismatches of %d\n", bad, checked);
    return 1;
  }
  printf("ok %d\n", checked);
  return 0;
}
