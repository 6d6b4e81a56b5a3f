// Division of a float by a constant in three instructions, with the quotient IEEE division gives.
//
//   q0 = x * y              y = the divisor's reciprocal, correctly rounded
//   e  = fma(-q0, b, x)     the remainder of the first guess, exact
//   q  = fma(e, y, q0)
// With a correctly rounded reciprocal and round-to-nearest, q is the correctly rounded x / b whenever nothing
// underflows or overflows on the way (Markstein's theorem); a compiler's own division costs about ten instructions
// (scaling for the whole exponent range, a hardware reciprocal, refinement, fix-up).  The block estimate divides
// bf16-rounded dot products by sqrt(head_dim): only 65 536 possible dividends, and tests/c_abi/div_check.c goes
// through all of them on the host -- this file is plain C as well -- and compares with the `/` operator: equal for
// every dividend of magnitude 2^-100 and more.  Infinite dividends keep their quotient.  Below 2^-100 the remainder
// underflows and the quotient may be one unit in the last place off, and a zero quotient may differ in its sign: logits
// of 1e-30, whose exponentials no such difference reaches.
#pragma once

#ifdef __HIP__
#define PBS_DIV_FN __host__ __device__ __forceinline__
#else
#define PBS_DIV_FN static inline
#endif

PBS_DIV_FN float pbs_div_by_const(float x, float b, float y) {
  const float q0 = x * y;
  const float e = __builtin_fmaf(-q0, b, x);
  const float q = __builtin_fmaf(e, y, q0);
  return __builtin_isinf(q0) ? q0 : q;
}
