/* Exhaustive host check of the two-operation quotient the quantize kernels use on their fast path
 * (fp-quant_amd/csrc/fpq_device.h: scale_element, mx_group_scale, nv_group_scale, div6_rn;
 * fp-quant_amd/csrc/fpq_quantize.hip: kKappa).
 *
 * The reference rounds the IEEE quotient, cast_to_fp4(x / scales) (src/quantization/quant_ops.py:57-71).
 * The kernels compute q = fma(x, k1, x * k2) with k1 = RN(1/s), k2 = RN(fma(-s, k1, 1) / s).  q is
 * not always RN(x / s); what must hold is that q and RN(x / s) have the same E2M1 code for every x.
 * A code can only differ where x / s is within a few ulp of one of the seven decision points
 * T = 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5, so for every divisor mantissa (2^23 of them; powers of two
 * scale every quantity exactly inside the exponent range the kernels accept) all x within 8 ulp of
 * s * T are compared, and the largest distance between q and the quotient seen anywhere is
 * reported: it must stay well inside those 8 ulp.
 *
 *   part "nv":   arbitrary s (NVFP4: E4M3 value times fl(1/global_scale))
 *   part "mx":   s = 2^k * fl(4/3), k1 = 0.75, k2 = -1.5 * 2^-26, every x in [0.1, 16)
 *   part "div6": RN(a / 6) by Markstein's correction, and fl(fl(2a)/12) == RN(a/6), every mantissa
 *
 * Prints one line per part; exit status 0 if nothing differs.  Build: gcc -O2 -mfma -ffp-contract=off
 * -fopenmp (fmaf must be a true fused multiply-add; the program checks that first).
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* E2M1 magnitude index of round-to-nearest-even, as cast_to_fp4 writes it */
static inline int code(float v) {
  const float a = fabsf(v);
  if (a <= 0.25f) return 0;
  if (a < 0.75f) return 1;
  if (a <= 1.25f) return 2;
  if (a < 1.75f) return 3;
  if (a <= 2.5f) return 4;
  if (a < 3.5f) return 5;
  if (a <= 5.0f) return 6;
  return 7;
}

int main(void) {
  /* fmaf must not round twice: 2^-24 survives only in a fused operation */
  volatile float one_plus = 1.0f + 0x1p-23f, minus_one = -1.0f;
  if (fmaf(one_plus, one_plus, minus_one) != 0x1p-22f + 0x1p-46f) { printf("fmaf is not fused\n"); return 2; }

  const float T[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
  long bad_nv = 0, n_nv = 0;
  int worst_nv = 0;
#pragma omp parallel for reduction(+ : bad_nv, n_nv) reduction(max : worst_nv) schedule(static)
  for (uint32_t m = 0; m < (1u << 23); ++m) {
    const float s = u2f(0x3f800000u | m);
    const float k1 = 1.0f / s;
    const float k2 = fmaf(-s, k1, 1.0f) / s;
    for (int i = 0; i < 7; ++i) {
      const uint32_t u0 = f2u(s * T[i]);
      for (int d = -8; d <= 8; ++d) {
        const float x = u2f(u0 + d);
        const float want = x / s, got = fmaf(x, k1, x * k2);
        int dist = (int)f2u(got) - (int)f2u(want);
        dist = dist < 0 ? -dist : dist;
        worst_nv = dist > worst_nv ? dist : worst_nv;
        bad_nv += code(got) != code(want);
        ++n_nv;
      }
    }
  }
  printf("nv: %ld comparisons, %ld code mismatches, largest distance to the IEEE quotient %d ulp\n", n_nv, bad_nv,
         worst_nv);

  const float c = 1.0f / 0.75f; /* fl(4/3), the mantissa of every MXFP4 working scale */
  const float kappa = -0x1.8p-26f;
  long bad_mx = 0, n_mx = 0;
  int worst_mx = 0;
  const uint32_t lo = f2u(0.1f), hi = f2u(16.0f);
#pragma omp parallel for reduction(+ : bad_mx, n_mx) reduction(max : worst_mx) schedule(static)
  for (uint32_t u = lo; u < hi; ++u) {
    const float x = u2f(u);
    const float want = x / c, got = fmaf(x, 0.75f, x * kappa);
    int dist = (int)f2u(got) - (int)f2u(want);
    dist = dist < 0 ? -dist : dist;
    worst_mx = dist > worst_mx ? dist : worst_mx;
    bad_mx += code(got) != code(want);
    ++n_mx;
  }
  printf("mx: %ld comparisons, %ld code mismatches, largest distance to the IEEE quotient %d ulp\n", n_mx, bad_mx,
         worst_mx);
  /* below 0.1 both quotients are under 0.25 (code 0), from 16 on both exceed 5 (code 7) */
  const int ends_ok = code(0.1f / c) == 0 && code(fmaf(0.1f, 0.75f, 0.1f * kappa)) == 0 && code(16.0f / c) == 7 &&
                      code(fmaf(16.0f, 0.75f, 16.0f * kappa)) == 7;

  const float c6 = 1.0f / 6.0f;
  long bad_div6 = 0, bad_12 = 0;
#pragma omp parallel for reduction(+ : bad_div6, bad_12) schedule(static)
  for (uint32_t m = 0; m < (1u << 24); ++m) {
    const float a = u2f(0x3f000000u + m); /* [0.5, 2): every mantissa in two binades */
    const float q = a * c6;
    const float q1 = fmaf(fmaf(-q, 6.0f, a), c6, q);
    bad_div6 += q1 != a / 6.0f;
    bad_12 += (a * 2.0f) / 12.0f != a / 6.0f;
  }
  printf("div6: %ld wrong Markstein quotients, %ld differences between fl(fl(2a)/12) and RN(a/6)\n", bad_div6, bad_12);
  return (bad_nv || bad_mx || bad_div6 || bad_12 || !ends_ok || worst_nv > 2 || worst_mx > 2) ? 1 : 0;
}
