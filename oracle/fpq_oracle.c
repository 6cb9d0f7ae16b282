/*
 * fpq_oracle.c — plain-C restatement of the rotate + quantize path (TEST INFRASTRUCTURE, NOT
 * PRODUCT).  Written independently of oracle/fpq_oracle.py so that the two can be checked
 * against each other; only tests/ and bench.py's CPU-baseline leg may load it.
 *
 * Follows (paths relative to the reference checkout):
 *   rotation matrix  inference_lib/src/fp_quant/module/linear.py:24-30 (Sylvester, +-norm)
 *   abs-max scale    src/quantization/quantizer.py:107-112
 *   E8M0 scale       src/quantization/quantizer.py:162-165, quant_ops.py:82-94
 *   E4M3 scale       src/quantization/quantizer.py:143-160,168
 *   E2M1 RNE         src/quantization/quant_ops.py:57-68
 *   packing          src/quantization/quant_ops.py:31-40 (zero -> 0x8 under policy 0)
 *   stored bytes     src/quantization/rtn.py:187-188, quant_ops.py:111-118
 *
 * All arithmetic is IEEE binary32, round to nearest even, no contraction (-ffp-contract=off).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* in-place FWHT of g floats, butterfly strides 1, 2, ..., g/2 */
static void fwht(float* v, int g) {
  for (int s = 1; s < g; s <<= 1)
    for (int i = 0; i < g; ++i)
      if ((i & s) == 0) { float a = v[i], b = v[i + s]; v[i] = a + b; v[i + s] = a - b; }
}

static int e2m1_mag(float a) {
  if (a <= 0.25f) return 0;
  if (a < 0.75f) return 1;
  if (a <= 1.25f) return 2;
  if (a < 1.75f) return 3;
  if (a <= 2.5f) return 4;
  if (a < 3.5f) return 5;
  if (a <= 5.0f) return 6;
  return 7;
}

static int e2m1_code(float v, int zero_policy) {
  int mag = e2m1_mag(fabsf(v));
  int neg = zero_policy == 0 ? (v < 0.0f || mag == 0) : (int)(f32_bits(v) >> 31);
  return mag | (neg << 3);
}

/* fp32 -> float8_e4m3fn byte, RNE, subnormals to 2^-9, (448,464] -> 448, above -> 0x7f */
static int e4m3_encode(float t) {
  int sign = (int)(f32_bits(t) >> 24) & 0x80;
  float a = fabsf(t);
  int e, byte;
  if (!(a <= 464.0f)) return 0x7f | sign;
  if (a < 0.015625f) return (int)nearbyintf(a * 512.0f) | sign;
  float m = frexpf(a, &e);                 /* a = m * 2^e, 0.5 <= m < 1 */
  float k = nearbyintf(m * 16.0f);         /* 8..16: 1.mmm * 8 */
  if (k == 16.0f) { k = 8.0f; e += 1; }
  byte = ((e - 1 + 7) << 3) | ((int)k - 8);
  return byte | sign;
}

static float e4m3_decode(int byte) {
  int mag = byte & 0x7f;
  float v = mag < 8 ? (float)mag * 0.001953125f : ldexpf(1.0f + (float)(mag & 7) / 8.0f, (mag >> 3) - 7);
  return (byte & 0x80) ? -v : v;
}

/* fp32 >= 0 -> float8_e8m0fnu byte: nearest power of two, halves up, < 2^-127 -> 0 */
static int e8m0_encode(float t) {
  uint32_t b = f32_bits(t), ex = (b >> 23) & 0xff, man = b & 0x7fffff;
  if (ex == 0) return man >= 0x600000 ? 1 : 0;
  int byte = (int)ex + (man >= 0x400000 ? 1 : 0);
  return byte > 255 ? 255 : byte;
}

/* rot: 0 hadamard, 1 identity.  fmt: 0 MXFP4 (group 32), 1 NVFP4 (group 16). */
int fpq_oracle_quantize(const uint16_t* x, long rows, long cols, int fmt, int rot, int g, float norm,
                        float global_scale, int zero_policy, uint8_t* codes, uint8_t* scales) {
  const int group = fmt == 0 ? 32 : 16;
  if (rot == 1) g = group;
  if (cols % g || cols % group) return -2;
  const float rg = global_scale == 0.0f ? 0.0f : 1.0f / global_scale;
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r) {
    float row[128];
    for (long c0 = 0; c0 < cols; c0 += g) {
      for (int i = 0; i < g; ++i) row[i] = bf16_to_f32(x[r * cols + c0 + i]);
      if (rot == 0) {
        for (int i = 0; i < g; ++i) row[i] = row[i] * norm;
        fwht(row, g);
      }
      for (int g0 = 0; g0 < g; g0 += group) {
        float a = 0.0f, s;
        int byte, zero = 0;
        for (int i = 0; i < group; ++i) a = fmaxf(a, fabsf(row[g0 + i]));
        float sc0 = (a * 2.0f) / 12.0f;
        if (fmt == 0) {
          float arg = sc0 * 6.0f;
          if (!(arg >= 1.17549435e-38f)) arg = 1.17549435e-38f;
          int e;
          (void)frexpf(arg, &e);
          e -= 1;
          if (e > 127) e = 127;
          s = ldexpf(1.0f, e - 2) / 0.75f;
          byte = e8m0_encode(s * 3.0f);
        } else {
          float t = sc0 * global_scale;
          if (t > 448.0f) t = 448.0f;
          if (t < -448.0f) t = -448.0f;
          s = e4m3_decode(e4m3_encode(t)) * rg;
          zero = s == 0.0f;
          byte = zero ? 0 : e4m3_encode(s * global_scale);
          if (zero) s = 1.0f;
        }
        scales[r * (cols / group) + (c0 + g0) / group] = (uint8_t)byte;
        for (int i = 0; i < group; i += 2) {
          float v0 = zero ? 0.0f : row[g0 + i] / s, v1 = zero ? 0.0f : row[g0 + i + 1] / s;
          codes[(r * cols + c0 + g0 + i) / 2] = (uint8_t)(e2m1_code(v0, zero_policy) | (e2m1_code(v1, zero_policy) << 4));
        }
      }
    }
  }
  return 0;
}
