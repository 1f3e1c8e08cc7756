/*
 * TEST INFRASTRUCTURE ONLY -- CPU checker for the OCP FP8 E4M3FN byte codec and the per-token
 * KV-cache quantizer.  Nothing in the product path (tileops_amd/) may load or call this file.
 *
 * What it restates:
 *   - OCP "FP8 Formats for Deep Learning" E4M3FN: 1 sign, 4 exponent (bias 7), 3 mantissa bits,
 *     no infinities, NaN = S.1111.111, max finite 448, subnormals m * 2^-9.  This is the format
 *     torch.float8_e4m3fn implements and gfx950's v_cvt_*_fp8 converts (gfx942 used the "fnuz" variant).
 *   - the per-token quantizer of the reference workload
 *     (workloads/fp8_quant.py:27-33, src/tileops/kernels/fp8_quant.py:44-60,
 *      workloads/gqa_fp8_utils.py:11-17):
 *        amax  = max(|x| over the last dim), clamped below at 1e-4
 *        scale = amax / 448                      (fp32)
 *        q     = fp8( clamp(x / scale, -448, 448) )   round-to-nearest-even
 *   - the dequant convention  x' = float(q) * scale  (tests/ops/attention/test_gqa_fp8.py:216-219).
 *
 * Pinned by tests/test_oracle_fp8.py: exhaustive 256-code decode against torch.float8_e4m3fn,
 * encode on a dense grid (every fp32 halfway point between adjacent codes and both neighbours)
 * against torch's cast, and decode(encode(x)) idempotence.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* Decode one E4M3FN byte to fp32 (exact). */
float fp8_e4m3fn_decode(uint8_t b) {
  int sign = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) return NAN;
  if (e == 0) v = ldexpf((float)m, -9);                 /* subnormal: m/8 * 2^-6 */
  else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return sign ? -v : v;
}

/* Encode fp32 to E4M3FN, round-to-nearest-even, NOT saturating: |x| that rounds above 448 -> NaN
 * (0x7F | sign), like torch's cast.  Callers that want saturation clamp first, as the reference does. */
uint8_t fp8_e4m3fn_encode(float x) {
  uint32_t bits;
  memcpy(&bits, &x, 4);
  uint8_t sign = (uint8_t)((bits >> 24) & 0x80);
  float a = fabsf(x);
  if (!(a == a)) return sign | 0x7F;          /* NaN */
  if (isinf(a)) return sign | 0x7F;
  /* 464 is the midpoint between 448 (even mantissa) and the NaN slot at 480: the tie itself rounds to 448,
   * anything above it rounds into the NaN slot; both fall out of the general path below. */
  if (a < ldexpf(1.0f, -10)) return sign;     /* below half of the smallest subnormal (2^-9) -> 0 ; tie at 2^-10 -> even (0) */
  int e;
  (void)frexpf(a, &e);                        /* a = f * 2^e, f in [0.5,1) -> unbiased exponent e-1 */
  int ue = e - 1;
  if (ue < -6) ue = -6;                       /* subnormal range shares the exponent of the smallest normal */
  /* quantum = 2^(ue-3); q = a / quantum, rounded to nearest even integer */
  float q = ldexpf(a, 3 - ue);
  float r = nearbyintf(q);                    /* default rounding mode: to nearest even */
  int qi = (int)r;
  if (ue == -6 && qi < 8) return sign | (uint8_t)qi;          /* subnormal (or zero) */
  if (qi == 16) { qi = 8; ue += 1; }                           /* mantissa overflow */
  int be = ue + 7;
  if (be > 15 || (be == 15 && qi - 8 == 7)) return sign | 0x7F;
  return sign | (uint8_t)((be << 3) | (qi - 8));
}

void fp8_e4m3fn_decode_n(const uint8_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; i++) dst[i] = fp8_e4m3fn_decode(src[i]);
}

void fp8_e4m3fn_encode_n(const float* src, uint8_t* dst, int64_t n) {
  for (int64_t i = 0; i < n; i++) dst[i] = fp8_e4m3fn_encode(src[i]);
}

/* Per-token quantizer: x is [rows, dim] fp32; writes q [rows, dim] bytes and scale [rows] fp32. */
void fp8_quant_per_token(const float* x, uint8_t* q, float* scale, int64_t rows, int64_t dim) {
  for (int64_t r = 0; r < rows; r++) {
    const float* xr = x + r * dim;
    float amax = 0.0f;
    for (int64_t j = 0; j < dim; j++) {
      float a = fabsf(xr[j]);
      if (a > amax) amax = a;
    }
    if (amax < 1e-4f) amax = 1e-4f;
    float s = amax / 448.0f;
    scale[r] = s;
    for (int64_t j = 0; j < dim; j++) {
      float t = xr[j] / s;
      if (t > 448.0f) t = 448.0f;
      if (t < -448.0f) t = -448.0f;
      q[r * dim + j] = fp8_e4m3fn_encode(t);
    }
  }
}
