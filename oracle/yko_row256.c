/* CPU oracle, part 3: the reference's own 256-channel row codec.  TEST INFRASTRUCTURE ONLY.
 *
 * These functions restate, operation for operation, the arithmetic the reference applies to a 256-channel K or V row:
 * the signed Walsh-Hadamard rotation, the flat int4 quantizer with one fp32 scale per row and MSB-first bit packing,
 * and the int8 row quantizer.  Every operation is a single IEEE fp32 add, subtract, multiply, divide or
 * round-to-nearest-even, in the order the reference performs it, so any correct implementation is bit-identical.
 */
#include "yko.h"
#include <math.h>
#include <string.h>

/* src/kvx_codec.cuh:28-32: sign of channel d from an integer hash of d+1 */
float yko_kvx_sign(int d) {
  uint32_t h = (uint32_t)d + 1u;
  h = (h ^ (h >> 16)) * 0x7feb352du;
  h = (h ^ (h >> 15)) * 0x846ca68bu;
  h ^= h >> 16;
  return (h & 1u) != 0u ? -1.f : 1.f;
}

/* src/kvx_codec.cuh:35-49: forward = signs, then 8 butterfly stages (h = 1..128; the element whose index has bit h set
 * becomes partner - self, the other self + partner), then x 1/16; inverse = the same butterflies and scale, signs last. */
void yko_kvx_rotate256(const float* x, float* y, int inverse) {
  float a[256], b[256];
  for (int d = 0; d < 256; ++d) a[d] = inverse ? x[d] : x[d] * yko_kvx_sign(d);
  for (int h = 1; h < 256; h *= 2) {
    for (int d = 0; d < 256; ++d) {
      const float self = a[d], other = a[d ^ h];
      b[d] = (d & h) ? other - self : self + other;
    }
    memcpy(a, b, sizeof a);
  }
  for (int d = 0; d < 256; ++d) {
    float v = a[d] * 0.0625f;
    if (inverse) v = v * yko_kvx_sign(d);
    y[d] = v;
  }
}

/* src/kvq_fast.cuh:194-198 (same arithmetic in src/kvq_gpu.cuh:85-86): am = max|r|, s7 = am / 7 (1 if 0),
 * q = clamp(rint(r / s7), -7, 7), field = q + 8, reconstruction q * s7.
 * Packing src/kvq_fast.cuh:226-233: field e occupies bits [4e, 4e+4) of an MSB-first stream of 32-bit words. */
void yko_flat4_encode256(const float* r, uint32_t* words32, float* scale, float* xq /* optional */) {
  float am = 0.f;
  for (int d = 0; d < 256; ++d) am = fmaxf(am, fabsf(r[d]));
  float s7 = am / 7.f;
  if (s7 == 0.f) s7 = 1.f;
  uint8_t fld[256];
  for (int d = 0; d < 256; ++d) {
    float q = rintf(r[d] / s7);
    q = fminf(fmaxf(q, -7.f), 7.f);
    fld[d] = (uint8_t)((int)q + 8);
    if (xq) xq[d] = q * s7;
  }
  for (int w = 0; w < 32; ++w) {
    uint32_t v = 0u;
    for (int i = 0; i < 32; ++i) {
      const int g = 32 * w + i, e = g / 4, jb = g - e * 4;
      v |= (((uint32_t)fld[e] >> (3 - jb)) & 1u) << (31 - i);
    }
    words32[w] = v;
  }
  *scale = s7;
}

/* src/kvq_attn.cuh:33-37,53-54: 4 bits at stream position 4d, (nib - 8) * s */
void yko_flat4_decode256(const uint32_t* words32, float scale, float* y) {
  for (int d = 0; d < 256; ++d) {
    const int pos = 4 * d, wi = pos >> 5, o = pos & 31;
    const uint64_t Z = ((uint64_t)words32[wi] << 32) | (uint64_t)((wi + 1 < 32) ? words32[wi + 1] : 0u);
    const int nib = (int)((Z >> (64 - o - 4)) & 15u);
    y[d] = (float)(nib - 8) * scale;
  }
}

/* src/kvx_codec.cuh:50-69 (integer mode): sc = max|x| / 127, q = sc > 0 ? rint(x / sc) : 0, clamped to +-127;
 * decode q * sc (src/kvx_probe.cu:15) */
void yko_int8_encode256(const float* x, int8_t* q, float* scale) {
  float am = 0.f;
  for (int d = 0; d < 256; ++d) am = fmaxf(am, fabsf(x[d]));
  const float sc = am / 127.f;
  for (int d = 0; d < 256; ++d) {
    int v = sc > 0.f ? (int)rintf(x[d] / sc) : 0;
    v = v < -127 ? -127 : (v > 127 ? 127 : v);
    q[d] = (int8_t)v;
  }
  *scale = sc;
}

/* The round trip of the reference's codec probe (src/kvx_probe.cu:7-20) for `rows` rows of 256 fp32 values:
 * [rotate] -> encode -> decode -> [inverse rotate].  mode 0: int8 rows (q8 [rows][256], words unused);
 * mode 1: flat int4 (words [rows][32], q8 unused). */
void yko_kvx_probe256(const float* x, int rows, int mode, int rot, int8_t* q8, uint32_t* words, float* scales, float* y) {
  for (int r = 0; r < rows; ++r) {
    float v[256], dq[256];
    if (rot) yko_kvx_rotate256(x + (size_t)r * 256, v, 0); else memcpy(v, x + (size_t)r * 256, sizeof v);
    if (mode == 0) {
      yko_int8_encode256(v, q8 + (size_t)r * 256, scales + r);
      for (int d = 0; d < 256; ++d) dq[d] = (float)q8[(size_t)r * 256 + d] * scales[r];
    } else {
      yko_flat4_encode256(v, words + (size_t)r * 32, scales + r, NULL);
      yko_flat4_decode256(words + (size_t)r * 32, scales[r], dq);
    }
    if (rot) yko_kvx_rotate256(dq, y + (size_t)r * 256, 1); else memcpy(y + (size_t)r * 256, dq, sizeof dq);
  }
}

/* ---- the step after attention for 256-channel heads (src/q35_kernels.cu:1420-1428, src/a8_prologue.cuh:87-98,122-133),
 *      with fp16 in the place of the reference's bf16 roundings ----
 * Per token and per pair of heads (512 consecutive values e = head * 256 + d):
 *   sg = f16(1 / (1 + expf(-gate)));  y2 = f16(y * sg);  u = y2 * sign[e]
 *   v  = f16(H512(u) * 2^-4.5)        (Sylvester Hadamard transform: stages h = 1 .. 256, the element whose index has bit h
 *                                      set becomes partner - self, the other self + partner; 0.0441941738... = 1/sqrt(512))
 *   alpha = max|v| / 127;  q = alpha > 0 ? rint(v / alpha) : 0, clamped to +-127
 * y16: attention outputs [M][n_heads][256] fp16 (already rotated back and rounded by the combiner); gate16 the same shape;
 * signs [n_heads * 256] (+1 / -1); qx [M][n_heads * 256] int8; alpha [M][n_heads * 256 / 512]. */
static float f16r_(float x) { return yko_h2f(yko_f2h(x)); }
void yko_attn_out256(const uint16_t* y16, const uint16_t* gate16, const int8_t* signs, int M, int n_heads, int8_t* qx, float* alpha) {
  const int N = n_heads * 256, nb = N / 512;
  for (int t = 0; t < M; ++t)
    for (int b = 0; b < nb; ++b) {
      float a[512], c[512];
      for (int i = 0; i < 512; ++i) {
        const size_t e = (size_t)t * N + (size_t)b * 512 + i;
        const float sg = f16r_(1.f / (1.f + expf(-yko_h2f(gate16[e]))));
        const float y2 = f16r_(yko_h2f(y16[e]) * sg);
        a[i] = y2 * (float)signs[b * 512 + i];
      }
      for (int h = 1; h < 512; h *= 2) {
        for (int i = 0; i < 512; ++i) { const float self = a[i], other = a[i ^ h]; c[i] = (i & h) ? other - self : self + other; }
        memcpy(a, c, sizeof a);
      }
      float am = 0.f;
      for (int i = 0; i < 512; ++i) { a[i] = f16r_(a[i] * 0.044194173824159216f); am = fmaxf(am, fabsf(a[i])); }
      const float al = am / 127.f;
      alpha[(size_t)t * nb + b] = al;
      for (int i = 0; i < 512; ++i) {
        int q = al > 0.f ? (int)rintf(a[i] / al) : 0;
        q = q < -127 ? -127 : (q > 127 ? 127 : q);
        qx[(size_t)t * N + (size_t)b * 512 + i] = (int8_t)q;
      }
    }
}
