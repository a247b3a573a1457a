/* CPU oracle, codec part.  TEST INFRASTRUCTURE ONLY - see yko.h.
 * Compile with -ffp-contract=off: the reference library is built with --fmad=false
 * (CMakeLists.txt:60-63), so no product is ever fused into an add. */
#include "yko.h"
#include <math.h>
#include <string.h>

/* ---------- fp16 <-> fp32 (reference: src/a8_prologue.cuh:36-38 wrap __half2float / __float2half_rn) ---------- */
float yko_h2f(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) u = sign;
    else { /* subnormal: value = man * 2^-24; normalise */
      int e = -1; uint32_t m = man;
      do { ++e; m <<= 1; } while ((m & 0x400u) == 0);
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (exp == 31) u = sign | 0x7f800000u | (man << 13);
  else u = sign | ((exp + 112u) << 23) | (man << 13);
  float f; memcpy(&f, &u, 4); return f;
}

uint16_t yko_f2h(float f) {
  uint32_t u; memcpy(&u, &f, 4);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (a > 0x7f800000u ? 0x200u | ((a >> 13) & 0x3ffu) : 0u)); /* inf / nan */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* >= 65520 rounds to inf */
  if (a < 0x33000001u) return (uint16_t)sign;                        /* <= 2^-25 rounds to zero (2^-25 is a tie -> even = 0) */
  const int e = (int)(a >> 23) - 127;                                /* unbiased exponent */
  uint32_t m = (a & 0x7fffffu) | 0x800000u;                          /* 24-bit significand */
  int shift;                                                         /* bits to drop */
  uint32_t base;
  if (e >= -14) { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }   /* normal: hidden bit goes into the exponent */
  else { shift = 13 + (-14 - e); base = 0; }                         /* subnormal: keep the hidden bit */
  const uint32_t kept = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
  uint32_t r = base + kept;
  if (rem > half || (rem == half && (kept & 1u))) ++r;               /* nearest even; a carry walks into the exponent correctly */
  return (uint16_t)(sign | r);
}

/* ---------- flat symmetric int4, group of 32 ----------
 * Reference arithmetic (src/kvq_fast.cuh:194-198, same in src/kvq_gpu.cuh:86):
 *   am = max|r|; s7 = am / 7 (IEEE divide); if (s7 == 0) s7 = 1;
 *   q = clamp(rintf(r / s7), -7, 7); field = q + 8; decoded value = q * s7.
 * Frozen choices where the measured format differs from the reference's row-256 / fp32-scale form:
 *   - the scale is stored as fp16; the encoder divides by the STORED (rounded) scale, as the reference divides by
 *     the scale it stores, so dequantization error is what the encoder minimised.  Rounding can push |r / s|
 *     slightly above 7: the clamp is live.
 *   - the zero guard applies to the stored scale: if the fp16 scale is 0 (all-zero group or underflow) it is 1.0.
 * Inputs must be finite. */
void yko_quant_group32(const uint16_t* x16, uint8_t* codes16, uint16_t* scale16) {
  float xf[YKO_GROUP], am = 0.f;
  for (int i = 0; i < YKO_GROUP; ++i) { xf[i] = yko_h2f(x16[i]); const float a = fabsf(xf[i]); if (a > am) am = a; }
  const float s32 = am / 7.0f;
  uint16_t s16 = yko_f2h(s32);
  if ((s16 & 0x7fffu) == 0) s16 = 0x3c00u;
  const float sd = yko_h2f(s16);
  uint8_t f[YKO_GROUP];
  for (int i = 0; i < YKO_GROUP; ++i) {
    float q = rintf(xf[i] / sd);               /* default rounding mode: nearest even */
    q = fminf(fmaxf(q, -7.f), 7.f);
    f[i] = (uint8_t)((int)q + 8);
  }
  yko_pack_nibbles(f, YKO_GROUP, codes16);
  *scale16 = s16;
}

/* decode: (nib - 8) * s, a product that is exact in fp32 (src/kvq_attn.cuh:52-54) */
void yko_dequant_group32(const uint8_t* codes16, uint16_t scale16, float* y32) {
  const float sd = yko_h2f(scale16);
  for (int j = 0; j < YKO_GROUP / 2; ++j) {
    y32[2 * j] = (float)((int)(codes16[j] & 15) - 8) * sd;
    y32[2 * j + 1] = (float)((int)(codes16[j] >> 4) - 8) * sd;
  }
}

/* two fields per byte, even index in the low nibble (src/post_kernels.cu:77-80) */
void yko_pack_nibbles(const uint8_t* fields, int n, uint8_t* bytes) {
  for (int j = 0; j < n / 2; ++j) bytes[j] = (uint8_t)((fields[2 * j] & 15) | ((fields[2 * j + 1] & 15) << 4));
}
void yko_unpack_nibbles(const uint8_t* bytes, int n, uint8_t* fields) {
  for (int j = 0; j < n / 2; ++j) { fields[2 * j] = bytes[j] & 15; fields[2 * j + 1] = bytes[j] >> 4; }
}

void yko_quant_rows(const uint16_t* x16, int rows, int dim, uint8_t* codes, uint16_t* scales) {
  const int ng = dim / YKO_GROUP;
  for (long r = 0; r < rows; ++r)
    for (int g = 0; g < ng; ++g)
      yko_quant_group32(x16 + r * dim + g * YKO_GROUP, codes + r * (dim / 2) + g * (YKO_GROUP / 2), scales + r * ng + g);
}
void yko_dequant_rows(const uint8_t* codes, const uint16_t* scales, int rows, int dim, float* y) {
  const int ng = dim / YKO_GROUP;
  for (long r = 0; r < rows; ++r)
    for (int g = 0; g < ng; ++g)
      yko_dequant_group32(codes + r * (dim / 2) + g * (YKO_GROUP / 2), scales[r * ng + g], y + r * dim + g * YKO_GROUP);
}

/* rows pos..pos+M-1 of every KV head are (over)written before any row of the pass is read
 * (src/engine35.cpp:911-913; row index src/q35_kernels.cu:42) */
void yko_cache_row(const yko_cache* c, int isv, size_t row, float* out) {
  const int D = c->head_dim;
  if (c->fmt == 1) {
    const uint32_t* words = (const uint32_t*)(isv ? c->vc : c->kc) + row * 32;
    yko_flat4_decode256(words, ((const float*)(isv ? c->vs : c->ks))[row], out);
  } else {
    const int ng = D / YKO_GROUP;
    yko_dequant_rows((isv ? c->vc : c->kc) + row * (D / 2), (isv ? c->vs : c->ks) + row * ng, 1, D, out);
  }
}

void yko_append(yko_cache* c, const uint16_t* k16, const uint16_t* v16, int M, int pos) {
  const int D = c->head_dim, ng = D / YKO_GROUP, KVH = c->n_kv_heads;
  for (int t = 0; t < M; ++t)
    for (int h = 0; h < KVH; ++h) {
      const size_t row = (size_t)h * c->max_ctx + (size_t)(pos + t);
      const size_t src = ((size_t)t * KVH + h) * D;
      if (c->fmt == 1) {                 /* D == 256: the reference's row codec on the fp32 value of every fp16 input */
        float x[256];
        for (int isv = 0; isv < 2; ++isv) {
          const uint16_t* s16 = (isv ? v16 : k16) + src;
          for (int d = 0; d < 256; ++d) x[d] = yko_h2f(s16[d]);
          yko_flat4_encode256(x, (uint32_t*)(isv ? c->vc : c->kc) + row * 32, (float*)(isv ? c->vs : c->ks) + row, NULL);
        }
        continue;
      }
      yko_quant_rows(k16 + src, 1, D, c->kc + row * (D / 2), c->ks + row * ng);
      yko_quant_rows(v16 + src, 1, D, c->vc + row * (D / 2), c->vs + row * ng);
    }
}
