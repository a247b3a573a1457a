/* CPU oracle, trellis-coded KV rows (the reference's KV4 / KV5 row formats).  TEST INFRASTRUCTURE ONLY.
 *
 * A row of 256 fp32 values is coded against a profile blob ("KVQP" v1, parsed as src/engine35.cpp:48-52 and
 * src/kvq_fast.hpp:52-76 do).  Per group g = (layer * 4 + kv head) * 2 + (0 K | 1 V) the blob names: mode (0 trellis,
 * 1 flat int4), kk bits per element, a table index, a guard position, m <= 2 directions U (fp16) that are projected
 * out, and an optional mean row mu (fp16).  Reference forms: src/kvq_gpu.cuh:51-147 (one row, one block),
 * src/kvq_fast.cuh:63-233 (production: one block per row x multiplier x chunk, then a select-and-pack block per row).
 * Both compute the same values in the same order; this file follows them:
 *
 *   r = y - mu; for j < m: c_j = f16(sum(r * u_j)), r -= c_j * u_j; rms = sqrt(sum(r * r) / 256), 0 -> 1.
 *   sums over 256 elements: inside each run of 32 the butterfly a[i] += a[i ^ o], o = 16 .. 1, then the 8 run sums are
 *   added in order starting from 0 (tbf_sum, src/kvq_fast.cuh:31-40).
 *   trellis (mode 0): for every multiplier mi: s = f16(rms * mult[mi]), 0 -> 1; xi = clamp(rint(r / s * 256), +-2048);
 *   each chunk of 64 elements is a path through 256 states that starts in state 0; state after element t is
 *   ((previous << kk) | field) & 255, its value ci[state]; integer cost sum (xi - ci)^2; among equal costs the smaller
 *   predecessor and the smaller final state win (src/kvq_fast.cuh:113-141).  The multiplier with the smallest squared
 *   error (summed as above over (r - (ci/256 * gain) * s)^2, first wins ties) is kept; the row stores the low kk bits
 *   of every state, s, and (c_0, c_1) as two fp16.
 *   flat (mode 1): the row quantizer of yko_flat4_encode256 on r (src/kvq_fast.cuh:194-198).
 *   words: element e occupies bits [kb * e, kb * e + kb) of an MSB-first stream of 32-bit words (src/kvq_fast.cuh:226-233).
 *   decode: src/kvq_attn.cuh:46-75 - the state of element e is the last 8 bits of the stream up to the end of its field,
 *   cut at the start of its chunk.
 */
#include "yko.h"
#include <math.h>
#include <string.h>

static unsigned u16_at(const uint8_t* p) { return (unsigned)p[0] | ((unsigned)p[1] << 8); }
static unsigned u32_at(const uint8_t* p) { return u16_at(p) | (u16_at(p + 2) << 16); }
static float f32_at(const uint8_t* p) { const unsigned u = u32_at(p); float f; memcpy(&f, &u, 4); return f; }
static float f16r(float v) { return yko_h2f(yko_f2h(v)); }

int yko_tb_check_blob(const uint8_t* b, size_t n) {
  if (n < 100 || memcmp(b, "KVQP", 4) != 0 || u16_at(b + 4) != 1 || u32_at(b + 8) != n) return -1;
  if (u16_at(b + 16) != 256) return -2;
  const unsigned nm = u16_at(b + 24), ngrp = u32_at(b + 28), off_m = u32_at(b + 32), off_t = u32_at(b + 36), off_g = u32_at(b + 40), nt = u16_at(b + 22);
  if (nm < 1 || nm > 16 || off_m + 4 * nm > n || off_t + 4 * nt > n || off_g + 4 * (size_t)ngrp > n) return -3;
  for (unsigned t = 0; t < nt; ++t) {
    const size_t to = u32_at(b + off_t + 4 * t);
    if (to + 12 + 512 > n || b[to] != 8 || b[to + 2] != 64 || b[to + 3] != 8) return -4;
  }
  for (unsigned g = 0; g < ngrp; ++g) {
    const size_t go = u32_at(b + off_g + 4 * g);
    if (go + 8 > n) return -5;
    const size_t need = go + 8 + (b[go + 5] ? 512 : 0) + 512 * (size_t)b[go + 4];
    if (need > n || b[go + 4] > 2 || b[go] > 1) return -5;
    if (b[go] == 0 && (b[go + 1] < 3 || b[go + 1] > 5 || b[go + 2] >= nt)) return -6;
  }
  return 0;
}

int yko_tb_group(const uint8_t* b, int g, int* fields6) {
  if ((unsigned)g >= u32_at(b + 28)) return -1;
  const size_t go = u32_at(b + u32_at(b + 40) + 4 * (size_t)g);
  for (int i = 0; i < 6; ++i) fields6[i] = b[go + i];      /* mode, kk, table, guard, m, has_mu */
  return 0;
}

static float sum256(const float* v) {
  float t = 0.f;
  for (int w = 0; w < 8; ++w) {
    float a[32], c[32];
    memcpy(a, v + 32 * w, sizeof a);
    for (int o = 16; o; o >>= 1) {
      for (int i = 0; i < 32; ++i) c[i] = a[i] + a[i ^ o];
      memcpy(a, c, sizeof a);
    }
    t = t + a[0];
  }
  return t;
}

/* One chunk of T elements through the 256-state trellis.  states[t] = state after element t; returns the path cost. */
int yko_tb_viterbi(const int* xi, int T, const int16_t* ci, int kk, uint8_t* states) {
  const int Kq = 1 << kk, UU = 256 >> kk;
  static _Thread_local uint8_t bp[64][256];
  int cost[2][256];
  for (int d = 0; d < 256; ++d) cost[0][d] = d ? 0x40000000 : 0;
  for (int t = 0; t < T; ++t) {
    const int* cp = cost[t & 1];
    int* cn = cost[(t + 1) & 1];
    for (int d = 0; d < 256; ++d) {
      const int u = d >> kk;
      int mn = cp[u], jb = 0;
      for (int j = 1; j < Kq; ++j) { const int cc = cp[j * UU + u]; if (cc < mn) { mn = cc; jb = j; } }
      const int dx = xi[t] - ci[d];
      cn[d] = dx * dx + mn;
      bp[t][d] = (uint8_t)jb;
    }
  }
  const int* cf = cost[T & 1];
  int st = 0;
  for (int d = 1; d < 256; ++d) if (cf[d] < cf[st]) st = d;
  const int total = cf[st];
  for (int t = T - 1; t >= 0; --t) {
    states[t] = (uint8_t)st;
    st = (bp[t][st] << (8 - kk)) | (st >> kk);
  }
  return total;
}

static float cdec(int ci, float gain) { return ((float)ci * 0.00390625f) * gain; }

/* y[256] -> x[256] (what the row decodes to), fields[256], scale, pc (two fp16), best multiplier.
 * Returns 0 if the row stays as it is (group out of range, or pos below the guard), 1 if it was coded. */
int yko_tb_encode_row(const uint8_t* b, int g, int pos, const float* y, float* x, uint8_t* fields, float* scale, uint32_t* pc_out, int* best_mi) {
  memcpy(x, y, 256 * sizeof(float));
  memset(fields, 0, 256); *scale = 1.f; *pc_out = 0; *best_mi = -1;
  if ((unsigned)g >= u32_at(b + 28)) return 0;
  const unsigned off_m = u32_at(b + 32), off_t = u32_at(b + 36), off_g = u32_at(b + 40);
  const int nm = (int)u16_at(b + 24);
  const size_t go = u32_at(b + off_g + 4 * (size_t)g);
  const int mode = b[go], kk = b[go + 1], tix = b[go + 2], guard = b[go + 3], m = b[go + 4], has_mu = b[go + 5];
  if (pos < guard) return 0;
  const uint8_t* mup = b + go + 8;
  const uint8_t* Up = mup + (has_mu ? 512 : 0);
  float r[256], mud[256], uj[2][256], cj[2] = {0.f, 0.f}, tmp[256];
  for (int d = 0; d < 256; ++d) { mud[d] = has_mu ? yko_h2f((uint16_t)u16_at(mup + 2 * d)) : 0.f; r[d] = has_mu ? y[d] - mud[d] : y[d]; }
  for (int j = 0; j < m; ++j) {
    for (int d = 0; d < 256; ++d) { uj[j][d] = yko_h2f((uint16_t)u16_at(Up + 2 * (j * 256 + d))); tmp[d] = r[d] * uj[j][d]; }
    cj[j] = f16r(sum256(tmp));
    for (int d = 0; d < 256; ++d) r[d] = r[d] - cj[j] * uj[j][d];
  }
  for (int d = 0; d < 256; ++d) tmp[d] = r[d] * r[d];
  float rms = sqrtf(sum256(tmp) / 256.f);
  if (rms == 0.f) rms = 1.f;
  float xq[256];
  if (mode == 1) {
    float am = 0.f;
    for (int d = 0; d < 256; ++d) am = fmaxf(am, fabsf(r[d]));
    float s7 = am / 7.f; if (s7 == 0.f) s7 = 1.f;
    for (int d = 0; d < 256; ++d) {
      float q = rintf(r[d] / s7); q = fminf(fmaxf(q, -7.f), 7.f);
      xq[d] = q * s7; fields[d] = (uint8_t)((int)q + 8);
    }
    *scale = s7;
  } else {
    const size_t to = u32_at(b + off_t + 4 * (size_t)tix);
    const float gain = f32_at(b + to + 4);
    int16_t ci[256];
    for (int d = 0; d < 256; ++d) ci[d] = (int16_t)u16_at(b + to + 12 + 2 * d);
    float best_e = 0.f; int have = 0;
    uint8_t st[256], best_st[256]; float best_s = 1.f;
    for (int mi = 0; mi < nm; ++mi) {
      float s = f16r(rms * f32_at(b + off_m + 4 * (size_t)mi)); if (s == 0.f) s = 1.f;
      int xi[256];
      for (int d = 0; d < 256; ++d) { const float t = rintf((r[d] / s) * 256.f); xi[d] = (int)fminf(fmaxf(t, -2048.f), 2048.f); }
      for (int c = 0; c < 4; ++c) yko_tb_viterbi(xi + 64 * c, 64, ci, kk, st + 64 * c);
      for (int d = 0; d < 256; ++d) { const float dd = r[d] - cdec(ci[st[d]], gain) * s; tmp[d] = dd * dd; }
      const float e = sum256(tmp);
      if (!have || e < best_e) { have = 1; best_e = e; *best_mi = mi; best_s = s; memcpy(best_st, st, 256); }
    }
    for (int d = 0; d < 256; ++d) { xq[d] = cdec(ci[best_st[d]], gain) * best_s; fields[d] = (uint8_t)(best_st[d] & ((1 << kk) - 1)); }
    *scale = best_s;
  }
  for (int d = 0; d < 256; ++d) {
    float v = xq[d];
    for (int j = 0; j < m; ++j) v = v + cj[j] * uj[j][d];
    if (has_mu) v = v + mud[d];
    x[d] = v;
  }
  *pc_out = (uint32_t)yko_f2h(cj[0]) | ((uint32_t)yko_f2h(cj[1]) << 16);
  return 1;
}

void yko_tb_pack(const uint8_t* fields, int kb, uint32_t* words) {
  memset(words, 0, 8 * (size_t)kb * 4);
  for (int e = 0; e < 256; ++e)
    for (int j = 0; j < kb; ++j) {
      const int bit = kb * e + j;
      words[bit >> 5] |= (((uint32_t)fields[e] >> (kb - 1 - j)) & 1u) << (31 - (bit & 31));
    }
}

static unsigned stream_bits(const uint32_t* w, int nwords, int pos, int n) {
  unsigned v = 0;
  for (int i = 0; i < n; ++i) { const int bit = pos + i; const unsigned x = (bit >> 5) < nwords ? (w[bit >> 5] >> (31 - (bit & 31))) & 1u : 0u; v = (v << 1) | x; }
  return v;
}

/* words (8 * kb) + scale + pc -> y[256]; the group's mode decides the meaning of the fields */
int yko_tb_decode_row(const uint8_t* b, int g, const uint32_t* words, float scale, uint32_t pc, float* y) {
  if ((unsigned)g >= u32_at(b + 28)) return -1;
  const size_t go = u32_at(b + u32_at(b + 40) + 4 * (size_t)g);
  const int mode = b[go], kk = b[go + 1], tix = b[go + 2], m = b[go + 4], has_mu = b[go + 5];
  const int kb = mode == 1 ? 4 : kk;
  const uint8_t* mup = b + go + 8;
  const uint8_t* Up = mup + (has_mu ? 512 : 0);
  const size_t to = mode == 0 ? u32_at(b + u32_at(b + 36) + 4 * (size_t)tix) : 0;
  for (int d = 0; d < 256; ++d) {
    float xq;
    if (mode == 1) xq = (float)((int)stream_bits(words, 8 * kb, 4 * d, 4) - 8) * scale;
    else {
      const int endb = kb * (d + 1), first = kb * (d & ~63), lo = endb - 8 > first ? endb - 8 : first;
      const unsigned state = stream_bits(words, 8 * kb, lo, endb - lo);
      xq = cdec((int16_t)u16_at(b + to + 12 + 2 * state), f32_at(b + to + 4)) * scale;
    }
    float x = xq;
    if (m > 0) x = x + yko_h2f((uint16_t)(pc & 0xffffu)) * yko_h2f((uint16_t)u16_at(Up + 2 * d));
    if (m > 1) x = x + yko_h2f((uint16_t)(pc >> 16)) * yko_h2f((uint16_t)u16_at(Up + 2 * (256 + d)));
    if (has_mu) x = x + yko_h2f((uint16_t)u16_at(mup + 2 * d));
    y[d] = x;
  }
  return 0;
}

/* rows [n][256] with group and position per row -> coded rows; OpenMP over rows */
void yko_tb_encode_rows(const uint8_t* b, const int* grp, const int* pos, int n, const float* y, float* x, uint32_t* words, int stride_words,
                        float* scale, uint32_t* pc, int* best_mi, int* coded) {
#pragma omp parallel for schedule(dynamic, 1)
  for (int i = 0; i < n; ++i) {
    uint8_t fields[256];
    int f6[6] = {0, 4, 0, 0, 0, 0};
    coded[i] = yko_tb_encode_row(b, grp[i], pos[i], y + 256 * (size_t)i, x + 256 * (size_t)i, fields, scale + i, pc + i, best_mi + i);
    memset(words + (size_t)i * stride_words, 0, 4 * (size_t)stride_words);
    if (coded[i] && yko_tb_group(b, grp[i], f6) == 0) yko_tb_pack(fields, f6[0] == 1 ? 4 : f6[1], words + (size_t)i * stride_words);
  }
}
