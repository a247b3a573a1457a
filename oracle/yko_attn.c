/* CPU oracle, attention part.  TEST INFRASTRUCTURE ONLY - see yko.h.
 * Compile with -ffp-contract=off (the reference is built with --fmad=false, CMakeLists.txt:60-63). */
#include "yko.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define YKO_MAXD 256

static inline int row_len(int pos, const uint8_t* depth, int t) { return pos + (depth ? (int)depth[t] : t) + 1; }
/* split policy of the packed kernels: 31 splits below 4096 keys, else 42 (src/q35_atxpk.cu:404-409, src/engine35.hpp:434-439) */
static inline int ref_splits(int len) { return len < 4096 ? 31 : 42; }

/* dot product with a fixed summation order: 16 strided partial sums, then a pairwise tree.
 * (The reference sums lane-strided partials and then butterflies them, src/attention_kv4q.cu:126-141;
 * any fixed order is within 1e-6 relative of any other, far inside the comparison tolerance.) */
static inline float dot16(const float* a, const float* b, int D) {
  float p[16];
  for (int j = 0; j < 16; ++j) p[j] = a[j] * b[j];
  for (int d = 16; d < D; d += 16)
    for (int j = 0; j < 16; ++j) p[j] = p[j] + a[d + j] * b[d + j];
  for (int w = 8; w; w >>= 1)
    for (int j = 0; j < w; ++j) p[j] = p[j] + p[j + w];
  return p[0];
}

/* One (kv head, split): stream the split's keys once, update every row of the window that sees the key.
 * Online softmax exactly as attn_softmax7 (src/attention_kv4q.cu:19-31): one exp per key,
 *   mn = max(m, s); e = exp(min(m,s) - mn); a = s > m ? e : 1; b = s > m ? 1 : e; l = l*a + b; acc = acc*a + b*v. */
static void split_task(const yko_cache* c, const float* qf /* [M][NH][D], pre-scaled */, int M, int pos, const uint8_t* depth,
                       int kvh, int split, int splits_arg, int Smax, float* pm, float* pl, float* pacc) {
  const int D = c->head_dim, NH = c->n_heads, G = NH / c->n_kv_heads;
  int lo_all = 0x7fffffff, hi_all = 0;
  int* lo = (int*)malloc(sizeof(int) * 2 * (size_t)M);
  int* hi = lo + M;
  for (int t = 0; t < M; ++t) {
    const int len = row_len(pos, depth, t), S = splits_arg > 0 ? splits_arg : ref_splits(len);
    const int per = (len + S - 1) / S;
    lo[t] = split * per; hi[t] = lo[t] + per < len ? lo[t] + per : len;
    if (split >= S || hi[t] < lo[t]) hi[t] = lo[t];
    if (hi[t] > lo[t]) { if (lo[t] < lo_all) lo_all = lo[t]; if (hi[t] > hi_all) hi_all = hi[t]; }
    for (int i = 0; i < G; ++i) {
      const size_t p = ((size_t)t * Smax + split) * NH + kvh * G + i;
      pm[p] = -1e30f; pl[p] = 0.f; memset(pacc + p * D, 0, sizeof(float) * D);
    }
  }
  float kd[YKO_MAXD], vd[YKO_MAXD];
  for (int key = lo_all; key < hi_all; ++key) {
    const size_t row = (size_t)kvh * c->max_ctx + key;
    yko_cache_row(c, 0, row, kd);
    yko_cache_row(c, 1, row, vd);
    for (int t = 0; t < M; ++t) {
      if (key < lo[t] || key >= hi[t]) continue;
      for (int i = 0; i < G; ++i) {
        const int head = kvh * G + i;
        const size_t p = ((size_t)t * Smax + split) * NH + head;
        const float s = dot16(qf + ((size_t)t * NH + head) * D, kd, D);
        const float m = pm[p], mn = fmaxf(m, s);
        const int gt = s > m;
        const float e = expf((gt ? m : s) - mn), a = gt ? e : 1.f, b = gt ? 1.f : e;
        pl[p] = pl[p] * a + b; pm[p] = mn;
        float* acc = pacc + p * D;
        for (int d = 0; d < D; ++d) acc[d] = acc[d] * a + b * vd[d];
      }
    }
  }
  free(lo);
}

/* combiner (src/attention_kv4q.cu:325-332; same algebra src/q35_kernels.cu:1412-1416):
 *   M2 = max_s pm; w_s = pm > -1e29 ? exp(pm - M2) : 0; L = sum w_s pl; o = sum w_s pacc; y = o / L */
void yko_combine(const float* pm, const float* pl, const float* pacc, int S, int rows, int dim, float* y) {
  for (int r = 0; r < rows; ++r) {
    float M2 = -1e30f;
    for (int s = 0; s < S; ++s) M2 = fmaxf(M2, pm[(size_t)s * rows + r]);
    float L = 0.f;
    for (int d = 0; d < dim; ++d) y[(size_t)r * dim + d] = 0.f;
    for (int s = 0; s < S; ++s) {
      const size_t p = (size_t)s * rows + r;
      const float w = pm[p] > -1e29f ? expf(pm[p] - M2) : 0.f;
      L = L + w * pl[p];
      for (int d = 0; d < dim; ++d) y[(size_t)r * dim + d] = y[(size_t)r * dim + d] + w * pacc[p * dim + d];
    }
    for (int d = 0; d < dim; ++d) y[(size_t)r * dim + d] = y[(size_t)r * dim + d] / L;
  }
}

void yko_attend_f32(const yko_cache* c, const uint16_t* q16, int M, int pos, const uint8_t* depth,
                    int splits, int threads, uint16_t* out16, float* out32) {
  const int D = c->head_dim, NH = c->n_heads, KVH = c->n_kv_heads;
  int Smax = splits > 0 ? splits : 42;
  const float qs = 1.0f / sqrtf((float)D);  /* 0.08838834764831845 at D=128, the constant of src/attention_kv4q.cu:77 */
  float* qf = (float*)malloc(sizeof(float) * (size_t)M * NH * D);
  for (size_t i = 0; i < (size_t)M * NH * D; ++i) qf[i] = yko_h2f(q16[i]) * qs;   /* scale folded into q (attention_kv4q.cu:81) */
  const size_t np = (size_t)M * Smax * NH;
  float* pm = (float*)malloc(sizeof(float) * np);
  float* pl = (float*)malloc(sizeof(float) * np);
  float* pacc = (float*)malloc(sizeof(float) * np * D);
  const int ntask = KVH * Smax;
  (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads > 1 ? threads : 1)
#endif
  for (int task = 0; task < ntask; ++task)
    split_task(c, qf, M, pos, depth, task / Smax, task % Smax, splits, Smax, pm, pl, pacc);
  /* combine per (row, head) */
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1)
#endif
  for (int r = 0; r < M * NH; ++r) {
    const int t = r / NH, head = r % NH;
    const int len = row_len(pos, depth, t), S = splits > 0 ? splits : ref_splits(len);
    float M2 = -1e30f;
    for (int s = 0; s < S; ++s) M2 = fmaxf(M2, pm[((size_t)t * Smax + s) * NH + head]);
    float L = 0.f, o[YKO_MAXD];
    for (int d = 0; d < D; ++d) o[d] = 0.f;
    for (int s = 0; s < S; ++s) {
      const size_t p = ((size_t)t * Smax + s) * NH + head;
      const float w = pm[p] > -1e29f ? expf(pm[p] - M2) : 0.f;
      L = L + w * pl[p];
      for (int d = 0; d < D; ++d) o[d] = o[d] + w * pacc[p * D + d];
    }
    for (int d = 0; d < D; ++d) {
      const float y = o[d] / L;
      if (out32) out32[(size_t)r * D + d] = y;
      if (out16) out16[(size_t)r * D + d] = yko_f2h(y);
    }
  }
  free(qf); free(pm); free(pl); free(pacc);
}

/* textbook: scores in double, subtract the row maximum, exponentiate, normalise, weight V */
void yko_attend_f64(const yko_cache* c, const uint16_t* q16, int M, int pos, const uint8_t* depth, double* out64) {
  const int D = c->head_dim, NH = c->n_heads, KVH = c->n_kv_heads, G = NH / KVH;
  const double qs = 1.0 / sqrt((double)D);
  int maxlen = 0;
  for (int t = 0; t < M; ++t) { const int l = row_len(pos, depth, t); if (l > maxlen) maxlen = l; }
  double* sc = (double*)malloc(sizeof(double) * (size_t)maxlen);
  float kd[YKO_MAXD];
  for (int t = 0; t < M; ++t) {
    const int len = row_len(pos, depth, t);
    for (int head = 0; head < NH; ++head) {
      const int kvh = head / G;
      const uint16_t* q = q16 + ((size_t)t * NH + head) * D;
      double mx = -INFINITY;
      for (int key = 0; key < len; ++key) {
        const size_t row = (size_t)kvh * c->max_ctx + key;
        yko_cache_row(c, 0, row, kd);
        double s = 0.0;
        for (int d = 0; d < D; ++d) s += (double)yko_h2f(q[d]) * (double)kd[d];
        s *= qs; sc[key] = s; if (s > mx) mx = s;
      }
      double L = 0.0; double* o = out64 + ((size_t)t * NH + head) * D;
      for (int d = 0; d < D; ++d) o[d] = 0.0;
      for (int key = 0; key < len; ++key) {
        const double w = exp(sc[key] - mx); L += w;
        const size_t row = (size_t)kvh * c->max_ctx + key;
        yko_cache_row(c, 1, row, kd);
        for (int d = 0; d < D; ++d) o[d] += w * (double)kd[d];
      }
      for (int d = 0; d < D; ++d) o[d] /= L;
    }
  }
  free(sc);
}

/* ---------- seeded inputs ---------- */
uint64_t yko_splitmix64(uint64_t x) {
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}
/* Box-Muller on two 32-bit uniforms taken from one 64-bit hash of (seed, i) */
double yko_normal(uint64_t seed, uint64_t i) {
  const uint64_t h = yko_splitmix64(yko_splitmix64(seed) ^ (i * 0xd1342543de82ef95ull + 0x632be59bd9b4e019ull));
  const double u1 = ((double)(uint32_t)(h >> 32) + 1.0) * (1.0 / 4294967296.0);   /* (0, 1] */
  const double u2 = (double)(uint32_t)h * (1.0 / 4294967296.0);                   /* [0, 1) */
  return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
}
void yko_outlier_channels(uint64_t seed, int dim, int* ch4) {
  uint64_t s = yko_splitmix64(seed ^ 0x6f75746c69657273ull);
  int n = 0;
  while (n < 4) {
    s = yko_splitmix64(s);
    const int c = (int)(s % (uint64_t)dim);
    int dup = 0;
    for (int j = 0; j < n; ++j) dup |= ch4[j] == c;
    if (!dup) ch4[n++] = c;
  }
}
void yko_fill_normal_f16(uint64_t seed, uint64_t first, uint64_t n, int dim, const int* ch4, float mult, uint16_t* out) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (int64_t j = 0; j < (int64_t)n; ++j) {
    const uint64_t e = first + (uint64_t)j;
    float x = (float)yko_normal(seed, e);
    if (ch4) { const int ch = (int)(e % (uint64_t)dim); if (ch == ch4[0] || ch == ch4[1] || ch == ch4[2] || ch == ch4[3]) x = x * mult; }
    out[j] = yko_f2h(x);
  }
}
