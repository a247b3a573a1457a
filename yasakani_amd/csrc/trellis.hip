// Trellis-coded KV rows (the reference's KV4 / KV5 row formats) on gfx950: encoder, packing, decoder.
//   reference: src/kvq_gpu.cuh:51-147 (one row per block), src/kvq_fast.cuh:63-233 (production: a block per
//   row x multiplier x chunk, then a select-and-pack block per row), decode src/kvq_attn.cuh:46-75.
// Every fp32 value is produced by the same sequence of single IEEE operations as there (explicit __f*_rn calls, sums in
// the reference's order: inside each run of 32 elements the butterfly a[i] += a[i ^ o], o = 16 .. 1, then the 8 run sums
// added in order), and the path search works on integers with the reference's tie rules, so rows are bit-identical.
//
// How the search is laid out is specific to wave64: a chunk of 64 elements is one path through 256 states and belongs to
// ONE wave; lane l holds the costs of states l, l + 64, l + 128, l + 192.  The predecessors of state d are the states
// p with p mod U == d >> kk (U = 256 >> kk), and 64 is a multiple of U, so all four states of a lane feed the same
// group u = l mod U: the minimum of a group is a per-lane minimum of 4 followed by a butterfly over the lane bits above
// log2(U) - 3 exchanges for 5-bit fields, 2 for 4-bit fields, done with a row rotation and the row / half swap
// instructions of gfx950 - with no barrier, no cost array in LDS and no LDS round trip.  The smallest predecessor among
// equal costs is found by a second butterfly on the candidate indices.  Back-pointers (one per group
// and step) go to a 2 KB LDS block private to the wave; one lane walks them back.
#include "yka_internal.h"
#include "rot256_device.h"
#include <hip/hip_fp16.h>

namespace yka {
namespace {

__device__ __forceinline__ unsigned tb_u16(const uint8_t* p) { return (unsigned)p[0] | ((unsigned)p[1] << 8); }
__device__ __forceinline__ unsigned tb_u32(const uint8_t* p) { return tb_u16(p) | (tb_u16(p + 2) << 16); }
__device__ __forceinline__ float tb_f32(const uint8_t* p) { return __uint_as_float(tb_u32(p)); }
__device__ __forceinline__ float tb_h2f(unsigned h) { return __half2float(__ushort_as_half((unsigned short)h)); }
// fp32 value -> nearest fp16 -> fp32.  The empty asm keeps the compiler from merging the operation that produced v with the
// conversion into one mixed-precision instruction, which would skip the fp32 rounding the reference performs in between
__device__ __forceinline__ float tb_f16r(float v) { asm volatile("" : "+v"(v)); return __half2float(__float2half_rn(v)); }
__device__ __forceinline__ float tb_cdec(int ci, float gain) { return __fmul_rn(__fmul_rn((float)ci, 0.00390625f), gain); }

struct Group { int nm, mode, kk, tix, guard, m, has_mu; unsigned go, off_m, off_t; bool ok; };
__device__ __forceinline__ Group tb_group(const uint8_t* b, int g) {
  Group P;
  P.nm = (int)tb_u16(b + 24); P.off_m = tb_u32(b + 32); P.off_t = tb_u32(b + 36);
  const unsigned off_g = tb_u32(b + 40), ngrp = tb_u32(b + 28);
  P.ok = (unsigned)g < ngrp;
  P.go = P.ok ? tb_u32(b + off_g + 4u * (unsigned)g) : 0u;
  P.mode = P.ok ? b[P.go] : 0; P.kk = P.ok ? b[P.go + 1] : 4; P.tix = P.ok ? b[P.go + 2] : 0; P.guard = P.ok ? b[P.go + 3] : 0;
  P.m = P.ok ? b[P.go + 4] : 0; P.has_mu = P.ok ? b[P.go + 5] : 0;
  return P;
}

// sum over the 256 threads of a block in the reference's order (tbf_sum, src/kvq_fast.cuh:31-40); red: 8 floats
__device__ __forceinline__ float block_sum(float* red, float v) {
#pragma unroll
  for (int o = 16; o; o >>= 1) v = __fadd_rn(v, __shfl_xor(v, o, 64));     // stays inside each half of the wave
  if ((threadIdx.x & 31) == 0) red[threadIdx.x >> 5] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < 8; ++w) t = __fadd_rn(t, red[w]);
  __syncthreads();
  return t;
}
__device__ __forceinline__ float block_max(float* red, float v) {
#pragma unroll
  for (int o = 16; o; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  if ((threadIdx.x & 31) == 0) red[threadIdx.x >> 5] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < 8; ++w) t = fmaxf(t, red[w]);
  __syncthreads();
  return t;
}

struct Row { float y; int g, pos; size_t out; int kind, kvh; size_t slot_off; bool ok; };
// row rj of the launch, element d.  Probe form: rows with their own group and position.  Cache form: rj = (token, K|V, kv head)
__device__ __forceinline__ Row tb_row(const TbEncArgs& A, int rj, int d, float* buf) {
  Row R;
  if (A.yin) {
    const int ri = A.row0 + rj;
    R.g = A.grp[ri]; R.pos = A.pos[ri]; R.y = A.yin[(size_t)ri * 256 + d]; R.out = (size_t)ri; R.kind = 0; R.kvh = 0;
    R.slot_off = 0; R.ok = true;
  } else {
    const int tok = rj / (2 * A.n_kv), rem = rj - tok * 2 * A.n_kv;
    R.kind = rem / A.n_kv; R.kvh = rem - R.kind * A.n_kv;
    R.slot_off = 0; R.ok = true;
    if (A.rows.pos) {                                                           // multi-stream pass: the row's own container and position
      R.pos = A.rows.pos[A.tok0 + tok];
      const int slot = A.rows.slot[A.tok0 + tok];
      R.ok = slot >= 0 && slot < A.rows.n_slots;
      R.slot_off = R.ok ? (size_t)slot * A.rows.slot_bytes : 0;
    } else {
      R.pos = *A.d_pos + A.tok0 + tok;
    }
    R.g = (A.layer * A.n_kv + R.kvh) * 2 + R.kind;
    const size_t e = ((size_t)(A.tok0 + tok) * A.n_kv + R.kvh) * 256 + d;
    R.y = A.k32 ? (R.kind ? A.v32 : A.k32)[e] : __half2float(__ushort_as_half((R.kind ? A.v16 : A.k16)[e]));
    R.out = (size_t)R.kvh * A.max_ctx + (size_t)max(0, min(R.pos, A.max_ctx - 1));
  }
  if (A.rot) R.y = rotate256(R.y, buf, false);
  return R;
}

struct Pre { float r, mud, cj0, cj1, uj0, uj1, rms; };
__device__ __forceinline__ Pre tb_pre(float* red, const uint8_t* b, const Group& P, float y) {
  const int d = threadIdx.x;
  const uint8_t* mup = b + P.go + 8;
  const uint8_t* Up = mup + (P.has_mu ? 512 : 0);
  Pre Q; Q.mud = 0.f; Q.cj0 = Q.cj1 = Q.uj0 = Q.uj1 = 0.f;
  float r = y;
  if (P.has_mu) { Q.mud = tb_h2f(tb_u16(mup + 2 * d)); r = __fsub_rn(y, Q.mud); }
  if (P.m > 0) { Q.uj0 = tb_h2f(tb_u16(Up + 2 * d));         Q.cj0 = tb_f16r(block_sum(red, __fmul_rn(r, Q.uj0))); r = __fsub_rn(r, __fmul_rn(Q.cj0, Q.uj0)); }
  if (P.m > 1) { Q.uj1 = tb_h2f(tb_u16(Up + 2 * (256 + d))); Q.cj1 = tb_f16r(block_sum(red, __fmul_rn(r, Q.uj1))); r = __fsub_rn(r, __fmul_rn(Q.cj1, Q.uj1)); }
  const float ssq = block_sum(red, __fmul_rn(r, r));
  float rms = sqrtf(__fdiv_rn(ssq, 256.f));
  if (rms == 0.f) rms = 1.f;
  Q.r = r; Q.rms = rms;
  return Q;
}

// min over the lane pair (l, l ^ O) without an LDS round trip: a row rotation for O = 8, the gfx950 row / half swaps for
// O = 16 and 32 (after swapping a register with a copy of itself the two results hold, in every lane, the values of the
// lane and of its partner)
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
template <int O>
__device__ __forceinline__ int pair_min(int v) {
  if constexpr (O == 8) return min(v, __builtin_amdgcn_update_dpp(v, v, 0x128, 0xf, 0xf, false));      // row_ror:8
  else if constexpr (O == 16) { const u32x2 r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false); return min((int)r[0], (int)r[1]); }
  else { const u32x2 r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false); return min((int)r[0], (int)r[1]); }
}
template <int U>
__device__ __forceinline__ int group_min(int v) {       // min over the lanes congruent modulo U (U = 8, 16, 32)
  if constexpr (U <= 8) v = pair_min<8>(v);
  if constexpr (U <= 16) v = pair_min<16>(v);
  return pair_min<32>(v);
}

// One chunk in one wave.  xi: the chunk's 64 integer targets (LDS), ci4: table values of the lane's four states,
// bp: 64 x 32 bytes of LDS private to the wave, st_out: 64 bytes of LDS private to the wave.
template <int KK>
__device__ __forceinline__ void wave_chunk(const int* xi, const int (&ci4)[4], uint8_t* bp, uint8_t* st_out) {
  constexpr int U = 256 >> KK, PER = 64 / U;          // PER = predecessor indices j a lane step covers: j = l / U + PER * k
  const int lane = threadIdx.x & 63;
  const int xreg = xi[lane];                           // target t lives in lane t
  // Costs are kept relative to a common offset (only differences decide) and, for 4- and 5-bit fields, carried as
  // cost * 2^KK + j with j the state's index among the predecessors of its group: ONE minimum then yields the smallest
  // cost and, among equal costs, the smallest predecessor.  At any step two states differ by at most two (three at 3
  // bits) steps' worth of squared error, < 2 * 3148^2, so the packed value fits 32 bits once the offset - the minimum of
  // group 0 - is subtracted at every step.  States that cannot be reached yet start 40,000,000 above state 0: more than
  // any path costs before every state is reachable, like the reference's 2^30, and small enough to be packed.
  constexpr bool kPacked = KK >= 4;
  constexpr int kFar = kPacked ? 40000000 : 0x40000000;
  int cost[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) cost[k] = (lane == 0 && k == 0) ? 0 : kFar;
#pragma unroll 1
  for (int t = 0; t < 64; ++t) {
    int mn, jb;
    if constexpr (kPacked) {
      int key[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) key[k] = (cost[k] << KK) | (lane / U + PER * k);
      const int km = group_min<U>(min(min(key[0], key[1]), min(key[2], key[3])));
      jb = km & ((1 << KK) - 1);
      mn = km >> KK;
      mn -= __builtin_amdgcn_readlane(mn, 0);           // the common offset: group 0's minimum
    } else {
      mn = group_min<U>(min(min(cost[0], cost[1]), min(cost[2], cost[3])));
      jb = 255;
#pragma unroll
      for (int k = 3; k >= 0; --k) jb = cost[k] == mn ? lane / U + PER * k : jb;
      jb = group_min<U>(jb);
    }
    if (lane < U) bp[t * 32 + lane] = (uint8_t)jb;
    const int x = __builtin_amdgcn_readlane(xreg, t);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      // the group this state continues is u = (lane + 64 k) >> KK; lane u holds its minimum (reading the minima into
      // scalar registers and selecting per lane was measured slower than this gather)
      const int m = __shfl(mn, (lane + 64 * k) >> KK, 64);
      const int dx = x - ci4[k];
      cost[k] = dx * dx + m;
    }
  }
  // smallest cost, then smallest state
  int bc = cost[0], bs = lane;
#pragma unroll
  for (int k = 1; k < 4; ++k) if (cost[k] < bc) { bc = cost[k]; bs = lane + 64 * k; }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int oc = __shfl_xor(bc, o, 64), os = __shfl_xor(bs, o, 64);
    if (oc < bc || (oc == bc && os < bs)) { bc = oc; bs = os; }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  if (lane == 0) {
    int st = bs;
    for (int t = 63; t >= 0; --t) {
      st_out[t] = (uint8_t)st;
      const int j = bp[t * 32 + (st >> KK)];
      st = (j << (8 - KK)) | (st >> KK);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// grid rows * nm, block 256: block = (row, multiplier); wave c = chunk c.  Writes the 256 states of the row under this
// multiplier and the 8 partial error sums to scratch.
__global__ void __launch_bounds__(256) tb_search_kernel(TbEncArgs A) {
  __shared__ float red[8];
  __shared__ float buf[256];
  __shared__ int xi[256];
  __shared__ uint8_t bp[4][64 * 32];
  __shared__ uint8_t stv[256];
  const int d = threadIdx.x, wave = d >> 6, lane = d & 63;
  const int rj = blockIdx.x / A.nm, mi = blockIdx.x - rj * A.nm;
  const uint8_t* b = A.blob;
  const Row R = tb_row(A, rj, d, buf);
  const Group P = tb_group(b, R.g);
  if (!P.ok || R.pos < P.guard || P.mode != 0) return;                     // uniform over the block
  const Pre Q = tb_pre(red, b, P, R.y);
  const unsigned to = tb_u32(b + P.off_t + 4u * (unsigned)P.tix);
  const float gain = tb_f32(b + to + 4);
  float s = tb_f16r(__fmul_rn(Q.rms, tb_f32(b + P.off_m + 4u * (unsigned)mi)));
  if (s == 0.f) s = 1.f;
  {
    const float t = rintf(__fmul_rn(__fdiv_rn(Q.r, s), 256.f));
    xi[d] = (int)fminf(fmaxf(t, -2048.f), 2048.f);
  }
  int ci4[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) ci4[k] = (int)(short)tb_u16(b + to + 12 + 2 * (lane + 64 * k));
  __syncthreads();
  switch (P.kk) {
    case 3: wave_chunk<3>(xi + 64 * wave, ci4, bp[wave], stv + 64 * wave); break;
    case 4: wave_chunk<4>(xi + 64 * wave, ci4, bp[wave], stv + 64 * wave); break;
    default: wave_chunk<5>(xi + 64 * wave, ci4, bp[wave], stv + 64 * wave); break;
  }
  // error of the chunk under this multiplier: element d of the row is lane `lane` of wave `wave`
  const int st = stv[d];
  const float rec = __fmul_rn(tb_cdec((int)(short)tb_u16(b + to + 12 + 2 * st), gain), s);
  const float dd = __fsub_rn(Q.r, rec);
  float v = __fmul_rn(dd, dd);
#pragma unroll
  for (int o = 16; o; o >>= 1) v = __fadd_rn(v, __shfl_xor(v, o, 64));
  const size_t job = (size_t)rj * A.nm + mi;
  if ((d & 31) == 0) reinterpret_cast<float*>(A.scr + A.scr_w_ofs)[job * 8 + (d >> 5)] = v;
  A.scr[job * 256 + d] = (uint8_t)st;
}

// word d of a row's MSB-first stream of KB-bit fields: the fields that overlap bits [32 d, 32 d + 32)
template <int KB>
__device__ __forceinline__ uint32_t pack_word(const uint8_t* fld, int d) {
  const int e0 = (32 * d) / KB;                          // first field with bits in the word (division by a constant)
  uint32_t w = 0u;
#pragma unroll
  for (int k = 0; k < 32 / KB + 2; ++k) {
    const int e = e0 + k, sh = 32 * d + 32 - KB * (e + 1);   // distance of the field's last bit from the word's last bit
    if (e < 256 && sh > -KB) w |= sh >= 0 ? (uint32_t)fld[e] << sh : (uint32_t)fld[e] >> -sh;
  }
  return w;
}

// grid rows, block 256: keeps the best multiplier (or runs the flat row quantizer), rebuilds the row, packs the fields
__global__ void __launch_bounds__(256) tb_select_kernel(TbEncArgs A) {
  __shared__ float red[8];
  __shared__ float buf[256];
  __shared__ uint8_t fld[256];
  const int d = threadIdx.x, nm = A.nm, rj = blockIdx.x;
  const uint8_t* b = A.blob;
  const Row R = tb_row(A, rj, d, buf);
  const Group P = tb_group(b, R.g);
  float x = R.y;
  int field = 0, kb = 4; float psc = 1.f; unsigned pc = 0u; bool pack = false;
  if (P.ok && R.pos >= P.guard) {
    const Pre Q = tb_pre(red, b, P, R.y);
    float xq = Q.r;
    if (P.mode == 1) {
      const float am = block_max(red, fabsf(Q.r));
      float s7 = __fdiv_rn(am, 7.f); if (s7 == 0.f) s7 = 1.f;
      float q = rintf(__fdiv_rn(Q.r, s7)); q = fminf(fmaxf(q, -7.f), 7.f); xq = __fmul_rn(q, s7);
      field = (int)q + 8; psc = s7; kb = 4; pack = true;
    } else if (P.mode == 0) {
      const float* const W = reinterpret_cast<const float*>(A.scr + A.scr_w_ofs) + (size_t)rj * nm * 8;
      float best_e = 0.f; int best = 0; bool have = false;
      for (int mi = 0; mi < nm; ++mi) {
        float e = 0.f;
#pragma unroll
        for (int w = 0; w < 8; ++w) e = __fadd_rn(e, W[mi * 8 + w]);
        if (!have || e < best_e) { have = true; best_e = e; best = mi; }
      }
      float s = tb_f16r(__fmul_rn(Q.rms, tb_f32(b + P.off_m + 4u * (unsigned)best))); if (s == 0.f) s = 1.f;
      const unsigned to = tb_u32(b + P.off_t + 4u * (unsigned)P.tix);
      const int st = A.scr[((size_t)rj * nm + best) * 256 + d];
      xq = __fmul_rn(tb_cdec((int)(short)tb_u16(b + to + 12 + 2 * st), tb_f32(b + to + 4)), s);
      field = st & ((1 << P.kk) - 1); psc = s; kb = P.kk; pack = true;
    }
    x = xq;
    if (P.m > 0) x = __fadd_rn(x, __fmul_rn(Q.cj0, Q.uj0));
    if (P.m > 1) x = __fadd_rn(x, __fmul_rn(Q.cj1, Q.uj1));
    if (P.has_mu) x = __fadd_rn(x, Q.mud);
    pc = (unsigned)__half_as_ushort(__float2half_rn(Q.cj0)) | ((unsigned)__half_as_ushort(__float2half_rn(Q.cj1)) << 16);
  }
  const bool in_range = A.yin || (R.ok && R.pos >= 0 && R.pos < A.max_ctx && (A.pos_limit == 0 || R.pos < A.pos_limit));
  uint8_t* const payb0 = R.kind ? A.pay1 : A.pay0;
  uint8_t* const payb = payb0 ? payb0 + R.slot_off : nullptr;
  if (payb && in_range) {
    uint32_t* const wrow = reinterpret_cast<uint32_t*>(payb + R.out * (size_t)A.stride);
    fld[d] = (uint8_t)field;
    __syncthreads();
    const int nw = A.stride >> 2;
    if (d < nw) {
      uint32_t w = 0u;
      if (pack && d < 8 * kb) w = kb == 5 ? pack_word<5>(fld, d) : kb == 4 ? pack_word<4>(fld, d) : pack_word<3>(fld, d);
      wrow[d] = w;
    }
    if (d == 0) {
      float* const scl = R.kind ? A.scl1 : A.scl0;
      if (scl) reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(scl) + R.slot_off)[R.out] = psc;
      if (A.side) { A.side[2 * R.out] = __float_as_uint(psc); A.side[2 * R.out + 1] = pc; }
      if (A.coded) A.coded[R.out] = pack ? 1 : 0;
    }
  }
  if (A.yout) A.yout[R.out * 256 + d] = x;
}

// decoder (tba_unpack_kernel, src/kvq_attn.cuh:46-75): grid rows, block 256
__device__ __forceinline__ unsigned stream_bits(const uint32_t* wp, int nwords, int pos, int n) {
  const int wi = pos >> 5, o = pos & 31;
  const unsigned long long Z = ((unsigned long long)wp[wi] << 32) | (unsigned long long)((wi + 1 < nwords) ? wp[wi + 1] : 0u);
  return (unsigned)((Z >> (64 - o - n)) & ((1ull << n) - 1ull));
}
__global__ void __launch_bounds__(256) tb_unpack_kernel(const uint8_t* blob, const int* grp, const int* pos, const uint8_t* pay, const uint32_t* side,
                                                        int stride, const float* yin, float* y) {
  __shared__ float tab[256];
  const int row = blockIdx.x, d = threadIdx.x;
  const int g = grp[row];
  float out = yin ? yin[(size_t)row * 256 + d] : 0.f;
  if ((unsigned)g < tb_u32(blob + 28)) {
    const Group P = tb_group(blob, g);
    if (pos[row] >= P.guard && P.mode <= 1) {
      const uint32_t* wp = reinterpret_cast<const uint32_t*>(pay + (size_t)row * stride);
      const float s = __uint_as_float(side[2 * (size_t)row]); const unsigned pc = side[2 * (size_t)row + 1];
      const int kb = P.mode == 1 ? 4 : P.kk, nw = 8 * kb;
      float xq;
      if (P.mode == 1) xq = __fmul_rn((float)((int)stream_bits(wp, nw, 4 * d, 4) - 8), s);
      else {
        const unsigned to = tb_u32(blob + P.off_t + 4u * (unsigned)P.tix);
        tab[d] = tb_cdec((int)(short)tb_u16(blob + to + 12 + 2 * d), tb_f32(blob + to + 4));
        __syncthreads();
        const int endb = kb * (d + 1), first = kb * (d & ~63), lo = max(endb - 8, first);
        xq = __fmul_rn(tab[stream_bits(wp, nw, lo, endb - lo)], s);
      }
      float x = xq;
      const uint8_t* mup = blob + P.go + 8; const uint8_t* Up = mup + (P.has_mu ? 512 : 0);
      if (P.m > 0) x = __fadd_rn(x, __fmul_rn(tb_h2f(pc & 0xffffu), tb_h2f(tb_u16(Up + 2 * d))));
      if (P.m > 1) x = __fadd_rn(x, __fmul_rn(tb_h2f(pc >> 16), tb_h2f(tb_u16(Up + 2 * (256 + d)))));
      if (P.has_mu) x = __fadd_rn(x, tb_h2f(tb_u16(mup + 2 * d)));
      out = x;
    }
  }
  y[(size_t)row * 256 + d] = out;
}

}  // namespace

void launch_tb_encode(const TbEncArgs& A, hipStream_t st) {
  if (A.nrow <= 0) return;
  if (A.has_trellis) hipLaunchKernelGGL(tb_search_kernel, dim3(A.nrow * A.nm), dim3(256), 0, st, A);
  hipLaunchKernelGGL(tb_select_kernel, dim3(A.nrow), dim3(256), 0, st, A);
}
void launch_tb_unpack(const uint8_t* blob, const int* grp, const int* pos, const uint8_t* pay, const uint32_t* side, int stride, const float* yin,
                      float* y, int rows, hipStream_t st) {
  if (rows > 0) hipLaunchKernelGGL(tb_unpack_kernel, dim3(rows), dim3(256), 0, st, blob, grp, pos, pay, side, stride, yin, y);
}

}  // namespace yka
