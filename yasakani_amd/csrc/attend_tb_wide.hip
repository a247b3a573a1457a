// Split-KV attention over trellis-coded rows (the reference's KV4 / KV5 packed streams) for windows of 3..64 query tokens.
// gfx950.  reference: launch_q35_prefill_atx_pk / q35_atxpk4_kernel on packed rows (src/q35_atxpk.hpp:21, src/q35_atxpk4.cuh:71-499).
//
// The compute side is the wide kernel of the flat 256-channel rows (attend256_wide.hip): a workgroup of 8 waves owns 128
// query rows and one split of the keys, every 32-key tile is decoded ONCE per workgroup into a double-buffered LDS image
// (K values as exact fp16 integers, V transposed, both scale vectors), a wave owns 16 rows with MFMA 16x16x32.  What
// differs is the decode: a thread turns 16 consecutive K elements of one key and the 8-channel V block of two adjacent
// keys into table values with one 32-bit LDS gather per PAIR of elements (the pair tables of attend_tb.hip, 16 / 32 KB
// per table, resident in LDS next to the tile images: 150 KB in all at 5 bits per element).  The table's integers stay
// exact; gain / 256 joins the softmax scale (K) and the final normalisation (V).  A V mean row is added to the
// normalised partial; a K mean row cancels in the softmax and is not applied.
// LDS image of one tile (42240 bytes):
//   K  [32 keys][544 B]    chunk c (16 bytes) of a key = channels 8c .. 8c+7
//   V  [256 channels][96 B] key 16kb + 4g + r sits at slot 8g + 4kb + r: the 8 keys whose probabilities an MFMA lane of
//                           group g holds are 16 contiguous bytes
//   SC [2][32] fp32        K scales, V scales of the tile's keys
#include "yka_internal.h"
#include <hip/hip_fp16.h>
#include <type_traits>

namespace yka {

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t as_u32(h2 h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ uint32_t funnel(uint32_t hi, uint32_t lo, uint32_t sh) { return __builtin_amdgcn_alignbit(hi, lo, sh); }   // (hi:lo) >> sh

constexpr int kD2 = 256;
constexpr float kLog2e = 1.4426950408889634f;
constexpr int NT = 512;                        // threads per workgroup (8 waves x 16 rows)
constexpr int kKPitch = 544, kVPitch = 96;     // conflict-free for the fragment reads (see attend256_wide.hip)
constexpr int kLdsK = 0, kLdsV = 32 * kKPitch, kLdsS = kLdsV + kD2 * kVPitch, kLdsBuf = kLdsS + 256;   // 42240
constexpr float kRaise = 8.f;                  // log2 slack before a running maximum is raised

// byte offset (entry index x 4) into a pair table for the KB + 8 bits that end at bit `endbit` (exclusive) of the bit
// string w[0] w[1] ... (MSB first); bits before w[0] count as zero.  endbit is a compile-time constant.
template <int KB>
__device__ __forceinline__ uint32_t pair_offset(const uint32_t* w, int endbit) {
  constexpr uint32_t mask4 = ((1u << (8 + KB)) - 1u) << 2;
  const int j = (endbit - 1) >> 5, r = 31 - ((endbit - 1) & 31);
  const uint32_t hi = j > 0 ? w[j - 1] : 0u;
  if (r >= 2) return (r == 2 ? w[j] : funnel(hi, w[j], (uint32_t)(r - 2))) & mask4;
  return (funnel(hi, w[j], (uint32_t)r) << 2) & mask4;
}
__device__ __forceinline__ uint32_t pair_at(const uint8_t* tab, uint32_t off) { return *reinterpret_cast<const uint32_t*>(tab + off); }

// One thread's share of a raw 32-key tile.  Every window starts 8 - KB bits before its first element, i.e. possibly in
// the word before a chunk (masked to zero there; the word before the very first row lies in a guard band the pool keeps
// in front of its payload), and may end a word past what it needs.
struct Raw {
  u32x4 k;                                     // K: elements 16c .. 16c+15 of key tid/16 (c = tid%16)
  u32x3 v[2];                                  // V: the 8-channel block tid/16 of keys 2(tid%16), 2(tid%16)+1
  uint32_t sc;                                 // (tid & 63) < 32: K scale of key tid&31, else V scale of key tid&31
};
// k, v: byte offsets of the thread's windows from kLaneBias bytes BEFORE the tile's first row.  The hardware adds the lane
// offset of a "scalar base + lane offset" access as an unsigned 32-bit number, and a window may begin 4 bytes before the
// row, so the scalar base is moved back by kLaneBias (into the guard band for the very first row) and the offsets stay
// positive.
constexpr int kLaneBias = 256;
struct LaneOffs { uint32_t k, v, sc; uint32_t shk, shv, keepk, keepv; };
template <int KB>
__device__ __forceinline__ LaneOffs lane_offs(int tid, int stride, uint32_t vscl_minus_kscl) {
  LaneOffs L;
  const int key = tid >> 4, c = tid & 15;
  {                                            // K: quarter c & 3 of chunk c >> 2
    const int s0 = KB * 16 * (c & 3) - (8 - KB), w0 = s0 >> 5;
    L.k = (uint32_t)(kLaneBias + key * stride + (c >> 2) * (8 * KB) + 4 * w0);
    L.shk = 32u - (uint32_t)(s0 & 31);
    L.keepk = (c & 3) == 0 ? 0u : 0xffffffffu;
  }
  {                                            // V: block w & 7 of chunk w >> 3, keys 2 kp and 2 kp + 1
    const int w = tid >> 4, kp = tid & 15;
    const int s0 = KB * 8 * (w & 7) - (8 - KB), w0 = s0 >> 5;
    L.v = (uint32_t)(kLaneBias + 2 * kp * stride + (w >> 3) * (8 * KB) + 4 * w0);
    L.shv = 32u - (uint32_t)(s0 & 31);
    L.keepv = (w & 7) == 0 ? 0u : 0xffffffffu;
  }
  const uint32_t t6 = tid & 63;
  L.sc = (t6 < 32 ? 0u : vscl_minus_kscl) + (t6 & 31) * 4u;
  return L;
}
// Loads as instructions ("wave-uniform base in scalar registers + 32-bit lane offset") so that they stay where they are
// written - right after the registers they land in were consumed, a whole tile step before their use.
__device__ __forceinline__ void load_raw(const uint8_t* krows, const uint8_t* vrows, const uint8_t* sc, int stride, const LaneOffs& L, Raw& R) {
  const uint32_t v1 = L.v + (uint32_t)stride;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(R.k) : "v"(L.k), "s"(krows));
  asm volatile("global_load_dwordx3 %0, %1, %2" : "=v"(R.v[0]) : "v"(L.v), "s"(vrows));
  asm volatile("global_load_dwordx3 %0, %1, %2" : "=v"(R.v[1]) : "v"(v1), "s"(vrows));
  asm volatile("global_load_dword %0, %1, %2" : "=v"(R.sc) : "v"(L.sc), "s"(sc));
}
__device__ __forceinline__ void wait_raw(Raw& R) {
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(R.k), "+v"(R.v[0]), "+v"(R.v[1]), "+v"(R.sc));
}

template <int KB>
__device__ __forceinline__ void decode_to_lds(uint8_t* buf, int tid, const Raw& R, const LaneOffs& L, const uint8_t* tabK, const uint8_t* tabV) {
  {                                            // K: 16 elements = 8 pair reads -> 32 contiguous bytes of the key's row
    const int key = tid >> 4, c = tid & 15;
    uint32_t y[3];
    y[0] = funnel(R.k[0] & L.keepk, R.k[1], L.shk);
    y[1] = funnel(R.k[1], R.k[2], L.shk);
    y[2] = funnel(R.k[2], R.k[3], L.shk);
    uint32_t d[8];
#pragma unroll
    for (int p = 0; p < 8; ++p) d[p] = pair_at(tabK, pair_offset<KB>(y, KB * 2 * p + 8 + KB));
    uint8_t* dst = buf + kLdsK + key * kKPitch + c * 32;
    *reinterpret_cast<uint4*>(dst) = make_uint4(d[0], d[1], d[2], d[3]);
    *reinterpret_cast<uint4*>(dst + 16) = make_uint4(d[4], d[5], d[6], d[7]);
  }
  {                                            // V: block w of keys (2kp, 2kp+1) -> 8 channel rows, two adjacent key slots each
    const int w = tid >> 4, key = 2 * (tid & 15);
    const int slot = 8 * ((key >> 2) & 3) + 4 * (key >> 4) + (key & 3);
    uint8_t* vb = buf + kLdsV + (8 * w) * kVPitch + slot * 2;
    uint32_t pr[2][4];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      uint32_t y[2];
      y[0] = funnel(R.v[kk][0] & L.keepv, R.v[kk][1], L.shv);
      y[1] = funnel(R.v[kk][1], R.v[kk][2], L.shv);
#pragma unroll
      for (int t = 0; t < 4; ++t) pr[kk][t] = pair_at(tabV, pair_offset<KB>(y, KB * 2 * t + 8 + KB));
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      *reinterpret_cast<uint32_t*>(vb + (2 * t) * kVPitch) = __builtin_amdgcn_perm(pr[1][t], pr[0][t], 0x05040100u);       // element 2t of both keys
      *reinterpret_cast<uint32_t*>(vb + (2 * t + 1) * kVPitch) = __builtin_amdgcn_perm(pr[1][t], pr[0][t], 0x07060302u);   // element 2t + 1
    }
  }
  reinterpret_cast<uint32_t*>(buf + kLdsS)[tid & 63] = R.sc;      // waves repeat each other (no divergent branch)
}

// grid (S, n_kv, ceil(6M / 128)), block 512; wave w owns rows [16 w, 16 (w+1)) of the block
template <int KB>
__global__ void __launch_bounds__(NT, 1) attend_tb_wide_kernel(TbAttnArgs A) {
  constexpr int kTabBytes = 4 << (8 + KB);
  __shared__ __align__(16) uint8_t lds[2][kLdsBuf];
  __shared__ __align__(16) uint8_t tabs[2 * kTabBytes];
  const uint8_t* const tabK = tabs;
  const uint8_t* const tabV = tabs + kTabBytes;
  const int split = blockIdx.x, kvh = blockIdx.y, rb = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int gK = (A.layer * A.n_kv + kvh) * 2, gV = gK + 1;
  {                                            // the K and V pair tables of this kv head: global (L2) -> LDS
    const uint4* srcK = reinterpret_cast<const uint4*>(A.pairs + (size_t)gK * (kTabBytes / 4));
    const uint4* srcV = reinterpret_cast<const uint4*>(A.pairs + (size_t)gV * (kTabBytes / 4));
    uint4* dst = reinterpret_cast<uint4*>(tabs);
#pragma unroll 4
    for (int x = tid; x < kTabBytes / 16; x += NT) { dst[x] = srcK[x]; dst[kTabBytes / 16 + x] = srcV[x]; }
  }
  const int pos = *A.d_pos;
  const int nrows = kG * A.M;
  constexpr int RPB = 128;

  // row of this lane column: R = rb*128 + wave*16 + i  ->  token R/6 of the slice, head kvh*6 + R%6
  const int row0 = rb * RPB + wave * 16;
  const int R = row0 + i;
  const bool vrow = R < nrows;
  const int tl = R / kG, head = kvh * kG + R % kG;
  int len = 0;
  if (vrow) { const int tg = A.tok0 + tl; len = min(pos + (A.depth ? (int)A.depth[tg] : tg) + 1, A.max_ctx); }
  // Q fragments: k-step t of 8, lane (row i, group g), element e <-> channel 8 (4t + g) + e
  h8 qf[8];
  {
    const uint16_t* qrow = A.q16 + ((size_t)tl * A.n_heads + head) * kD2 + 8 * g;
#pragma unroll
    for (int t = 0; t < 8; ++t) qf[t] = __builtin_bit_cast(h8, vrow ? *reinterpret_cast<const uint4*>(qrow + 32 * t) : make_uint4(0, 0, 0, 0));
  }
  const bool has_rows = row0 < nrows;                       // wave uniform

  // key range of the workgroup: its splits cut [0, maxlen) of the block's longest row into 32-key tiles
  const int tok_lo = (rb * RPB) / kG, tok_hi = min(A.M, (rb * RPB + RPB + kG - 1) / kG);
  int maxdep = 0, mindep = 0x7fffffff;
  for (int t = tok_lo; t < tok_hi; ++t) { const int tg = A.tok0 + t; const int dp = A.depth ? (int)A.depth[tg] : tg; maxdep = max(maxdep, dp); mindep = min(mindep, dp); }
  const int maxlen = min(pos + maxdep + 1, A.max_ctx), minlen = min(pos + mindep + 1, A.max_ctx);
  const int ntiles = (maxlen + 31) >> 5, tps = (ntiles + A.S - 1) / A.S;
  const int tile0 = split * tps, tile1 = min(ntiles, tile0 + tps);

  const float sc_log2 = kLog2e * 0.0625f * A.gfac[gK];      // log2(e) / sqrt(256) x gain / 256 of the K table (positive)
  float m_run = -1e30f, l_run = 0.f;           // m_run in log2 units, shared by the four lanes of a row
  f4 o[16];
#pragma unroll
  for (int b = 0; b < 16; ++b) o[b] = f4{0.f, 0.f, 0.f, 0.f};

  Raw raw{};                                   // raw words of the next tile
  const size_t prow0 = (size_t)kvh * A.max_ctx;
  const LaneOffs offs = lane_offs<KB>(tid, A.stride, (uint32_t)(reinterpret_cast<const uint8_t*>(A.vscl) - reinterpret_cast<const uint8_t*>(A.kscl)));
  auto load_tile_raw = [&](int T, Raw& r) __attribute__((always_inline)) {
    const size_t row = prow0 + ((size_t)T << 5);
    load_raw(A.kpay + row * A.stride - kLaneBias, A.vpay + row * A.stride - kLaneBias, reinterpret_cast<const uint8_t*>(A.kscl + row), A.stride, offs, r);
  };
  __syncthreads();                             // pair tables
  if (tile0 < tile1) {
    load_tile_raw(tile0, raw);
    wait_raw(raw);
    decode_to_lds<KB>(lds[0], tid, raw, offs, tabK, tabV);
    load_tile_raw(min(tile0 + 1, tile1 - 1), raw);
  }
  __syncthreads();

  // One tile: `rs` holds the raw words of tile T+1, which are decoded into the other LDS buffer (unconditionally: after
  // the last tile that buffer is read by nobody) and replaced by the request for tile T+2 (past the end: the last tile
  // again); cb is a literal at both call sites.
  auto tile_step = [&](auto compute_tag, const int T, const int cb, Raw& rs) __attribute__((always_inline)) {
    constexpr bool kCompute = decltype(compute_tag)::value;
    const uint8_t* buf = lds[cb];
    wait_raw(rs);
    decode_to_lds<KB>(lds[cb ^ 1], tid, rs, offs, tabK, tabV);
    load_tile_raw(min(T + 2, tile1 - 1), rs);
    if constexpr (kCompute) {
      const int t0 = T << 5;
      // ---- scores: per 16-key block 8 chained MFMAs over the 256 channels, then one multiply by the key's scale ----
      float s[8];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const f4 ksc = *reinterpret_cast<const f4*>(buf + kLdsS + (16 * kb + 4 * g) * 4);
        h8 kf[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)
          kf[t] = __builtin_bit_cast(h8, *reinterpret_cast<const uint4*>(buf + kLdsK + (16 * kb + i) * kKPitch + (4 * t + g) * 16));
        f4 part = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 8; ++t) part = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[t], qf[t], part, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) s[4 * kb + r] = part[r] * ksc[r];          // key t0 + 16kb + 4g + r against row i
        // all fragment reads of the block first, then its MFMA chain: the chain does not wait for LDS between links
        __builtin_amdgcn_sched_group_barrier(0x100, 9, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      }
      // V scales of the lane's 8 keys, and the first half of the V fragments: their latency runs under the softmax
      const f4 vsc0 = *reinterpret_cast<const f4*>(buf + kLdsS + 128 + (4 * g) * 4);
      const f4 vsc1 = *reinterpret_cast<const f4*>(buf + kLdsS + 128 + (16 + 4 * g) * 4);
      h8 vf[8];
#pragma unroll
      for (int b = 0; b < 8; ++b)
        vf[b] = __builtin_bit_cast(h8, *reinterpret_cast<const uint4*>(buf + kLdsV + (16 * b + i) * kVPitch + g * 16));
      if (t0 + 32 > minlen) {
#pragma unroll
        for (int e = 0; e < 8; ++e) { const int key = t0 + 16 * (e >> 2) + 4 * g + (e & 3); s[e] = key < len ? s[e] : -INFINITY; }
      }
      // ---- online softmax with a lazily raised maximum (p = 2^(s * sc_log2 - m_run)) ----
      float tmax = s[0];
#pragma unroll
      for (int e = 1; e < 8; ++e) tmax = fmaxf(tmax, s[e]);
      tmax *= sc_log2;
      if (__any(tmax > m_run + kRaise)) {
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new; l_run *= alpha;
#pragma unroll
        for (int b = 0; b < 16; ++b) { o[b][0] *= alpha; o[b][1] *= alpha; o[b][2] *= alpha; o[b][3] *= alpha; }
      }
      h8 pf;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], sc_log2, -m_run));
        l_run += p;
        pf[e] = (_Float16)(p * (e < 4 ? vsc0[e & 3] : vsc1[e & 3]));            // the V scale of the key rides on its probability
      }
      // ---- O^T += V^T P^T : accumulator b covers channels 16b .. 16b+15, one MFMA contracts the tile's 32 keys ----
#pragma unroll
      for (int b = 0; b < 8; ++b) o[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[b], pf, o[b], 0, 0, 0);
#pragma unroll
      for (int b = 0; b < 8; ++b)
        vf[b] = __builtin_bit_cast(h8, *reinterpret_cast<const uint4*>(buf + kLdsV + (16 * (b + 8) + i) * kVPitch + g * 16));
#pragma unroll
      for (int b = 0; b < 8; ++b) o[b + 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[b], pf, o[b + 8], 0, 0, 0);
    }
    __syncthreads();
  };
  auto run = [&](auto compute_tag) __attribute__((always_inline)) {
    for (int T = tile0; T < tile1; T += 2) {
      tile_step(compute_tag, T, 0, raw);
      if (T + 1 < tile1) tile_step(compute_tag, T + 1, 1, raw);
    }
  };
  if (has_rows) run(std::true_type{}); else run(std::false_type{});
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // the loads past the last tile
  if (!has_rows) return;                       // no barrier follows
  // ---- partials: normalised fp16.  o[b][r] of lane (row i, group g) is channel 16b + 4g + r.  Rows go through LDS (the
  //      tile buffers are free after the last barrier) so that every store instruction writes whole 512-byte rows ----
  constexpr int kOPitch = 2 * kD2 + 16;                      // bytes per staged row
  uint8_t* stage = &lds[0][0] + wave * 16 * kOPitch;         // 8 waves x 8448 bytes of the 84480
  float l = l_run;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  const size_t pidx = ((size_t)tl * A.S + split) * A.n_heads + head;
  if (vrow && g == 0) { A.pm[pidx] = m_run; A.pl[pidx] = l; }
  const float inv = l > 0.f ? A.gfac[gV] / l : 0.f;          // gain / 256 of the V table joins the normalisation
#pragma unroll
  for (int b = 0; b < 16; ++b) {
    f4 mu = f4{0.f, 0.f, 0.f, 0.f};
    if (A.mu && l > 0.f) mu = *reinterpret_cast<const f4*>(A.mu + (size_t)gV * 256 + 16 * b + 4 * g);
    const h2 lo = {(_Float16)(o[b][0] * inv + mu[0]), (_Float16)(o[b][1] * inv + mu[1])}, hi = {(_Float16)(o[b][2] * inv + mu[2]), (_Float16)(o[b][3] * inv + mu[3])};
    *reinterpret_cast<uint2*>(stage + i * kOPitch + (16 * b + 4 * g) * 2) = make_uint2(as_u32(lo), as_u32(hi));
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");     // the wave reads back what its own lanes wrote
  const int chunk = lane & 31;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int jr = 2 * k + (lane >> 5);
    const int Rr = row0 + jr;
    if (Rr < nrows) {
      const size_t p = ((size_t)(Rr / kG) * A.S + split) * A.n_heads + kvh * kG + Rr % kG;
      const uint4 v = *reinterpret_cast<const uint4*>(stage + jr * kOPitch + chunk * 16);
      *reinterpret_cast<uint4*>(A.pacc16 + p * kD2 + chunk * 8) = v;
    }
  }
}

}  // namespace

void launch_attend_tb_wide(const TbAttnArgs& A, int kb, hipStream_t st) {
  const int rows = kG * A.M, rb = (rows + 127) / 128;
  const dim3 grid(A.S, A.n_kv, rb);
  if (kb == 4) hipLaunchKernelGGL(attend_tb_wide_kernel<4>, grid, dim3(NT), 0, st, A);
  else hipLaunchKernelGGL(attend_tb_wide_kernel<5>, grid, dim3(NT), 0, st, A);
}

}  // namespace yka
