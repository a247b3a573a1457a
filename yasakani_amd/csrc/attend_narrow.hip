// Split-KV attention over the int4 cache for row tiles of at most 2 tokens x 6 heads (single-token decode and the
// building block for any window), plus the split combiner.  gfx950 (wave64, MFMA 16x16x32 f16).
//
// What it computes is the reference's split-KV pass (src/attention_kv4q.cu:71-146, production form
// src/q35_atxpk3.cuh:131-477): for every query row, an online softmax over the keys of one split, written as
// (m, l, acc) partials, merged by a combiner (src/attention_kv4q.cu:325-332).  How it computes it is specific to
// CDNA4:
//   * one wave owns a 32-key tile.  K rows are read as one 16-byte chunk per lane; the page layout puts one dword of
//     every scale group into that chunk, so MFMA step m contracts exactly the 32 channels of group m.  V is read as
//     one dword per (lane, token) so that a lane ends up with 8 tokens of the same 8 channels - the operand shape
//     the token-contracting MFMA needs;
//   * codes become fp16 without integer conversion.  V: a nibble OR-ed into the mantissa of 1024.0 is 1024+n (or
//     1024+16n for the odd nibble of a byte); subtracting 1032 (1152) gives n-8 (16(n-8)) exactly.  K: a nibble left in
//     place in a zero word IS an fp16, the subnormal n * 2^-24, and the matrix pipe takes subnormal inputs unflushed: an
//     AND per pair of codes is the whole conversion, the offset -8 rides in the MFMA's initial accumulator as
//     -8 * 2^-24 * sum(q) per (row, scale group), and the 2^24 is folded into the exponent's scale;
//   * K stays exact: the MFMA multiplies Q by the integer codes, and the fp16 group scale is applied to the fp32
//     partial sum of each group (rounding q*scale to fp16 first costs 7e-4 relative L2 on inputs with outlier
//     channels, most of the 1e-3 budget).  V is scaled in fp16 (one rounding, 2e-4);
//   * scores S^T = K Q^T come out of the MFMA with one query row per lane column, which is already the B-operand
//     layout of O^T += V^T P^T: probabilities never move between lanes;
//   * running maxima are shared by the 4 lane groups of a row through two cross-lane exchanges per tile;
//   * a wave that has more than two tiles to walk keeps two raw tiles in registers: the 16 loads of the tile after the
//     one it works on are in flight while it dequantizes and multiplies (2 waves per SIMD, 8 per CU, two tiles each).
//     Against 4 waves per SIMD with one tile each this measures the same at 32k tokens per head, 17 % faster at 262k
//     and 10 % faster with 32 streams in one launch.  Waves with one or two tiles load them straight away;
//   * quantize-on-append is fused into the decode launch (a launch costs about 2.5 us here, the same order as the
//     whole KV stream): the workgroup whose tiles contain a row appended by this pass quantizes and stores that row
//     before it loads the tile;
//   * the split merge is a second launch by default.  It can ride in the same launch when the caller hands over a
//     ticket array: every workgroup of a (kv head, row tile) column stores its partials with agent-scope stores (written
//     through its XCD's L2, which the other XCDs do not see), waits until they are acknowledged, and takes a ticket; the
//     workgroup that draws the last one reads the column's partials back with agent-scope loads and writes the final
//     rows.  No cache-wide write-back or invalidate is involved (a device-scope release fence in every workgroup measured
//     4x slower than a second launch), but the last workgroup still pays three dependent trips to memory after its
//     tiles - stores acknowledged, ticket, loads - and that measures slower than the gap between two kernels: 14.7
//     against 8.6 us per layer call at 4k tokens, 18.9 against 12.0 at 32k, 34.0 against 24.9 at 131k (one token; two
//     tokens add another 7 to 14 us).
#include <type_traits>
#include "codec_device.h"
#include "sign_device.h"
#include "tile32_device.h"

namespace yka {

// Agent-scope accesses for data that workgroups on different XCDs hand to each other inside one launch: relaxed atomics,
// which the compiler turns into plain stores and loads with the scope bit that makes them go past the XCD-local L2.
__device__ __forceinline__ void st_agent(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float ld_agent(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent16(uint16_t* p, uint4 v) {     // 16 bytes, 16-byte aligned
  uint64_t* q = reinterpret_cast<uint64_t*>(p);
  __hip_atomic_store(q, (uint64_t)v.x | ((uint64_t)v.y << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(q + 1, (uint64_t)v.z | ((uint64_t)v.w << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint4 ld_agent16(const uint16_t* p) {
  const uint64_t* q = reinterpret_cast<const uint64_t*>(p);
  const uint64_t a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_uint4((uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32));
}

// The workgroup's partials are out (or its "no keys" markers): wait until the stores are acknowledged, take a ticket of
// the column.  True for the workgroup that drew the last one: every partial of the column is then visible to agent-scope
// loads.  The ticket is an acquire-release operation at agent scope behind a workgroup barrier, so the order "partials,
// then ticket" (writers) and "ticket, then partials" (the merging workgroup) holds by the memory model and not only by
// the explicit wait.  The counter is also put back to zero; the host zeroes it in front of every launch regardless.
__device__ __forceinline__ bool last_of_column(const AttnArgs& A, int* s_ticket) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int* t = A.tickets + blockIdx.y * gridDim.z + blockIdx.z;
  if (threadIdx.x == 0) {
    const int old = __hip_atomic_fetch_add(t, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    if (old == A.S - 1) __hip_atomic_store(t, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_ticket = old;
  }
  __syncthreads();
  return *s_ticket == A.S - 1;
}

// The combiner of one column (reference: src/attention_kv4q.cu:325-332), run by its last workgroup: 256 threads, rows =
// the column's tokens x 6 heads.  Per token: thread t weighs split t of each head (w = 2^(m - max m) * l), then 16 split
// lanes x 16 channel lanes sum w * acc/l over the splits, K splits in flight per lane and head; K * 16 >= S.  All six
// heads are in flight at once when K is 4 (one memory round trip: decode up to 64 splits), one head at a time otherwise.
// lds: 6 * 256 + 4 * 6 * 128 + 64 floats.
template <int TPT, int K>
__device__ __forceinline__ void combine_column(const AttnArgs& A, int kvh, int rt, float* lds) {
  constexpr int HB = K <= 4 ? kG : 1;                  // heads per batch of loads
  float* s_w = lds;                                    // [6][256] weights
  float* s_o = lds + kG * 256;                         // [4 waves][6 heads][128]
  float* s_red = s_o + 4 * kG * kD;                    // [4][6] maxima, then [4][6] weight sums
  const int tid = threadIdx.x, wave = tid >> 6, sl = tid >> 4, c8 = (tid & 15) * 8;
  const int ntok = min(TPT, A.M - TPT * rt);
  for (int tk = 0; tk < ntok; ++tk) {
    const int tj = TPT * rt + tk;
    const size_t p0 = (size_t)tj * A.S * A.n_heads + kvh * kG;        // (split s, head h) lives at p0 + s * n_heads + h
    const size_t stride = (size_t)A.n_heads * kD;
    float pmv[kG], plv[kG];
#pragma unroll
    for (int h = 0; h < kG; ++h) {
      pmv[h] = tid < A.S ? ld_agent(A.pm + p0 + (size_t)tid * A.n_heads + h) : -1e30f;
      plv[h] = tid < A.S ? ld_agent(A.pl + p0 + (size_t)tid * A.n_heads + h) : 0.f;
    }
    uint4 u[HB][K];
    auto request = [&](int h0) __attribute__((always_inline)) {
#pragma unroll
      for (int hh = 0; hh < HB; ++hh)
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const int sp = sl + 16 * k;
          u[hh][k] = sp < A.S ? ld_agent16(A.pacc16 + (p0 + h0 + hh) * kD + (size_t)sp * stride + c8) : make_uint4(0, 0, 0, 0);
        }
    };
    request(0);
    // maxima over the splits, per head
    float mx[kG];
#pragma unroll
    for (int h = 0; h < kG; ++h) {
      mx[h] = pmv[h];
#pragma unroll
      for (int o = 32; o; o >>= 1) mx[h] = fmaxf(mx[h], __shfl_xor(mx[h], o, 64));
    }
    __syncthreads();                                   // the previous token's readers of s_red / s_w / s_o are done
    if ((tid & 63) == 0)
#pragma unroll
      for (int h = 0; h < kG; ++h) s_red[wave * kG + h] = mx[h];
    __syncthreads();
    float wsum[kG];
#pragma unroll
    for (int h = 0; h < kG; ++h) {
      const float M2 = fmaxf(fmaxf(s_red[h], s_red[kG + h]), fmaxf(s_red[2 * kG + h], s_red[3 * kG + h]));
      const float w = (tid < A.S && pmv[h] > -1e29f) ? exp2f(pmv[h] - M2) * plv[h] : 0.f;
      s_w[h * 256 + tid] = w;
      wsum[h] = w;
#pragma unroll
      for (int o = 32; o; o >>= 1) wsum[h] += __shfl_xor(wsum[h], o, 64);
    }
    __syncthreads();                                   // maxima read by everyone, weights written
    if ((tid & 63) == 0)
#pragma unroll
      for (int h = 0; h < kG; ++h) s_red[wave * kG + h] = wsum[h];
    // weighted sums over the splits
#pragma unroll
    for (int h0 = 0; h0 < kG; h0 += HB) {
      if (h0) request(h0);
#pragma unroll
      for (int hh = 0; hh < HB; ++hh) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const int sp = sl + 16 * k;
          const float w = sp < A.S ? s_w[(h0 + hh) * 256 + sp] : 0.f;
          const uint4 r = w != 0.f ? u[hh][k] : make_uint4(0, 0, 0, 0);   // a row of weight 0 may hold anything
          const h8 v = __builtin_bit_cast(h8, r);
#pragma unroll
          for (int c = 0; c < 8; ++c) acc[c] += w * (float)v[c];
        }
        // the wave's 4 split lanes (lane bits 4 and 5), then the 4 waves through LDS
#pragma unroll
        for (int c = 0; c < 8; ++c) { acc[c] += __shfl_xor(acc[c], 16, 64); acc[c] += __shfl_xor(acc[c], 32, 64); }
        if ((tid & 48) == 0) {
          float* d = s_o + (wave * kG + h0 + hh) * kD + c8;
          *reinterpret_cast<float4*>(d) = make_float4(acc[0], acc[1], acc[2], acc[3]);
          *reinterpret_cast<float4*>(d + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
        }
      }
    }
    __syncthreads();
    if (tid < kG * 16) {                               // 16 lanes per head, 8 channels each: one 16-byte store
      const int h = tid >> 4;
      const float L = s_red[h] + s_red[kG + h] + s_red[2 * kG + h] + s_red[3 * kG + h];
      const float inv = L > 0.f ? 1.f / L : 0.f;       // a row that saw no key at all (a rejected row of a multi-stream pass)
      float yv[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const float o = s_o[(0 * kG + h) * kD + c8 + c] + s_o[(1 * kG + h) * kD + c8 + c] + s_o[(2 * kG + h) * kD + c8 + c] + s_o[(3 * kG + h) * kD + c8 + c];
        yv[c] = o * inv;
      }
      *reinterpret_cast<uint4*>(A.out16 + ((size_t)tj * A.n_heads + kvh * kG + h) * kD + c8) = pack_out8(yv, A.out_bf16);
    }
  }
}

// grid (S, n_kv, ceil(M/TPT)), block 256 (4 waves).  Workgroup = (split, kv head, row tile of TPT tokens x 6 heads):
// TPT = 2 for a single-stream pass; MS (multi-stream pass, reference: src/q35_atxpk_ms.cu:13-33): one token per tile,
// which reads the container and the position its row map names.
template <bool MS>
__global__ void __launch_bounds__(256, 2) attend_narrow_kernel(AttnArgs A) {
  __shared__ float s_m[4][16], s_l[4][16];
  __shared__ __align__(16) float s_acc[4][16][kD + 4];     // 8448 floats; the fused combiner needs 4672 of them
  __shared__ int s_ticket;
  constexpr int TPT = MS ? 1 : 2;
  const bool fused = A.tickets != nullptr;                 // uniform over the grid
  const int split = blockIdx.x, kvh = blockIdx.y, rt = blockIdx.z;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // a scalar: tile indices and page pointers are wave uniform
  const int lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
  int pos; bool row_ok = true;
  if (MS) {
    pos = A.rows.pos[rt];
    const int slot = A.rows.slot[rt];
    row_ok = pos >= 0 && pos < A.kv.max_ctx && slot >= 0 && slot < A.rows.n_slots;   // a bad row reads nothing and yields zeros
    A.kv = slot_view(A.kv, A.rows, row_ok ? slot : 0);
  } else {
    pos = *A.d_pos;
  }

  // query row of this lane column: j = i -> (token TPT*rt + i/6, head kvh*6 + i%6); the other columns are padding
  const int tl = TPT * rt + i / kG;                // token index inside the slice
  const bool vrow = i < TPT * kG && tl < A.M && row_ok;
  const int head = kvh * kG + i % kG;
  int len = 0;
  if (vrow) {
    if (MS) len = pos + 1;
    else { const int tg = A.tok0 + tl; len = pos + (A.depth ? (int)A.depth[tg] : tg) + 1; }
    len = min(len, A.kv.max_ctx);
  }
  int maxlen = len, minlen = vrow ? len : 0x7fffffff;
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) { maxlen = max(maxlen, __shfl_xor(maxlen, o, 64)); minlen = min(minlen, __shfl_xor(minlen, o, 64)); }
  maxlen = __builtin_amdgcn_readfirstlane(maxlen); minlen = __builtin_amdgcn_readfirstlane(minlen);
  // The grid is sized for long contexts; how many of its splits a row tile uses follows from the length it finds on the
  // device: at least two 32-key tiles per workgroup.  The other workgroups leave the "no keys" marker and exit, and
  // the combiner does not read their rows.
  const int ntiles = (maxlen + 31) >> 5;
  const int s_used = min(A.S, max(1, ntiles >> 1));
  if (split >= s_used) {
    const int j = threadIdx.x, tj = TPT * rt + j / kG;
    if (j < TPT * kG && tj < A.M) {
      const size_t p = ((size_t)tj * A.S + split) * A.n_heads + kvh * kG + j % kG;
      if (fused) { st_agent(A.pm + p, -1e30f); st_agent(A.pl + p, 0.f); }
      else { A.pm[p] = -1e30f; A.pl[p] = 0.f; }
    }
    if (fused && last_of_column(A, &s_ticket)) {
      if (A.S <= 64) combine_column<TPT, 4>(A, kvh, rt, &s_acc[0][0][0]); else combine_column<TPT, 16>(A, kvh, rt, &s_acc[0][0][0]);
    }
    return;
  }
  const int tps = (ntiles + s_used - 1) / s_used;
  const int tile0 = split * tps, tile1 = min(ntiles, tile0 + tps);

  // ---- fused quantize-on-append (decode, M <= 2, one row tile): a row of this pass is written by the one workgroup
  //      whose tile range holds it - the only workgroup of this kv head that will read it in this launch.  Writer and
  //      readers are waves of one workgroup, i.e. of one CU and one (write-through) L1, so workgroup-scope fences
  //      around the barrier order the stores before the loads without any cache maintenance. ----
  if (!MS && A.k16) {
    bool mine = false;
    for (int t = 0; t < A.M; ++t) {
      const int r = pos + A.tok0 + t;              // k16/v16 point at row 0 of the pass, this slice starts at row tok0
      // A row no query row of this launch can see (a depth table may say so) lies past the last tile when it opens a new
      // one: nobody reads it now, the last workgroup in use stores it.  All conditions are uniform over the workgroup.
      const bool held = (r >> 5) >= tile0 && (r >> 5) < tile1, unseen = (r >> 5) >= ntiles && split == s_used - 1;
      if (r < 0 || r >= A.kv.max_ctx || !(held || unseen)) continue;
      mine = true;
      const bool isv = threadIdx.x >= 128;
      const uint16_t* src = (isv ? A.v16 : A.k16) + ((size_t)(A.tok0 + t) * A.kv.n_kv + kvh) * kD;
      quant_store_row(A.kv, kvh, r, isv, src, threadIdx.x & 127);
    }
    if (mine) {                      // uniform over the workgroup
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __syncthreads();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
  }

  // Q fragments: B operand of S^T = K Q^T.  MFMA step m (= scale group m), lane (row i, lane group g), element e
  // <-> channel 32m + 8g + pi(e), pi = [0,4,1,5,2,6,3,7] (the order dq_dword_int produces); odd channels carry 1/4, even ones 4.
  // The four loads are written as instructions and only requested here: the first tiles are requested right behind them
  // and q_ready<N> then waits for the query alone, leaving the N tile loads in flight - one trip to memory before the
  // first MFMA instead of two.  Padding lanes read row 0 of the slice (memory that exists) and drop it.
  // q_ready is called once in every branch below.  It does not name the query registers as operands of its wait (a
  // wait site per branch that redefines them makes the compiler place copies of the registers in front of one of the
  // waits, i.e. copies of registers whose loads are still in flight); instead the wait hands out a zero that is OR-ed
  // into the raw words, so that nothing computed from them can be scheduled ahead of it.
  h8 qf[4];
  f4 kinit[4];                 // initial accumulators of the score MFMAs: the code offset -8, see dq_dword_sub
  u32x4 qraw[4];
  {
    const uint16_t* qrow = A.q16 + (vrow ? ((size_t)tl * A.n_heads + head) * kD : (size_t)0) + 8 * g;
#pragma unroll
    for (int m = 0; m < 4; ++m) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qraw[m]) : "v"(qrow + 32 * m));
  }
  auto q_ready = [&](auto n_younger) __attribute__((always_inline)) {
    uint32_t z;
    asm volatile("s_waitcnt vmcnt(%1)\n\tv_mov_b32 %0, 0" : "=v"(z) : "n"(decltype(n_younger)::value));
    // the odd nibble of a byte enters the MFMA as 16 n: its query channels carry 1/4 and the others 4, so that both
    // kinds of products are 4 q n and neither factor costs fp16 range at one end only (a plain 1/16 on the odd channels
    // pushes queries below 1e-3 into the subnormals); the 4 leaves with the softmax scale
    const _Float16 se = (_Float16)4.f, so = (_Float16)0.25f;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const h8 c = __builtin_bit_cast(h8, vrow ? (qraw[m] | u32x4{z, z, z, z}) : u32x4{0u, 0u, 0u, 0u});
      qf[m] = h8{c[0] * se, c[4] * se, c[1] * so, c[5] * so, c[2] * se, c[6] * se, c[3] * so, c[7] * so};
      // -8 * 2^-24 * (sum of the row's 32 query channels of group m): the lane's 8 channels, then its 3 sister lanes
      float qs = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) qs += (float)c[e];
      qs += __shfl_xor(qs, 16, 64);
      qs += __shfl_xor(qs, 32, 64);
      const float c0 = -32.f * kTwoM24 * qs;       // -8 per code, in the units of the products: 4 q n 2^-24
      kinit[m] = f4{c0, c0, c0, c0};
    }
  };
  const float sc_log2 = 0.25f * kTwo24 * kLog2e / sqrtf((float)kD);   // scores carry the 2^-24 of the subnormal codes and the 4 of the query fragments

  float m_run = -1e30f, l_run = 0.f;
  f4 o[8];
#pragma unroll
  for (int b = 0; b < 8; ++b) o[b] = f4{0.f, 0.f, 0.f, 0.f};

  const LaneOffs offs = lane_offs(i, g);
  uint32_t magic = kMagic;
  asm volatile("" : "+v"(magic));
  // one 32-key tile: scores, online softmax, O += P V
  auto tile = [&](const int T, const RawTile& cur) __attribute__((always_inline)) {
    const int t0 = T << 5;
    const bool need_mask = t0 + 32 > minlen;         // wave uniform: only the last tiles of a row can hold keys past its length
    // ---- scores: two 16-key MFMA tiles; step m contracts scale group m, its fp32 sum is scaled afterwards ----
    float s[8];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const uint32_t w[4] = {cur.kw[kt][0], cur.kw[kt][1], cur.kw[kt][2], cur.kw[kt][3]};
      f4 part[4];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        h2 k4[4];
        dq_dword_sub(w[m], k4);
        const h8 kf = h8{k4[0][0], k4[0][1], k4[1][0], k4[1][1], k4[2][0], k4[2][1], k4[3][0], k4[3][1]};
        part[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[m], kinit[m], 0, 0, 0);
      }
      // part[m][r] = sum over group m of q * code for key t0 + 16kt + 4g + r and row i
      const uint32_t sw[8] = {cur.ks[kt][0][0], cur.ks[kt][0][1], cur.ks[kt][0][2], cur.ks[kt][0][3],
                              cur.ks[kt][1][0], cur.ks[kt][1][1], cur.ks[kt][1][2], cur.ks[kt][1][3]};
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const h2 s01 = as_h2(sw[2 * r]), s23 = as_h2(sw[2 * r + 1]);
        float dot = __builtin_fmaf(part[0][r], (float)s01[0], 0.f);
        dot = __builtin_fmaf(part[1][r], (float)s01[1], dot);
        dot = __builtin_fmaf(part[2][r], (float)s23[0], dot);
        dot = __builtin_fmaf(part[3][r], (float)s23[1], dot);
        s[4 * kt + r] = dot;                           // raw units; log2(e)/sqrt(d) is folded into the exponent below
      }
    }
    if (need_mask) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { const int key = t0 + 16 * (e >> 2) + 4 * g + (e & 3); s[e] = key < len ? s[e] : -INFINITY; }
    }
    // ---- online softmax (one running maximum per row, shared by its 4 lane groups) ----
    float tmax = s[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) tmax = fmaxf(tmax, s[e]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax * sc_log2);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);    // 0 on the first tile (m_run = -1e30): nothing to rescale yet
    const bool first = m_run < -1e29f;
    m_run = m_new;
    if (__any(alpha != 1.f && !first)) {
      l_run *= alpha;
#pragma unroll
      for (int b = 0; b < 8; ++b) { o[b][0] *= alpha; o[b][1] *= alpha; o[b][2] *= alpha; o[b][3] *= alpha; }
    }
    h8 pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) { const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], sc_log2, -m_new)); l_run += p; pf[e] = (_Float16)p; }
    // ---- O^T += V^T P^T : 8 MFMAs, MFMA b covers channels 8*i' + b ----
    h2 va[8][4];
#pragma unroll
    for (int pe = 0; pe < 4; ++pe) {
      const uint32_t spk = cur.vs[pe >> 1][pe & 1];                            // scales of tokens (2pe, 2pe+1) of this lane
      const h2 s2 = as_h2(spk), s2q = s2 * h2{(_Float16)0.0625f, (_Float16)0.0625f};
      const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f}, c1152 = {(_Float16)1152.f, (_Float16)1152.f};
      const uint32_t w0 = cur.vw[2 * pe], w1 = cur.vw[2 * pe + 1];
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        // byte bb of both tokens side by side: low half = token 2pe, high half = token 2pe+1
        const uint32_t x = __builtin_amdgcn_perm(w1, w0, 0x0c040c00u + bb * 0x00010001u);
        va[2 * bb][pe] = (as_h2(nib(x, 0x000f000fu, magic)) - c1032) * s2;
        va[2 * bb + 1][pe] = (as_h2(nib(x, 0x00f000f0u, magic)) - c1152) * s2q;
      }
    }
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const h8 vf = h8{va[b][0][0], va[b][0][1], va[b][1][0], va[b][1][1], va[b][2][0], va[b][2][1], va[b][3][0], va[b][3][1]};
      o[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, o[b], 0, 0, 0);
    }
  };
  // The wave's tiles are T0, T0 + 4, ...; while it works on one, the next is in flight in the other register set.  Every
  // branch here is wave uniform, so the number of loads in flight at each wait is known: 16 if a younger tile was
  // requested, 0 otherwise.  The wait that names the tile's registers is unconditional (a conditional one would make
  // the compiler merge two versions of those registers, with copies placed before the wait); when there is no younger
  // tile a full wait without operands precedes it.
  {
    RawTile ta, tb;
    auto request = [&](int T, RawTile& r) __attribute__((always_inline)) { load_tile(kv_page_uniform(A.kv, kvh, T << 5), (T << 5) % kPageTok, offs, r); };
    const int T0 = tile0 + wave;
    if (T0 + 8 < tile1) {                              // three tiles or more: the next tile is always in flight
      request(T0, ta);
      request(T0 + 4, tb);
      q_ready(std::integral_constant<int, 2 * kTileLoads>{});
      for (int T = T0; T < tile1; T += 8) {
        if (T + 4 >= tile1) asm volatile("s_waitcnt vmcnt(0)");
        wait_tile<kTileLoads>(ta);
        tile(T, ta);
        if (T + 8 < tile1) request(T + 8, ta);
        if (T + 4 >= tile1) break;
        if (T + 8 >= tile1) asm volatile("s_waitcnt vmcnt(0)");
        wait_tile<kTileLoads>(tb);
        tile(T + 4, tb);
        if (T + 12 < tile1) request(T + 12, tb);
      }
    } else if (T0 < tile1) {
      // one or two tiles (single-stream decode up to 32k): the second is requested after the first has been used -
      // measured 2 % faster than both at once.  Separate registers and no loop: nothing for the compiler to merge.
      RawTile t1;
      request(T0, t1);
      q_ready(std::integral_constant<int, kTileLoads>{});
      wait_tile<0>(t1);
      tile(T0, t1);
      if (T0 + 4 < tile1) {
        RawTile t2;
        request(T0 + 4, t2);
        wait_tile<0>(t2);
        tile(T0 + 4, t2);
      }
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // a wave without tiles: the query requests are answered before their registers are given up
    }
  }
  // ---- merge the 4 waves of the workgroup, write one partial per (row, split) ----
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (g == 0) { s_m[wave][i] = m_run; s_l[wave][i] = l_run; }
  // o[b][r] of lane (row i, group g) is channel 8 (4g + r) + b: eight consecutive channels per r, two 16-byte writes
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float* d = &s_acc[wave][i][8 * (4 * g + r)];
    *reinterpret_cast<float4*>(d) = make_float4(o[0][r], o[1][r], o[2][r], o[3][r]);
    *reinterpret_cast<float4*>(d + 4) = make_float4(o[4][r], o[5][r], o[6][r], o[7][r]);
  }
  __syncthreads();
  // 16 lanes per row, 8 channels each: one 16-byte store per lane
  if (threadIdx.x < TPT * kG * 16) {
    const int j = threadIdx.x >> 4, c8 = (threadIdx.x & 15) * 8;
    const int tj = TPT * rt + j / kG;
    if (tj < A.M) {
      const float m0 = s_m[0][j], m1 = s_m[1][j], m2 = s_m[2][j], m3 = s_m[3][j];
      const float M2 = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));
      const float w[4] = {exp2f(m0 - M2), exp2f(m1 - M2), exp2f(m2 - M2), exp2f(m3 - M2)};
      const size_t p = ((size_t)tj * A.S + split) * A.n_heads + kvh * kG + j % kG;
      const float L = w[0] * s_l[0][j] + w[1] * s_l[1][j] + w[2] * s_l[2][j] + w[3] * s_l[3][j];
      float4 a0[4], a1[4];                                    // all eight reads first: one LDS round trip, not eight
#pragma unroll
      for (int wv = 0; wv < 4; ++wv) { a0[wv] = *reinterpret_cast<const float4*>(&s_acc[wv][j][c8]); a1[wv] = *reinterpret_cast<const float4*>(&s_acc[wv][j][c8 + 4]); }
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int wv = 0; wv < 4; ++wv) {
        acc[0] += w[wv] * a0[wv].x; acc[1] += w[wv] * a0[wv].y; acc[2] += w[wv] * a0[wv].z; acc[3] += w[wv] * a0[wv].w;
        acc[4] += w[wv] * a1[wv].x; acc[5] += w[wv] * a1[wv].y; acc[6] += w[wv] * a1[wv].z; acc[7] += w[wv] * a1[wv].w;
      }
      const float inv = L > 0.f ? 1.f / L : 0.f;            // one division per lane, not one per channel
      h8 v;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (_Float16)(acc[e] * inv);
      if (fused) {
        st_agent16(A.pacc16 + p * kD + c8, __builtin_bit_cast(uint4, v));
        if (c8 == 0) { st_agent(A.pm + p, M2); st_agent(A.pl + p, L); }
      } else {
        *reinterpret_cast<uint4*>(A.pacc16 + p * kD + c8) = __builtin_bit_cast(uint4, v);
        if (c8 == 0) { A.pm[p] = M2; A.pl[p] = L; }
      }
    }
  }
  if (fused && last_of_column(A, &s_ticket)) {   // the barrier inside also ends every read of s_acc above
    if (A.S <= 64) combine_column<TPT, 4>(A, kvh, rt, &s_acc[0][0][0]); else combine_column<TPT, 16>(A, kvh, rt, &s_acc[0][0][0]);
  }
}

void launch_attend_narrow(const AttnArgs& A, hipStream_t st) {
  if (A.rows.pos) hipLaunchKernelGGL(attend_narrow_kernel<true>, dim3(A.S, A.kv.n_kv, A.M), dim3(256), 0, st, A);
  else hipLaunchKernelGGL(attend_narrow_kernel<false>, dim3(A.S, A.kv.n_kv, (A.M + 1) / 2), dim3(256), 0, st, A);
}

// combiner (reference: src/attention_kv4q.cu:325-332): M2 = max pm; w_s = pm_s > -1e29 ? 2^(pm_s - M2) * pl_s : 0;
// y = sum w_s * (acc_s / l_s) / sum w_s.  grid (n_heads, M), block 256: 16 lanes x 8 channels cover a row, 16 split
// lanes run in parallel and are summed through LDS.  S <= 256.
// kInFlight = partial rows a split lane requests before it uses any: 16 covers 256 splits in one memory round trip, 8
// covers the 128 splits of decode over long contexts (few, long workgroups); 4 keeps the register count low where
// thousands of workgroups run (wide windows).
template <int kInFlight>
__global__ void __launch_bounds__(256) combine_kernel(CombineArgs A) {
  __shared__ float s_w[256];
  __shared__ float s_o[16][kD + 4];
  __shared__ float s_wsum[16];
  const int head = blockIdx.x, tok = blockIdx.y, tid = threadIdx.x;
  const size_t p0 = (size_t)tok * A.S * A.n_heads + head;      // split s lives at p0 + s * n_heads
  // 16 split lanes; each takes splits sl, sl+16, ... (at most kInFlight of them: the launcher picks kInFlight so that
  // 16 * kInFlight >= S).  Their partial rows are requested first, together with the (m, l) pairs the weights come
  // from: one memory round trip instead of two.  A row of weight 0 may be one that no workgroup wrote: it is zeroed
  // before use.
  const int sl = tid >> 4, c8 = (tid & 15) * 8;
  const uint16_t* src = A.pacc16 + p0 * kD + c8;
  const size_t stride = (size_t)A.n_heads * kD;
  uint4 u[kInFlight];
#pragma unroll
  for (int k = 0; k < kInFlight; ++k) {
    const int sp = sl + 16 * k;
    u[k] = sp < A.S ? *reinterpret_cast<const uint4*>(src + (size_t)sp * stride) : make_uint4(0, 0, 0, 0);
  }
  // weights: every thread looks at one split
  float pmv = -1e30f, plv = 0.f;
  if (tid < A.S) { pmv = A.pm[p0 + (size_t)tid * A.n_heads]; plv = A.pl[p0 + (size_t)tid * A.n_heads]; }
  float M2 = pmv;
#pragma unroll
  for (int o = 32; o; o >>= 1) M2 = fmaxf(M2, __shfl_xor(M2, o, 64));
  if ((tid & 63) == 0) s_wsum[tid >> 6] = M2;
  __syncthreads();
  M2 = fmaxf(fmaxf(s_wsum[0], s_wsum[1]), fmaxf(s_wsum[2], s_wsum[3]));
  s_w[tid] = (tid < A.S && pmv > -1e29f) ? exp2f(pmv - M2) * plv : 0.f;
  __syncthreads();
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float wsum = 0.f;
#pragma unroll
  for (int k = 0; k < kInFlight; ++k) {
    const int sp = sl + 16 * k;
    const float w = sp < A.S ? s_w[sp] : 0.f;
    const uint4 r = w != 0.f ? u[k] : make_uint4(0, 0, 0, 0);
    const h8 v = __builtin_bit_cast(h8, r);
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] += w * (float)v[c];
    wsum += w;
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) s_o[sl][c8 + c] = acc[c];
  if ((tid & 15) == 0) s_wsum[sl] = wsum;
  __syncthreads();
  float y = 0.f;
  if (tid < kD) {
    float o = 0.f, L = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) { o += s_o[k][tid]; L += s_wsum[k]; }
    y = L > 0.f ? o / L : 0.f;                     // a row that saw no key at all (a rejected row of a multi-stream pass)
  }
  if (A.unrot) {                                   // uniform over the grid
    // inverse signed Hadamard rotation over the row's 128 channels (threads 0..127 = two waves)
#pragma unroll
    for (int h = 1; h < 64; h *= 2) {
      const float b = __shfl_xor(y, h, 64);
      y = (tid & h) ? b - y : y + b;
    }
    __syncthreads();
    if (tid < kD) s_w[tid] = y;
    __syncthreads();
    if (tid < kD) {
      const float b = s_w[tid ^ 64];
      y = (tid & 64) ? b - y : y + b;
      y = y * 0.0625f * channel_sign(tid);         // signs last on the way back (src/kvx_codec.cuh:28-32)
    }
  }
  if (tid < kD) A.out16[((size_t)tok * A.n_heads + head) * kD + tid] = A.out_bf16 ? f2bf_bits(y) : __half_as_ushort(__float2half_rn(y));
}
// The combiner for wide passes (many rows, at most 32 splits, no un-rotation): one wave per (token, head) row, four
// waves per workgroup, no LDS and no barrier.  Lane = (split lane 0..3, 8 channels); a split lane takes splits sl, sl + 4,
// ... (at most 8), requests their rows together with the (m, l) pairs, and the four split lanes are summed by two
// cross-lane exchanges.  Same arithmetic as combine_kernel up to the order of the sums.
__global__ void __launch_bounds__(256) combine_rows_kernel(CombineArgs A) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);               // row = tok * n_heads + head
  if (row >= A.M * A.n_heads) return;
  const int tok = row / A.n_heads, head = row % A.n_heads, lane = threadIdx.x & 63, sl = lane >> 4, c8 = (lane & 15) * 8;
  const size_t p0 = (size_t)tok * A.S * A.n_heads + head;
  const size_t stride = (size_t)A.n_heads * kD;
  uint4 u[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int sp = sl + 4 * k;
    u[k] = sp < A.S ? *reinterpret_cast<const uint4*>(A.pacc16 + p0 * kD + (size_t)sp * stride + c8) : make_uint4(0, 0, 0, 0);
  }
  // lane t < S looks at split t; the maximum and every weight then come from cross-lane reads
  float pmv = -1e30f, plv = 0.f;
  if (lane < A.S) { pmv = A.pm[p0 + (size_t)lane * A.n_heads]; plv = A.pl[p0 + (size_t)lane * A.n_heads]; }
  float M2 = pmv;
#pragma unroll
  for (int o = 32; o; o >>= 1) M2 = fmaxf(M2, __shfl_xor(M2, o, 64));
  const float wl = (lane < A.S && pmv > -1e29f) ? exp2f(pmv - M2) * plv : 0.f;     // weight of split `lane`
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float wsum = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int sp = sl + 4 * k;                                       // < 32: a lane of this wave
    const float w = __shfl(wl, sp, 64);
    const uint4 r = w != 0.f ? u[k] : make_uint4(0, 0, 0, 0);         // a row of weight 0 may be one that no workgroup wrote
    const h8 v = __builtin_bit_cast(h8, r);
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] += w * (float)v[c];
    wsum += w;
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) { acc[c] += __shfl_xor(acc[c], 16, 64); acc[c] += __shfl_xor(acc[c], 32, 64); }
  wsum += __shfl_xor(wsum, 16, 64); wsum += __shfl_xor(wsum, 32, 64);
  if (sl == 0) {
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
    float yv[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) yv[c] = acc[c] * inv;
    *reinterpret_cast<uint4*>(A.out16 + (size_t)row * kD + c8) = pack_out8(yv, A.out_bf16);
  }
}
void launch_combine(const CombineArgs& A, hipStream_t st) {
  if (A.S <= 32 && !A.unrot && A.M >= 8) { hipLaunchKernelGGL(combine_rows_kernel, dim3((A.M * A.n_heads + 3) / 4), dim3(256), 0, st, A); return; }
  if (A.S > 128) hipLaunchKernelGGL(combine_kernel<16>, dim3(A.n_heads, A.M), dim3(256), 0, st, A);   // S <= 256
  else if (A.S > 64) hipLaunchKernelGGL(combine_kernel<8>, dim3(A.n_heads, A.M), dim3(256), 0, st, A);
  else hipLaunchKernelGGL(combine_kernel<4>, dim3(A.n_heads, A.M), dim3(256), 0, st, A);
}

}  // namespace yka
