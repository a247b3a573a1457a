// Split-KV attention over the reference's own 256-channel rows for windows of 3..64 query tokens.  gfx950.
//
// Same mathematics as attend256_kernel (one fp32 scale per row: the score of a key is the integer dot product times its
// scale, the V scale of a key rides on its probability; reference window shape src/q35_atxpk4.cuh:71-499, row geometry
// src/q35_atxpk.cu:391-411).  What differs is who dequantizes, as in the 128-channel wide kernel:
//   * a workgroup of 8 waves owns 128 query rows (token-major, 6 heads per token) and one split of the keys; every
//     32-key tile is dequantized ONCE per workgroup into LDS - K as exact integer codes in fp16, V as exact integer
//     codes transposed (channel-major, the operand shape of the token-contracting MFMA), both scale vectors as they are;
//   * a wave owns 16 rows (MFMA 16x16x32: 16 accumulator tiles of 4 registers cover the 256 output channels, the query
//     fragments take 32 registers), so that two waves fit a SIMD;
//   * LDS is double buffered: tile n+1 is dequantized while tile n is consumed; one barrier per tile; the tile loads are
//     explicit instructions two tiles ahead with their own waits;
//   * quantize-on-append rides in the launch: a workgroup stores the rows of the pass that fall into the tiles of its own
//     split before it reads them (32 lanes per row, a word of 8 channels each).
// LDS image of one tile (42240 bytes):
//   K  [32 keys][544 B]    chunk c (16 bytes) of a key = word c of its row = channels 8c + [7,3,6,2,5,1,4,0]
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
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
__device__ __forceinline__ uint32_t as_u32(h2 h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ uint32_t nib(uint32_t w, uint32_t magic) { return (w & 0x000f000fu) | (magic & ~0x000f000fu); }

constexpr int kD2 = 256;
constexpr int kP2Kw = 0, kP2Vw = 32768, kP2Ks = 65536, kP2Vs = 66560;
constexpr uint32_t kMagic = 0x64006400u;
constexpr float kLog2e = 1.4426950408889634f;
constexpr int NT = 512;                        // threads per workgroup (8 waves x 16 rows)
// Row pitches: a 128-bit LDS read of a wave is served 16 lanes at a time, and the 16 are lanes {0-7, 24-31}, {8-15, 16-23}
// (and the same in the upper half) - measured.  With lane = row i + 16 * group g, i.e. (i 0-7, g) together with
// (i 8-15, g+1), the 16 lanes of a pass fall into 16 different 4-bank groups iff the pitch is 2 * odd chunks of 16 bytes:
// 34 chunks for K rows, 6 for V rows.  (33 and 5 chunks, free of conflicts for 16 consecutive lanes, measure a 2-way
// conflict on every fragment read.)
constexpr int kKPitch = 544, kVPitch = 96;
constexpr int kLdsK = 0, kLdsV = 32 * kKPitch, kLdsS = kLdsV + kD2 * kVPitch, kLdsBuf = kLdsS + 256;   // 42240
constexpr float kRaise = 8.f;                  // log2 slack before a running maximum is raised

__device__ __forceinline__ uint8_t* page256w(const KvView& kv, int kvh, int t) {
  const int lp = t / kPageTok;
  int pp = lp;
  if (kv.table) pp = table_entry_scalar(kv.table, lp);
  return kv.base + (size_t)(pp * kv.n_kv + kvh) * kPage256Bytes;
}

struct Raw {                                   // one thread's share of a raw 32-key tile
  uint32_t kw[2];                              // K words c, c+16 of key tid/16 (c = tid%16)
  uint32_t vw[2];                              // V word tid/16 of keys 2*(tid%16), 2*(tid%16)+1
  uint32_t sc;                                 // (tid & 63) < 32: K scale of key tid&31, else V scale of key tid&31
};
struct LaneOffs { uint32_t k, v, sc; };
__device__ __forceinline__ LaneOffs lane_offs(int tid) {
  const uint32_t t6 = tid & 63;
  return LaneOffs{kP2Kw + (uint32_t)(tid >> 4) * 128u + (uint32_t)(tid & 15) * 4u, kP2Vw + (uint32_t)(tid & 15) * 256u + (uint32_t)(tid >> 4) * 4u,
                  (t6 < 32 ? kP2Ks : kP2Vs) + (t6 & 31) * 4u};
}
// Loads as instructions ("wave-uniform base in scalar registers + 32-bit lane offset"), so that they can stay in flight
// across loop steps with a wait of their own: wait_raw<N> leaves the N younger loads in flight.
__device__ __forceinline__ void load_raw(const uint8_t* pg, int tp, const LaneOffs& L, Raw& R) {
  const uint8_t* rows = pg + (uint32_t)tp * 128u;          // code rows of the tile (K and V planes)
  const uint8_t* sc = pg + (uint32_t)tp * 4u;              // scale entries of the tile
  asm volatile("global_load_dword %0, %1, %2" : "=v"(R.kw[0]) : "v"(L.k), "s"(rows));
  asm volatile("global_load_dword %0, %1, %2 offset:64" : "=v"(R.kw[1]) : "v"(L.k), "s"(rows));
  asm volatile("global_load_dword %0, %1, %2" : "=v"(R.vw[0]) : "v"(L.v), "s"(rows));
  asm volatile("global_load_dword %0, %1, %2 offset:128" : "=v"(R.vw[1]) : "v"(L.v), "s"(rows));
  asm volatile("global_load_dword %0, %1, %2" : "=v"(R.sc) : "v"(L.sc), "s"(sc));
}
template <int N>
__device__ __forceinline__ void wait_raw(Raw& R) {
  asm volatile("s_waitcnt vmcnt(%5)" : "+v"(R.kw[0]), "+v"(R.kw[1]), "+v"(R.vw[0]), "+v"(R.vw[1]), "+v"(R.sc) : "n"(N));
}

// 8 codes of a word (MSB-first 4-bit fields) -> 8 fp16 integers n-8 in the element order [7,3,6,2,5,1,4,0]
__device__ __forceinline__ uint4 dq_word(uint32_t w, uint32_t magic) {
  const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f};
  uint4 o;
  o.x = as_u32(as_h2(nib(w, magic)) - c1032);
  o.y = as_u32(as_h2(nib(w >> 4, magic)) - c1032);
  o.z = as_u32(as_h2(nib(w >> 8, magic)) - c1032);
  o.w = as_u32(as_h2(nib(w >> 12, magic)) - c1032);
  return o;
}

__device__ __forceinline__ void dequant_to_lds(uint8_t* buf, int tid, const Raw& R, uint32_t magic) {
  const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f};
  {                                            // K: words c and c+16 of one key -> two 16-byte chunks; 16 lanes write 256 contiguous bytes
    const int key = tid >> 4, c = tid & 15;
    uint8_t* dst = buf + kLdsK + key * kKPitch + c * 16;
    *reinterpret_cast<uint4*>(dst) = dq_word(R.kw[0], magic);
    *reinterpret_cast<uint4*>(dst + 256) = dq_word(R.kw[1], magic);
  }
  {                                            // V: word w of keys (2kp, 2kp+1) -> 8 channel rows, two adjacent key slots each.
    // The 16 key pairs are the fast lane index: the lanes of a wave write 16 consecutive dwords of 4 rows (a 2-way bank
    // conflict); with the word as the fast index 16 lanes would hit one bank.
    const int w = tid >> 4, key = 2 * (tid & 15);
    const int slot = 8 * ((key >> 2) & 3) + 4 * (key >> 4) + (key & 3);
    uint8_t* vb = buf + kLdsV + (8 * w) * kVPitch + slot * 2;
#pragma unroll
    for (int bb = 0; bb < 4; ++bb) {
      // byte bb of both keys side by side (low half = key 2kp, high half = key 2kp+1): its low nibble is element 7-2bb
      // of the word, its high nibble element 6-2bb
      const uint32_t x = __builtin_amdgcn_perm(R.vw[1], R.vw[0], 0x0c040c00u + bb * 0x00010001u);
      *reinterpret_cast<uint32_t*>(vb + (7 - 2 * bb) * kVPitch) = as_u32(as_h2(nib(x, magic)) - c1032);
      *reinterpret_cast<uint32_t*>(vb + (6 - 2 * bb) * kVPitch) = as_u32(as_h2(nib(x >> 4, magic)) - c1032);
    }
  }
  reinterpret_cast<uint32_t*>(buf + kLdsS)[tid & 63] = R.sc;      // waves repeat each other (no divergent branch)
}

// One 256-channel row by 32 lanes: lane c holds channels 8c .. 8c+7 as 8 fp16 in `raw` and builds word c.  Bit-identical
// to the row quantizer of the append kernel: the maximum of the row is exact in any order, everything behind it is the
// same sequence of IEEE operations per channel.  All 32 lanes of the row call it; `store` is uniform over them.
__device__ __forceinline__ void quant_store_word256(const KvView& kv, int kvh, int pos, bool isv, uint4 raw, int c, bool store) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  float x[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = __half2float(__ushort_as_half((uint16_t)(w[e >> 1] >> (16 * (e & 1)))));
  float am = fabsf(x[0]);
#pragma unroll
  for (int e = 1; e < 8; ++e) am = fmaxf(am, fabsf(x[e]));
#pragma unroll
  for (int o = 1; o < 32; o <<= 1) am = fmaxf(am, __shfl_xor(am, o, 64));
  float s7 = __fdiv_rn(am, 7.f);
  if (s7 == 0.f) s7 = 1.f;
  uint32_t word = 0u;                          // channel 8c + e in bits [28 - 4e, 32 - 4e): the first field on top
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float q = rintf(__fdiv_rn(x[e], s7));
    q = fminf(fmaxf(q, -7.f), 7.f);
    word |= (uint32_t)((int)q + 8) << (28 - 4 * e);
  }
  if (store) {
    const int lp = pos / kPageTok, tp = pos % kPageTok;
    const int pp = kv.table ? kv.table[lp] : lp;             // rows of one wave may lie in two pages: a load per lane
    uint8_t* pg = kv.base + (size_t)(pp * kv.n_kv + kvh) * kPage256Bytes;
    reinterpret_cast<uint32_t*>(pg + (isv ? kP2Vw : kP2Kw))[tp * 32 + c] = word;
    if (c == 0) reinterpret_cast<float*>(pg + (isv ? kP2Vs : kP2Ks))[tp] = s7;
  }
}

}  // namespace

// grid (S, n_kv, ceil(6M / 128)), block 512; wave w owns rows [16 w, 16 (w+1)) of the block
__global__ void __launch_bounds__(NT, 1) attend256_wide_kernel(AttnArgs A) {
  __shared__ __align__(16) uint8_t lds[2][kLdsBuf];
  const int split = blockIdx.x, kvh = blockIdx.y, rb = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int pos = *A.d_pos;
  const int nrows = kG * A.M;
  constexpr int RPB = 128;

  // row of this lane column: R = rb*128 + wave*16 + i  ->  token R/6 of the slice, head kvh*6 + R%6
  const int row0 = rb * RPB + wave * 16;
  const int R = row0 + i;
  const bool vrow = R < nrows;
  const int tl = R / kG, head = kvh * kG + R % kG;
  int len = 0;
  if (vrow) { const int tg = A.tok0 + tl; len = min(pos + (A.depth ? (int)A.depth[tg] : tg) + 1, A.kv.max_ctx); }
  // Q fragments: k-step t of 8, lane (row i, group g), element e <-> channel 8 (4t + g) + [7,3,6,2,5,1,4,0][e]
  h8 qf[8];
  {
    const uint16_t* qrow = A.q16 + ((size_t)tl * A.n_heads + head) * kD2 + 8 * g;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      uint4 u = vrow ? *reinterpret_cast<const uint4*>(qrow + 32 * t) : make_uint4(0, 0, 0, 0);
      const h8 c = __builtin_bit_cast(h8, u);
      qf[t] = h8{c[7], c[3], c[6], c[2], c[5], c[1], c[4], c[0]};
    }
  }
  const bool has_rows = row0 < nrows;                       // wave uniform

  // key range of the workgroup: its splits cut [0, maxlen) of the block's longest row into 32-key tiles
  const int tok_lo = (rb * RPB) / kG, tok_hi = min(A.M, (rb * RPB + RPB + kG - 1) / kG);
  int maxdep = 0, mindep = 0x7fffffff;
  for (int t = tok_lo; t < tok_hi; ++t) { const int tg = A.tok0 + t; const int dp = A.depth ? (int)A.depth[tg] : tg; maxdep = max(maxdep, dp); mindep = min(mindep, dp); }
  const int maxlen = min(pos + maxdep + 1, A.kv.max_ctx), minlen = min(pos + mindep + 1, A.kv.max_ctx);
  const int ntiles = (maxlen + 31) >> 5, tps = (ntiles + A.S - 1) / A.S;
  const int tile0 = split * tps, tile1 = min(ntiles, tile0 + tps);

  // ---- fused quantize-on-append (a slice of at most 64 tokens): a workgroup stores the rows of this pass that lie in
  //      the tiles of its own range before it reads them, so no workgroup reads a row another one has to store.  Row
  //      blocks of one kv head write identical bytes where their ranges overlap.  A row past the last tile of the last
  //      row block (no query row of the pass sees it: a depth table may say so) is stored by that block's last split.
  //      Writer and readers are waves of one CU and one write-through L1: workgroup-scope fences order the stores.
  //      Every condition that guards the barrier is uniform over the workgroup. ----
  if (A.k16) {
    static_assert(kMaxSlice <= 64, "8 steps of 16 rows cover K and V of a slice");
    const int r0 = pos + A.tok0;
    const int Tn0 = r0 >> 5, Tn1 = (r0 + A.M - 1) >> 5;
    const bool last_wg = split == A.S - 1 && rb == (int)gridDim.z - 1;
    if ((Tn0 < tile1 && Tn1 >= tile0) || (last_wg && Tn1 >= ntiles)) {
      const int slot = tid >> 5, c = tid & 31;
      uint4 rawv[8];
      bool mine[8];
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int hh = it * 16 + slot, t = hh >> 1, r = r0 + t, T = r >> 5;
        mine[it] = t < A.M && r >= 0 && r < A.kv.max_ctx && ((T >= tile0 && T < tile1) || (last_wg && T >= ntiles));
        const uint16_t* src = ((hh & 1) ? A.v16 : A.k16) + ((size_t)(A.tok0 + t) * A.kv.n_kv + kvh) * kD2 + 8 * c;
        rawv[it] = mine[it] ? *reinterpret_cast<const uint4*>(src) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int hh = it * 16 + slot;
        quant_store_word256(A.kv, kvh, r0 + (hh >> 1), hh & 1, rawv[it], c, mine[it]);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __syncthreads();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      asm volatile("" ::: "memory");           // the tile loads below are instructions the compiler does not see as loads
    }
  }

  const float sc_log2 = kLog2e * 0.0625f;      // log2(e) / sqrt(256)
  float m_run = -1e30f, l_run = 0.f;           // m_run in log2 units, shared by the four lanes of a row
  f4 o[16];
#pragma unroll
  for (int b = 0; b < 16; ++b) o[b] = f4{0.f, 0.f, 0.f, 0.f};

  Raw raw0{}, raw1{};                          // raw codes of the next two tiles: loads run two tiles ahead of their use
  const LaneOffs offs = lane_offs(tid);
  uint32_t magic = kMagic;
  asm volatile("" : "+v"(magic));
  auto load_tile_raw = [&](int T, Raw& r) __attribute__((always_inline)) { load_raw(page256w(A.kv, kvh, T << 5), (T << 5) % kPageTok, offs, r); };
  if (tile0 < tile1) {
    load_tile_raw(tile0, raw0);
    wait_raw<0>(raw0);
    dequant_to_lds(lds[0], tid, raw0, magic);
    load_tile_raw(min(tile0 + 1, tile1 - 1), raw1);
    load_tile_raw(min(tile0 + 2, tile1 - 1), raw0);
  }
  __syncthreads();

  // One tile: `rs` holds the raw codes of tile T+1, which are dequantized into the other LDS buffer (unconditionally:
  // after the last tile that buffer is read by nobody) and replaced by the request for tile T+3 (past the end: the last
  // tile again, so that the count of loads in flight is static); cb is a literal at both call sites.
  auto tile_step = [&](auto compute_tag, const int T, const int cb, Raw& rs) __attribute__((always_inline)) {
    constexpr bool kCompute = decltype(compute_tag)::value;
    const uint8_t* buf = lds[cb];
    wait_raw<5>(rs);                           // the five loads of the other register set stay in flight
    dequant_to_lds(lds[cb ^ 1], tid, rs, magic);
    load_tile_raw(min(T + 3, tile1 - 1), rs);
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
      tile_step(compute_tag, T, 0, raw1);
      if (T + 1 < tile1) tile_step(compute_tag, T + 1, 1, raw0);
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
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int b = 0; b < 16; ++b) {
    const h2 lo = {(_Float16)(o[b][0] * inv), (_Float16)(o[b][1] * inv)}, hi = {(_Float16)(o[b][2] * inv), (_Float16)(o[b][3] * inv)};
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

void launch_attend256_wide(const AttnArgs& A, hipStream_t st) {
  const int rows = kG * A.M, rb = (rows + 127) / 128;
  hipLaunchKernelGGL(attend256_wide_kernel, dim3(A.S, A.kv.n_kv, rb), dim3(NT), 0, st, A);
}

}  // namespace yka
