// Split-KV attention for windows of 3..64 query tokens (verify windows) and for prefill chunks cut into slices of up to
// 1024 tokens (one launch per slice, every workgroup 128 rows of it).  gfx950.
//
// Same mathematics as the narrow kernel (reference: src/q35_atxpk4.cuh:71-499 for the window shape, row geometry
// src/q35_atxpk.cu:391-411): every row t of the window runs an online softmax over the keys [0, len(t)) of its
// split and leaves (m, l, acc) partials for the combiner.  What differs is who dequantizes and how the work of a
// compute unit is laid out in time:
//   * one workgroup of 8 waves per compute unit owns up to 128 query rows (token-major, 6 heads per token) and one
//     split of the keys.  The waves form two groups of four; group g walks the tiles tile0 + g, tile0 + g + 2, ... of
//     the split, each with its own softmax state, and the two states are merged through LDS at the end: one partial
//     row per (row, split), half as many splits as workgroups of four waves would need to fill the chip;
//   * a group dequantizes each of its 32-key tiles ONCE into LDS - K as exact integer codes in fp16 (n-8, odd nibbles
//     16(n-8)), V scaled and transposed (channel-major, the operand shape of the token-contracting MFMA) - and every
//     wave of the group reads its MFMA fragments from there;
//   * a wave owns one tile of 32 rows (MFMA 32x32x16: one K or V fragment read from LDS serves 32 rows) and stays
//     under 256 registers, so the two waves of a SIMD (one of each group) fit and all MFMA results live in ordinary
//     VGPRs (no accumulator-file copies);
//   * a step of a group has two phases with a workgroup barrier after each: a MATRIX phase (the PV product of the
//     previous tile, the score MFMAs of this tile with the scale multiply-adds in their shadow, fragment reads) and a
//     VECTOR phase (softmax, dequantization of the group's next tile, requests for the tile after that).  The groups run
//     half a step apart: while one is in its matrix phase the other is in its vector phase, so the two waves of a SIMD
//     never compete for the matrix pipe and vector work of one wave runs under the MFMAs of the other.  Two waves
//     left to themselves do not find this arrangement: measured, two independent 4-wave workgroups per compute unit
//     take as long as the same two one after the other;
//   * the group scales of K are applied to the fp32 partial sum of each 32-channel group (two chained MFMAs per
//     group), so K is never rounded; V carries one fp16 rounding.  The scales in LDS carry log2(e)/sqrt(d) and the
//     chain of multiply-adds starts from minus the row's running maximum: a score leaves it as the exponent of its
//     probability;
//   * the running maximum of a row is only raised when a score exceeds it by more than 2^8: accumulators stay in
//     their registers untouched on almost every tile;
//   * LDS is double buffered per group; the raw tile loads run two tiles ahead as explicit load instructions with
//     their own counter waits;
//   * the last split owns the tiles that hold the rows this pass appends and quantizes them itself before reading
//     them (quantize-on-append without a launch of its own).
// The values the instruction-form loads produce must reach their wait in the registers they were loaded into: they are
// loop carried in fixed registers, every request is waited for before the loop's registers are given up, and every
// parity test would fail on a copy made before its wait.
// LDS image of one tile (19456 bytes):
//   K  [32 keys][272 B]   chunk 4m+g of a key = channels 32m+8g..+7 in the order n0,n4,n1,n5,n2,n6,n3,n7; the 272-byte
//                          pitch makes the lanes of a fragment read hit distinct banks
//   V  [128 rows][80 B]   channel 8*dw+c lives in row 16*sigma(c)+dw, sigma(c) = 2*(c&3) + (c>>2): the 16 lanes that
//                          dequantize one byte position write 16 consecutive rows, and an output lane ends up with runs
//                          of 8 consecutive channels.  Inside a row token 16u+8a+4h+b sits at position 16u+8h+4a+b, so
//                          the 8 tokens an MFMA lane needs are 16 contiguous bytes
//   S  [4 groups][4 a][2 h][4 b] fp32   K group scale of key 8a+4h+b: every lane needs the scales of 16 keys x 4 groups,
//                          the same for all 32 lanes of a wave half; converted to fp32 once per workgroup, each lane reads
//                          four of them per instruction (a broadcast read) and multiplies with a plain fp32 FMA
// Partial results leave through the same LDS after the last tile so that every store writes whole 256-byte rows.
#include "codec_device.h"
#include <hip/hip_fp16.h>
#include <type_traits>

namespace yka {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

namespace {

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
__device__ __forceinline__ uint32_t as_u32(h2 h) { return __builtin_bit_cast(uint32_t, h); }

constexpr uint32_t kMagic = 0x64006400u;
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kKPitch = 272, kVPitch = 80;
constexpr int kLdsK = 0, kLdsV = 32 * kKPitch, kLdsS = kLdsV + 128 * kVPitch, kLdsBuf = kLdsS + 512;   // 19456
constexpr int NT = 512;                        // threads per workgroup: two groups of four waves
constexpr int NTG = 256;                       // threads per group
constexpr float kRaise = 8.f;                  // log2 slack before a running maximum is raised

struct Raw {                                   // one thread's share of a raw 32-key tile
  uint32_t kw[2];
  uint32_t vw[2];
  uint32_t vs;
  uint32_t ks;                                 // fp16 scale of (key (tid & 127) / 4, group tid % 4)
};

// Byte offsets of one thread inside a page, fixed for the whole kernel; the page pointer and the tile's first token
// are wave uniform, so every load is "scalar base + 32-bit lane offset".
struct LaneOffs { uint32_t k, v, vs, ks; };
__device__ __forceinline__ LaneOffs lane_offs(int tid, int h) {
  const uint32_t pair = tid >> 4, dw = tid & 15;
  (void)h;
  return LaneOffs{(uint32_t)tid * 4u, kPageVc + pair * 128u + dw * 4u, kPageVs + (dw >> 2) * (kPageTok * 2u) + pair * 4u,
                  kPageKs + ((uint32_t)tid & 127u) * 2u};
}
// The tile loads are written as instructions: they stay in flight across two loop steps, and the counter wait the
// compiler would place at the loop header (it merges the header's predecessors conservatively) drains all of them.
// Every load here is "wave-uniform base in scalar registers + 32-bit lane offset"; wait_raw<N> ties the six registers
// of a tile to a wait that leaves the N younger loads in flight.  Loads return in order and nothing stores in the loop.
template <int IMM>
__device__ __forceinline__ uint32_t gload32(const uint8_t* base, uint32_t off) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(v) : "v"(off), "s"(base), "n"(IMM));
  return v;
}
__device__ __forceinline__ uint32_t gload16(const uint8_t* base, uint32_t off) {
  uint32_t v;
  asm volatile("global_load_ushort %0, %1, %2" : "=v"(v) : "v"(off), "s"(base));
  return v;
}
__device__ __forceinline__ void load_raw(const uint8_t* pg, int tp, const LaneOffs& L, Raw& R) {
  const uint8_t* kt = pg + (uint32_t)tp * 64u;            // K and V code rows of the tile start here (+ plane offset)
  R.kw[0] = gload32<0>(kt, L.k);
  R.kw[1] = gload32<NTG * 4>(kt, L.k);
  R.vw[0] = gload32<0>(kt, L.v);
  R.vw[1] = gload32<64>(kt, L.v);
  R.vs = gload32<0>(pg + (uint32_t)tp * 2u, L.vs);
  R.ks = gload16(pg + (uint32_t)tp * 8u, L.ks);
}
template <int N>
__device__ __forceinline__ void wait_raw(Raw& R) {
  asm volatile("s_waitcnt vmcnt(%6)" : "+v"(R.kw[0]), "+v"(R.kw[1]), "+v"(R.vw[0]), "+v"(R.vw[1]), "+v"(R.vs), "+v"(R.ks) : "n"(N));
}

// (w & mask) | magic as one bit-field insert: `magic` (0x64006400, no bit inside either nibble mask) is kept opaque to
// the optimizer so that the select form survives to instruction selection
__device__ __forceinline__ uint32_t nib(uint32_t w, uint32_t mask, uint32_t magic) { return (w & mask) | (magic & ~mask); }

__device__ __forceinline__ void dequant_to_lds(uint8_t* buf, int tid, const Raw& R, uint32_t magic, float sc_log2) {
  const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f}, c1152 = {(_Float16)1152.f, (_Float16)1152.f};
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int idx = tid + u * NTG, key = idx >> 4, p = idx & 15;      // physical dword p = 4g+m of the key row
    const uint32_t w = R.kw[u], t = w >> 8;
    uint4 o;
    o.x = as_u32(as_h2(nib(w, 0x000f000fu, magic)) - c1032);
    o.y = as_u32(as_h2(nib(w, 0x00f000f0u, magic)) - c1152);
    o.z = as_u32(as_h2(nib(t, 0x000f000fu, magic)) - c1032);
    o.w = as_u32(as_h2(nib(t, 0x00f000f0u, magic)) - c1152);
    *reinterpret_cast<uint4*>(buf + kLdsK + key * kKPitch + (4 * (p & 3) + (p >> 2)) * 16) = o;
  }
  {                                                                  // K group scales as fp32, [group][a][h][b] for key 8a+4h+b,
    const int key = (tid & 127) >> 2, m = tid & 3;                   // times log2(e)/sqrt(d): scores come out in log2 units
    reinterpret_cast<float*>(buf + kLdsS)[m * 32 + (key >> 3) * 8 + (key & 7)] = (float)as_h2(R.ks)[0] * sc_log2;   // waves 2 and 3 repeat waves 0 and 1 (no divergent branch)
  }
  {
    const int pair = tid >> 4, dw = tid & 15;
    const int t0 = 2 * pair;                                         // token 16u + 8a + 4h + b -> position 16u + 8h + 4a + b
    const int posn = (t0 & 16) + 8 * ((t0 >> 2) & 1) + 4 * ((t0 >> 3) & 1) + (t0 & 3);
    const h2 s2 = as_h2(R.vs), s2q = s2 * h2{(_Float16)0.0625f, (_Float16)0.0625f};
    const uint32_t w0 = R.vw[0], w1 = R.vw[1];
    uint8_t* vb = buf + kLdsV + dw * kVPitch + posn * 2;
#pragma unroll
    for (int bb = 0; bb < 4; ++bb) {
      // byte bb of both tokens side by side (low half = token t0, high half = token t0+1)
      const uint32_t x = __builtin_amdgcn_perm(w1, w0, 0x0c040c00u + bb * 0x00010001u);
      const h2 lo = (as_h2(nib(x, 0x000f000fu, magic)) - c1032) * s2;       // channel c = 2bb
      const h2 hi = (as_h2(nib(x, 0x00f000f0u, magic)) - c1152) * s2q;      // channel c = 2bb+1
      const int c0 = 2 * bb, c1 = 2 * bb + 1;
      *reinterpret_cast<uint32_t*>(vb + 16 * (2 * (c0 & 3) + (c0 >> 2)) * kVPitch) = as_u32(lo);
      *reinterpret_cast<uint32_t*>(vb + 16 * (2 * (c1 & 3) + (c1 >> 2)) * kVPitch) = as_u32(hi);
    }
  }
}

}  // namespace

// Workgroup = (split, kv head, row block), block 512; wave w of either group owns rows [32 w, 32 (w+1)) of the block.
// The row blocks of one (split, kv head) pair read the same KV tiles, and each of the 8 XCDs has an L2 of its own, so the
// grid is one-dimensional and laid out for the dispatcher's round robin (workgroup i runs on XCD i mod 8, strictly: a
// workgroup waits for a CU of ITS XCD, so the grid holds exactly pairs x n_rb workgroups and no padding).  XCD x gets
// n_x = total / 8 (+1 if x < total mod 8) workgroups.  The first F * n_rb of them, F = (total / 8) / n_rb, are the row
// blocks of F whole pairs (the k-th is row block k mod n_rb of pair x + 8 (k / n_rb)): all row blocks of such a pair run
// on one XCD at about the same time and each tile leaves HBM once.  The workgroups left over on every XCD take the
// remaining pairs in order.
__global__ void __launch_bounds__(NT) attend_wide_kernel(AttnArgs A) {
  __shared__ __align__(16) uint8_t lds[2][2][kLdsBuf];               // [group][buffer]
  const int n_rb = (kG * A.M + A.rows_per_block - 1) / A.rows_per_block;
  int pair, rb;
  {
    const int total = gridDim.x, x = blockIdx.x & 7, k = blockIdx.x >> 3, F = (total >> 3) / n_rb;
    if (k < F * n_rb) { pair = x + 8 * (k / n_rb); rb = k % n_rb; }
    else {
      const int base_e = (total >> 3) - F * n_rb;                     // leftover workgroups of an XCD, +1 on the first total mod 8
      const int jj = x * base_e + min(x, total & 7) + (k - F * n_rb);
      pair = 8 * F + jj / n_rb; rb = jj % n_rb;
    }
  }
  const int split = pair % A.S, kvh = pair / A.S;
  const int tid = threadIdx.x, gt = tid & (NTG - 1);                  // gt: thread index inside the group
  const int grp = __builtin_amdgcn_readfirstlane(tid >> 8);           // wave uniform
  const int wave = __builtin_amdgcn_readfirstlane(gt >> 6), lane = tid & 63, j = lane & 31, h = lane >> 5;
  const int pos = *A.d_pos;
  const int nrows = kG * A.M;

  // row of this lane: R = rb*rows_per_block + wave*32 + j  ->  token R/6 of the slice, head kvh*6 + R%6
  const int RPB = A.rows_per_block;
  const int row0 = rb * RPB + wave * 32;
  const int R = row0 + j;
  const bool vrow = R < nrows && R < (rb + 1) * RPB;
  const int tl = R / kG, head = kvh * kG + R % kG;
  int len = 0;
  if (vrow) { const int tg = A.tok0 + tl; len = min(pos + (A.depth ? (int)A.depth[tg] : tg) + 1, A.kv.max_ctx); }
  const size_t pidx = ((size_t)tl * A.S + split) * A.n_heads + head;
  // B operand of S^T = K Q^T, k-step ks: lane (row j, half h) holds chunk 2ks+h = (group ks/2, sub-chunk 2(ks&1)+h)
  h8 qf[8];
  {
    const uint16_t* qrow = A.q16 + ((size_t)tl * A.n_heads + head) * kD;
    // the odd nibble of a byte is 16 (n - 8) in the K image: its query channels carry 1/4 and the others 4 (products 4 q n
    // either way; a plain 1/16 would push small queries into the fp16 subnormals), the 4 leaves with the softmax scale
    const _Float16 se = (_Float16)4.f, so = (_Float16)0.25f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      uint4 u = vrow ? *reinterpret_cast<const uint4*>(qrow + 32 * (ks >> 1) + 8 * (2 * (ks & 1) + h)) : make_uint4(0, 0, 0, 0);
      const h8 c = __builtin_bit_cast(h8, u);
      qf[ks] = h8{c[0] * se, c[4] * se, c[1] * so, c[5] * so, c[2] * se, c[6] * se, c[3] * so, c[7] * so};
    }
  }
  const bool has_rows = row0 < min(nrows, (rb + 1) * RPB);             // wave uniform

  // key range of the workgroup: its splits cut [0, maxlen) of the block's longest row into 32-key tiles
  const int tok_lo = (rb * RPB) / kG, tok_hi = min(A.M, (rb * RPB + RPB + kG - 1) / kG);
  int maxdep = 0, mindep = 0x7fffffff;
  for (int t = tok_lo; t < tok_hi; ++t) { const int tg = A.tok0 + t; const int dp = A.depth ? (int)A.depth[tg] : tg; maxdep = max(maxdep, dp); mindep = min(mindep, dp); }
  const int maxlen = min(pos + maxdep + 1, A.kv.max_ctx), minlen = min(pos + mindep + 1, A.kv.max_ctx);
  // The last split owns the tiles that hold rows of this slice (from tile Tw on), the other splits share the cached
  // context before them evenly: the rows a pass appends are then read by the workgroups of one split only, which
  // is what lets them be quantized and stored by those workgroups themselves (below) instead of by a launch of
  // their own.
  const int ntiles = (maxlen + 31) >> 5;
  // The window split takes an even share of the cached context as well, less window_cost tiles for the quantization it
  // does first (measured: about the time of 7 tiles for 64 rows): every workgroup of the launch then finishes at about
  // the same time (with the window tiles alone, 12 of the 252 workgroups of a 64-row pass were idle after two tiles and
  // the others walked 51 tiles instead of 49).
  const int kWindowCost = A.k16 ? 1 + A.M / 10 : 0;
  const int Tnew = min(ntiles, max(0, pos + A.tok0) >> 5);            // first tile that holds a row of this slice
  const int Tw = A.S > 1 ? min(Tnew, (A.S - 1) * ((ntiles + kWindowCost + A.S - 1) / A.S)) : Tnew;
  // A pass wider than one slice (a prefill chunk: its rows were appended by a launch of their own) has no window split:
  // its key range is cut evenly.
  int tile0, tile1;
  if (A.S == 1) { tile0 = 0; tile1 = ntiles; }
  else if (A.M > kMaxSlice) { const int tps = (ntiles + A.S - 1) / A.S; tile0 = min(ntiles, split * tps); tile1 = min(ntiles, tile0 + tps); }
  else if (split == A.S - 1) { tile0 = Tw; tile1 = ntiles; }
  else { const int tps = (Tw + A.S - 2) / (A.S - 1); tile0 = split * tps; tile1 = min(Tw, tile0 + tps); }
  // ---- fused quantize-on-append: every workgroup of the window split stores the slice's rows up to its own last
  //      token (the row blocks of one kv head write identical bytes: each row is the same sequence of IEEE operations
  //      on the same inputs whoever computes it) and reads them back after a workgroup barrier: writer and readers
  //      are waves of one CU and one write-through L1.  Group 0 quantizes; the barrier is the workgroup's. ----
  if (A.k16 && split == A.S - 1) {
    // 16 lanes per 128-channel row, 16 rows (K and V of 8 tokens) per step; all loads of the slice (at most 64 tokens)
    // are requested before the first row is quantized
    static_assert(kMaxSlice <= 64, "8 steps of 16 rows cover K and V of a slice");
    if (grp == 0) {
      const int c = gt & 15, slot = gt >> 4;
      uint4 rawv[8];
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int hh = it * 16 + slot, t = hh >> 1;
        const uint16_t* src = ((hh & 1) ? A.v16 : A.k16) + ((size_t)(A.tok0 + t) * A.kv.n_kv + kvh) * kD + 8 * c;
        rawv[it] = t < tok_hi ? *reinterpret_cast<const uint4*>(src) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int hh = it * 16 + slot, t = hh >> 1, r = pos + A.tok0 + t;
        if (t < tok_hi && r >= 0 && r < A.kv.max_ctx) quant_store_chunk8(A.kv, kvh, r, hh & 1, rawv[it], c);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    asm volatile("" ::: "memory");             // the tile loads below are instructions the compiler does not see as loads
  }

  // tiles of this group: tile0 + grp + 2u, u = 0 .. nu-1; both groups walk nsteps steps (a group one tile short idles in
  // its last step) so that every wave of the workgroup meets the same number of barriers
  const int ntl = max(0, tile1 - tile0);
  const int nsteps = (ntl + 1) >> 1, nu = (ntl + 1 - grp) >> 1;
  auto tile_of = [&](int u) __attribute__((always_inline)) { return tile0 + grp + 2 * min(u, nu - 1); };   // past the end: the last tile again

  float m_run = -1e30f, l_run = 0.f;           // m_run in log2 units, shared by the two lanes of a row
  f16v o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;

  const float sc_log2 = 0.25f * kLog2e / sqrtf((float)kD);      // 1/4: the query fragments carry a factor 4
  Raw raw0{}, raw1{};                          // raw codes of the group's next two tiles: loads run two tiles ahead of their use
  const LaneOffs offs = lane_offs(gt, h);
  uint32_t magic = kMagic;
  asm volatile("" : "+v"(magic));
  auto load_tile_raw = [&](int T, Raw& r) __attribute__((always_inline)) { load_raw(kv_page_uniform(A.kv, kvh, T << 5), (T << 5) % kPageTok, offs, r); };
  if (nu > 0) {
    load_tile_raw(tile_of(0), raw0);
    wait_raw<0>(raw0);
    dequant_to_lds(lds[grp][0], gt, raw0, magic, sc_log2);
    load_tile_raw(tile_of(1), raw1);
    load_tile_raw(tile_of(2), raw0);
  }
  __syncthreads();

  // The probabilities and the V fragments of a tile stay in registers across the two barriers of a step; their eight
  // MFMAs open the NEXT matrix phase.  The first one multiplies zeros; the product of the last tile follows the loop.
  h8 pf[2], vfr[8];
#pragma unroll
  for (int c = 0; c < 8; ++c)
#pragma unroll
    for (int e = 0; e < 8; ++e) { vfr[c][e] = (_Float16)0.f; pf[c & 1][e] = (_Float16)0.f; }
  auto pv = [&]() __attribute__((always_inline)) {                            // O^T += V^T P^T : d-tile dt (32 rows of the V image), k-step u (16 tokens)
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int u = 0; u < 2; ++u) o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vfr[2 * dt + u], pf[u], o[dt], 0, 0, 0);
  };
  float s[16];                                 // exponents of the tile in hand: written by the matrix phase, used by the vector phase
  float m_sub = 0.f;
  bool first = true;
#pragma unroll
  for (int r = 0; r < 16; ++r) s[r] = -INFINITY;

  // ---- matrix phase of the group's tile u (buffer cb of the group): PV of the tile before, scores of this one ----
  auto matrix_phase = [&](const int u, const int cb) __attribute__((always_inline)) {
    if (!has_rows) return;                     // wave uniform
    const uint8_t* buf = lds[grp][cb];
    h8 kfr[8];
#pragma unroll
    for (int c = 0; c < 8; ++c)
      kfr[c] = __builtin_bit_cast(h8, *reinterpret_cast<const uint4*>(buf + kLdsK + j * kKPitch + (4 * (c >> 1) + 2 * (c & 1) + h) * 16));
    pv();
    // scores: per scale group two chained MFMAs (32 channels), then the fp32 sum times the group scale.  A row that has
    // seen no key yet (m_run is the "no keys" marker) starts its chain from 0.
    first = m_run < -1e29f;
    m_sub = first ? 0.f : m_run;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      float4 sc4[4];                           // fp32 scales of group m for the lane's 16 keys, the same for all 32 lanes of a half
#pragma unroll
      for (int a = 0; a < 4; ++a) sc4[a] = *reinterpret_cast<const float4*>(buf + kLdsS + ((m * 4 + a) * 2 + h) * 16);
      f16v part;
#pragma unroll
      for (int r = 0; r < 16; ++r) part[r] = 0.f;
      part = __builtin_amdgcn_mfma_f32_32x32x16_f16(kfr[2 * m], qf[2 * m], part, 0, 0, 0);
      part = __builtin_amdgcn_mfma_f32_32x32x16_f16(kfr[2 * m + 1], qf[2 * m + 1], part, 0, 0, 0);
      // part[r]: key 8(r/4) + 4h + r%4 of the tile against row j
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float sh = (&sc4[r >> 2].x)[r & 3];
        s[r] = __builtin_fmaf(part[r], sh, m == 0 ? -m_sub : s[r]);
      }
    }
    // the V fragments are requested here and used in the next matrix phase: their latency runs under the vector phase
#pragma unroll
    for (int c = 0; c < 8; ++c)
      vfr[c] = __builtin_bit_cast(h8, *reinterpret_cast<const uint4*>(buf + kLdsV + (32 * (c >> 1) + j) * kVPitch + (16 * (c & 1) + 8 * h) * 2));
  };
  // ---- vector phase of tile u: softmax of its scores; `rs` holds the raw codes of tile u+1, which are dequantized into
  //      the group's other buffer (unconditionally: after the last tile that buffer is read by nobody) and replaced by
  //      the request for tile u+3 ----
  auto vector_phase = [&](const int u, const int cb, Raw& rs) __attribute__((always_inline)) {
    // The wave in its vector phase goes first when both waves of a SIMD have an instruction to issue.  At equal priority
    // the older wave (group 0) wins in both of its phases and the younger group sets the pace of every phase: its vector
    // phase, the longer stream, measured 1,580 cycles against group 0's 1,190.  With this, both groups take about 1,200
    // cycles in either phase.
    __builtin_amdgcn_s_setprio(2);
    if (has_rows) {
      const int t0 = tile_of(u) << 5;
      // online softmax with a lazily raised maximum: a row's offset m_run only moves when a score exceeds it by more
      // than 2^kRaise (or when the row sees its first keys).  The row sum is taken from the fp16 probabilities the PV
      // product uses (two per dot2).
      if (t0 + 32 > minlen) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = t0 + 8 * (r >> 2) + 4 * h + (r & 3);
          s[r] = key < len ? s[r] : -INFINITY;
        }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s[r]);
      if (__any(tmax > (first ? -INFINITY : kRaise))) {
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const bool seen = tmax > -INFINITY;                       // false: every key of the tile lies past the row's length
        const float d = first ? (seen ? tmax : 0.f) : fmaxf(tmax, 0.f);
        const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-d);   // a first tile finds zeros in l and o
        if (!first || seen) m_run = m_sub + d;
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] -= d;
      }
      float lsum0 = 0.f, lsum1 = 0.f;
      const h2 ones = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
      for (int r = 0; r < 16; r += 4) {
        const h2 p01 = {(_Float16)__builtin_amdgcn_exp2f(s[r]), (_Float16)__builtin_amdgcn_exp2f(s[r + 1])};
        const h2 p23 = {(_Float16)__builtin_amdgcn_exp2f(s[r + 2]), (_Float16)__builtin_amdgcn_exp2f(s[r + 3])};
        lsum0 = __builtin_amdgcn_fdot2(p01, ones, lsum0, false);
        lsum1 = __builtin_amdgcn_fdot2(p23, ones, lsum1, false);
        pf[r >> 3][r & 7] = p01[0]; pf[r >> 3][(r & 7) + 1] = p01[1]; pf[r >> 3][(r & 7) + 2] = p23[0]; pf[r >> 3][(r & 7) + 3] = p23[1];
      }
      l_run += lsum0 + lsum1;
    }
    wait_raw<6>(rs);                           // the six loads of the other register set stay in flight
    dequant_to_lds(lds[grp][cb ^ 1], gt, rs, magic, sc_log2);
    load_tile_raw(tile_of(u + 3), rs);         // always issued (past the end: the last tile again), so that the count of loads in flight is static
    __builtin_amdgcn_s_setprio(0);
  };
  // Group 1 starts one barrier late and group 0 ends with one barrier more: the groups stay a phase apart, and every
  // wave executes 2 * nsteps + 1 barriers whatever its group (a group one tile short only meets the barriers of its
  // last step).  cb and the register set are literals at every call site.
  if (grp == 1) __syncthreads();
  for (int u = 0; u < nu; u += 2) {
    matrix_phase(u, 0);
    __syncthreads();
    vector_phase(u, 0, raw1);
    __syncthreads();
    if (u + 1 < nu) {
      matrix_phase(u + 1, 1);
      __syncthreads();
      vector_phase(u + 1, 1, raw0);
      __syncthreads();
    }
  }
  for (int u = nu; u < nsteps; ++u) { __syncthreads(); __syncthreads(); }
  if (grp == 0) __syncthreads();
  // every request has been answered before the registers it names are given up
  wait_raw<0>(raw0);
  wait_raw<0>(raw1);
  if (has_rows) pv();

  // ---- the two groups' states of a row are merged: group 1 leaves its registers in LDS (the tile buffers are free
  //      after the last barrier), group 0 folds them into its own.  Wave w of either group holds the same rows in the
  //      same registers, so the exchange is a plain register image: [wave][register][lane]. ----
  float* xo = reinterpret_cast<float*>(&lds[0][0][0]);               // 4 waves x 64 registers x 64 lanes = 65536 bytes
  float* xm = xo + 4 * 64 * 64;                                       // then m and l, [wave][lane]: 2048 bytes
  float* xl = xm + 4 * 64;
  static_assert(4 * 64 * 64 * 4 + 2 * 4 * 64 * 4 <= 4 * kLdsBuf, "the register image of group 1 fits the tile buffers");
  if (grp == 1 && has_rows) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) xo[(wave * 64 + dt * 16 + r) * 64 + lane] = o[dt][r];
    xm[wave * 64 + lane] = m_run; xl[wave * 64 + lane] = l_run;
  }
  __syncthreads();
  if (grp == 1 || !has_rows) return;           // no barrier follows
  {
    const float mb = xm[wave * 64 + lane], lb = xl[wave * 64 + lane];
    const float m2 = fmaxf(m_run, mb);
    const float wa = __builtin_amdgcn_exp2f(m_run - m2), wb = __builtin_amdgcn_exp2f(mb - m2);   // both markers: 2^0, sums stay 0
    m_run = m2; l_run = wa * l_run + wb * lb;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][r] = wa * o[dt][r] + wb * xo[(wave * 64 + dt * 16 + r) * 64 + lane];
  }
  // ---- partials: normalised fp16.  o[dt][4a+b] of lane (row j, half h) is V-image row 32dt + 8a + 4h + b, i.e.
  //      channel 64(a&1) + 32h + 8b + 4(a>>1) + dt: for each (a&1, b) the lane owns 8 consecutive channels.
  //      Rows go through LDS so that every store instruction writes whole 256-byte rows: 16 lanes per row instead of
  //      64 scattered 16-byte pieces.  A wave stages its rows inside the part of the register image only it has read. ----
  constexpr int kOPitch = 2 * kD + 16;                       // bytes per staged row
  static_assert(32 * kOPitch <= 64 * 64 * 4, "a wave's staging area lies inside its own part of the register image");
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");     // the image has been read before the wave overwrites it
  uint8_t* stage = &lds[0][0][0] + wave * (64 * 64 * 4);     // 4 waves x 8704 bytes, 16384 bytes apart
  float l = l_run;
  l += __shfl_xor(l, 32, 64);
  if (vrow && h == 0) { A.pm[pidx] = m_run; A.pl[pidx] = l; }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int a0 = 0; a0 < 2; ++a0)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      h8 v;
#pragma unroll
      for (int c = 0; c < 8; ++c) v[c] = (_Float16)(o[c & 3][4 * (2 * (c >> 2) + a0) + b] * inv);
      *reinterpret_cast<uint4*>(stage + j * kOPitch + (64 * a0 + 32 * h + 8 * b) * 2) = __builtin_bit_cast(uint4, v);
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");     // the wave reads back what its own lanes wrote
  const int chunk = lane & 15;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int jr = 4 * k + (lane >> 4);
    const int Rr = row0 + jr;
    if (Rr < nrows && Rr < (rb + 1) * RPB) {
      const size_t p = ((size_t)(Rr / kG) * A.S + split) * A.n_heads + kvh * kG + Rr % kG;
      const uint4 v = *reinterpret_cast<const uint4*>(stage + jr * kOPitch + chunk * 16);
      *reinterpret_cast<uint4*>(A.pacc16 + p * kD + chunk * 8) = v;
    }
  }
}

void launch_attend_wide(const AttnArgs& A, hipStream_t st) {
  const int rows = kG * A.M, rb = (rows + A.rows_per_block - 1) / A.rows_per_block;
  hipLaunchKernelGGL(attend_wide_kernel, dim3(A.S * A.kv.n_kv * rb), dim3(NT), 0, st, A);
}

}  // namespace yka
