// One wave's view of a 32-key tile of the int4 cache, shared by the kernels in which a wave owns whole tiles (the decode
// kernel, attend_narrow.hip, and the kernel for windows of 3..16 rows, attend_mid.hip): what a lane loads, where from,
// the load instructions with their counter waits, and the code -> fp16 conversions.  gfx950.
#pragma once
#include "yka_internal.h"

namespace yka {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
__device__ __forceinline__ uint32_t as_u32(h2 h) { return __builtin_bit_cast(uint32_t, h); }

constexpr uint32_t kMagic = 0x64006400u;  // two fp16 1024.0
constexpr float kLog2e = 1.4426950408889634f;

// 8 codes of one dword -> 4 half2 in element order [n0,n4 | n1,n5 | n2,n6 | n3,n7] holding n-8 for even nibbles and
// 16(n-8) for odd ones, all exact.  The factor 16 is undone by the query fragment.
// (w & mask) | magic written as a bit-field insert; `magic` (0x64006400, no bit inside either nibble mask) is kept opaque
// to the optimizer so that the pair is selected as one and-or instruction
__device__ __forceinline__ uint32_t nib(uint32_t w, uint32_t mask, uint32_t magic) { return (w & mask) | (magic & ~mask); }
__device__ __forceinline__ void dq_dword_int(uint32_t w, h2* out, uint32_t magic) {
  const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f}, c1152 = {(_Float16)1152.f, (_Float16)1152.f};
  const uint32_t t = w >> 8;
  out[0] = as_h2(nib(w, 0x000f000fu, magic)) - c1032;
  out[1] = as_h2(nib(w, 0x00f000f0u, magic)) - c1152;
  out[2] = as_h2(nib(t, 0x000f000fu, magic)) - c1032;
  out[3] = as_h2(nib(t, 0x00f000f0u, magic)) - c1152;
}

// K codes for the score MFMA need no arithmetic at all: a nibble left in place in an otherwise zero fp16 is the
// subnormal n * 2^-24 (16 n * 2^-24 for the odd nibble of a byte), which the matrix pipe multiplies exactly like any
// other fp16.  The offset of the code (-8 per channel) becomes -8 * sum(q) per (row, scale group), which the MFMA gets as
// its initial accumulator, and the factor 2^24 is folded into the exponent's scale.  Same element order as dq_dword_int.
__device__ __forceinline__ void dq_dword_sub(uint32_t w, h2* out) {
  const uint32_t t = w >> 8;
  out[0] = as_h2(w & 0x000f000fu);
  out[1] = as_h2(w & 0x00f000f0u);
  out[2] = as_h2(t & 0x000f000fu);
  out[3] = as_h2(t & 0x00f000f0u);
}
constexpr float kTwo24 = 16777216.f, kTwoM24 = 1.f / 16777216.f;

struct RawTile {       // what one lane holds of a 32-key tile before dequantization
  u32x4 kw[2];         // K codes: key 16*kt + (lane&15), dword m = channels 32m + 8*(lane>>4) .. +7
  u32x4 ks[2][2];      // K scales of the 4 keys whose scores this lane receives: [kt][..] = keys 16kt+4g+r, 4 fp16 each
  uint32_t vw[8];      // V codes: token tau(e), channels 8*(lane&15) .. +7
  u32x2 vs[2];         // V scales, group (lane&15)/4, tokens 16h+4g .. +3 (4 fp16)
};
// token slot e of lane group g inside a 32-key tile: the keys whose scores this lane receives from the two score MFMAs
__device__ __forceinline__ int tau(int g, int e) { return 16 * (e >> 2) + 4 * g + (e & 3); }

// Byte offsets of one lane inside a page, fixed for the whole kernel.  The page pointer and the tile's first token are
// wave uniform, so every load is "scalar base + 32-bit lane offset + immediate".
struct LaneOffs { uint32_t kc, ks, vs, vc; };
__device__ __forceinline__ LaneOffs lane_offs(int i, int g) {
  return LaneOffs{kPageKc + (uint32_t)i * 64u + 16u * g, kPageKs + 32u * g, kPageVs + ((uint32_t)(i >> 2) * kPageTok + 4u * g) * 2u,
                  kPageVc + 256u * g + 4u * i};
}
// The 16 loads of a tile are written as instructions: a wave keeps the tile after the one it works on in flight, and a
// wait the compiler places (it assumes the fewest loads in flight over all paths into a loop) would drain it.  The cache
// is read once per call: streaming (nontemporal) loads, which a plain read kernel on this GPU measures 10-15 % faster
// than default ones.  wait_tile<N> ties the tile's registers to a wait that leaves the N younger loads in flight.
#define YKA_GL(width, dst, off, base, imm) asm volatile("global_load_" width " %0, %1, %2 offset:%3 nt" : "=v"(dst) : "v"(off), "s"(base), "n"(imm))
// pg = start of the (page, kv head) block, tp = index of the tile's first token inside the page (both wave uniform)
__device__ __forceinline__ void load_tile(const uint8_t* pg, int tp, const LaneOffs& L, RawTile& R) {
  const uint8_t* c64 = pg + (uint32_t)tp * 64u;     // code rows (K and V planes) of the tile
  const uint8_t* s8 = pg + (uint32_t)tp * 8u;       // K scale rows
  const uint8_t* s2 = pg + (uint32_t)tp * 2u;       // V scale columns
  YKA_GL("dwordx4", R.kw[0], L.kc, c64, 0);      YKA_GL("dwordx4", R.kw[1], L.kc, c64, 1024);
  YKA_GL("dwordx4", R.ks[0][0], L.ks, s8, 0);    YKA_GL("dwordx4", R.ks[0][1], L.ks, s8, 16);
  YKA_GL("dwordx4", R.ks[1][0], L.ks, s8, 128);  YKA_GL("dwordx4", R.ks[1][1], L.ks, s8, 144);
  YKA_GL("dwordx2", R.vs[0], L.vs, s2, 0);       YKA_GL("dwordx2", R.vs[1], L.vs, s2, 32);
  // token tau(g, e) = 16 (e >> 2) + 4 g + (e & 3)
  YKA_GL("dword", R.vw[0], L.vc, c64, 0);    YKA_GL("dword", R.vw[1], L.vc, c64, 64);   YKA_GL("dword", R.vw[2], L.vc, c64, 128);  YKA_GL("dword", R.vw[3], L.vc, c64, 192);
  YKA_GL("dword", R.vw[4], L.vc, c64, 1024); YKA_GL("dword", R.vw[5], L.vc, c64, 1088); YKA_GL("dword", R.vw[6], L.vc, c64, 1152); YKA_GL("dword", R.vw[7], L.vc, c64, 1216);
}
#undef YKA_GL
constexpr int kTileLoads = 16;
template <int N>
__device__ __forceinline__ void wait_tile(RawTile& R) {
  asm volatile("s_waitcnt vmcnt(%16)"
               : "+v"(R.kw[0]), "+v"(R.kw[1]), "+v"(R.ks[0][0]), "+v"(R.ks[0][1]), "+v"(R.ks[1][0]), "+v"(R.ks[1][1]), "+v"(R.vs[0]), "+v"(R.vs[1]),
                 "+v"(R.vw[0]), "+v"(R.vw[1]), "+v"(R.vw[2]), "+v"(R.vw[3]), "+v"(R.vw[4]), "+v"(R.vw[5]), "+v"(R.vw[6]), "+v"(R.vw[7])
               : "n"(N));
}

}  // namespace yka
