// Split-KV attention for windows of 3..16 query tokens (the draft lengths speculative decoding uses; reference shapes:
// src/q35_atx.cu:350-572, grids of 8 and 16 tokens in src/q35_atxpk4.cuh:520-537).  gfx950 (wave64, MFMA 16x16x32 f16).
//
// Same mathematics as the other two kernels: every row of the window runs an online softmax over the keys of one split
// and leaves (m, l, acc / l) partials for the combiner.  The shape of the work is the decode kernel's, not the wide
// kernel's: a window of at most 16 tokens x 6 heads is at most six MFMA row tiles of 16 rows, few enough for ONE wave to
// keep all their accumulators in registers (192 of the 512 a wave owns when it has its SIMD to itself).  So
//   * a wave owns whole 32-key tiles, loads them with 14 explicit loads (the next tile is in flight while the current one
//     is worked on) and dequantizes each tile ONCE into MFMA operands that stay in registers: K as two exact scaled images
//     (code x the upper 8 bits of the fp16 group scale, code x its lower 3 bits: both exact in fp16), V scaled in fp16;
//   * it then walks the window's row tiles: query fragments come from LDS (staged once per workgroup in operand order:
//     one conflict-free 16-byte read per lane and scale group), 16 score MFMAs chained over both images (the fp32
//     accumulation adds them exactly: K is never rounded, and no multiply-add per score is left), softmax with a lazily
//     raised running maximum, 8 PV MFMAs into that row tile's accumulators.  Dequantization is paid once per tile instead
//     of once per row tile, there is no LDS round trip for K / V and no barrier inside the loop;
//   * one workgroup (4 waves, one per SIMD) per compute unit; its waves take the tiles of the split round robin and are
//     merged through LDS at the end, one row tile at a time (two buffers, one barrier per row tile);
//   * the rows the pass appends are quantized and stored by the workgroups whose tiles hold them, before they load those
//     tiles (same arithmetic and same stores as the append kernel: bit-identical rows).
// Windows wider than one block (16 * NRT / 6 tokens) run as several row blocks (grid z), each streaming the keys again.
#include <algorithm>
#include "codec_device.h"
#include "tile32_device.h"

namespace yka {

namespace {
constexpr float kRaiseMid = 8.f;               // log2 slack before a running maximum is raised
constexpr int kAccPitch = kD + 4;              // floats per staged row of the wave merge

// Where the matrix results live.  A wave that has its SIMD to itself owns 512 registers, half of them accumulator
// registers.  Left to the compiler, every matrix instruction of such a kernel gets an accumulator-register result: the
// score partial sums, which the vector unit consumes at once, come back through one copy instruction per value, and the
// PV accumulators, which should never leave the accumulator file, are copied to ordinary registers at the head of
// every loop iteration.  So this file is compiled with matrix results in ordinary registers (Makefile:
// -amdgpu-mfma-vgpr-form), which is right for the score instructions (the compiler still schedules them and keeps their
// result hazards), and the PV instructions are written out with their accumulators in the accumulator file: there they
// stay wherever they are live, the compiler moves them only on the rare rescale path and in the epilogue.
// The compiler does not know that the written-out instructions are matrix instructions, so the waits it would add are
// explicit.  A vector instruction's result is not forwarded to a matrix instruction issued right behind it (seen: with
// no idle slot between the last conversion that writes the probabilities and the first PV instruction, that instruction
// multiplied the registers' previous contents - one accumulator in eight wrong; the compiler keeps 2 slots): in the loop
// the PV instructions read probabilities written a whole step earlier, operand_ready covers the one place where they
// follow at once.  pv_done puts 16 idle slots between the last PV instruction and the epilogue's reads of a row tile's
// accumulators (the compiler keeps 8).  Inside the loop an accumulator is next touched a whole tile later.
// What a lane holds of a raw 32-key tile in this kernel.  The K group scales are those of the lane's OWN keys (16kt + i,
// the rows of its K operand: 4 fp16 = one 8-byte load per key half), because here the scales go into the operand, not
// onto the scores.  14 loads per tile.
struct MidTile {
  u32x4 kw[2];         // K codes: key 16*kt + i, dword m = channels 32m + 8g .. +7
  u32x2 ksa[2];        // K scales of key 16*kt + i, groups 0..3
  uint32_t vw[8];      // V codes: token tau(g, e), channels 8i .. +7
  u32x2 vs[2];         // V scales, group i/4, tokens 16h + 4g .. +3
};
#define YKA_GL(width, dst, off, base, imm) asm volatile("global_load_" width " %0, %1, %2 offset:%3 nt" : "=v"(dst) : "v"(off), "s"(base), "n"(imm))
__device__ __forceinline__ void load_mid_tile(const uint8_t* pg, int tp, const LaneOffs& L, uint32_t ksa_off, MidTile& R) {
  const uint8_t* c64 = pg + (uint32_t)tp * 64u;     // code rows (K and V planes) of the tile
  const uint8_t* s8 = pg + (uint32_t)tp * 8u;       // K scale rows
  const uint8_t* s2 = pg + (uint32_t)tp * 2u;       // V scale columns
  YKA_GL("dwordx4", R.kw[0], L.kc, c64, 0);      YKA_GL("dwordx4", R.kw[1], L.kc, c64, 1024);
  YKA_GL("dwordx2", R.ksa[0], ksa_off, s8, 0);   YKA_GL("dwordx2", R.ksa[1], ksa_off, s8, 128);
  YKA_GL("dwordx2", R.vs[0], L.vs, s2, 0);       YKA_GL("dwordx2", R.vs[1], L.vs, s2, 32);
  YKA_GL("dword", R.vw[0], L.vc, c64, 0);    YKA_GL("dword", R.vw[1], L.vc, c64, 64);   YKA_GL("dword", R.vw[2], L.vc, c64, 128);  YKA_GL("dword", R.vw[3], L.vc, c64, 192);
  YKA_GL("dword", R.vw[4], L.vc, c64, 1024); YKA_GL("dword", R.vw[5], L.vc, c64, 1088); YKA_GL("dword", R.vw[6], L.vc, c64, 1152); YKA_GL("dword", R.vw[7], L.vc, c64, 1216);
}
#undef YKA_GL
__device__ __forceinline__ void wait_mid_tile(MidTile& R) {
  asm volatile("s_waitcnt vmcnt(0)"
               : "+v"(R.kw[0]), "+v"(R.kw[1]), "+v"(R.ksa[0]), "+v"(R.ksa[1]), "+v"(R.vs[0]), "+v"(R.vs[1]),
                 "+v"(R.vw[0]), "+v"(R.vw[1]), "+v"(R.vw[2]), "+v"(R.vw[3]), "+v"(R.vw[4]), "+v"(R.vw[5]), "+v"(R.vw[6]), "+v"(R.vw[7]));
}

__device__ __forceinline__ void operand_ready(h8& p) {
  asm volatile("s_nop 2" : "+v"(p));
}
__device__ __forceinline__ void mfma_pv(f4& o, const h8& v, const h8& p) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(o) : "v"(v), "v"(p));
}
__device__ __forceinline__ void pv_done(f4 (&o)[8]) {
  asm volatile("s_nop 15" : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(o[4]), "+a"(o[5]), "+a"(o[6]), "+a"(o[7]));
}
}  // namespace

// grid (S, n_kv, row blocks), block 256.  Row R = 16 rt + i of a block is (token tokb + R / 6, head kvh * 6 + R % 6).
// One wave per SIMD for every instantiation.  (Two waves per SIMD were tried for NRT = 2, whose registers nearly fit:
// the compiler then spills under pressure, and what it spilled were the destination registers of tile loads still in
// flight - copied to the accumulator file right behind the load instruction and reused as the next load's address.
// The static check in tests/test_isa_inflight_loads.py reports exactly that; it has to pass before this file runs on
// a GPU.)
template <int NRT>
__global__ void __launch_bounds__(256, 1) attend_mid_kernel(AttnArgs A) {
  constexpr int TB = (16 * NRT) / kG;          // tokens per row block
  __shared__ __align__(16) uint4 s_q[NRT * 4 * 64];                 // [row tile][scale group][lane]: B operands of the score MFMAs
  // wave merge: up to four row tiles are staged at once (one barrier for the whole merge), more go through two buffers
  // in turn (one barrier per row tile)
  constexpr int kStage = NRT <= 4 ? NRT : 2;
  __shared__ __align__(16) float s_acc[kStage][4][16][kAccPitch];
  __shared__ float s_m[NRT][4][16], s_l[NRT][4][16];
  const int split = blockIdx.x, kvh = blockIdx.y, rb = blockIdx.z;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int tokb = rb * TB, ntok = min(TB, A.M - tokb), nrows = kG * ntok;

  // The tiles of a row block are dealt out to ALL waves of its workgroups round robin: wave gw = 4 split + wave takes the
  // tiles gw, gw + W, gw + 2 W, ... (W = 4 S waves).  Which tile a wave starts with therefore does not depend on the
  // position, and its loads go out before anything else: the position, the query rows and the first tile arrive in ONE
  // trip to memory.  (The tile exists whatever the position is: it lies inside the container.  If it turns out to be
  // beyond the keys this pass sees, or to hold rows this pass is about to store, what was loaded is dropped.)
  const int W = 4 * A.S, gw = 4 * split + wave;
  const LaneOffs offs = lane_offs(i, g);
  const uint32_t ksa_off = kPageKs + 8u * i;       // K scales of key i of a key half: [token][4] fp16
  auto request = [&](int T, MidTile& r) __attribute__((always_inline)) { load_mid_tile(kv_page_uniform(A.kv, kvh, T << 5), (T << 5) % kPageTok, offs, ksa_off, r); };
  MidTile raw;
  request(min(gw, A.kv.max_ctx / 32 - 1), raw);

  // ---- the same trip: the position, the depth entries and the query rows (wave w stages scale group w of every
  //      row tile) ----
  uint4 qraw[NRT];
  int dep[NRT];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    const int R = 16 * rt + i;
    const bool v = R < nrows;
    const int tl = tokb + R / kG, head = kvh * kG + R % kG;
    qraw[rt] = v ? *reinterpret_cast<const uint4*>(A.q16 + ((size_t)tl * A.n_heads + head) * kD + 32 * wave + 8 * g) : make_uint4(0, 0, 0, 0);
    const int tg = A.tok0 + tl;
    dep[rt] = v ? (A.depth ? (int)A.depth[tg] : tg) : -1;
  }
  const int pos = *A.d_pos;
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    const h8 c = __builtin_bit_cast(h8, qraw[rt]);
    const h8 f = h8{c[0], c[4], c[1], c[5], c[2], c[6], c[3], c[7]};       // the element order the K dequantization produces
    s_q[(rt * 4 + wave) * 64 + lane] = __builtin_bit_cast(uint4, f);
  }
  int lenr[NRT];
  int maxlen = 0, minlen = 0x7fffffff;
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    lenr[rt] = dep[rt] >= 0 ? min(pos + dep[rt] + 1, A.kv.max_ctx) : 0;
    maxlen = max(maxlen, lenr[rt]);
    if (dep[rt] >= 0) minlen = min(minlen, lenr[rt]);
  }
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) { maxlen = max(maxlen, __shfl_xor(maxlen, o, 64)); minlen = min(minlen, __shfl_xor(minlen, o, 64)); }
  maxlen = __builtin_amdgcn_readfirstlane(maxlen); minlen = __builtin_amdgcn_readfirstlane(minlen);

  // The grid is sized for the context the caller expects.  A workgroup none of whose waves has a tile (short contexts)
  // leaves the "no keys" marker and exits; the others hold tile counts that differ by at most one.
  const int ntiles = (maxlen + 31) >> 5;
  auto owned = [&](int T) { return (T % W) >> 2 == split; };         // does a wave of this workgroup own tile T
  if (4 * split >= ntiles) {
    if (tid < nrows) {
      const size_t p = ((size_t)(tokb + tid / kG) * A.S + split) * A.n_heads + kvh * kG + tid % kG;
      A.pm[p] = -1e30f; A.pl[p] = 0.f;
    }
    wait_mid_tile(raw);                            // the loads are answered before their registers are given up
    return;
  }

  // ---- fused quantize-on-append.  A block reads rows of the pass up to its own last token; it stores those of them that
  //      lie in its tiles before it loads the tiles (writer and readers are waves of one CU and one write-through L1:
  //      workgroup-scope fences around the barrier).  Row blocks of one kv head write identical bytes.  A row no query
  //      row can see (a depth table may say so) lies past the last tile when it opens a new one: the workgroup of the
  //      last row block that would own that tile stores it. ----
  bool stale = false;                                          // this wave's first tile holds rows this workgroup stores below
  if (A.k16) {
    const int nvis = min(A.M, tokb + ntok);                    // rows of the slice this block may read
    const int nst = rb == (int)gridDim.z - 1 ? A.M : nvis;     // rows it stores if they are its own
    const int r_lo = pos + A.tok0, r_hi = r_lo + nst - 1;
    const bool lastb = rb == (int)gridDim.z - 1;
    bool any_mine = false;                                     // uniform over the workgroup; a slice spans at most 3 tiles
    for (int T = r_lo >> 5; T <= r_hi >> 5; ++T) any_mine |= owned(T);
    stale = any_mine && gw >= (r_lo >> 5) && gw <= (r_hi >> 5);
    if (any_mine) {
      const int c = tid & 15, slot = tid >> 4;                 // 16 lanes per 128-channel row, 16 rows (K and V of 8 tokens) per step
      for (int h0 = 0; h0 < 2 * nst; h0 += 32) {
        uint4 rawv[2];
#pragma unroll
        for (int it = 0; it < 2; ++it) {
          const int hh = h0 + it * 16 + slot, t = hh >> 1;
          const uint16_t* src = ((hh & 1) ? A.v16 : A.k16) + ((size_t)(A.tok0 + t) * A.kv.n_kv + kvh) * kD + 8 * c;
          rawv[it] = t < nst ? *reinterpret_cast<const uint4*>(src) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
          const int hh = h0 + it * 16 + slot, t = hh >> 1, r = pos + A.tok0 + t;
          // rows this block may read; the last block also stores the rows nobody reads (past every visible tile)
          const bool mine = owned(r >> 5) && (t < nvis || (lastb && (r >> 5) >= ntiles));
          if (t < nst && r >= 0 && r < A.kv.max_ctx && mine) quant_store_chunk8(A.kv, kvh, r, hh & 1, rawv[it], c);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    }
    __syncthreads();
    if (any_mine) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    asm volatile("" ::: "memory");               // the tile loads below are instructions the compiler does not see as loads
  } else {
    __syncthreads();                             // the query fragments are in LDS
  }

  const float sc_log2 = kLog2e / sqrtf((float)kD);
  float m_run[NRT], l_run[NRT];
  f4 o[NRT][8];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    m_run[rt] = -1e30f; l_run[rt] = 0.f;
#pragma unroll
    for (int b = 0; b < 8; ++b) { o[rt][b] = f4{0.f, 0.f, 0.f, 0.f}; asm("" : "+a"(o[rt][b])); }
  }
  uint32_t magic = kMagic;
  asm volatile("" : "+v"(magic));

  // one 32-key tile against every row tile of the block
  auto tile = [&](const int T, MidTile& cur, auto&& request_next) __attribute__((always_inline)) {
    const int t0 = T << 5;
    const bool need_mask = t0 + 32 > minlen;     // uniform: only the last tiles hold keys past a row's length
    // ---- the tile's MFMA operands, once: K codes as exact integers (A operand of S^T = K Q^T: key 16kt + i, channels
    //      32m + 8g ..), V scaled (A operand of O^T += V^T P^T: channel 8i + b, tokens tau(g, .)) ----
    // K: code x scale, exact, as the sum of two fp16 images.  The fp16 group scale s (11 significant bits) is cut into
    // hi = its upper 8 bits and lo = s - hi (3 bits): (n - 8) has 3 bits, so (n - 8) * hi and (n - 8) * lo are both
    // exact in fp16 (lo's last bit is s's last bit: no underflow that s itself does not have), and the score MFMAs, which
    // accumulate in fp32, add the two products of every channel without rounding either.  All eight MFMAs of a key half
    // (4 groups x hi, lo) chain into ONE accumulator: a score leaves the matrix pipe finished but for the softmax scale -
    // no multiply-add per score and scale group on the vector unit, a quarter of the partial-sum registers.
    h8 kf[2][2][4];                              // [key half][hi | lo][scale group]
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const uint32_t sw[2] = {cur.ksa[kt][0], cur.ksa[kt][1]};
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const uint32_t pair = sw[m >> 1];
        const uint32_t hi_pair = pair & 0xfff8fff8u;
        const h2 lo_pair = as_h2(pair) - as_h2(hi_pair);
        const _Float16 sh = as_h2(hi_pair)[m & 1], sl = lo_pair[m & 1];
        const h2 sh2 = {sh, sh}, sl2 = {sl, sl};
        const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f};
        const uint32_t w = cur.kw[kt][m];
        // codes n0,n4 | n1,n5 | n2,n6 | n3,n7 as n - 8 (every nibble shifted down to bit 0 / 16: no factor 16 on the odd ones)
        const h2 c0 = as_h2(nib(w, 0x000f000fu, magic)) - c1032, c1 = as_h2(nib(w >> 4, 0x000f000fu, magic)) - c1032;
        const h2 c2 = as_h2(nib(w >> 8, 0x000f000fu, magic)) - c1032, c3 = as_h2(nib(w >> 12, 0x000f000fu, magic)) - c1032;
        const h2 a0 = c0 * sh2, a1 = c1 * sh2, a2 = c2 * sh2, a3 = c3 * sh2;
        const h2 b0 = c0 * sl2, b1 = c1 * sl2, b2 = c2 * sl2, b3 = c3 * sl2;
        kf[kt][0][m] = h8{a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
        kf[kt][1][m] = h8{b0[0], b0[1], b1[0], b1[1], b2[0], b2[1], b3[0], b3[1]};
      }
    }
    h8 vf[8];
    {
      h2 va[8][4];
#pragma unroll
      for (int pe = 0; pe < 4; ++pe) {
        const uint32_t spk = cur.vs[pe >> 1][pe & 1];                            // scales of tokens (2pe, 2pe+1) of this lane
        const h2 s2 = as_h2(spk), s2q = s2 * h2{(_Float16)0.0625f, (_Float16)0.0625f};
        const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f}, c1152 = {(_Float16)1152.f, (_Float16)1152.f};
        const uint32_t w0 = cur.vw[2 * pe], w1 = cur.vw[2 * pe + 1];
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const uint32_t x = __builtin_amdgcn_perm(w1, w0, 0x0c040c00u + bb * 0x00010001u);   // byte bb of both tokens side by side
          va[2 * bb][pe] = (as_h2(nib(x, 0x000f000fu, magic)) - c1032) * s2;
          va[2 * bb + 1][pe] = (as_h2(nib(x, 0x00f000f0u, magic)) - c1152) * s2q;
        }
      }
#pragma unroll
      for (int b = 0; b < 8; ++b)
        vf[b] = h8{va[b][0][0], va[b][0][1], va[b][1][0], va[b][1][1], va[b][2][0], va[b][2][1], va[b][3][0], va[b][3][1]};
    }
    // Everything derived from the raw tile exists before the next tile is requested, and nothing of the raw tile is
    // live when its registers are loaded again: the register set that is waited for at the top of the loop is then the
    // one the request writes (a value kept alive across the request makes the compiler move the whole set with copies
    // placed in front of the wait, i.e. copies of registers whose loads are still in flight; code sunk towards its first
    // use does the same).
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int hl = 0; hl < 2; ++hl) asm volatile("" : "+v"(kf[kt][hl][0]), "+v"(kf[kt][hl][1]), "+v"(kf[kt][hl][2]), "+v"(kf[kt][hl][3]));
    asm volatile("" : "+v"(vf[0]), "+v"(vf[1]), "+v"(vf[2]), "+v"(vf[3]), "+v"(vf[4]), "+v"(vf[5]), "+v"(vf[6]), "+v"(vf[7]));
    __builtin_amdgcn_sched_barrier(0);
    request_next();                              // the raw registers are free: the next tile's loads run under the row tiles
    __builtin_amdgcn_sched_barrier(0);

    // ---- the row tiles, as a software pipeline of depth one in both matrix products: step rt issues the score MFMAs of
    //      row tile rt + 1, turns the partial sums of row tile rt into probabilities (vector work) and issues the PV
    //      MFMAs of row tile rt - 1 between the exponentials.  A wave alone on its SIMD has nobody to fill the slots in
    //      which it waits for its own matrix results; here every MFMA result is consumed one step after it was asked for.
    //      Scheduling barriers keep the steps apart: the registers hold two sets of partial sums, not six. ----
    h8 qf[2][4];
    f4 part[2][2];                               // [set][key half]: finished dot products q . (code x scale)
    h8 pf[2];
    auto load_q = [&](int rt, h8 (&q)[4]) __attribute__((always_inline)) {
#pragma unroll
      for (int m = 0; m < 4; ++m) q[m] = __builtin_bit_cast(h8, s_q[(rt * 4 + m) * 64 + lane]);
    };
    auto scores = [&](const h8 (&q)[4], f4 (&pp)[2]) __attribute__((always_inline)) {
      pp[0] = f4{0.f, 0.f, 0.f, 0.f}; pp[1] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int hl = 0; hl < 2; ++hl)
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)           // the two chains alternate: an MFMA never waits for the one before it
            pp[kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[kt][hl][m], q[m], pp[kt], 0, 0, 0);
    };
    load_q(0, qf[0]);
    scores(qf[0], part[0]);
    if (NRT > 1) load_q(1, qf[1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      const int cs = rt & 1, ns = cs ^ 1;
      if (rt + 1 < NRT) scores(qf[ns], part[ns]);                  // asked for now, consumed in the next step
      if (rt + 2 < NRT) load_q(rt + 2, qf[cs]);                    // the fragments of row tile rt were last read one step ago
      // part[cs][kt][r] = q . k for key t0 + 16kt + 4g + r and row i of row tile rt
      const bool first = m_run[rt] < -1e29f;     // the row has seen no key yet
      const float msub = first ? 0.f : m_run[rt];
      float e[8];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) e[4 * kt + r] = __builtin_fmaf(part[cs][kt][r], sc_log2, -msub);   // exponent of the probability, relative to the running maximum
      if (need_mask) {
#pragma unroll
        for (int k = 0; k < 8; ++k) { const int key = t0 + tau(g, k); e[k] = key < lenr[rt] ? e[k] : -INFINITY; }
      }
      // online softmax with a lazily raised maximum: the row's offset only moves when a score exceeds it by more than
      // 2^kRaiseMid (or on the row's first keys), so the accumulators are rescaled on almost no tile
      float tmax = fmaxf(fmaxf(fmaxf(e[0], e[1]), fmaxf(e[2], e[3])), fmaxf(fmaxf(e[4], e[5]), fmaxf(e[6], e[7])));
      if (__any(tmax > (first ? -INFINITY : kRaiseMid))) {
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const bool seen = tmax > -INFINITY;      // false: every key of the tile lies past the row's length
        const float d = first ? (seen ? tmax : 0.f) : fmaxf(tmax, 0.f);
        const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-d);
        if (!first || seen) m_run[rt] = msub + d;
        if (__any(!first)) {                     // a wave on its first tile finds zeros in l and o: nothing to rescale
          l_run[rt] *= alpha;
#pragma unroll
          for (int b = 0; b < 8; ++b) {
            asm volatile("" : "+a"(o[rt][b]));    // the copy out of the accumulator file stays on this (rare) path
            o[rt][b][0] *= alpha; o[rt][b][1] *= alpha; o[rt][b][2] *= alpha; o[rt][b][3] *= alpha;
            asm volatile("" : "+a"(o[rt][b]));    // and the value is back there before the join: both ways into it agree
          }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) e[k] -= d;
      }
      __builtin_amdgcn_sched_barrier(0);
      // exponentials of row tile rt between the PV MFMAs of row tile rt - 1 (two per pair of probabilities)
      const h2 ones = {(_Float16)1.f, (_Float16)1.f};
      float ls = 0.f;
#pragma unroll
      for (int k = 0; k < 8; k += 2) {
        if (rt > 0) { mfma_pv(o[rt - 1][k], vf[k], pf[ns]); mfma_pv(o[rt - 1][k + 1], vf[k + 1], pf[ns]); }
        asm volatile("" : "+v"(e[k]), "+v"(e[k + 1]));            // this pair's exponentials are issued behind that pair of MFMAs, not ahead of all of them
        h2 p = {(_Float16)__builtin_amdgcn_exp2f(e[k]), (_Float16)__builtin_amdgcn_exp2f(e[k + 1])};
        asm volatile("" : "+v"(p));                               // ... and ahead of the next pair (nor sunk to their first use in the next step)
        ls = __builtin_amdgcn_fdot2(p, ones, ls, false);         // the row sum is taken from the fp16 probabilities the PV product uses
        pf[cs][k] = p[0]; pf[cs][k + 1] = p[1];
      }
      __builtin_amdgcn_sched_barrier(0);
      l_run[rt] += ls;
    }
    operand_ready(pf[(NRT - 1) & 1]);
#pragma unroll
    for (int b = 0; b < 8; ++b) mfma_pv(o[NRT - 1][b], vf[b], pf[(NRT - 1) & 1]);
    // The compiler may move accumulators between registers where control flow joins (it does at the loop's exit) and does
    // not know that the instructions above are still writing them: their passes are drained here, once per tile.
    asm volatile("s_nop 7" : "+a"(o[NRT - 1][0]), "+a"(o[NRT - 1][1]), "+a"(o[NRT - 1][2]), "+a"(o[NRT - 1][3]),
                             "+a"(o[NRT - 1][4]), "+a"(o[NRT - 1][5]), "+a"(o[NRT - 1][6]), "+a"(o[NRT - 1][7]));
    __builtin_amdgcn_sched_barrier(0);
  };

  // The wave's tiles are gw, gw + W, ...  One register set: the request for the next tile goes out as soon as the
  // current one has been turned into operands, and is in flight during the whole walk over the row tiles.  It is always
  // issued (past the end: the current tile again) so that the number of loads in flight at a wait is static.  The first
  // tile was requested at the top of the kernel; a wave whose first tile holds rows that this workgroup has just stored
  // asks for it again (short contexts only: the first W tiles).  Every value of the register set that reaches the loop
  // has passed a wait.
  wait_mid_tile(raw);
  if (stale) {                                     // wave uniform
    MidTile again;
    request(gw, again);
    wait_mid_tile(again);
    raw = again;
  }
  if (gw < ntiles) {
    for (int T = gw;;) {
      tile(T, raw, [&]() __attribute__((always_inline)) { request(T + W < ntiles ? T + W : T, raw); });
      wait_mid_tile(raw);
      T += W;
      if (T >= ntiles) break;
    }
  }
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) pv_done(o[rt]);

  // ---- merge the 4 waves: every wave stages its accumulators, then thread (row j, 8 channels) weighs the four and writes
  //      one normalised fp16 partial row piece.  o[rt][b][r] of lane (row i, group g) is channel 8 (4g + r) + b. ----
  auto stage = [&](int rt) __attribute__((always_inline)) {
    float l = l_run[rt];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (g == 0) { s_m[rt][wave][i] = m_run[rt]; s_l[rt][wave][i] = l; }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float* d = &s_acc[rt % kStage][wave][i][8 * (4 * g + r)];
      *reinterpret_cast<float4*>(d) = make_float4(o[rt][0][r], o[rt][1][r], o[rt][2][r], o[rt][3][r]);
      *reinterpret_cast<float4*>(d + 4) = make_float4(o[rt][4][r], o[rt][5][r], o[rt][6][r], o[rt][7][r]);
    }
  };
  auto reduce = [&](int rt) __attribute__((always_inline)) {
    const int j = tid >> 4, c8 = (tid & 15) * 8, R = 16 * rt + j;
    if (R < nrows) {
      const float m0 = s_m[rt][0][j], m1 = s_m[rt][1][j], m2 = s_m[rt][2][j], m3 = s_m[rt][3][j];
      const float M2 = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));
      const float w[4] = {exp2f(m0 - M2), exp2f(m1 - M2), exp2f(m2 - M2), exp2f(m3 - M2)};
      const float L = w[0] * s_l[rt][0][j] + w[1] * s_l[rt][1][j] + w[2] * s_l[rt][2][j] + w[3] * s_l[rt][3][j];
      float4 a0[4], a1[4];
#pragma unroll
      for (int wv = 0; wv < 4; ++wv) { a0[wv] = *reinterpret_cast<const float4*>(&s_acc[rt % kStage][wv][j][c8]); a1[wv] = *reinterpret_cast<const float4*>(&s_acc[rt % kStage][wv][j][c8 + 4]); }
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int wv = 0; wv < 4; ++wv) {
        acc[0] += w[wv] * a0[wv].x; acc[1] += w[wv] * a0[wv].y; acc[2] += w[wv] * a0[wv].z; acc[3] += w[wv] * a0[wv].w;
        acc[4] += w[wv] * a1[wv].x; acc[5] += w[wv] * a1[wv].y; acc[6] += w[wv] * a1[wv].z; acc[7] += w[wv] * a1[wv].w;
      }
      const float inv = L > 0.f ? 1.f / L : 0.f;
      h8 v;
#pragma unroll
      for (int c = 0; c < 8; ++c) v[c] = (_Float16)(acc[c] * inv);
      const size_t p = ((size_t)(tokb + R / kG) * A.S + split) * A.n_heads + kvh * kG + R % kG;
      *reinterpret_cast<uint4*>(A.pacc16 + p * kD + c8) = __builtin_bit_cast(uint4, v);
      if (c8 == 0) { A.pm[p] = M2; A.pl[p] = L; }
    }
  };
  if constexpr (NRT <= 4) {
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt)
      if (16 * rt < nrows) stage(rt);              // uniform
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt)
      if (16 * rt < nrows) reduce(rt);
  } else {
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      if (16 * rt >= nrows) break;                 // uniform
      stage(rt);
      __syncthreads();
      reduce(rt);
    }
  }
}

int mid_row_tiles(int M) { return (kG * std::min(M, 16) + 15) / 16; }   // row tiles of a block: 16 tokens at most

void launch_attend_mid(const AttnArgs& A, hipStream_t st) {
  // the narrowest kernel whose block holds the window (or 16-token blocks for wider windows)
  const int nrt = std::max(2, mid_row_tiles(A.M));
  const int tb = (16 * nrt) / kG, nb = (A.M + tb - 1) / tb;
  const dim3 grid(A.S, A.kv.n_kv, nb), block(256);
  switch (nrt) {
    case 2: hipLaunchKernelGGL(attend_mid_kernel<2>, grid, block, 0, st, A); break;
    case 3: hipLaunchKernelGGL(attend_mid_kernel<3>, grid, block, 0, st, A); break;
    case 4: hipLaunchKernelGGL(attend_mid_kernel<4>, grid, block, 0, st, A); break;
    case 5: hipLaunchKernelGGL(attend_mid_kernel<5>, grid, block, 0, st, A); break;
    default: hipLaunchKernelGGL(attend_mid_kernel<6>, grid, block, 0, st, A); break;
  }
}

}  // namespace yka
