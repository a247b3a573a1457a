// Split-KV attention over trellis-coded rows (the reference's KV4 / KV5 packed streams), gfx950, wave64, MFMA 16x16x32 f16.
//   reference: launch_q35_atx_pk (src/q35_atxpk.hpp:14-17; decode helpers src/q35_atxpk.cu:70-106, scalar form
//   tba_attention_kernel, src/kvq_attn.cuh:120-310).  Rows live as the reference lays them out: payload
//   (kvh * max_ctx + pos) * stride bytes, one fp32 scale per row in a parallel array (src/q35_atxpk3.cuh:196-200).
// A row is 4 chunks of 64 elements; element e of a chunk decodes to table[state] * scale with state = the last 8 bits of
// the chunk's MSB-first stream up to the end of field e.  What is specific to this GPU:
//   * the tile geometry of the 256-channel flat kernel (attend256.hip): a wave owns 32 keys, lane (i, g) holds key i's
//     chunk g for the scores - so a lane decodes a whole chunk from its own 8 or 10 words, no neighbour needed - and
//     the 8-channel block i + 16 hh of the 8 tokens whose probabilities it receives for O^T += V^T P^T;
//   * the table holds the reference's integers (|value| <= 1100, exact in fp16); the factor gain / 256 and the row scale
//     are applied in fp32 to the MFMA's sums (K) or ride on the probability and the final accumulator (V), so no table
//     value is rounded (the reference rounds its table to bf16);
//   * one LDS read decodes TWO elements: the states of elements e and e + 1 are both contained in the 8 + kb stream bits
//     that end with field e + 1, so a table of 2^(8 + kb) entries of two fp16 values (16 KB at 4 bits, 32 KB at 5, per
//     table; built when the profile is set, copied into LDS by every workgroup, in the space the wave merge uses
//     afterwards) turns one funnel shift, one mask and one 32-bit gather into a finished pair of MFMA operand halves.
//     The reference keeps a 4096-entry pair table for 4-bit rows (src/q35_atxpk3.cuh:66-78);
//   * a mean row of K shifts every score of a query row by the same q.mu and cancels in the softmax: it is not added.
//     A mean row of V is added to the normalised partial (the probabilities of a split sum to one).
#include "yka_internal.h"
#include <hip/hip_fp16.h>

namespace yka {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kD2 = 256;

__device__ __forceinline__ uint32_t funnel(uint32_t hi, uint32_t lo, uint32_t sh) { return __builtin_amdgcn_alignbit(hi, lo, sh); }   // (hi:lo) >> sh
// byte offset (entry index x 4) of the pair entry for the KB + 8 stream bits that end at bit `endbit` (exclusive) of a chunk
// held as words w[]; bits before the chunk start count as zero.  Everything but w is a compile-time constant.
template <int KB>
__device__ __forceinline__ uint32_t pair_offset(const uint32_t* w, int endbit) {
  constexpr uint32_t mask4 = ((1u << (8 + KB)) - 1u) << 2;
  const int j = (endbit - 1) >> 5, r = 31 - ((endbit - 1) & 31);            // word of the last bit, bits to its right
  const uint32_t hi = j > 0 ? w[j - 1] : 0u;
  if (r >= 2) return (r == 2 ? w[j] : funnel(hi, w[j], (uint32_t)(r - 2))) & mask4;
  return (funnel(hi, w[j], (uint32_t)r) << 2) & mask4;
}
__device__ __forceinline__ uint32_t pair_at(const uint8_t* tab, uint32_t off) { return *reinterpret_cast<const uint32_t*>(tab + off); }

// 8 consecutive elements Q0 .. Q0 + 7 (Q0 a compile-time multiple of 8) of a chunk held as 2 KB words
template <int KB, int Q0>
__device__ __forceinline__ h8 chunk_vals(const uint32_t* w, const uint8_t* tab) {
  uint32_t d[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) d[p] = pair_at(tab, pair_offset<KB>(w, KB * (Q0 + 2 * p + 2)));
  return __builtin_bit_cast(h8, uint4{d[0], d[1], d[2], d[3]});
}

// MS: multi-stream pass (reference: src/q35_atxpk_ms.cu:13-33, which runs on packed rows) - one token per row tile, which
// reads the container and the position its row map names
template <int KB, bool MS>
__global__ void __launch_bounds__(256, 2) attend_tb_kernel(TbAttnArgs A) {
  constexpr int TPT = MS ? 1 : 2;                    // tokens per row tile
  constexpr int NW = 2 * KB;                         // words per chunk
  constexpr int kTabBytes = 4 << (8 + KB);           // one pair table
  constexpr int kAccBytes = 4 * 16 * (kD2 + 4) * 4;
  __shared__ float s_m[4][16], s_l[4][16];
  __shared__ __align__(16) float s_wn[16][4];
  __shared__ __align__(16) uint8_t s_buf[kAccBytes > 2 * kTabBytes ? kAccBytes : 2 * kTabBytes];   // pair tables, then the wave merge
  float (*s_acc)[16][kD2 + 4] = reinterpret_cast<float (*)[16][kD2 + 4]>(s_buf);
  const uint8_t* const s_tabK = s_buf;
  const uint8_t* const s_tabV = s_buf + kTabBytes;
  const int split = blockIdx.x, kvh = blockIdx.y, rt = blockIdx.z;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
  const int gK = (A.layer * A.n_kv + kvh) * 2, gV = gK + 1;
  int pos; bool row_ok = true;
  if (MS) {
    pos = A.rows.pos[rt];
    const int slot = A.rows.slot[rt];
    row_ok = pos >= 0 && pos < A.max_ctx && slot >= 0 && slot < A.rows.n_slots;   // a bad row reads nothing and yields zeros
    const size_t off = row_ok ? (size_t)slot * A.rows.slot_bytes : 0;
    A.kpay += off; A.vpay += off;
    A.kscl = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(A.kscl) + off);
    A.vscl = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(A.vscl) + off);
  } else {
    pos = *A.d_pos;
  }
  const int tl = TPT * rt + i / kG;
  const bool vrow = i < TPT * kG && tl < A.M && row_ok;
  const int head = kvh * kG + i % kG;
  int len = 0;
  if (vrow) {
    if (MS) len = pos + 1;
    else { const int tg = A.tok0 + tl; len = pos + (A.depth ? (int)A.depth[tg] : tg) + 1; }
    len = min(len, A.max_ctx);
  }
  int maxlen = len, minlen = vrow ? len : 0x7fffffff;
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) { maxlen = max(maxlen, __shfl_xor(maxlen, o, 64)); minlen = min(minlen, __shfl_xor(minlen, o, 64)); }
  maxlen = __builtin_amdgcn_readfirstlane(maxlen); minlen = __builtin_amdgcn_readfirstlane(minlen);
  const int ntiles = (maxlen + 31) >> 5;
  const int s_used = min(A.S, max(1, ntiles >> 1));
  if (split >= s_used) {                             // the "no keys" marker; the combiner does not read such rows
    const int j = threadIdx.x, tj = TPT * rt + j / kG;
    if (j < TPT * kG && tj < A.M) {
      const size_t p = ((size_t)tj * A.S + split) * A.n_heads + kvh * kG + j % kG;
      A.pm[p] = -1e30f; A.pl[p] = 0.f;
    }
    return;
  }
  {                                                  // the K and V pair tables of this kv head: global (L2) -> LDS
    const uint4* srcK = reinterpret_cast<const uint4*>(A.pairs + (size_t)gK * (kTabBytes / 4));
    const uint4* srcV = reinterpret_cast<const uint4*>(A.pairs + (size_t)gV * (kTabBytes / 4));
    uint4* dst = reinterpret_cast<uint4*>(s_buf);
#pragma unroll 4
    for (int x = threadIdx.x; x < kTabBytes / 16; x += 256) { dst[x] = srcK[x]; dst[kTabBytes / 16 + x] = srcV[x]; }
  }
  __syncthreads();
  const int tps = (ntiles + s_used - 1) / s_used;
  const int tile0 = split * tps, tile1 = min(ntiles, tile0 + tps);

  h8 qf[8];                                          // k-step t: channels 64 g + 8 t .. + 7 of row i
  {
    const uint16_t* qrow = A.q16 + ((size_t)tl * A.n_heads + head) * kD2 + 64 * g;
#pragma unroll
    for (int t = 0; t < 8; ++t) qf[t] = __builtin_bit_cast(h8, vrow ? *reinterpret_cast<const uint4*>(qrow + 8 * t) : make_uint4(0, 0, 0, 0));
  }
  const float sc_log2 = kLog2e * 0.0625f * A.gfac[gK];      // log2(e) / sqrt(256) x gain / 256 of the K table
  const size_t row0 = (size_t)kvh * A.max_ctx;
  const uint8_t* const kbase = A.kpay + row0 * A.stride + (uint32_t)g * (4u * NW);
  const float* const kscl = A.kscl + row0;
  const float* const vscl = A.vscl + row0;
  // V: lane (i, g) needs, for hh = 0, 1, the 8 elements of block cb = i + 16 hh of 8 tokens.  Inside its chunk the block
  // starts at bit KB * 8 * c (c = cb & 7); the window that also holds the 8 - KB bits before it (zero at a chunk start)
  // starts at bit s0 = KB * 8 * c - (8 - KB), i.e. in word w0 = floor(s0 / 32) at offset off - never 0 for KB 4 or 5.
  const int c8 = i & 7;
  const int s0 = KB * 8 * c8 - (8 - KB);
  const int w0 = s0 >> 5;                            // -1 for the first block of a chunk
  const uint32_t sh = 32u - (uint32_t)(s0 & 31);
  // byte offset, inside a V row, of the window's first word for hh = 0, 1.  For the first block of a chunk that is the
  // word BEFORE the chunk (w0 = -1): it is loaded like any other (the word before row 0 of the V payload is the last
  // word of the K payload, the word after a row's last chunk is the next row or the scale array: same allocation) and
  // masked to zero; words past the window's last needed bit are never used.
  uint32_t vo[2];
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) vo[hh] = (uint32_t)((i + 16 * hh) >> 3) * (4u * NW) + 4u * (uint32_t)w0;
  const uint32_t keep0 = c8 == 0 ? 0u : 0xffffffffu;

  float m_run = -1e30f, l_run = 0.f;
  f4 o[16];
#pragma unroll
  for (int b = 0; b < 16; ++b) o[b] = f4{0.f, 0.f, 0.f, 0.f};

  // K words and K scales of a tile are requested one tile ahead (right after the scores of the tile before have consumed
  // the registers they land in); V words at the top of their own tile, a whole score phase before their first use
  uint32_t kw[2][NW];
  f4 ksc[2];
  auto load_k = [&](int T) __attribute__((always_inline)) {
    const int t0 = T << 5;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const uint8_t* kr = kbase + (size_t)(t0 + 16 * kt + i) * A.stride;
      if (KB == 4) {
        const uint4 a = *reinterpret_cast<const uint4*>(kr), b = *reinterpret_cast<const uint4*>(kr + 16);
        kw[kt][0] = a.x; kw[kt][1] = a.y; kw[kt][2] = a.z; kw[kt][3] = a.w; kw[kt][4] = b.x; kw[kt][5] = b.y; kw[kt][6] = b.z; kw[kt][7] = b.w;
      } else {
        __builtin_memcpy(&kw[kt][0], __builtin_assume_aligned(kr, 8), 16);          // 40-byte chunks: 8-byte aligned
        __builtin_memcpy(&kw[kt][4], __builtin_assume_aligned(kr + 16, 8), 16);
        __builtin_memcpy(&kw[kt][8], __builtin_assume_aligned(kr + 32, 8), 8);
      }
      ksc[kt] = *reinterpret_cast<const f4*>(kscl + t0 + 16 * kt + 4 * g);
    }
  };
  if (tile0 + wave < tile1) load_k(tile0 + wave);
  for (int T = tile0 + wave; T < tile1; T += 4) {
    const int t0 = T << 5;
    f4 vsc[2];
    uint32_t vw[2][8][3];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) vsc[kt] = *reinterpret_cast<const f4*>(vscl + t0 + 16 * kt + 4 * g);
    // V windows of the channel blocks hh = 0 now (their latency runs under the score phase), those of hh = 1 after the
    // score phase (under the softmax and the first half of the PV product): the registers are needed in between
    auto load_v = [&](int hh) __attribute__((always_inline)) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int tok = t0 + 16 * (e >> 2) + 4 * g + (e & 3);
        const uint8_t* vr = A.vpay + (row0 + tok) * A.stride;
        vw[hh][e][2] = 0u;
        __builtin_memcpy(&vw[hh][e][0], __builtin_assume_aligned(vr + (int32_t)vo[hh], 4), KB == 5 ? 12 : 8);
        vw[hh][e][0] &= keep0;
      }
    };
    load_v(0);
    const bool need_mask = t0 + 32 > minlen;
    // ---- scores ----
    float s[8];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      // at 4 bits per element all 32 table reads of the key block are issued ahead of the MFMA chain, so that the chain
      // does not wait for LDS between links (measured 6 % on the decode kernel); at 5 bits the registers do not allow it
      f4 part = f4{0.f, 0.f, 0.f, 0.f};
      if constexpr (KB == 4) {
        h8 kf[8];
        kf[0] = chunk_vals<KB, 0>(kw[kt], s_tabK); kf[1] = chunk_vals<KB, 8>(kw[kt], s_tabK);
        kf[2] = chunk_vals<KB, 16>(kw[kt], s_tabK); kf[3] = chunk_vals<KB, 24>(kw[kt], s_tabK);
        kf[4] = chunk_vals<KB, 32>(kw[kt], s_tabK); kf[5] = chunk_vals<KB, 40>(kw[kt], s_tabK);
        kf[6] = chunk_vals<KB, 48>(kw[kt], s_tabK); kf[7] = chunk_vals<KB, 56>(kw[kt], s_tabK);
#pragma unroll
        for (int t = 0; t < 8; ++t) part = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[t], qf[t], part, 0, 0, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 70, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 32, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      } else {
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 0>(kw[kt], s_tabK), qf[0], part, 0, 0, 0);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 8>(kw[kt], s_tabK), qf[1], part, 0, 0, 0);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 16>(kw[kt], s_tabK), qf[2], part, 0, 0, 0);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 24>(kw[kt], s_tabK), qf[3], part, 0, 0, 0);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 32>(kw[kt], s_tabK), qf[4], part, 0, 0, 0);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 40>(kw[kt], s_tabK), qf[5], part, 0, 0, 0);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 48>(kw[kt], s_tabK), qf[6], part, 0, 0, 0);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_vals<KB, 56>(kw[kt], s_tabK), qf[7], part, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) s[4 * kt + r] = part[r] * ksc[kt][r];          // key t0 + 16 kt + 4 g + r against row i
    }
    load_v(1);
    if (T + 4 < tile1) load_k(T + 4);
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
    const float m_new = fmaxf(m_run, tmax * sc_log2);          // the table's gain is positive (checked when the profile is set)
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    const bool first_tile = m_run < -1e29f;
    m_run = m_new;
    if (__any(alpha != 1.f && !first_tile)) {
      l_run *= alpha;
#pragma unroll
      for (int b = 0; b < 16; ++b) { o[b][0] *= alpha; o[b][1] *= alpha; o[b][2] *= alpha; o[b][3] *= alpha; }
    }
    h8 pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], sc_log2, -m_new));
      l_run += p;
      pf[e] = (_Float16)(p * vsc[e >> 2][e & 3]);            // the V scale of the key rides on its probability
    }
    // ---- O^T += V^T P^T: accumulator hh * 8 + el covers channel 8 (i + 16 hh) + el ----
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      uint32_t y0[8], y1[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        y0[e] = funnel(vw[hh][e][0], vw[hh][e][1], sh);
        y1[e] = funnel(vw[hh][e][1], vw[hh][e][2], sh);
      }
#pragma unroll
      for (int el = 0; el < 8; el += 2) {                      // elements el, el + 1 = bits [KB el, KB el + KB + 8) of y0:y1
        constexpr uint32_t mask4 = ((1u << (8 + KB)) - 1u) << 2;
        const int q = KB * el + 8 + KB;                        // end of the pair's bits
        uint32_t pr[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          uint32_t off;
          if (q <= 30) off = (y0[e] >> (30 - q)) & mask4;
          else if (q <= 32) off = (y0[e] << (q - 30)) & mask4;
          else off = funnel(y0[e], y1[e], (uint32_t)(62 - q)) & mask4;
          pr[e] = pair_at(s_tabV, off);
        }
        uint32_t a[4], b[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          a[t] = __builtin_amdgcn_perm(pr[2 * t + 1], pr[2 * t], 0x05040100u);     // element el of tokens 2t, 2t + 1
          b[t] = __builtin_amdgcn_perm(pr[2 * t + 1], pr[2 * t], 0x07060302u);     // element el + 1
        }
        o[hh * 8 + el] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, uint4{a[0], a[1], a[2], a[3]}), pf, o[hh * 8 + el], 0, 0, 0);
        o[hh * 8 + el + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, uint4{b[0], b[1], b[2], b[3]}), pf, o[hh * 8 + el + 1], 0, 0, 0);
      }
    }
  }
  __syncthreads();                                   // every wave is done with the tables: their space now holds the merge
  // ---- merge the 4 waves, write one partial per (row, split): o[hh*8 + el][r] = channel 8 (4g + r + 16 hh) + el of row i ----
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (g == 0) { s_m[wave][i] = m_run; s_l[wave][i] = l_run; }
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int el = 0; el < 8; ++el)
#pragma unroll
      for (int r = 0; r < 4; ++r) s_acc[wave][i][8 * (4 * g + r + 16 * hh) + el] = o[hh * 8 + el][r];
  __syncthreads();
  // per row: the weight of each wave's accumulator, already divided by the row's sum and multiplied by gain / 256 of the
  // V table - computed once per row by 4 lanes, not once per output element
  if (threadIdx.x < 64) {
    const int j = threadIdx.x >> 2, w = threadIdx.x & 3;
    const float mw = s_m[w][j];
    float M2 = fmaxf(mw, __shfl_xor(mw, 1, 64));
    M2 = fmaxf(M2, __shfl_xor(M2, 2, 64));
    const float ww = exp2f(mw - M2);
    float L = ww * s_l[w][j];
    L += __shfl_xor(L, 1, 64);
    L += __shfl_xor(L, 2, 64);
    s_wn[j][w] = L > 0.f ? ww * A.gfac[gV] / L : 0.f;
    const int tj = TPT * rt + j / kG;
    if (w == 0 && j < TPT * kG && tj < A.M) {
      const size_t p = ((size_t)tj * A.S + split) * A.n_heads + kvh * kG + j % kG;
      A.pm[p] = M2; A.pl[p] = L;
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < TPT * kG * kD2; idx += 256) {
    const int j = idx >> 8, d = idx & (kD2 - 1);
    const int tj = TPT * rt + j / kG;
    if (tj >= A.M) continue;
    const f4 w4 = *reinterpret_cast<const f4*>(s_wn[j]);
    const size_t p = ((size_t)tj * A.S + split) * A.n_heads + kvh * kG + j % kG;
    float y = w4[0] * s_acc[0][j][d] + w4[1] * s_acc[1][j][d] + w4[2] * s_acc[2][j][d] + w4[3] * s_acc[3][j][d];
    if (A.mu && w4[0] + w4[1] + w4[2] + w4[3] > 0.f) y += A.mu[(size_t)gV * 256 + d];
    A.pacc16[p * kD2 + d] = __half_as_ushort(__float2half_rn(y));
  }
}

}  // namespace

void launch_attend_tb(const TbAttnArgs& A, int kb, hipStream_t st) {
  if (A.rows.pos) {
    const dim3 grid(A.S, A.n_kv, A.M);
    if (kb == 4) hipLaunchKernelGGL((attend_tb_kernel<4, true>), grid, dim3(256), 0, st, A);
    else hipLaunchKernelGGL((attend_tb_kernel<5, true>), grid, dim3(256), 0, st, A);
    return;
  }
  const dim3 grid(A.S, A.n_kv, (A.M + 1) / 2);
  if (kb == 4) hipLaunchKernelGGL((attend_tb_kernel<4, false>), grid, dim3(256), 0, st, A);
  else hipLaunchKernelGGL((attend_tb_kernel<5, false>), grid, dim3(256), 0, st, A);
}

}  // namespace yka
