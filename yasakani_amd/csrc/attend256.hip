// The reference's own KV rows on gfx950: head_dim 256, flat int4 with ONE fp32 scale per row, 4-bit fields MSB first in
// 32-bit words (src/kvq_fast.cuh:194-198,226-233; decode src/kvq_attn.cuh:33-37,53-54).  Quantize-on-append, the
// canonical image, split-KV attention for row tiles of 2 tokens x 6 heads, and the combiner.
//
// Page of one (page, kv head): 256 tokens, 67584 bytes
//   +0      K words  [256][32] uint32      +65536  K scales [256] fp32
//   +32768  V words  [256][32] uint32      +66560  V scales [256] fp32
// Attention follows the 128-channel narrow kernel (same MFMA 16x16x32 layouts: S^T = K Q^T leaves one query row per lane
// column, which is the B-operand layout of O^T += V^T P^T), with what one scale per row allows:
//   * the score of a key is (sum over 256 channels of q * code) * scale: 8 chained MFMAs and ONE multiply;
//   * V codes stay exact integers in the MFMA; the V scale of a key is folded into its probability (p * scale, rounded
//     to fp16 once), the softmax denominator uses the unscaled p.
// Nibble -> fp16: ((w >> s) & 0x000f000f) | 0x64006400 is (1024 + n) in both halves; minus 1032 gives n - 8.  Shift s
// selects elements 7 - s/4 (low half) and 3 - s/4 (high half) of the word, so a word yields its 8 codes in the order
// [7,3,6,2,5,1,4,0]; the query fragments are loaded in the same order.
#include "yka_internal.h"
#include "rot256_device.h"
#include <hip/hip_fp16.h>

namespace yka {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kD2 = 256;
constexpr int kP2Kw = 0, kP2Vw = 32768, kP2Ks = 65536, kP2Vs = 66560;
constexpr uint32_t kMagic = 0x64006400u;
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
__device__ __forceinline__ uint32_t nib(uint32_t w, uint32_t magic) { return (w & 0x000f000fu) | (magic & ~0x000f000fu); }

// start of the (page, kv head) block of token t; t uniform over the wave (table entry through the scalar path)
__device__ __forceinline__ uint8_t* page256(const KvView& kv, int kvh, int t) {
  const int lp = t / kPageTok;
  int pp = lp;
  if (kv.table) pp = table_entry_scalar(kv.table, lp);
  return kv.base + (size_t)(pp * kv.n_kv + kvh) * kPage256Bytes;
}

// One row of 256 values (thread d holds channel d) -> 32 words + one fp32 scale at token `pos` of kv head `kvh`.  Called by
// all 256 threads of a workgroup (three barriers inside); red[4] and fld[256] are its LDS scratch.
__device__ __forceinline__ void quant_store_row256(const KvView& kv, int kvh, int pos, bool isv, float x, int d, float* red, uint8_t* fld) {
  float am = fabsf(x);
#pragma unroll
  for (int o = 32; o; o >>= 1) am = fmaxf(am, __shfl_xor(am, o, 64));
  __syncthreads();                               // the scratch of a previous row is no longer read
  if ((d & 63) == 0) red[d >> 6] = am;
  __syncthreads();
  am = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float s7 = __fdiv_rn(am, 7.f);
  if (s7 == 0.f) s7 = 1.f;
  float q = rintf(__fdiv_rn(x, s7));
  q = fminf(fmaxf(q, -7.f), 7.f);
  fld[d] = (uint8_t)((int)q + 8);
  __syncthreads();
  uint8_t* pg = page256(kv, kvh, pos);
  const int tp = pos % kPageTok;
  if (d < 32) {                                  // word d = fields 8d .. 8d+7, the first in the top nibble
    uint32_t w = 0u;
#pragma unroll
    for (int k = 0; k < 8; ++k) w |= (uint32_t)fld[8 * d + k] << (28 - 4 * k);
    reinterpret_cast<uint32_t*>(pg + (isv ? kP2Vw : kP2Kw))[tp * 32 + d] = w;
  }
  if (d == 0) reinterpret_cast<float*>(pg + (isv ? kP2Vs : kP2Ks))[tp] = s7;
}

// ---- quantize-on-append: grid (M, n_kv * 2), block 256 = one row, thread = channel ----
__global__ void __launch_bounds__(256) append256_kernel(AppendArgs A) {
  __shared__ float red[4];
  __shared__ float buf[256];
  __shared__ uint8_t fld[256];
  const int tok = blockIdx.x, kvh = blockIdx.y >> 1, isv = blockIdx.y & 1, d = threadIdx.x;
  int pos;
  if (A.rows.pos) {                                // multi-stream pass: the row's own container and position
    pos = A.rows.pos[tok];
    const int slot = A.rows.slot[tok];
    if (pos < 0 || pos >= A.kv.max_ctx || slot < 0 || slot >= A.rows.n_slots) return;
    A.kv = slot_view(A.kv, A.rows, slot);
  } else {
    pos = *A.d_pos + tok;
    if (pos < 0 || pos >= A.kv.max_ctx) return;
  }
  const size_t e = ((size_t)tok * A.kv.n_kv + kvh) * kD2 + d;
  float x = A.k32 ? (isv ? A.v32 : A.k32)[e] : __half2float(__ushort_as_half((isv ? A.v16 : A.k16)[e]));
  if (A.rot) x = rotate256(x, buf, false);
  quant_store_row256(A.kv, kvh, pos, isv, x, d, red, fld);
}

// ---- the step between the QKV projection and the cache for 256-channel heads, fused with quantize-on-append
//      (src/q35_kernels.cu:1030-1065 in the reference's own order of operations, with fp16 in the place of its bf16
//      roundings): the projected value is rounded to 16 bits first (:1030); per-head RMS normalisation (sum of squares:
//      butterfly inside each run of 32 channels, then the 8 run sums folded in sequence, :1051-1056), partial rotary
//      embedding with the rotate-half pairing, optional 256-point signed rotation; Q rows leave as fp16, K and V rows go
//      through the row quantizer as fp32 values; gate rows (if given) leave as the rounded projection (:1048).
//      grid (n_heads + 2 n_kv [+ n_heads gate rows], M), block 256 = one head row. ----
__device__ __forceinline__ float f16r256(float x) { asm volatile("" : "+v"(x)); return __half2float(__float2half_rn(x)); }
__global__ void __launch_bounds__(256) attn_post256_kernel(PostArgs A) {
  __shared__ float buf[256];
  __shared__ float red[8];
  __shared__ uint8_t fld[256];
  const int blk = blockIdx.x, tok = blockIdx.y, d = threadIdx.x;
  const int NH = A.n_heads, KVH = A.kv.n_kv;
  const int pos = *A.d_pos + tok;
  if (pos < 0 || pos >= A.kv.max_ctx || (A.rd > 0 && pos >= A.rope_rows)) return;   // rows outside the container are dropped
  if (blk >= NH + 2 * KVH) {                       // gate rows: the projection rounded to the 16-bit type
    const size_t e = ((size_t)tok * NH + (blk - NH - 2 * KVH)) * kD2 + d;
    A.gate16[e] = A.io_bf16 ? f2bf_bits(A.xgate[e]) : __half_as_ushort(__float2half_rn(A.xgate[e]));
    return;
  }
  const bool isq = blk < NH, isk = !isq && blk < NH + KVH;
  const int head = isq ? blk : (isk ? blk - NH : blk - NH - KVH);
  const float* src = isq ? A.xq + ((size_t)tok * NH + head) * kD2
                         : (isk ? A.xk : A.xv) + ((size_t)tok * KVH + head) * kD2;
  const float y = f16r256(src[d]);
  float out;
  if (isq || isk) {
    float ss = __fmul_rn(y, y);
#pragma unroll
    for (int o = 16; o; o >>= 1) ss = __fadd_rn(ss, __shfl_xor(ss, o, 64));
    if ((d & 31) == 0) red[d >> 5] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) tot = __fadd_rn(tot, red[w]);
    // sqrtf, not __fsqrt_rn: only the former is correctly rounded on this target
    const float r = __fdiv_rn(1.f, sqrtf(__fadd_rn(__fdiv_rn(tot, 256.f), A.eps)));
    const float w = __half2float(__ushort_as_half((isq ? A.qn_w16 : A.kn_w16)[d]));
    const float xn = f16r256(__fmul_rn(__fmul_rn(y, r), __fadd_rn(1.f, w)));
    out = xn;
    const int hr = A.rd >> 1;
    if (hr > 0) {
      buf[d] = xn;
      __syncthreads();
      if (d < A.rd) {
        const int i = d < hr ? d : d - hr;
        const float2 cs = reinterpret_cast<const float2*>(A.rope)[(size_t)pos * hr + i];
        const float partner = d < hr ? -buf[d + hr] : buf[d - hr];
        out = f16r256(__fadd_rn(f16r256(__fmul_rn(xn, cs.x)), f16r256(__fmul_rn(partner, cs.y))));
      }
    }
    if (A.rot) out = rotate256(out, buf, false);
  } else {
    out = A.rot ? rotate256(y, buf, false) : y;
  }
  if (isq) {
    asm volatile("" : "+v"(out));                  // the rotation's last multiply is rounded to fp32 before the fp16 rounding
    A.q16[((size_t)tok * NH + head) * kD2 + d] = A.io_bf16 ? f2bf_bits(out) : __half_as_ushort(__float2half_rn(out));
  } else if (A.k32_out) {
    (isk ? A.k32_out : A.v32_out)[((size_t)tok * KVH + head) * kD2 + d] = out;
  } else {
    quant_store_row256(A.kv, head, pos, !isk, out, d, red, fld);
  }
}

// ---- canonical image <-> pages: grid (n, n_kv), block 64: lanes 0..31 move K words, 32..63 V words ----
// rotated query rows: grid rows, block 256
__global__ void __launch_bounds__(256) rotate_q256_kernel(const float* x32, uint16_t* q16) {
  __shared__ float buf[256];
  const size_t e = (size_t)blockIdx.x * kD2 + threadIdx.x;
  q16[e] = __half_as_ushort(__float2half_rn(rotate256(x32[e], buf, false)));
}

template <bool IMPORT>
__global__ void __launch_bounds__(64) xfer256_kernel(KvView kv, int pos0, int n, uint32_t* kw, float* ks, uint32_t* vw, float* vs) {
  const int t = blockIdx.x, kvh = blockIdx.y, j = threadIdx.x & 31, isv = threadIdx.x >> 5;
  uint8_t* pg = page256(kv, kvh, pos0 + t);
  const int tp = (pos0 + t) % kPageTok;
  uint32_t* pw = reinterpret_cast<uint32_t*>(pg + (isv ? kP2Vw : kP2Kw)) + tp * 32 + j;
  float* ps = reinterpret_cast<float*>(pg + (isv ? kP2Vs : kP2Ks)) + tp;
  const size_t row = (size_t)kvh * n + t;
  uint32_t* cw = (isv ? vw : kw) + row * 32 + j;
  float* cs = (isv ? vs : ks) + row;
  if (IMPORT) { *pw = *cw; if (j == 0) *ps = *cs; }
  else { *cw = *pw; if (j == 0) *cs = *ps; }
}

struct Raw256 {        // what one lane holds of a 32-key tile
  uint4 kw[2][2];      // K words of key 16kt + (lane & 15): words 8g .. 8g+7 (g = lane >> 4) = channels 64g .. 64g+63
  f4 ksc[2], vsc[2];   // scales of the 4 keys whose scores this lane receives: keys 16kt + 4g + r
  uint32_t vw[2][8];   // V word (lane & 15) + 16 hh of token tau(g, e)
};
struct Offs256 { uint32_t kw, sc, vw; };

__device__ __forceinline__ void load_tile256(const uint8_t* pg, int tp, const Offs256& L, Raw256& R) {
  const uint8_t* rows = pg + (uint32_t)tp * 128u;          // code rows of the tile (K and V planes)
  const uint8_t* sc = pg + (uint32_t)tp * 4u;              // scale entries of the tile
#pragma unroll
  for (int kt = 0; kt < 2; ++kt) {
    R.kw[kt][0] = *reinterpret_cast<const uint4*>(rows + kP2Kw + L.kw + 2048 * kt);
    R.kw[kt][1] = *reinterpret_cast<const uint4*>(rows + kP2Kw + L.kw + 2048 * kt + 16);
    R.ksc[kt] = *reinterpret_cast<const f4*>(sc + kP2Ks + L.sc + 64 * kt);
    R.vsc[kt] = *reinterpret_cast<const f4*>(sc + kP2Vs + L.sc + 64 * kt);
  }
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int e = 0; e < 8; ++e)                             // token tau(g, e) = 16 (e >> 2) + 4 g + (e & 3)
      R.vw[hh][e] = *reinterpret_cast<const uint32_t*>(rows + kP2Vw + L.vw + (16 * (e >> 2) + (e & 3)) * 128 + 64 * hh);
}

}  // namespace

// grid (S, n_kv, ceil(M/TPT)), block 256 (4 waves, 2 waves per SIMD).  Workgroup = (split, kv head, TPT tokens x 6 heads):
// TPT = 2 for a single-stream pass; MS (multi-stream pass, reference: src/q35_atxpk_ms.cu:13-33): one token per row
// tile, which reads the container and the position its row map names.
template <bool MS>
__global__ void __launch_bounds__(256, 2) attend256_kernel(AttnArgs A) {
  constexpr int TPT = MS ? 1 : 2;
  __shared__ float s_m[4][16], s_l[4][16];
  __shared__ __align__(16) float s_wn[16][4];
  __shared__ float s_acc[4][16][kD2 + 4];
  const int split = blockIdx.x, kvh = blockIdx.y, rt = blockIdx.z;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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
  const int tl = TPT * rt + i / kG;
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
  // as many of the launched splits as the length found on the device justifies (two 32-key tiles per workgroup at
  // least); the others leave the "no keys" marker, whose rows the combiner does not read
  const int ntiles = (maxlen + 31) >> 5;
  const int s_used = min(A.S, max(1, ntiles >> 1));
  if (split >= s_used) {
    const int j = threadIdx.x, tj = TPT * rt + j / kG;
    if (j < TPT * kG && tj < A.M) {
      const size_t p = ((size_t)tj * A.S + split) * A.n_heads + kvh * kG + j % kG;
      A.pm[p] = -1e30f; A.pl[p] = 0.f;
    }
    return;
  }
  const int tps = (ntiles + s_used - 1) / s_used;
  const int tile0 = split * tps, tile1 = min(ntiles, tile0 + tps);

  // ---- fused quantize-on-append (rows of at most 2 tokens, one row tile): a row of this pass is written by the one
  //      workgroup whose tile range holds it - the only workgroup of this kv head that reads it in this launch; writer
  //      and readers are waves of one CU and one write-through L1, so workgroup-scope fences order the stores ----
  if (!MS && A.k16) {
    __shared__ float a_red[4];
    __shared__ uint8_t a_fld[256];
    bool mine = false;
    for (int t = 0; t < A.M; ++t) {
      const int r = pos + A.tok0 + t;
      // A row no query row of this launch can see (a depth table may say so) lies past the last tile when it opens a new
      // one: nobody reads it now, the last workgroup in use stores it.  All conditions are uniform over the workgroup.
      const bool held = (r >> 5) >= tile0 && (r >> 5) < tile1, unseen = (r >> 5) >= ntiles && split == s_used - 1;
      if (r < 0 || r >= A.kv.max_ctx || !(held || unseen)) continue;
      mine = true;
      const size_t e = ((size_t)(A.tok0 + t) * A.kv.n_kv + kvh) * kD2 + threadIdx.x;
      quant_store_row256(A.kv, kvh, r, false, __half2float(__ushort_as_half(A.k16[e])), threadIdx.x, a_red, a_fld);
      quant_store_row256(A.kv, kvh, r, true, __half2float(__ushort_as_half(A.v16[e])), threadIdx.x, a_red, a_fld);
    }
    if (mine) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __syncthreads();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
  }

  // Q fragments: k-step t of 8, lane (row i, group g), element e <-> channel 64g + 8t + [7,3,6,2,5,1,4,0][e]
  h8 qf[8];
  {
    const uint16_t* qrow = A.q16 + ((size_t)tl * A.n_heads + head) * kD2 + 64 * g;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      uint4 u = vrow ? *reinterpret_cast<const uint4*>(qrow + 8 * t) : make_uint4(0, 0, 0, 0);
      const h8 c = __builtin_bit_cast(h8, u);
      qf[t] = h8{c[7], c[3], c[6], c[2], c[5], c[1], c[4], c[0]};
    }
  }
  const float sc_log2 = kLog2e * 0.0625f;          // log2(e) / sqrt(256)
  const h2 c1032 = {(_Float16)1032.f, (_Float16)1032.f};
  uint32_t magic = kMagic;
  asm volatile("" : "+v"(magic));
  const Offs256 offs{(uint32_t)i * 128u + 32u * g, 16u * g, 512u * g + 4u * i};

  float m_run = -1e30f, l_run = 0.f;
  f4 o[16];
#pragma unroll
  for (int b = 0; b < 16; ++b) o[b] = f4{0.f, 0.f, 0.f, 0.f};

  Raw256 cur;
  for (int T = tile0 + wave; T < tile1; T += 4) {
    load_tile256(page256(A.kv, kvh, T << 5), (T << 5) % kPageTok, offs, cur);
    const int t0 = T << 5;
    const bool need_mask = t0 + 32 > minlen;
    // ---- scores: per 16-key tile 8 chained MFMAs (one per word of the lane), then one multiply by the key's scale ----
    float s[8];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const uint32_t w[8] = {cur.kw[kt][0].x, cur.kw[kt][0].y, cur.kw[kt][0].z, cur.kw[kt][0].w,
                             cur.kw[kt][1].x, cur.kw[kt][1].y, cur.kw[kt][1].z, cur.kw[kt][1].w};
      f4 part = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const h2 p0 = as_h2(nib(w[t], magic)) - c1032, p1 = as_h2(nib(w[t] >> 4, magic)) - c1032;
        const h2 p2 = as_h2(nib(w[t] >> 8, magic)) - c1032, p3 = as_h2(nib(w[t] >> 12, magic)) - c1032;
        const h8 kf = h8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[t], part, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) s[4 * kt + r] = part[r] * cur.ksc[kt][r];      // key t0 + 16kt + 4g + r against row i
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
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    const bool first = m_run < -1e29f;
    m_run = m_new;
    if (__any(alpha != 1.f && !first)) {
      l_run *= alpha;
#pragma unroll
      for (int b = 0; b < 16; ++b) { o[b][0] *= alpha; o[b][1] *= alpha; o[b][2] *= alpha; o[b][3] *= alpha; }
    }
    h8 pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], sc_log2, -m_new));
      l_run += p;
      pf[e] = (_Float16)(p * cur.vsc[e >> 2][e & 3]);       // the V scale of the key rides on its probability
    }
    // ---- O^T += V^T P^T: word (lane & 15) + 16 hh of 8 tokens; byte bb of those words holds elements 7-2bb (low
    //      nibble) and 6-2bb (high nibble): accumulator hh*8 + element covers channels 8 * word + element ----
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        h2 lo[4], hi[4];
#pragma unroll
        for (int pe = 0; pe < 4; ++pe) {
          const uint32_t x = __builtin_amdgcn_perm(cur.vw[hh][2 * pe + 1], cur.vw[hh][2 * pe], 0x0c040c00u + bb * 0x00010001u);
          lo[pe] = as_h2(nib(x, magic)) - c1032;
          hi[pe] = as_h2(nib(x >> 4, magic)) - c1032;
        }
        const h8 vlo = h8{lo[0][0], lo[0][1], lo[1][0], lo[1][1], lo[2][0], lo[2][1], lo[3][0], lo[3][1]};
        const h8 vhi = h8{hi[0][0], hi[0][1], hi[1][0], hi[1][1], hi[2][0], hi[2][1], hi[3][0], hi[3][1]};
        o[hh * 8 + 7 - 2 * bb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vlo, pf, o[hh * 8 + 7 - 2 * bb], 0, 0, 0);
        o[hh * 8 + 6 - 2 * bb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vhi, pf, o[hh * 8 + 6 - 2 * bb], 0, 0, 0);
      }
  }
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
  // per row: the weight of each wave's accumulator, already divided by the row's sum - computed once per row by 4 lanes,
  // not once per output element
  if (threadIdx.x < 64) {
    const int j = threadIdx.x >> 2, w = threadIdx.x & 3;
    const float mw = s_m[w][j];
    float M2 = fmaxf(mw, __shfl_xor(mw, 1, 64));
    M2 = fmaxf(M2, __shfl_xor(M2, 2, 64));
    const float ww = exp2f(mw - M2);
    float L = ww * s_l[w][j];
    L += __shfl_xor(L, 1, 64);
    L += __shfl_xor(L, 2, 64);
    s_wn[j][w] = L > 0.f ? ww / L : 0.f;
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
    const float y = w4[0] * s_acc[0][j][d] + w4[1] * s_acc[1][j][d] + w4[2] * s_acc[2][j][d] + w4[3] * s_acc[3][j][d];
    A.pacc16[p * kD2 + d] = __half_as_ushort(__float2half_rn(y));
  }
}

// combiner (src/attention_kv4q.cu:325-332) for 256-channel rows: grid (n_heads, M), block 256 = 8 split lanes x 32 channel
// lanes of 8 channels; the split lanes run in parallel and are summed through LDS.  S <= 256.  kInFlight = partial rows a
// split lane requests before it uses any: 16 covers 128 splits (decode: few, long workgroups; 32 for up to 256 splits), 4 covers
// 32 and keeps the register count low where thousands of workgroups run (wide windows).
template <int kInFlight>
__global__ void __launch_bounds__(256) combine256_kernel(CombineArgs A) {
  __shared__ float s_w[256];
  __shared__ float s_o[8][kD2 + 4];
  __shared__ float s_wsum[8];
  const int head = blockIdx.x, tok = blockIdx.y, tid = threadIdx.x;
  const size_t p0 = (size_t)tok * A.S * A.n_heads + head;
  // 8 split lanes; each takes splits sl, sl + 8, ... (at most kInFlight of them: the launcher picks kInFlight so that
  // 8 * kInFlight >= S).  Their partial rows are requested first, together with the (m, l) pairs the weights come from:
  // one memory round trip instead of two.  A row of weight 0 may be one that no workgroup wrote: it is zeroed before use.
  const int sl = tid >> 5, c8 = (tid & 31) * 8;
  const uint16_t* src = A.pacc16 + p0 * kD2 + c8;
  const size_t stride = (size_t)A.n_heads * kD2;
  uint4 u[kInFlight];
#pragma unroll
  for (int k = 0; k < kInFlight; ++k) {
    const int sp = sl + 8 * k;
    u[k] = sp < A.S ? *reinterpret_cast<const uint4*>(src + (size_t)sp * stride) : make_uint4(0, 0, 0, 0);
  }
  float pmv = -1e30f, plv = 0.f;
  if (tid < A.S) { pmv = A.pm[p0 + (size_t)tid * A.n_heads]; plv = A.pl[p0 + (size_t)tid * A.n_heads]; }
  float M2 = pmv;
#pragma unroll
  for (int o = 32; o; o >>= 1) M2 = fmaxf(M2, __shfl_xor(M2, o, 64));
  if ((tid & 63) == 0) s_wsum[tid >> 6] = M2;
  __syncthreads();
  M2 = fmaxf(fmaxf(s_wsum[0], s_wsum[1]), fmaxf(s_wsum[2], s_wsum[3]));
  __syncthreads();
  s_w[tid] = (tid < A.S && pmv > -1e29f) ? exp2f(pmv - M2) * plv : 0.f;
  __syncthreads();
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float wsum = 0.f;
#pragma unroll
  for (int k = 0; k < kInFlight; ++k) {
    const int sp = sl + 8 * k;
    const float w = sp < A.S ? s_w[sp] : 0.f;
    const uint4 r = w != 0.f ? u[k] : make_uint4(0, 0, 0, 0);
    const h8 v = __builtin_bit_cast(h8, r);
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] += w * (float)v[c];
    wsum += w;
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) s_o[sl][c8 + c] = acc[c];
  if ((tid & 31) == 0) s_wsum[sl] = wsum;
  __syncthreads();
  float o = 0.f, L = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) { o += s_o[k][tid]; L += s_wsum[k]; }
  float y = L > 0.f ? __fdiv_rn(o, L) : 0.f;
  if (A.unrot) y = rotate256(y, s_w, true);        // inverse of the rotation of the V rows (src/q35_kernels.cu:1421); s_w is free again
  A.out16[((size_t)tok * A.n_heads + head) * kD2 + tid] = A.out_bf16 ? f2bf_bits(y) : __half_as_ushort(__float2half_rn(y));
}

void launch_attn_post256(const PostArgs& A, hipStream_t st) {
  hipLaunchKernelGGL(attn_post256_kernel, dim3(A.n_heads + 2 * A.kv.n_kv + (A.gate16 ? A.n_heads : 0), A.M), dim3(256), 0, st, A);
}
void launch_append256(const AppendArgs& A, hipStream_t st) {
  hipLaunchKernelGGL(append256_kernel, dim3(A.M, A.kv.n_kv * 2), dim3(256), 0, st, A);
}
void launch_rotate_q256(const float* x32, int rows, uint16_t* q16, hipStream_t st) {
  hipLaunchKernelGGL(rotate_q256_kernel, dim3(rows), dim3(256), 0, st, x32, q16);
}
void launch_attend256(const AttnArgs& A, hipStream_t st) {
  if (A.rows.pos) hipLaunchKernelGGL(attend256_kernel<true>, dim3(A.S, A.kv.n_kv, A.M), dim3(256), 0, st, A);
  else hipLaunchKernelGGL(attend256_kernel<false>, dim3(A.S, A.kv.n_kv, (A.M + 1) / 2), dim3(256), 0, st, A);
}
void launch_combine256(const CombineArgs& A, hipStream_t st) {
  // 8 split lanes x kInFlight rows each must cover the S <= 256 splits
  if (A.S > 128) hipLaunchKernelGGL(combine256_kernel<32>, dim3(A.n_heads, A.M), dim3(256), 0, st, A);
  else if (A.S > 32) hipLaunchKernelGGL(combine256_kernel<16>, dim3(A.n_heads, A.M), dim3(256), 0, st, A);
  else hipLaunchKernelGGL(combine256_kernel<4>, dim3(A.n_heads, A.M), dim3(256), 0, st, A);
}
void launch_export_rows256(const KvView& kv, int pos0, int n, uint32_t* kw, float* ks, uint32_t* vw, float* vs, hipStream_t st) {
  hipLaunchKernelGGL(xfer256_kernel<false>, dim3(n, kv.n_kv), dim3(64), 0, st, kv, pos0, n, kw, ks, vw, vs);
}
void launch_import_rows256(const KvView& kv, int pos0, int n, const uint32_t* kw, const float* ks, const uint32_t* vw, const float* vs, hipStream_t st) {
  hipLaunchKernelGGL(xfer256_kernel<true>, dim3(n, kv.n_kv), dim3(64), 0, st, kv, pos0, n, const_cast<uint32_t*>(kw), const_cast<float*>(ks),
                     const_cast<uint32_t*>(vw), const_cast<float*>(vs));
}

}  // namespace yka
