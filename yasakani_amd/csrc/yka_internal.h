// Internal declarations shared by the translation units of libyka.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace yka {

// ---- fixed shape of the path ----
constexpr int kD = 128;          // head_dim
constexpr int kG = 6;            // query heads per KV head
constexpr int kGroup = 32;       // channels per scale group
constexpr int kNG = kD / kGroup; // scale groups per row (4)
constexpr int kPageTok = 256;    // tokens per page
// ---- physical page of one (page, kv head): 256 tokens, 36864 bytes, four planes ----
//   +0      K codes  [256][64]  byte j of a row: channel 2j low nibble, 2j+1 high nibble, value q+8; the 16 dwords of a
//                                row are stored in the order physical 4g+m = logical 4m+g, so that the 16-byte chunk g
//                                holds channels {32m + 8g .. 32m + 8g + 7 : m = 0..3} - one dword of every scale group
//   +16384  V codes  [256][64]  plain channel order
//   +32768  K scales [256][4]   fp16, token major
//   +34816  V scales [4][256]   fp16, group major (4 consecutive tokens of one group are 8 contiguous bytes)
constexpr int kPageKc = 0, kPageVc = 16384, kPageKs = 32768, kPageVs = 34816, kPageBytes = 36864;
__host__ __device__ inline int k_phys_dword(int logical) { return 4 * (logical & 3) + (logical >> 2); }
constexpr int kPage256Bytes = 67584;   // page of the 256-channel row format (attend256.hip): 256 x (128 + 128) code bytes + 2 x 256 fp32 scales
constexpr int kMaxSlice = 64;    // rows per attention slice (kVerifyMax of the reference, engine35.hpp:157)

// One layer's container.  The page of token t of kv head h starts at
//   base + (p * n_kv + h) * 36864,   p = table ? table[t / 256] : t / 256
struct KvView {
  uint8_t* base;
  const int32_t* table;  // nullptr in contiguous mode
  int n_kv;
  int max_ctx;
};
__host__ __device__ inline size_t kv_page_bytes(int n_kv) { return (size_t)n_kv * kPageBytes; }

// Multi-stream passes (reference: Q35MsRows, src/q35.hpp:28-35): row t of the pass belongs to the stream whose container
// is slot[t] and sits at position pos[t] of it.  Containers are slot_bytes apart (page tables slot_pages entries apart),
// starting from the view the arguments carry.  pos == nullptr: single-stream pass.
struct RowMap { const int* pos = nullptr; const int* slot = nullptr; int n_slots = 0; size_t slot_bytes = 0; int slot_pages = 0; };
__device__ __forceinline__ KvView slot_view(KvView v, const RowMap& R, int slot) {
  v.base += (size_t)slot * R.slot_bytes;
  if (v.table) v.table += (size_t)slot * R.slot_pages;
  return v;
}

// k32 / v32 / rot: 256-channel rows only (attend256.hip) - fp32 source rows instead of fp16 ones, and the signed Hadamard
// rotation applied to every row before it is quantized (src/q35_kernels.cu:1036,1060 + launch_tb_requant)
struct AppendArgs { KvView kv; const uint16_t* k16; const uint16_t* v16; const int* d_pos; int M; RowMap rows;
                    const float* k32 = nullptr; const float* v32 = nullptr; int rot = 0; };

// partial results of the split-KV kernels (same roles as pm/pl/pacc of the reference, args.hpp:10):
//   pm, pl [rows_tok][S][n_heads] fp32; pacc16 [rows_tok][S][n_heads][128] fp16 = acc / l (normalised, so that fp16
//   costs nothing measurable: every split's row is a convex combination of V rows).  pm is in log2 units; empty
//   split: pm = -1e30, pl = 0, pacc16 = 0.
struct AttnArgs {
  KvView kv; const uint16_t* q16; const int* d_pos; const uint8_t* depth;
  int M;        // rows (tokens) of this slice
  int tok0;     // index of the slice's first row inside the pass (row t sees keys [0, *d_pos + depth(tok0+t) + 1))
  int n_heads;
  int S;        // splits
  int rows_per_block;  // wide kernel: query rows one workgroup owns (multiple of 32)
  float* pm; float* pl; uint16_t* pacc16;
  // k16/v16 != nullptr: fused quantize-on-append - the workgroups whose tiles hold the new rows quantize and store them
  // before reading them.  Narrow kernel (M <= 2): rows [0, M) of the pass; wide kernel: k16/v16 point at row 0 of the
  // pass and the slice stores its own rows tok0 .. tok0 + M - 1.
  const uint16_t* k16; const uint16_t* v16;
  RowMap rows;  // narrow kernel only: multi-stream pass, one token per workgroup column, no depth table, no fused append
  // narrow kernel only: tickets != nullptr folds the split combine into the launch - every workgroup of a (kv head, row
  // tile) column takes a ticket from tickets[kv head * gridDim.z + row tile] once its partials are out, and the one that
  // draws the last ticket merges the column's partials into out16 and puts the counter back to zero
  int* tickets = nullptr; uint16_t* out16 = nullptr; int out_bf16 = 0;
};
// unrot != 0: the output row gets the inverse signed Hadamard rotation (7 butterfly stages, x 1/16, signs) before it is
// rounded to fp16 - the counterpart of rotating V rows on their way into the cache (src/q35_kernels.cu:1421)
struct CombineArgs { const float* pm; const float* pl; const uint16_t* pacc16; int S; int M; int n_heads; uint16_t* out16; int unrot;
                     int out_bf16 = 0; };   // outputs leave as bf16 (rounded once from the fp32 result) instead of fp16
// projection outputs xq [M][n_heads][128], xk / xv [M][n_kv][128] fp32 -> q16 and the cache rows at *d_pos + t
struct PostArgs {
  KvView kv; const float* xq; const float* xk; const float* xv; int M; int n_heads; const int* d_pos;
  const uint16_t* qn_w16; const uint16_t* kn_w16; float eps;
  const float* rope; int rd; int rope_rows;      // rope [rope_rows][rd/2] (cos, sin) pairs; rd = 0: no rotary step
  int rot; uint16_t* q16;
  // 256-channel heads only: if set, the finished K / V rows are written here as fp32 [M][n_kv][256] instead of being
  // quantized into kv (a handle with trellis-coded rows runs its encoder on them afterwards)
  float* k32_out = nullptr; float* v32_out = nullptr;
  // the gate half of the Q projection [M][n_heads][head_dim] fp32 -> gate16 (same shape, 16-bit), or nullptr
  const float* xgate = nullptr; uint16_t* gate16 = nullptr;
  int io_bf16 = 0;   // 16-bit rows that leave (q16, gate16) are bf16 instead of fp16
};

// Trellis-coded rows (trellis.hip; reference TbFastArgs, src/kvq_fast.hpp:16-37).  Probe form (yin != nullptr): rows
// row0 .. row0 + nrow - 1 of yin with their own group and position; results indexed by row.  Cache form: row rj of the
// launch is (token rj / (2 n_kv), K | V, kv head) of the pass, read from k32 / v32 [M][n_kv][256]; its payload goes to
// pay0 (K) / pay1 (V) + (kvh * max_ctx + pos) * stride and its scale to scl0 / scl1 [kvh * max_ctx + pos].
struct TbEncArgs {
  const uint8_t* blob; int nm; int has_trellis;
  // what the host looked up in the blob (see tb_descriptors in abi.hip): [ngrp][8] words
  //   { mode | bits << 8 | table << 16 | guard << 24, directions | has_mean << 8, byte offset of the mean row, of the
  //     first direction, index (in int16 units, from desc) of the group's table as aligned int16, gain bits, 0, 0 }
  // followed by the tables; mult_off: byte offset of the scale multipliers in the blob
  const uint32_t* desc; int ngrp; unsigned mult_off;
  const float* k32; const float* v32; const uint16_t* k16; const uint16_t* v16;   // cache form: fp32 rows, or fp16 rows if k32 == nullptr
  const int* d_pos; int layer, tok0, n_kv, max_ctx, rot;
  const float* yin; const int* grp; const int* pos; int row0;
  float* yout; uint32_t* side; int* coded;
  int nrow;
  uint8_t* scr; size_t scr_w_ofs;     // scratch: states [nrow * nm][256] bytes, then at scr_w_ofs error sums [nrow * nm][8] fp32
  uint8_t* pay0; uint8_t* pay1; float* scl0; float* scl1; int stride;
  int pos_limit;                      // cache form: rows at positions >= pos_limit are not stored (0: no limit besides max_ctx)
  RowMap rows;                        // cache form, multi-stream pass: token t sits at rows.pos[t] of container rows.slot[t] (pay / scl = container 0)
};
// attention over trellis-coded rows (attend_tb.hip).  pairs [groups][2^(8 + kb)]: entry i = the table's integers, as two
// fp16 values, of the states (i >> kb) & 255 and i & 255 (two consecutive elements from 8 + kb stream bits); gfac [groups]:
// gain / 256; mu [groups][256] fp32 mean rows (zero rows where a group has none) or nullptr if no group has one
struct TbAttnArgs {
  const uint8_t* kpay; const uint8_t* vpay; const float* kscl; const float* vscl; int max_ctx, n_kv, stride;
  const uint32_t* pairs; const float* gfac; const float* mu; int layer;
  const uint16_t* q16; const int* d_pos; const uint8_t* depth; int M, tok0, n_heads, S;
  float* pm; float* pl; uint16_t* pacc16;
  RowMap rows;  // narrow kernel only: multi-stream pass (one token per workgroup column; kpay .. vscl = container 0, `layer` = the profile's layer)
};
void launch_attend_tb(const TbAttnArgs&, int kb, hipStream_t);        // row tiles of 2 tokens x 6 heads (decode; any width)
void launch_attend_tb_wide(const TbAttnArgs&, int kb, hipStream_t);   // 3..64 rows: 128 query rows per workgroup, tiles decoded once into LDS
void launch_tb_encode(const TbEncArgs&, hipStream_t);
void launch_tb_unpack(const uint8_t* blob, const int* grp, const int* pos, const uint8_t* pay, const uint32_t* side, int stride, const float* yin,
                      float* y, int rows, hipStream_t);

// launchers (each checks nothing: the C layer validates shapes first)
void launch_append(const AppendArgs&, hipStream_t);
void launch_attend_narrow(const AttnArgs&, hipStream_t);   // 16-row tiles: 2 tokens x 6 heads per workgroup column
void launch_attend_wide(const AttnArgs&, hipStream_t);     // 3..64 tokens, and prefill slices
void launch_attend_mid(const AttnArgs&, hipStream_t);      // 3..16 tokens: a wave owns whole tiles, row tiles of 16 rows (wider: blocks of 16 tokens)
void launch_combine(const CombineArgs&, hipStream_t);
void launch_attn_post(const PostArgs&, hipStream_t);
void launch_attn_post256(const PostArgs&, hipStream_t);    // the same step for 256-channel heads (attend256.hip)
// the reference's own rows, head_dim 256 (attend256.hip): same argument structs, 67584-byte pages
void launch_append256(const AppendArgs&, hipStream_t);
void launch_rotate_q256(const float* x32, int rows, uint16_t* q16, hipStream_t);   // rotated query rows, rounded to fp16
void launch_attend256(const AttnArgs&, hipStream_t);       // row tiles of 2 tokens x 6 heads (decode; any width)
void launch_attend256_wide(const AttnArgs&, hipStream_t);  // 3..64 rows: 128 query rows per workgroup, tiles dequantized once into LDS
void launch_combine256(const CombineArgs&, hipStream_t);
void launch_export_rows256(const KvView&, int pos0, int n, uint32_t* kw, float* ks, uint32_t* vw, float* vs, hipStream_t);
void launch_import_rows256(const KvView&, int pos0, int n, const uint32_t* kw, const float* ks, const uint32_t* vw, const float* vs, hipStream_t);
// canonical <-> physical
void launch_export_rows(const KvView&, int pos0, int n, uint8_t* kc, uint16_t* ks, uint8_t* vc, uint16_t* vs, hipStream_t);
void launch_import_rows(const KvView&, int pos0, int n, const uint8_t* kc, const uint16_t* ks, const uint8_t* vc, const uint16_t* vs, hipStream_t);
void launch_dequant_rows(const KvView&, int pos0, int n, float* k, float* v, hipStream_t);
void launch_codec_probe(const uint16_t* x16, int rows, uint8_t* codes, uint16_t* scales, float* y, hipStream_t);
void launch_set_int(int* p, int v, hipStream_t);
void launch_zero_ints(int* p, int n, hipStream_t);   // a fill kernel (safe inside a captured graph, unlike a memset node)
// bf16 rows -> fp16 rows (round to nearest even; exact for magnitudes fp16 holds), n values each; any pointer pair may be null
void launch_bf16_to_f16(const uint16_t* a, uint16_t* a16, size_t na, const uint16_t* b, uint16_t* b16, const uint16_t* c, uint16_t* c16, size_t nbc, hipStream_t);
// the reference's own 256-channel row format (row256.hip): mode 0 = int8 rows, 1 = flat int4 (32 MSB-first words per row)
void launch_row256_encode(const float* x, int rows, int mode, int rot, int8_t* q8, uint32_t* words, float* scales, hipStream_t);
void launch_row256_decode(int rows, int mode, int rot, const int8_t* q8, const uint32_t* words, const float* scales, float* y, hipStream_t);
// the step after attention for 256-channel heads: gate, signs, 512-point Hadamard transform, int8 groups of 512 (n_heads even)
void launch_attn_out256(const uint16_t* y16, const uint16_t* gate16, const int8_t* signs, int M, int n_heads, int lo, int8_t* qx, float* alpha, hipStream_t);

// machine probe (probe.hip): fixed instruction mixes that time themselves; rec gets (shader cycles, wall ticks) per wave
void launch_probe_mix(int nv, bool mfma, float* sink, unsigned long long* rec, int iters, int iters_b, int split, int blocks, int threads, hipStream_t);
void launch_probe_mfma16(float* sink, unsigned long long* rec, int iters, int blocks, hipStream_t);
void launch_probe_valu(int op, float* sink, unsigned long long* rec, int iters, int blocks, int threads, hipStream_t);
void launch_probe_cross(int op, float* sink, unsigned long long* rec, int iters, int iters_b, int blocks, hipStream_t);
void launch_probe_read(bool nt, const void* src, size_t bytes, float* sink, int blocks, hipStream_t);

// fp32 -> bf16 bit pattern, round to nearest even (finite inputs)
__device__ __forceinline__ uint16_t f2bf_bits(float x) {
  const uint32_t u = __float_as_uint(x);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float bf_bits2f(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
// 8 fp32 results -> 16 bytes of fp16 or bf16
__device__ __forceinline__ uint4 pack_out8(const float* y, int bf16) {
  uint32_t w[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint16_t lo = bf16 ? f2bf_bits(y[2 * k]) : __half_as_ushort(__float2half_rn(y[2 * k]));
    const uint16_t hi = bf16 ? f2bf_bits(y[2 * k + 1]) : __half_as_ushort(__float2half_rn(y[2 * k + 1]));
    w[k] = (uint32_t)lo | ((uint32_t)hi << 16);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// start of the (page, kv head) block that holds token t
__device__ __forceinline__ uint8_t* kv_page(const KvView& kv, int kvh, int t) {
  const int lp = t / kPageTok;
  const int pp = kv.table ? kv.table[lp] : lp;
  return kv.base + (size_t)(pp * kv.n_kv + kvh) * kPageBytes;
}

// table[index] through the scalar data path; pointer and index are forced into scalar registers (they are uniform over
// the wave by contract, but the compiler cannot always prove it, e.g. inside a branch on a wave-uniform condition)
__device__ __forceinline__ int table_entry_scalar(const int32_t* table, int index) {
  const uint64_t a = (uint64_t)(uintptr_t)table;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  const uint64_t base = ((uint64_t)hi << 32) | lo;
  const int off = __builtin_amdgcn_readfirstlane(index * 4);
  int v;
  asm volatile("s_load_dword %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(base), "s"(off) : "memory");
  return v;
}

// The same for a token index that is uniform over the wave (the attention kernels' tile loops).  The page-table entry is
// fetched through the scalar data path: a vector load would share its completion counter with the tile loads a wave
// keeps in flight, so waiting for the entry would wait for all of them.  (Read only; the table is written by the host.)
__device__ __forceinline__ uint8_t* kv_page_uniform(const KvView& kv, int kvh, int t) {
  const int lp = t / kPageTok;
  int pp = lp;
  if (kv.table) pp = table_entry_scalar(kv.table, lp);
  return kv.base + (size_t)(pp * kv.n_kv + kvh) * kPageBytes;
}

}  // namespace yka
