/* CPU oracle for the int4-KV GQA attention path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library is the checker: tests, the smoke run and the cpu_baseline leg of
 * the benchmark may call it.  The product (the HIP library) never links, loads
 * or calls anything declared here.
 *
 * Every function is a plain-C restatement of the reference's arithmetic for the
 * path, adapted to the measured format (24 query heads / 4 KV heads /
 * head_dim 128, symmetric signed int4 with one fp16 scale per 32-channel
 * group).  Each cites the reference lines it follows.  Pinning status:
 *
 *   yko_h2f / yko_f2h        pinned: exhaustive / dense comparison with numpy float16
 *   yko_quant_group32        pinned: closed-form properties, ties-to-even cases,
 *                            exhaustive 1-value groups, independent fp64/numpy
 *                            restatement on random groups
 *   yko_dequant_group32      pinned: exact product, all 15 codes x all fp16 scales
 *   yko_pack / yko_unpack    pinned: all 256 byte values, v1 nibble order
 *   yko_attend_f32           pinned: fp64 textbook softmax(QK^T/sqrt(d))V (numpy),
 *                            split-count independence, uniform-V / dominant-key
 *                            closed forms, window == single rows
 *   yko_attend_f64           pinned: same closed forms + numpy
 *   (both, cache format 1)   pinned: numpy softmax on rows decoded with numpy bit unpacking, split independence,
 *                            window == single rows, uniform-V / dominant-key closed forms (head_dim 256)
 *   yko_combine              pinned: algebraic identity vs unsplit evaluation,
 *                            empty-split sentinel
 *   yko_kvx_sign             pinned: independent arbitrary-precision evaluation of the integer hash
 *   yko_kvx_rotate256        pinned: Sylvester Hadamard matrix (scipy) times the sign vector, in fp64;
 *                            involution; norm preservation
 *   yko_flat4_encode256 /    pinned: closed-form properties (zero row, max element -> +-7, ties to even),
 *   yko_flat4_decode256      independent numpy restatement; packing against numpy.unpackbits on the
 *                            big-endian byte image of the words
 *   yko_int8_encode256       pinned: closed-form properties, independent numpy restatement
 *   yko_attn_out256          pinned: scipy Sylvester matrix of order 512 (exact on integer inputs with an open gate),
 *                            numpy fp64 sigmoid gate within the fp16 roundings, closed forms of the int8 groups
 *   yko_rotate128            pinned: scipy Sylvester matrix (exact on integer rows), forward x inverse = identity,
 *                            q.k invariance
 *   yko_attn_post            pinned: numpy fp64 RMS normalisation and complex-multiplication rotary form within the
 *                            fp16 roundings, position 0 = no rotary change, pair-norm preservation, V rows pass through
 *   yko_attn_post256         pinned the same way on 256 channels; its rotation is yko_kvx_rotate256 (pinned above), so the
 *                            rotated rows are checked against the un-rotated ones through scipy's Sylvester matrix
 *   yko_tb_viterbi           pinned: exhaustive search over all paths on short chunks (minimum cost, and among equal
 *                            costs the path the tie rules name, on tables with repeated values)
 *   yko_tb_pack /            pinned: numpy.unpackbits on the big-endian byte image of the words; the sliding 8-bit
 *   yko_tb_decode_row        window against the state recursion; decode(encode(y)) == the encoder's own x, bit for bit
 *   yko_tb_encode_row        pinned as an algorithm: projections / rms against numpy fp64 within fp32 rounding, the kept
 *                            multiplier against a direct error evaluation of every multiplier, flat mode against
 *                            yko_flat4_encode256.  PARITY UNPINNED against real profiles: the reference's tables live
 *                            in a profile blob (kvq_u5.bin) that is not in its repository; tests use synthetic blobs
 *
 * The reference holds no golden vectors or known-answer tests for this path, so
 * none are replayed here; the checks above are what the mathematics fixes.
 */
#ifndef YKO_H
#define YKO_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define YKO_GROUP 32 /* channels per scale group */

/* ---- fp16 helpers (reference: src/a8_prologue.cuh:36-38, __float2half_rn / __half2float) ---- */
float yko_h2f(uint16_t h);
uint16_t yko_f2h(float f); /* round to nearest even, IEEE overflow to inf, subnormals kept */

/* ---- codec (reference: src/kvq_fast.cuh:194-198, src/kvq_gpu.cuh:85-86, decode src/kvq_attn.cuh:52-54,
 *      nibble order src/post_kernels.cu:77-80) ----
 * x16: 32 fp16 bit patterns.  codes: 16 bytes, element 2j in the low nibble of byte j,
 * element 2j+1 in the high nibble, each stored as q+8 (1..15).  scale16: fp16 bit pattern. */
void yko_quant_group32(const uint16_t* x16, uint8_t* codes16, uint16_t* scale16);
void yko_dequant_group32(const uint8_t* codes16, uint16_t scale16, float* y32);
/* rows of `dim` channels (dim % 32 == 0): codes [rows][dim/2], scales [rows][dim/32] */
void yko_quant_rows(const uint16_t* x16, int rows, int dim, uint8_t* codes, uint16_t* scales);
void yko_dequant_rows(const uint8_t* codes, const uint16_t* scales, int rows, int dim, float* y);
void yko_pack_nibbles(const uint8_t* fields, int n, uint8_t* bytes); /* n even; fields 0..15 */
void yko_unpack_nibbles(const uint8_t* bytes, int n, uint8_t* fields);

/* ---- the reference's own 256-channel row codec (yko_row256.c) ---- */
float yko_kvx_sign(int d);                                              /* src/kvx_codec.cuh:28-32 */
void yko_kvx_rotate256(const float* x, float* y, int inverse);          /* src/kvx_codec.cuh:35-49 */
/* flat int4, one fp32 scale per row, MSB-first 4-bit fields in 32 words (src/kvq_fast.cuh:194-198,226-233) */
void yko_flat4_encode256(const float* r, uint32_t* words32, float* scale, float* xq);
void yko_flat4_decode256(const uint32_t* words32, float scale, float* y);   /* src/kvq_attn.cuh:33-37,53-54 */
void yko_int8_encode256(const float* x, int8_t* q, float* scale);        /* src/kvx_codec.cuh:50-69 */
/* round trip of the reference's codec probe (src/kvx_probe.cu:7-20); mode 0 int8 rows, mode 1 flat int4 */
void yko_kvx_probe256(const float* x, int rows, int mode, int rot, int8_t* q8, uint32_t* words, float* scales, float* y);
/* the step after attention for 256-channel heads: sigmoid gate, signs, 512-point Hadamard transform, int8 groups of 512
 * (src/q35_kernels.cu:1420-1428, src/a8_prologue.cuh:87-98,122-133) */
void yko_attn_out256(const uint16_t* y16, const uint16_t* gate16, const int8_t* signs, int M, int n_heads, int8_t* qx, float* alpha);

/* ---- between the QKV projection and the cache (yko_post.c; src/q35_kernels.cu:1013-1065 for 128-channel heads) ---- */
void yko_rotate128(const float* x, float* y, int inverse, float factor);
void yko_post_qk_row(const float* y, const uint16_t* w16, float eps, const float* cs, int rd, int rot, float rot_factor, uint16_t* out16);
void yko_post_v_row(const float* y, int rot, uint16_t* out16);
void yko_attn_post(const float* xq, const float* xk, const float* xv, int M, int n_heads, int n_kv,
                   const uint16_t* qn_w16, const uint16_t* kn_w16, float eps, const float* rope, int rd, int pos,
                   int rot, uint16_t* q16, uint16_t* k16, uint16_t* v16);
void yko_unrotate_out(const float* y32, int rows, uint16_t* out16);
/* the same step for 256-channel heads (src/q35_kernels.cu:1037-1065): Q rows as fp16, K / V rows as the fp32 rows the
 * row quantizer takes */
void yko_post256_qk_row(const float* y, const uint16_t* w16, float eps, const float* cs, int rd, int rot, float* o32);
void yko_attn_post256(const float* xq, const float* xk, const float* xv, int M, int n_heads, int n_kv,
                      const uint16_t* qn_w16, const uint16_t* kn_w16, float eps, const float* rope, int rd, int pos,
                      int rot, uint16_t* q16, float* k32, float* v32);

/* ---- trellis-coded rows (src/kvq_gpu.cuh:51-147, src/kvq_fast.cuh:63-233, decode src/kvq_attn.cuh:46-75) ---- */
int yko_tb_check_blob(const uint8_t* blob, size_t n);                 /* 0 if a KVQP v1 blob this codec can use */
int yko_tb_group(const uint8_t* blob, int g, int* fields6);           /* mode, kk, table, guard, m, has_mu */
int yko_tb_viterbi(const int* xi, int T, const int16_t* ci, int kk, uint8_t* states);
int yko_tb_encode_row(const uint8_t* blob, int g, int pos, const float* y, float* x, uint8_t* fields, float* scale,
                      uint32_t* pc, int* best_mi);
void yko_tb_pack(const uint8_t* fields, int kb, uint32_t* words);
int yko_tb_decode_row(const uint8_t* blob, int g, const uint32_t* words, float scale, uint32_t pc, float* y);
void yko_tb_encode_rows(const uint8_t* blob, const int* grp, const int* pos, int n, const float* y, float* x, uint32_t* words,
                        int stride_words, float* scale, uint32_t* pc, int* best_mi, int* coded);

/* ---- canonical cache image used by the oracle and by the export/import hooks of the product ----
 * One layer: kc/vc [kvh][max_ctx][dim/2] bytes, ks/vs [kvh][max_ctx][dim/32] fp16 bit patterns. */
typedef struct {
  int n_heads, n_kv_heads, head_dim, max_ctx;
  uint8_t* kc; uint16_t* ks; uint8_t* vc; uint16_t* vs;
  /* fmt 0: the format above.  fmt 1 (head_dim 256 only): the reference's own rows - kc/vc point to uint32 words
   * [kvh][max_ctx][32] (4-bit fields, MSB first), ks/vs to float scales [kvh][max_ctx], one per row
   * (src/kvq_fast.cuh:194-198,226-233).  Append widens the fp16 inputs to fp32 and encodes them with
   * yko_flat4_encode256; attention decodes rows with yko_flat4_decode256. */
  int fmt;
} yko_cache;
/* row `row` (= kvh * max_ctx + token) of K (isv 0) or V (isv 1), dequantized to fp32 */
void yko_cache_row(const yko_cache* c, int isv, size_t row, float* out);

/* quantize-on-append (reference ordering: src/engine35.cpp:911-913 - rows are written before attention reads them;
 * row placement src/q35_kernels.cu:1038,1064): k16/v16 [M][kvh][dim] -> rows pos..pos+M-1 */
void yko_append(yko_cache* c, const uint16_t* k16, const uint16_t* v16, int M, int pos);

/* ---- attention ----
 * q16 [M][n_heads][dim]; row t of the window sees keys [0, pos + depth(t) + 1) with depth(t) = depth ? depth[t] : t
 * (reference: src/q35_atx.cu:110-118).  out16 [M][n_heads][dim] fp16.
 * splits <= 0 selects the reference policy (31 below 4096 keys, else 42: src/q35_atxpk.cu:404-409).
 * fp32 streaming form follows src/attention_kv4q.cu:19-31,71-146 (online softmax per split, sentinels m=-1e30,l=0)
 * and the combiner src/attention_kv4q.cu:325-332.  threads <= 1: scalar single thread (the oracle proper);
 * threads > 1: same loop nest spread over (kv head x split) with OpenMP (the timed CPU baseline). */
void yko_attend_f32(const yko_cache* c, const uint16_t* q16, int M, int pos, const uint8_t* depth,
                    int splits, int threads, uint16_t* out16, float* out32 /* optional, pre-rounding */);
/* textbook two-pass softmax in double on the dequantized tensors; out64 [M][n_heads][dim] */
void yko_attend_f64(const yko_cache* c, const uint16_t* q16, int M, int pos, const uint8_t* depth, double* out64);
/* combiner alone: pm,pl [S][rows], pacc [S][rows][dim] -> y [rows][dim] (src/attention_kv4q.cu:325-332) */
void yko_combine(const float* pm, const float* pl, const float* pacc, int S, int rows, int dim, float* y);

/* ---- seeded synthetic inputs (counter based: value i of stream `seed` does not depend on any other) ---- */
uint64_t yko_splitmix64(uint64_t x);
double yko_normal(uint64_t seed, uint64_t i);            /* N(0,1) */
void yko_outlier_channels(uint64_t seed, int dim, int* ch4); /* 4 distinct channel indices */
/* fills fp16 bit patterns of N(0,1) * (mult on the 4 outlier channels, 1 elsewhere); n = rows*dim */
void yko_fill_normal_f16(uint64_t seed, uint64_t first, uint64_t n, int dim, const int* ch4, float mult, uint16_t* out);

#ifdef __cplusplus
}
#endif
#endif
