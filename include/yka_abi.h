/* C ABI of the MI355X int4-KV GQA attention library (libyka.so).
 *
 * Conventions follow the reference's include/yskn_abi.h and src/c_api.cpp:
 *   - opaque handle, created by an open call and released by a close call (yskn_abi.h:21-24);
 *   - every call returns int: 0 = ok, -1 = error; the message of the last error of the calling thread is
 *     returned by yka_last_error() (c_api.cpp:17,33,49);
 *   - the stream is passed as void* (yskn_abi.h:19 "void* cuda_stream"); here it is a hipStream_t;
 *   - the position of the pass lives on the device (const int* d_pos) and is read by the kernels, never by the
 *     host, so a captured graph replays at new positions (engine35.cpp:2365-2375, q35_atxpk3.cuh:183);
 *   - the launch path (yka_append / yka_attend / yka_append_attend) allocates nothing, synchronises nothing and
 *     sets no function attribute: everything is reserved in yka_kv_open (engine35.cpp:323-326);
 *   - hooks that take host pointers allocate, copy, launch, synchronise and free inside (src/kvx_probe.cu).
 * One caller at a time per handle; any host thread may call (the device of the handle is made current first,
 * as on_gpu does in c_api.cpp:22-31).  One stream in flight per handle as well: a handle owns ONE set of split
 * partials, one device position word and (trellis rows) one encoder scratch, which every launch and every replay of a
 * pass captured from it uses.  Work of one handle issued on two streams, or a replay issued while an earlier call on
 * the handle may still run on another stream, races on them; order such work with events or keep it on one stream
 * (the reference replays its passes on the one stream of its engine, engine35.cpp:1977-1988).
 *
 * Formats, selected by head_dim at open:
 *   128: symmetric signed int4 codes stored as q+8, two per byte, even channel in the low nibble; one fp16 scale per
 *        (token, kv head, 32-channel group) - the measured format; every entry point below exists for it;
 *   256: the reference's own rows - flat int4 with ONE fp32 scale per (token, kv head) row, 4-bit fields MSB first in
 *        32 uint32 words (kvq_fast.cuh:194-198,226-233; decode kvq_attn.cuh:33-37,53-54).  Open / close / options /
 *        page table / append / attend / append_attend / layer_call_host / append_host / replicate / captured passes /
 *        attn_bench work on it; its canonical image goes through yka_kv_export_rows256 / yka_kv_import_rows256; the
 *        other entry points return an error.
 * Q, new K/V and outputs are fp16 bit patterns, [rows][heads][head_dim].
 */
#ifndef YKA_ABI_H
#define YKA_ABI_H
#include <stddef.h>
#include <stdint.h>
#define YKA_API __attribute__((visibility("default")))
#ifdef __cplusplus
extern "C" {
#endif

typedef struct yka_kv yka_kv;

typedef struct yka_kv_config {
  int32_t n_layers;    /* KV containers (the reference keeps one per full-attention layer, engine35.cpp:303-329) */
  int32_t n_heads;     /* query heads (24) */
  int32_t n_kv_heads;  /* KV heads (4); n_heads / n_kv_heads must be 6 */
  int32_t head_dim;    /* 128, or 256 for the reference's own rows */
  int32_t max_ctx;     /* tokens reserved per layer; multiple of 256 */
  int32_t max_rows;    /* most query rows one call may carry (64 = kVerifyMax, engine35.hpp:157; up to 2048 = PM_ for prefill) */
  int32_t paged;       /* 0: token t of a KV head lives in page t/256; 1: pages go through a per-layer page table */
  int32_t device;      /* HIP device ordinal */
} yka_kv_config;

/* replaces the KV reservation of yskn_open (yskn_abi.h:22; engine35.cpp:303-329). NULL on error.  Refused before any
 * device call: a configuration outside the ranges above, more than 1024 KV heads, or n_layers x max_ctx x n_kv_heads that
 * describes more than 1 TiB of cache. */
YKA_API yka_kv* yka_kv_open(const yka_kv_config* cfg);
/* replaces yskn_close (yskn_abi.h:23) for the KV containers */
YKA_API void yka_kv_close(yka_kv* kv);
/* replaces yskn_last_error (yskn_abi.h:30): thread-local message of the last failed call */
YKA_API const char* yka_last_error(void);
/* replaces yskn_build_info (yskn_abi.h:84): "hip=<version>;arch=gfx950;..." */
YKA_API const char* yka_build_info(void);
/* replaces yskn_set_opt (yskn_abi.h:87) for the options of this path.
 * key 1: split count of the narrow kernel (decode, rows of at most 2 tokens; at most 256); key 2: split count of the wide kernel;
 * key 3: 1 forces the narrow kernel for every width (cross-check of the wide kernel), 0 = automatic;
 * key 4: 1 = attention outputs get the inverse signed Hadamard rotation before they are rounded to fp16 (for caches
 *        filled by yka_attn_post or yka_append256_f32 with rotate = 1; the reference un-rotates in its output step,
 *        q35_kernels.cu:1421);
 * key 5: context length (tokens) the caller expects, used only to size the decode grid (the reference picks its split
 *        count from the length known on the host, engine35.hpp:434-439); 0 = the max_ctx of the handle.  Any actual
 *        position stays correct: positions are read on the device and the kernel uses as many of the launched
 *        splits as the length it finds there justifies;
 * key 6: handles with trellis-coded rows, multi-stream passes only: the profile layer whose groups code and decode the
 *        rows (the containers of such a handle are the streams of that one layer; the reference passes the layer in
 *        TbFastArgs::layer / Q35PkArgs::layer);
 * key 7: 1 = the decode kernel (128-channel rows of at most 2 tokens, multi-stream passes, no option key 4) merges its
 *        splits inside the attention launch: the workgroup that finishes a column last combines it.  0 (default) = a
 *        second launch combines.  Same results to within the summation order.  On MI355X the second launch is the faster
 *        form (12.0 against 18.9 us per layer call at 32k tokens): the hand-over between XCDs costs three dependent
 *        trips to memory (store acknowledged, ticket, loads), more than the gap between two kernels;
 * key 8: widest window (rows) that runs on the kernel for small windows (a wave owns whole tiles and walks the window's row
 *        tiles; 128-channel rows only).  0 = never, at most 64 (wider windows than 16 rows then run as blocks of 16
 *        tokens).  Default 10: measured faster than the 128-row workgroups of the wide kernel up to there;
 * key 9: split count of that kernel (0 = automatic);
 * key 10: tokens per prefill slice (passes wider than 64 rows), 0 = 1024; 128 .. 4096;
 * key 11: 16-bit row type at the boundary: 0 = fp16 (default), 1 = bf16, the type of the reference's activations
 *        (q35_kernels.cu:1048,1062: Q, gate and attention outputs are bf16 there).  With 1, d_q16 / d_k16 / d_v16 of every
 *        entry point are bf16 and are converted to fp16 by one extra launch per call (round to nearest; exact for
 *        magnitudes between 2^-14 and 65504, i.e. for normalised activations), attention outputs are rounded once from
 *        their fp32 value to bf16, and yka_attn_post writes q16 / gate16 as bf16.  Setting it to 1 the first time reserves
 *        the staging rows (max_rows of Q, K and V): do that before capturing passes; the call is not on the launch path. */
YKA_API int yka_set_opt(yka_kv* kv, int key, int value);

/* Paged mode: logical page p of `layer` (-1 = every layer) lives in physical page h_table[p]; n_pages = max_ctx/256
 * entries forming a permutation.  No counterpart in the reference (rows are addressed (kvh*max_ctx+pos)*row_bytes,
 * q35_atxpk3.cuh:196-200); added for the 256-token shuffled-page configuration. Synchronous. */
YKA_API int yka_kv_set_page_table(yka_kv* kv, int layer, const int32_t* h_table, int n_pages);

/* Quantize-on-append: rows *d_pos .. *d_pos+M-1 of every KV head of `layer` are overwritten with the int4 codes and
 * fp16 scales of d_k16 / d_v16 ([M][n_kv_heads][128] fp16, device).  Replaces the KV store of launch_q35_attn_post
 * followed by launch_tb_requant (q35_kernels.cu:1038,1064,1084-1092; call site engine35.cpp:911-913) and, for the
 * v1 engine, the K/V part of launch_qkv_post (post_kernels.cu:55-81). */
YKA_API int yka_append(yka_kv* kv, int layer, const uint16_t* d_k16, const uint16_t* d_v16, int M,
                       const int* d_pos, void* hip_stream);

/* Attention over the cache: row t of d_q16 ([M][n_heads][128] fp16) attends to keys [0, *d_pos + depth(t) + 1),
 * depth(t) = d_depth ? d_depth[t] : t (q35_atx.cu:110-118); writes d_out16 [M][n_heads][128] fp16.  A depth table names rows
 * of the pass, so depth(t) <= t: a larger value reaches past the rows this pass appends, into rows nobody has written
 * (the table lives on the device and is not checked).
 * Replaces launch_q35_prefill_atx_pk / launch_q35_atx_pk + launch_q35_combine (q35_atxpk.hpp:15-24, q35.hpp:153-156;
 * call site engine35.cpp:921-934) and launch_attention + launch_attn_combine of the v1 engine (args.hpp:36-37). */
YKA_API int yka_attend(yka_kv* kv, int layer, const uint16_t* d_q16, int M, const int* d_pos,
                       const uint8_t* d_depth, uint16_t* d_out16, void* hip_stream);

/* One layer call = the effect of yka_append followed by yka_attend on the same stream: the sequence of
 * Engine35::attn_block (engine35.cpp:911-934).  The rows are quantized inside the attention launches (each 64-row
 * slice stores its own rows before it reads them; bit-identical to yka_append), so a layer call is two launches:
 * attention and the split combiner.  M may be as large as max_rows; a pass wider than 64 rows is a prefill chunk: its rows
 * are appended by one launch, then slices of up to 1024 tokens (option key 10) run through the wide kernel, one attention
 * and one combiner launch per slice (attn_block cuts such passes into 64-row slices, engine35.cpp:935-947). */
YKA_API int yka_append_attend(yka_kv* kv, int layer, const uint16_t* d_q16, const uint16_t* d_k16,
                              const uint16_t* d_v16, int M, const int* d_pos, const uint8_t* d_depth,
                              uint16_t* d_out16, void* hip_stream);

/* The same layer call for callers that cannot allocate and must not depend on memory the handle allocated for its split
 * partials (code under graph capture that is handed a foreign handle, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same inputs, outputs and results as yka_append_attend - the same kernels
 * and split counts, bit for bit - but the split partials live in a static array inside the library's device code
 * (9,733,120 bytes, held by every GPU the library is used on until the process ends) whose device address is looked up
 * once per device when a handle is opened there.  Limits: head_dim 128 handles, 1 <= M <= 64 rows (one slice), at most
 * 24 query heads; anything else returns -1 with a message.  The call allocates nothing, frees nothing, synchronises
 * nothing.  Every call on one GPU uses that GPU's one array: calls that overlap on a GPU (two streams, two handles) race
 * on it; calls on one stream, or otherwise ordered, are safe.  No partial has to start at zero: every launch writes
 * every partial it later reads.  The last kilobyte holds the split tickets option key 7 uses: a fill kernel in front of
 * every launch that uses them puts them to zero, so a launch that ended half way cannot disturb a later one. */
YKA_API int yka_append_attend_static(yka_kv* kv, int layer, const uint16_t* d_q16, const uint16_t* d_k16,
                                     const uint16_t* d_v16, int M, const int* d_pos, const uint8_t* d_depth,
                                     uint16_t* d_out16, void* hip_stream);

/* Test hook, no counterpart in the reference: overwrites the handle's OWN split workspace (the one yka_append_attend and
 * yka_attend use) with NaN bit patterns, synchronously.  A call that gives right results afterwards did not read it
 * without writing it first - in particular yka_append_attend_static, which must not touch it at all. */
YKA_API int yka_kv_poison_workspace(yka_kv* kv);

/* Multi-stream pass (batched decode): row t of the pass belongs to the stream whose KV container is d_row_slot[t]
 * (a container index in [0, n_layers): the handle's containers are then one per stream of the layer being run) and sits
 * at position d_row_pos[t] of it.  If d_k16 / d_v16 are given, row t of them is quantized into that row first; then row
 * t of d_q16 attends to keys [0, d_row_pos[t]] of its container.  Rows of one stream may follow each other at
 * consecutive positions (a stream's last token and its draft tokens).  A row whose slot or position is out of range is
 * dropped and yields zeros.  Replaces launch_q35_attn_post_ms / launch_tb_requant_ms, launch_q35_atx_pk_ms and
 * launch_q35_combine_ms (q35.hpp:28-35,109-112,157; q35_atxpk.hpp:18-20; kernel src/q35_atxpk_ms.cu).  The reference caps
 * such a pass at 16 rows (Q35_SST, q35.hpp:20); here M may be up to max_rows.  Works on both row formats (head_dim 128
 * and 256: the reference's multi-stream kernel runs on its 256-channel rows).  Allocates nothing, synchronises nothing. */
YKA_API int yka_append_attend_ms(yka_kv* kv, const uint16_t* d_q16, const uint16_t* d_k16, const uint16_t* d_v16, int M,
                                 const int* d_row_pos, const int* d_row_slot, uint16_t* d_out16, void* hip_stream);

/* head_dim 256: quantize-on-append from fp32 rows, d_k32 / d_v32 [M][n_kv_heads][256].  With rotate != 0 every row first
 * gets the signed Walsh-Hadamard rotation (kvx_codec.cuh:28-49), then the flat int4 row codec - the arithmetic of
 * kvx_rotate followed by the flat mode of the row quantizer (q35_kernels.cu:1036,1060; kvq_fast.cuh:194-198), bit for
 * bit.  Allocates nothing, synchronises nothing. */
YKA_API int yka_append256_f32(yka_kv* kv, int layer, const float* d_k32, const float* d_v32, int M, const int* d_pos,
                              int rotate, void* hip_stream);
/* head_dim 256: rotated query rows, d_x32 [rows][256] fp32 -> d_q16 [rows][256] fp16 (q35_kernels.cu:1060,1062 with fp16
 * in the place of the reference's bf16).  Attention over a rotated cache then needs option key 4 (outputs un-rotated). */
YKA_API int yka_rotate_q256(const float* d_x32, int rows, uint16_t* d_q16, void* hip_stream);

/* The step after attention for 256-channel heads; replaces the output part of launch_q35_combine (q35.hpp:153-156,
 * q35_kernels.cu:1420-1428 with a8_group512_tail, a8_prologue.cuh:87-98,122-133), fp16 where the reference rounds to bf16:
 * per token and per pair of heads (512 values) y * f16(sigmoid(gate)) -> f16 -> x sign -> 512-point Hadamard transform
 * x 1/sqrt(512) -> f16 -> one scale alpha = max|v| / 127 and int8 codes.  d_y16 = attention outputs [M][n_heads][256]
 * (what yka_attend wrote, un-rotated if option key 4 is set), d_gate16 the same shape, d_signs [n_heads * 256] (+1/-1),
 * d_qx [M][n_heads * 256] int8, d_alpha [M][n_heads * 256 / 512] fp32.  Allocates nothing, synchronises nothing. */
YKA_API int yka_attn_out256(const uint16_t* d_y16, const uint16_t* d_gate16, const int8_t* d_signs, int M, int n_heads,
                            int8_t* d_qx, float* d_alpha, void* hip_stream);
/* The same step writing the reference's interleaved small-batch layout of the int8 operand (Q35CombineArgs::lo;
 * a8_lo_off, a8_prologue.cuh:121,132; q35_kernels.cu:1428): at most 8 tokens; d_qx [n_heads / 2][4096], element i of
 * token t of group g at g * 4096 + (i/256)*2048 + ((i/16)%4)*512 + t*64 + ((i/64)%4)*16 + i%16 (bytes of tokens that are
 * not part of the pass are left as they are); d_alpha as above. */
YKA_API int yka_attn_out256_lo(const uint16_t* d_y16, const uint16_t* d_gate16, const int8_t* d_signs, int M, int n_heads,
                               int8_t* d_qx, float* d_alpha, void* hip_stream);

/* The step between the QKV projection and the cache, fused with quantize-on-append; replaces launch_q35_attn_post
 * (q35.hpp:97-105, q35_kernels.cu:1013-1065) + launch_tb_requant (q35_kernels.cu:1084-1092) for 128-channel heads:
 * per head, Q and K rows are RMS-normalised (x / sqrt(mean x^2 + eps) * (1 + w)), get the rotary embedding on their
 * first rope_dims channels (pairing d <-> d + rope_dims/2, table row = position) and, if rotate, the signed
 * Walsh-Hadamard rotation (kvx_codec.cuh:28-49 for 128 channels; K and V x 1/8, Q x 1/16); V rows are only rotated.
 * Q rows are written to d_q16 [M][n_heads][128] fp16; K and V rows are rounded to fp16 and quantized into rows
 * *d_pos .. *d_pos+M-1 of `layer` exactly as yka_append would store them.  d_xq [M][n_heads][128], d_xk, d_xv
 * [M][n_kv_heads][128] are the projection's fp32 outputs (the reference's split-K recombination and per-column factors,
 * q35_kernels.cu:1027-1032, happen before this call).  Allocates nothing, synchronises nothing.
 * On a handle opened with head_dim 256 (the reference's own head size) the same call works on 256-channel rows: the
 * normalisation divides by 256, the rotation is the 256-point kvx_rotate (x 1/16 for Q, K and V), Q rows leave as fp16
 * [M][n_heads][256], and K / V rows go through the flat row quantizer (kvq_fast.cuh:194-198) as fp32 values, i.e. what
 * yka_append256_f32 stores for them. */
typedef struct yka_post_params {
  const uint16_t* d_qn_w16;  /* [head_dim] fp16 norm weights of Q heads, applied as (1 + w) (q35_kernels.cu:1057) */
  const uint16_t* d_kn_w16;  /* [head_dim] the same for K heads */
  float eps;
  const float* d_rope;       /* [rope_rows][rope_dims/2][2] fp32 (cos, sin) by position (q35_kernels.cu:1101-1107) */
  int32_t rope_dims;         /* even, 0..head_dim; 0 = no rotary step (the reference rotates 64 of 256 channels, q35.hpp:13) */
  int32_t rope_rows;         /* rows whose position is not below rope_rows are dropped */
  int32_t rotate;            /* 0 / 1 */
  const float* d_xgate;      /* the gate half of the Q projection, [M][n_heads][head_dim] fp32, or NULL (the reference's Q
                              * projection carries query and gate side by side, q35_kernels.cu:1017,1048) */
  uint16_t* d_gate16;        /* [M][n_heads][head_dim]: the gate rows rounded to the handle's 16-bit row type, the operand
                              * yka_attn_out256 later takes (q35_kernels.cu:1048); NULL together with d_xgate */
} yka_post_params;
YKA_API int yka_attn_post(yka_kv* kv, int layer, const float* d_xq, const float* d_xk, const float* d_xv, int M,
                          const int* d_pos, const yka_post_params* params, uint16_t* d_q16, void* hip_stream);

/* ---- hooks with host pointers (model: src/kvx_probe.cu) ---- */

/* Host-pointer form of yka_append_attend_ms (k16 / v16 may be NULL = attend only). */
YKA_API int yka_ms_call_host(yka_kv* kv, const uint16_t* q16, const uint16_t* k16, const uint16_t* v16, int M,
                             const int32_t* row_pos, const int32_t* row_slot, uint16_t* out16);

/* Host-pointer forms of yka_attn_out256 and yka_attn_out256_lo (qx [n_heads / 2][4096], zero where no token wrote). */
YKA_API int yka_attn_out256_host(const uint16_t* y16, const uint16_t* gate16, const int8_t* signs, int M, int n_heads,
                                 int8_t* qx, float* alpha);
YKA_API int yka_attn_out256_lo_host(const uint16_t* y16, const uint16_t* gate16, const int8_t* signs, int M, int n_heads,
                                    int8_t* qx, float* alpha);
/* Host-pointer forms of yka_append256_f32 and yka_rotate_q256. */
YKA_API int yka_append256_f32_host(yka_kv* kv, int layer, const float* k32, const float* v32, int M, int pos, int rotate);
YKA_API int yka_rotate_q256_host(const float* x32, int rows, uint16_t* q16);

/* Host-pointer form of yka_attn_post: uploads everything, sets the device position to `pos`, runs, downloads q16 (and
 * gate16 if xgate / gate16 are given; both NULL = no gate rows). */
YKA_API int yka_attn_post_host(yka_kv* kv, int layer, const float* xq, const float* xk, const float* xv, int M, int pos,
                               const uint16_t* qn_w16, const uint16_t* kn_w16, float eps, const float* rope,
                               int rope_dims, int rope_rows, int rotate, uint16_t* q16, const float* xgate, uint16_t* gate16);

/* Codec round trip on the GPU, replaces yskn_kvx_probe (kvx_probe.cu:22-36): x16 [rows][128] fp16 ->
 * codes [rows][64], scales [rows][4] fp16, y [rows][128] fp32 dequantized. */
YKA_API int yka_codec_probe(const uint16_t* x16, int rows, uint8_t* codes, uint16_t* scales, float* y);

/* Round trip through the reference's own 256-channel row format, replaces yskn_kvx_probe for it (kvx_probe.cu:7-36):
 * x [rows][256] fp32 -> [signed Walsh-Hadamard rotation, kvx_codec.cuh:28-49, if rot] -> encode -> decode ->
 * [inverse rotation] -> y [rows][256].  mode 0: int8 rows, q8 [rows][256], scale = max|x|/127 (kvx_codec.cuh:50-69);
 * mode 1: flat int4, words [rows][32] with field e in bits [4e, 4e+4) of an MSB-first stream, scale = max|x|/7
 * (kvq_fast.cuh:194-198,226-233; decode kvq_attn.cuh:33-37,53-54).  scales [rows] fp32.  The array of the other mode
 * may be NULL.  Results are bit-identical to the reference's arithmetic. */
YKA_API int yka_kvx256_probe(const float* x, int rows, int mode, int rot, int8_t* q8, uint32_t* words, float* scales, float* y);

/* Trellis-coded rows (the reference's KV4 / KV5 row formats): encode, pack, unpack.  Replaces yskn_tbp_pack_unpack
 * (kvx_probe.cu:123-188; kernels launch_tb_fast, kvq_fast.cuh:63-233, and tba_unpack_kernel, kvq_attn.cuh:46-75).
 * blob: a "KVQP" v1 profile (host memory); x [rows][256] fp32; grp / pos [rows]: the group ((layer * kv heads + kv head)
 * * 2 + K|V) and the position of every row; stride: bytes between payload rows (>= 160).  Outputs, all host memory:
 * y_fq [rows][256] = what each row decodes to according to the encoder; pay [rows][stride]: 8 * kb MSB-first words per
 * coded row (kb = the group's bits per element, 4 for flat groups), zero otherwise; side [rows][2]: the row's fp32 scale
 * and two fp16 projection coefficients; y_dec [rows][256] = the decoder's result from pay and side (x for rows that stay
 * uncoded: position below the group's guard, or no such group).  ms_out (may be NULL): milliseconds of the encode and
 * of the unpack launches, as the reference's hook reports them (kvx_probe.cu:160).  The argument list is that of
 * yskn_tbp_pack_unpack.  Bit-identical to the reference's arithmetic for the same blob.  Synchronous; allocates. */
YKA_API int yka_tb_pack_unpack(const uint8_t* blob, size_t blob_len, const float* x, const int* grp, const int* pos, int rows,
                               int stride, float* y_fq, uint8_t* pay, uint32_t* side, float* y_dec, float* ms_out);

/* Switches a handle opened with head_dim 256 (not paged) to trellis-coded rows under the given "KVQP" v1 profile (host
 * memory; copied).  Replaces the profile loading of the engine (YSKN_TB_PROFILE, engine35.cpp:38-66) and its packed KV
 * streams (kp / vp / kps / vps of Q35PkArgs, q35_atxpk.hpp:14).  As the reference asks before it keeps packed rows for a
 * layer (kvqaxpk_packable, kvq_atxpk.hpp:61-72) every group of the handle's layers must be trellis-coded with the same 4
 * or 5 bits per element, guard position 0 and no projected directions; mean rows are allowed.  Rows are then laid out as
 * the reference lays them out: payload (kv head * max_ctx + pos) * 32 * bits bytes, one fp32 scale per row in a parallel
 * array (q35_atxpk3.cuh:196-200).  From then on yka_append / yka_append256_f32 / yka_append_attend encode rows with the
 * trellis encoder (launch_tb_requant -> launch_tb_fast, q35_kernels.cu:1084-1092) and yka_attend / yka_append_attend
 * read them (launch_q35_atx_pk); yka_attn_post hands its finished K / V rows to the encoder (as launch_q35_attn_post is
 * followed by launch_tb_requant); the multi-stream pass runs on them with the groups of the layer option
 * key 6 names (launch_tb_fast_ms, kvq_fast.cuh:236-392; launch_q35_atx_pk_ms, q35_atxpk.hpp:18-20); the flat-row export /
 * import refuse.  The profile's layers are model layers: a single-stream call names one of them, so its `layer` must be
 * below both n_layers of the handle and the number of layers the profile has groups for.
 * Synchronous; allocates (the only call of the trellis path that does). */
YKA_API int yka_kv_set_profile(yka_kv* kv, const uint8_t* blob, size_t blob_len);
/* bits per element of the handle's trellis-coded rows, 0 if it has no profile */
YKA_API int yka_kv_profile_bits(const yka_kv* kv);
/* rows [pos0, pos0 + n) of one layer of a handle with a profile: kw / vw [n_kv_heads][n][8 * bits] payload words,
 * ks / vs [n_kv_heads][n] scales (host memory).  Test hook; synchronous. */
YKA_API int yka_kv_export_rows_tb(yka_kv* kv, int layer, int pos0, int n, uint32_t* kw, float* ks, uint32_t* vw, float* vs);

/* Canonical image of rows [pos0, pos0+n) of one layer, independent of the physical layout:
 * kc/vc [n_kv_heads][n][64], ks/vs [n_kv_heads][n][4].  export = device -> host, import = host -> device.
 * (The reference reads its containers back only inside its hooks, e.g. kvx_probe.cu:369.) Synchronous. */
YKA_API int yka_kv_export_rows(yka_kv* kv, int layer, int pos0, int n, uint8_t* kc, uint16_t* ks, uint8_t* vc, uint16_t* vs);
YKA_API int yka_kv_import_rows(yka_kv* kv, int layer, int pos0, int n, const uint8_t* kc, const uint16_t* ks,
                               const uint8_t* vc, const uint16_t* vs);
/* The same for head_dim 256: kw/vw [n_kv_heads][n][32] uint32 words, ks/vs [n_kv_heads][n] fp32 row scales. */
YKA_API int yka_kv_export_rows256(yka_kv* kv, int layer, int pos0, int n, uint32_t* kw, float* ks, uint32_t* vw, float* vs);
YKA_API int yka_kv_import_rows256(yka_kv* kv, int layer, int pos0, int n, const uint32_t* kw, const float* ks,
                                  const uint32_t* vw, const float* vs);
/* dequantize rows on the GPU (decoder probe, replaces tba_unpack_kernel's use in yskn_tbp_pack_unpack,
 * kvx_probe.cu:123-170): k, v [n_kv_heads][n][128] fp32 */
YKA_API int yka_kv_dequant_rows(yka_kv* kv, int layer, int pos0, int n, float* k, float* v);
/* copy the content of layer `src` into every other layer (device to device), as the bench hook tiles one set of
 * encoded rows over `nlayers` containers (kvx_probe.cu:373-386). Synchronous. */
YKA_API int yka_kv_replicate_layer(yka_kv* kv, int src);

/* Host-pointer form of one layer call: uploads q/k/v ([M][..][128] fp16; k16/v16 may be NULL = attend only),
 * sets the device position to `pos`, runs append + attend on an internal stream, downloads out16.
 * depth may be NULL.  The single-call analogue of the run/combine lambda of yskn_atxpk_bench (kvx_probe.cu:388-401). */
YKA_API int yka_layer_call_host(yka_kv* kv, int layer, const uint16_t* q16, const uint16_t* k16, const uint16_t* v16,
                                int M, int pos, const uint8_t* depth, uint16_t* out16);

/* Host-pointer form of yka_append alone (fills a container from fp16 rows; model: the encode step of
 * yskn_atxpk_bench, kvx_probe.cu:361-369). */
YKA_API int yka_append_host(yka_kv* kv, int layer, const uint16_t* k16, const uint16_t* v16, int M, int pos);

/* Captured passes.  The reference replays each pass shape from a CUDA graph (Engine35::run_pass, engine35.cpp:1977-1988;
 * decode loop engine35.cpp:2365-2375).  yka_pass_capture records, for each of the n listed layers in order, one layer
 * call (mode 0: append + attend, 1: attend only, 2: attention kernel alone) with the given device buffers into a
 * hipGraph; yka_pass_launch replays it on `hip_stream`.  Positions are read from d_pos at replay time.  All layer
 * calls of one graph share d_out16 and the handle's partial workspace, so they run in order. */
typedef struct yka_pass yka_pass;
YKA_API yka_pass* yka_pass_capture(yka_kv* kv, const int32_t* layers, int n, const uint16_t* d_q16, const uint16_t* d_k16,
                                   const uint16_t* d_v16, int M, const int* d_pos, const uint8_t* d_depth,
                                   uint16_t* d_out16, int mode);
YKA_API int yka_pass_launch(yka_pass* p, void* hip_stream);
YKA_API void yka_pass_destroy(yka_pass* p);

/* Timed sweeps, replaces yskn_atxpk_bench (kvx_probe.cu:322-449): with q/k/v uploaded once and the device position
 * fixed at `pos`, runs one warm sweep over all layers and then `reps` timed sweeps (hipEvents on the internal
 * stream), each sweep = one layer call per layer on distinct containers.  mode 0 = append + attend, 1 = attend only,
 * 2 = the dominant attention kernel alone (no append, no combine).  ms[r] = time of sweep r in milliseconds.
 * use_graph != 0 replays the sweep from a captured hipGraph (the reference replays captured passes,
 * engine35.cpp:1977-1988).  inv (may be NULL) receives the reference's built-in invariant (kvx_probe.cu:419-441), taken
 * on container 0 after the timed sweeps: the M-row pass against M one-row passes at positions pos .. pos + M - 1 -
 * inv[0] = rows whose outputs differ in any bit, inv[1] = rows compared, inv[2] = output values that differ, inv[3] =
 * the largest distance between two such values in units of the fp16 spacing.  (The reference demands bit equality of
 * its one kernel family; here windows of 3+ rows and single rows run on different kernels, whose roundings differ in
 * the last place, so inv reports how far.) */
YKA_API int yka_attn_bench(yka_kv* kv, const uint16_t* q16, const uint16_t* k16, const uint16_t* v16, int M, int pos,
                           int mode, int use_graph, int reps, float* ms, uint16_t* out16_last, int* inv);

/* Machine probe: fixed instruction mixes that time themselves, for the figures the kernels are designed around and the
 * roofline is read against.  Model: the timing part of the reference's bench hooks (kvx_probe.cu:407-413).  Synchronous;
 * allocates.  `blocks` workgroups of `threads` (256 or 512) lanes; every kind runs once untimed, then once timed.
 *   kind 0: per wave, iters x 4 x (one v_mfma_f32_32x32x16_f16 followed by p0 independent v_fma_f32), p0 in {0,2,4,6,8}
 *   kind 1: per wave, iters x 8 v_mfma_f32_16x16x32_f16 (256 lanes)
 *   kind 2: per wave, iters x 32 instructions of one vector opcode: p0 = 0 v_exp_f32, 1 v_pk_mul_f16, 2 v_cvt_pk_f16_f32,
 *           3 v_max3_f32, 4 v_and_or_b32, 5 v_pk_add_f16, 6 v_perm_b32, 7 v_mul_f32, 8 v_fma_f32
 *   kind 3: 512 lanes; waves 0-3 of a workgroup run kind 0 with p0 = 0, waves 4-7 run p0 iterations of 32 v_fma_f32: two
 *           waves per SIMD, one of each kind
 *   kind 4: streaming read of iters MiB in 16-byte pieces; p0 != 0: nontemporal loads
 *   kind 5: 512 lanes; waves 0-3 run kind 0 with p0 = 0 (iters x 4 MFMAs), waves 4-7 run (2/3 iters) x 32 instructions
 *           of the vector opcode p0 of kind 2 (0..7): how far the matrix pipe and that opcode run side by side
 * out[0] = milliseconds of the timed launch (events); out[1], out[2] = mean shader-clock cycles and mean wall-clock
 * ticks a wave measured around its loop (kinds 3 and 5: waves 0-3); out[3], out[4] the same for waves 4-7 of kinds 3, 5;
 * out[5] = wall-clock ticks per millisecond. */
YKA_API int yka_machine_probe(int kind, int p0, int iters, int blocks, int threads, double* out);

#ifdef __cplusplus
}
#endif
#endif
