// Quantize-on-append and the codec probes.  Compiled with -ffp-contract=off: the codec is bit-exact by contract,
// and the reference builds with --fmad=false (CMakeLists.txt:60-63).
// The quantizer itself lives in codec_device.h (shared with the fused decode kernel).
#include <algorithm>
#include "codec_device.h"

namespace yka {

// grid (M, n_kv * 2), block 128: blockIdx.y = kvh * 2 + (0: K, 1: V); thread = channel.
// Rows land at *d_pos + tok (reference: q35_kernels.cu:1038,1064 write the pass's rows before attention reads them).
__global__ void __launch_bounds__(128) append_kernel(AppendArgs A) {
  const int tok = blockIdx.x, kvh = blockIdx.y >> 1, isv = blockIdx.y & 1, d = threadIdx.x;
  const uint16_t* src = (isv ? A.v16 : A.k16) + ((size_t)tok * A.kv.n_kv + kvh) * kD;
  if (A.rows.pos) {                                // multi-stream pass: the row's own container and position
    const int pos = A.rows.pos[tok], slot = A.rows.slot[tok];
    if (pos < 0 || pos >= A.kv.max_ctx || slot < 0 || slot >= A.rows.n_slots) return;
    quant_store_row(slot_view(A.kv, A.rows, slot), kvh, pos, isv != 0, src, d);
    return;
  }
  const int pos = *A.d_pos + tok;
  if (pos < 0 || pos >= A.kv.max_ctx) return;
  quant_store_row(A.kv, kvh, pos, isv != 0, src, d);
}
void launch_append(const AppendArgs& A, hipStream_t st) {
  hipLaunchKernelGGL(append_kernel, dim3(A.M, A.kv.n_kv * 2), dim3(128), 0, st, A);
}

// codec round trip: x16 [rows][128] -> codes [rows][64], scales [rows][4], y [rows][128] fp32
__global__ void __launch_bounds__(128) codec_probe_kernel(const uint16_t* x16, int rows, uint8_t* codes, uint16_t* scales, float* y) {
  const int row = blockIdx.x, d = threadIdx.x;
  if (row >= rows) return;
  const float x = h2f_bits(x16[(size_t)row * kD + d]);
  int code; uint16_t s16;
  quant_lane(x, code, s16);
  const int nb = __shfl_xor(code, 1, 64);
  if ((d & 1) == 0) codes[(size_t)row * (kD / 2) + (d >> 1)] = (uint8_t)((code & 15) | ((nb & 15) << 4));
  if ((d & 31) == 0) scales[(size_t)row * kNG + (d >> 5)] = s16;
  // decode: (nib - 8) * s, exact in fp32 (reference: src/kvq_attn.cuh:52-54)
  y[(size_t)row * kD + d] = __fmul_rn((float)(code - 8), h2f_bits(s16));
}
void launch_codec_probe(const uint16_t* x16, int rows, uint8_t* codes, uint16_t* scales, float* y, hipStream_t st) {
  hipLaunchKernelGGL(codec_probe_kernel, dim3(rows), dim3(128), 0, st, x16, rows, codes, scales, y);
}

// canonical image <-> physical pages.  grid (n, n_kv), block 64: lane j moves byte j of K and V codes; lanes 0..3 the scales.
template <bool IMPORT>
__global__ void __launch_bounds__(64) xfer_rows_kernel(KvView kv, int pos0, int n, uint8_t* kc, uint16_t* ks, uint8_t* vc, uint16_t* vs) {
  const int t = blockIdx.x, kvh = blockIdx.y, j = threadIdx.x;
  uint8_t* pg = kv_page(kv, kvh, pos0 + t);
  const int tp = (pos0 + t) % kPageTok;
  uint8_t* pk = pg + kPageKc + tp * 64 + k_code_byte(j);
  uint8_t* pv = pg + kPageVc + tp * 64 + j;
  uint16_t* pks = reinterpret_cast<uint16_t*>(pg + kPageKs) + tp * kNG + j;      // j < 4 only
  uint16_t* pvs = reinterpret_cast<uint16_t*>(pg + kPageVs) + j * kPageTok + tp; // j < 4 only
  const size_t row = (size_t)kvh * n + t;
  if (IMPORT) {
    *pk = kc[row * 64 + j]; *pv = vc[row * 64 + j];
    if (j < kNG) { *pks = ks[row * kNG + j]; *pvs = vs[row * kNG + j]; }
  } else {
    kc[row * 64 + j] = *pk; vc[row * 64 + j] = *pv;
    if (j < kNG) { ks[row * kNG + j] = *pks; vs[row * kNG + j] = *pvs; }
  }
}
void launch_export_rows(const KvView& kv, int pos0, int n, uint8_t* kc, uint16_t* ks, uint8_t* vc, uint16_t* vs, hipStream_t st) {
  hipLaunchKernelGGL(xfer_rows_kernel<false>, dim3(n, kv.n_kv), dim3(64), 0, st, kv, pos0, n, kc, ks, vc, vs);
}
void launch_import_rows(const KvView& kv, int pos0, int n, const uint8_t* kc, const uint16_t* ks, const uint8_t* vc, const uint16_t* vs, hipStream_t st) {
  hipLaunchKernelGGL(xfer_rows_kernel<true>, dim3(n, kv.n_kv), dim3(64), 0, st, kv, pos0, n,
                     const_cast<uint8_t*>(kc), const_cast<uint16_t*>(ks), const_cast<uint8_t*>(vc), const_cast<uint16_t*>(vs));
}

// decoder probe: k, v [n_kv][n][128] fp32 = (nib - 8) * scale
__global__ void __launch_bounds__(128) dequant_rows_kernel(KvView kv, int pos0, int n, float* k, float* v) {
  const int t = blockIdx.x, kvh = blockIdx.y, d = threadIdx.x;
  const uint8_t* pg = kv_page(kv, kvh, pos0 + t);
  const int tp = (pos0 + t) % kPageTok;
  const size_t o = ((size_t)kvh * n + t) * kD + d;
  const int kb = pg[kPageKc + tp * 64 + k_code_byte(d >> 1)], vb = pg[kPageVc + tp * 64 + (d >> 1)];
  const int kn = (d & 1) ? (kb >> 4) : (kb & 15), vn = (d & 1) ? (vb >> 4) : (vb & 15);
  k[o] = __fmul_rn((float)(kn - 8), h2f_bits(reinterpret_cast<const uint16_t*>(pg + kPageKs)[tp * kNG + (d >> 5)]));
  v[o] = __fmul_rn((float)(vn - 8), h2f_bits(reinterpret_cast<const uint16_t*>(pg + kPageVs)[(d >> 5) * kPageTok + tp]));
}
void launch_dequant_rows(const KvView& kv, int pos0, int n, float* k, float* v, hipStream_t st) {
  hipLaunchKernelGGL(dequant_rows_kernel, dim3(n, kv.n_kv), dim3(128), 0, st, kv, pos0, n, k, v);
}

__global__ void set_int_kernel(int* p, int v) { *p = v; }
// bf16 -> fp16 for the rows a caller hands over in bf16 (handles opened for bf16 rows): 8 values per thread; blockIdx.y
// selects the array.  The fp32 value of every bf16 is rounded to fp16 (exact for magnitudes between 2^-14 and 65504).
__global__ void __launch_bounds__(256) bf16_to_f16_kernel(const uint16_t* a, uint16_t* a16, size_t na, const uint16_t* b, uint16_t* b16,
                                                          const uint16_t* c, uint16_t* c16, size_t nbc) {
  const uint16_t* src = blockIdx.y == 0 ? a : blockIdx.y == 1 ? b : c;
  uint16_t* dst = blockIdx.y == 0 ? a16 : blockIdx.y == 1 ? b16 : c16;
  const size_t n = blockIdx.y == 0 ? na : nbc;
  const size_t e = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (!src || e >= n) return;
  const uint4 r = *reinterpret_cast<const uint4*>(src + e);
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
  uint32_t o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint16_t lo = __half_as_ushort(__float2half_rn(bf_bits2f((uint16_t)w[k]))), hi = __half_as_ushort(__float2half_rn(bf_bits2f((uint16_t)(w[k] >> 16))));
    o[k] = (uint32_t)lo | ((uint32_t)hi << 16);
  }
  *reinterpret_cast<uint4*>(dst + e) = make_uint4(o[0], o[1], o[2], o[3]);
}
void launch_bf16_to_f16(const uint16_t* a, uint16_t* a16, size_t na, const uint16_t* b, uint16_t* b16, const uint16_t* c, uint16_t* c16, size_t nbc,
                        hipStream_t st) {
  const size_t n = std::max(na, b ? nbc : (size_t)0);
  hipLaunchKernelGGL(bf16_to_f16_kernel, dim3((unsigned)((n / 8 + 255) / 256), b ? 3 : 1), dim3(256), 0, st, a, a16, na, b, b16, c, c16, nbc);
}

__global__ void zero_ints_kernel(int* p, int n) { const int i = blockIdx.x * 256 + threadIdx.x; if (i < n) p[i] = 0; }
void launch_zero_ints(int* p, int n, hipStream_t st) { hipLaunchKernelGGL(zero_ints_kernel, dim3((n + 255) / 256), dim3(256), 0, st, p, n); }
void launch_set_int(int* p, int v, hipStream_t st) { hipLaunchKernelGGL(set_int_kernel, dim3(1), dim3(1), 0, st, p, v); }

}  // namespace yka
