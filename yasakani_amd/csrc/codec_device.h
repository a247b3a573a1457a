// Device-side quantizer shared by the append kernel and by the fused decode kernel.
//
// Arithmetic per 32-channel group (reference: src/kvq_fast.cuh:194-198, src/kvq_gpu.cuh:85-86):
//   am = max|x|; s = fp16(am / 7); if (s == 0) s = 1; q = clamp(rint(x / s), -7, 7); stored nibble = q + 8.
// The division is by the stored (fp16-rounded) scale, as the reference divides by the scale it stores.
// Only IEEE divides, conversions and min/max appear here: nothing a compiler could contract into an FMA.
#pragma once
#include "yka_internal.h"
#include <hip/hip_fp16.h>

namespace yka {

__device__ __forceinline__ float h2f_bits(uint16_t b) { return __half2float(__ushort_as_half(b)); }
// physical byte of a K row that holds logical byte j (channels 2j, 2j+1)
__device__ __forceinline__ int k_code_byte(int j) { return 4 * k_phys_dword(j >> 2) + (j & 3); }

// one lane = one channel; lanes of a 32-lane half-wave form one scale group
__device__ __forceinline__ void quant_lane(float x, int& code, uint16_t& s16) {
  float am = fabsf(x);
#pragma unroll
  for (int o = 16; o; o >>= 1) am = fmaxf(am, __shfl_xor(am, o, 32));
  const float s32 = __fdiv_rn(am, 7.0f);
  s16 = __half_as_ushort(__float2half_rn(s32));
  if ((s16 & 0x7fffu) == 0) s16 = 0x3c00u;
  const float sd = h2f_bits(s16);
  float q = rintf(__fdiv_rn(x, sd));
  q = fminf(fmaxf(q, -7.f), 7.f);
  code = (int)q + 8;
}

// Quantizes channel d (0..127) of one fp16 row and stores its share of the row at token `pos` of kv head `kvh`.
// Must be called by all 128 lanes of two full waves (d = lane index over the row); isv selects the V planes.
__device__ __forceinline__ void quant_store_value(const KvView& kv, int kvh, int pos, bool isv, float x, int d);
__device__ __forceinline__ void quant_store_row(const KvView& kv, int kvh, int pos, bool isv, const uint16_t* src_row, int d) {
  quant_store_value(kv, kvh, pos, isv, h2f_bits(src_row[d]), d);
}
// the same with the (fp16-valued) channel already in a register
__device__ __forceinline__ void quant_store_value(const KvView& kv, int kvh, int pos, bool isv, float x, int d) {
  int code; uint16_t s16;
  quant_lane(x, code, s16);
  const int nb = __shfl_xor(code, 1, 64);
  uint8_t* pg = kv_page(kv, kvh, pos);
  const int tp = pos % kPageTok;
  if ((d & 1) == 0) {
    const uint8_t byte = (uint8_t)((code & 15) | ((nb & 15) << 4));
    if (isv) pg[kPageVc + tp * 64 + (d >> 1)] = byte;
    else pg[kPageKc + tp * 64 + k_code_byte(d >> 1)] = byte;
  }
  if ((d & 31) == 0) {
    if (isv) reinterpret_cast<uint16_t*>(pg + kPageVs)[(d >> 5) * kPageTok + tp] = s16;
    else reinterpret_cast<uint16_t*>(pg + kPageKs)[tp * kNG + (d >> 5)] = s16;
  }
}

// The same quantizer with 16 lanes per row: lane c (0..15, four consecutive lanes = one scale group) owns channels
// 8c .. 8c+7, given as 8 fp16 in `raw`.  Bit-identical to quant_store_value: the group maximum is exact in any order,
// everything after it is the same sequence of IEEE operations per channel.  Must be called by all 16 lanes of a row.
__device__ __forceinline__ void quant_store_chunk8(const KvView& kv, int kvh, int pos, bool isv, uint4 raw, int c) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  float x[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = h2f_bits((uint16_t)(w[e >> 1] >> (16 * (e & 1))));
  float am = fabsf(x[0]);
#pragma unroll
  for (int e = 1; e < 8; ++e) am = fmaxf(am, fabsf(x[e]));
  am = fmaxf(am, __shfl_xor(am, 1, 64));
  am = fmaxf(am, __shfl_xor(am, 2, 64));
  const float s32 = __fdiv_rn(am, 7.0f);
  uint16_t s16 = __half_as_ushort(__float2half_rn(s32));
  if ((s16 & 0x7fffu) == 0) s16 = 0x3c00u;
  const float sd = h2f_bits(s16);
  uint32_t word = 0;                           // channel 8c+e in bits [4e, 4e+4): even channel = low nibble of its byte
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float q = rintf(__fdiv_rn(x[e], sd));
    q = fminf(fmaxf(q, -7.f), 7.f);
    word |= (uint32_t)((int)q + 8) << (4 * e);
  }
  uint8_t* pg = kv_page(kv, kvh, pos);
  const int tp = pos % kPageTok, g = c >> 2;
  if (isv) *reinterpret_cast<uint32_t*>(pg + kPageVc + tp * 64 + 4 * c) = word;
  else *reinterpret_cast<uint32_t*>(pg + kPageKc + tp * 64 + 4 * k_phys_dword(c)) = word;
  if ((c & 3) == 0) {
    if (isv) reinterpret_cast<uint16_t*>(pg + kPageVs)[g * kPageTok + tp] = s16;
    else reinterpret_cast<uint16_t*>(pg + kPageKs)[tp * kNG + g] = s16;
  }
}

}  // namespace yka
