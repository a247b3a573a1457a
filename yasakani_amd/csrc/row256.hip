// The reference's own 256-channel row codec on gfx950: signed Walsh-Hadamard rotation, flat int4 with one fp32 scale
// per row and MSB-first packing, int8 rows.  Compiled with -ffp-contract=off: every value is produced by the same
// sequence of single IEEE fp32 operations as in the reference, so results are bit-identical to it.
//   rotation   src/kvx_codec.cuh:28-49        flat int4  src/kvq_fast.cuh:194-198, packing :226-233
//   int8 rows  src/kvx_codec.cuh:50-69        decode     src/kvq_attn.cuh:33-37,53-54
// One workgroup of 256 threads (4 waves) per row, thread d owns channel d.
#include "yka_internal.h"
#include "rot256_device.h"
#include <hip/hip_fp16.h>

namespace yka {
namespace {

__device__ __forceinline__ float row_absmax(float v, float* red) {
  float m = fabsf(v);
#pragma unroll
  for (int o = 32; o; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__global__ void __launch_bounds__(256) row256_encode_kernel(const float* x, int mode, int rot, int8_t* q8, uint32_t* words, float* scales) {
  __shared__ float buf[256];
  __shared__ float red[4];
  __shared__ uint8_t fld[256];
  const int row = blockIdx.x, d = threadIdx.x;
  float v = x[(size_t)row * 256 + d];
  if (rot) v = rotate256(v, buf, false);
  const float am = row_absmax(v, red);
  if (mode == 0) {
    const float sc = __fdiv_rn(am, 127.f);
    int q = sc > 0.f ? __float2int_rn(__fdiv_rn(v, sc)) : 0;
    q = max(-127, min(127, q));
    q8[(size_t)row * 256 + d] = (int8_t)q;
    if (d == 0) scales[row] = sc;
  } else {
    float s7 = __fdiv_rn(am, 7.f);
    if (s7 == 0.f) s7 = 1.f;
    float q = rintf(__fdiv_rn(v, s7));
    q = fminf(fmaxf(q, -7.f), 7.f);
    fld[d] = (uint8_t)((int)q + 8);
    __syncthreads();
    if (d < 32) {                               // word d = fields 8d .. 8d+7, the first in the top nibble
      uint32_t w = 0u;
#pragma unroll
      for (int i = 0; i < 8; ++i) w |= (uint32_t)fld[8 * d + i] << (28 - 4 * i);
      words[(size_t)row * 32 + d] = w;
    }
    if (d == 0) scales[row] = s7;
  }
}

__global__ void __launch_bounds__(256) row256_decode_kernel(int mode, int rot, const int8_t* q8, const uint32_t* words, const float* scales, float* y) {
  __shared__ float buf[256];
  const int row = blockIdx.x, d = threadIdx.x;
  const float s = scales[row];
  float v;
  if (mode == 0) v = __fmul_rn((float)q8[(size_t)row * 256 + d], s);
  else {
    const uint32_t w = words[(size_t)row * 32 + (d >> 3)];
    const int nib = (int)((w >> (28 - 4 * (d & 7))) & 15u);
    v = __fmul_rn((float)(nib - 8), s);
  }
  if (rot) v = rotate256(v, buf, true);
  y[(size_t)row * 256 + d] = v;
}

// The step after attention for 256-channel heads (src/q35_kernels.cu:1420-1428, src/a8_prologue.cuh:87-98,122-133), fp16 in
// the place of the reference's bf16 roundings: sigmoid gate, signs, 512-point Hadamard transform x 1/sqrt(512), fp16
// rounding, int8 with one scale per group of 512.  grid (n_heads / 2, M), block 512: thread = element of the group.
// lo != 0: the reference's interleaved layout for passes of at most 8 tokens (a8_lo_off, src/a8_prologue.cuh:121,132; qx base
// + group * 4096): element i of token t of a group sits at (i/256)*2048 + ((i/16)%4)*512 + t*64 + ((i/64)%4)*16 + i%16.
__global__ void __launch_bounds__(512) attn_out256_kernel(const uint16_t* y16, const uint16_t* gate16, const int8_t* signs, int n_heads,
                                                          int lo, int8_t* qx, float* alpha) {
  __shared__ float buf[512];
  __shared__ float red[8];
  const int blk = blockIdx.x, tok = blockIdx.y, tid = threadIdx.x;
  const int N = n_heads * 256;
  const size_t e = (size_t)tok * N + (size_t)blk * 512 + tid;
  const float gate = __half2float(__ushort_as_half(gate16[e]));
  float sg = __fdiv_rn(1.f, __fadd_rn(1.f, expf(-gate)));
  asm volatile("" : "+v"(sg));                     // two roundings (fp32, then fp16), never one of the exact quotient
  sg = __half2float(__float2half_rn(sg));
  float y2 = __fmul_rn(__half2float(__ushort_as_half(y16[e])), sg);
  asm volatile("" : "+v"(y2));
  y2 = __half2float(__float2half_rn(y2));
  float v = __fmul_rn(y2, (float)signs[blk * 512 + tid]);
#pragma unroll
  for (int h = 1; h < 64; h *= 2) {
    const float q = __shfl_xor(v, h, 64);
    v = (tid & h) ? __fsub_rn(q, v) : __fadd_rn(v, q);
  }
#pragma unroll
  for (int h = 64; h < 512; h *= 2) {
    __syncthreads();
    buf[tid] = v;
    __syncthreads();
    const float q = buf[tid ^ h];
    v = (tid & h) ? __fsub_rn(q, v) : __fadd_rn(v, q);
  }
  v = __fmul_rn(v, 0.044194173824159216f);
  asm volatile("" : "+v"(v));
  v = __half2float(__float2half_rn(v));
  float am = fabsf(v);
#pragma unroll
  for (int o = 32; o; o >>= 1) am = fmaxf(am, __shfl_xor(am, o, 64));
  if ((tid & 63) == 0) red[tid >> 6] = am;
  __syncthreads();
  am = fmaxf(fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])), fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7])));
  const float al = __fdiv_rn(am, 127.f);
  if (tid == 0) alpha[(size_t)tok * (N / 512) + blk] = al;
  int q = al > 0.f ? __float2int_rn(__fdiv_rn(v, al)) : 0;
  q = max(-127, min(127, q));
  if (lo) qx[(size_t)blk * 4096 + (((tid >> 8) << 11) | (((tid >> 4) & 3) << 9) | (tok << 6) | (((tid >> 6) & 3) << 4) | (tid & 15))] = (int8_t)q;
  else qx[e] = (int8_t)q;
}

}  // namespace

void launch_attn_out256(const uint16_t* y16, const uint16_t* gate16, const int8_t* signs, int M, int n_heads, int lo, int8_t* qx, float* alpha, hipStream_t st) {
  hipLaunchKernelGGL(attn_out256_kernel, dim3(n_heads / 2, M), dim3(512), 0, st, y16, gate16, signs, n_heads, lo, qx, alpha);
}

void launch_row256_encode(const float* x, int rows, int mode, int rot, int8_t* q8, uint32_t* words, float* scales, hipStream_t st) {
  hipLaunchKernelGGL(row256_encode_kernel, dim3(rows), dim3(256), 0, st, x, mode, rot, q8, words, scales);
}
void launch_row256_decode(int rows, int mode, int rot, const int8_t* q8, const uint32_t* words, const float* scales, float* y, hipStream_t st) {
  hipLaunchKernelGGL(row256_decode_kernel, dim3(rows), dim3(256), 0, st, mode, rot, q8, words, scales, y);
}

}  // namespace yka
