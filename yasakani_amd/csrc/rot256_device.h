// Signed Walsh-Hadamard rotation over 256 channels, one channel per thread of a 256-thread workgroup
// (reference: src/kvx_codec.cuh:28-49).  Every value is produced by the same single IEEE fp32 operations, in the same
// order, as in the reference; include only from translation units compiled with -ffp-contract=off.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "sign_device.h"

namespace yka {

// The butterfly stages are element-wise, so where the partner lives does not change a bit of the result: partners at
// distance 1..32 are in the same wave (cross-lane exchange), 64 and 128 go through LDS.
__device__ __forceinline__ float rotate256(float x, float* buf, bool inverse) {
  const int d = threadIdx.x;
  float a = inverse ? x : __fmul_rn(x, channel_sign(d));
#pragma unroll
  for (int h = 1; h < 64; h *= 2) {
    const float b = __shfl_xor(a, h, 64);
    a = (d & h) ? __fsub_rn(b, a) : __fadd_rn(a, b);
  }
#pragma unroll
  for (int h = 64; h < 256; h *= 2) {
    __syncthreads();
    buf[d] = a;
    __syncthreads();
    const float b = buf[d ^ h];
    a = (d & h) ? __fsub_rn(b, a) : __fadd_rn(a, b);
  }
  float y = __fmul_rn(a, 0.0625f);
  if (inverse) y = __fmul_rn(y, channel_sign(d));
  return y;
}

}  // namespace yka
