// Sign (+1 or -1) attached to channel d of a rotated head: the low bit of a 32-bit avalanche hash of d + 1
// (xor-shift 16, multiply 0x7feb352d, xor-shift 15, multiply 0x846ca68b, xor-shift 16).  The reference derives its
// rotation signs the same way (src/kvx_codec.cuh:28-32), so rotated rows are interchangeable.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace yka {

__device__ __forceinline__ uint32_t avalanche32(uint32_t h) {
  h = (h ^ (h >> 16)) * 0x7feb352du;
  h = (h ^ (h >> 15)) * 0x846ca68bu;
  return h ^ (h >> 16);
}

__device__ __forceinline__ float channel_sign(int d) {
  return (avalanche32((uint32_t)d + 1u) & 1u) != 0u ? -1.f : 1.f;
}

}  // namespace yka
