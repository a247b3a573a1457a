// The step between the QKV projection and the cache for 128-channel heads, fused with quantize-on-append:
// per-head RMS normalisation, partial rotary embedding, optional signed Walsh-Hadamard rotation; Q rows leave as fp16,
// K and V rows go straight into the int4 cache without a round trip through HBM as fp16.
// Follows q35_attn_post_kernel (src/q35_kernels.cu:1013-1065) in its own order of operations, with fp16 in the place of
// the reference's bf16 roundings and a correctly rounded 1/sqrt in the place of its rsqrtf (which puts its bit pattern
// out of reach: the kernel is pinned bit for bit against a CPU restatement of the sequence below, kept with the tests).
// Compiled with -ffp-contract=off; every value is a fixed sequence of single IEEE operations:
//   y = f16(projected value), for Q, K, V and gate rows alike (:1030)
//   ss = sum y^2: butterfly a += a[lane ^ o], o = 16..1, inside each run of 32 channels (:1051), then the 4 run sums
//   folded in sequence from 0 (:1055-1056)
//   r = 1 / sqrt(ss / 128 + eps);  xn = f16(y * r * (1 + w))
//   rotary, pairing d <-> d + rd/2:  f16(f16(xn * cos) + f16(-+ partner * sin))
//   rotation: signs (src/kvx_codec.cuh:28-32), 7 butterfly stages (src/kvx_codec.cuh:40-45), x 1/8 for K and V,
//   x 1/16 for Q (and for the inverse applied to attention outputs): (1/8)(1/16) 128 = 1.
#include "codec_device.h"
#include "sign_device.h"

namespace yka {
namespace {

// Round an fp32 value to fp16 and back.  The empty asm keeps the value's producer (an fp32 multiply) from being merged
// with the conversion into one mixed-precision instruction that rounds the exact product once: the arithmetic here is
// defined as two roundings (fp32, then fp16), and the two differ when the fp32 product lands on an fp16 tie.
__device__ __forceinline__ float f16r(float x) { asm volatile("" : "+v"(x)); return __half2float(__float2half_rn(x)); }

// forward rotation of one 128-channel row held one channel per thread (2 waves); buf: 128 floats of LDS
__device__ __forceinline__ float rotate128_fwd(float x, float* buf, float factor) {
  const int d = threadIdx.x;
  float a = __fmul_rn(x, channel_sign(d));
#pragma unroll
  for (int h = 1; h < 64; h *= 2) {
    const float b = __shfl_xor(a, h, 64);
    a = (d & h) ? __fsub_rn(b, a) : __fadd_rn(a, b);
  }
  __syncthreads();
  buf[d] = a;
  __syncthreads();
  const float b = buf[d ^ 64];
  a = (d & 64) ? __fsub_rn(b, a) : __fadd_rn(a, b);
  return __fmul_rn(a, factor);
}

}  // namespace

// grid (n_heads + 2 n_kv [+ n_heads], M), block 128: blocks [0, n_heads) are Q heads, then the K heads, then the V heads,
// then (if the caller hands over the gate half of the Q projection) the gate rows
__global__ void __launch_bounds__(128) attn_post_kernel(PostArgs A) {
  __shared__ float buf[128];
  __shared__ float red[4];
  const int blk = blockIdx.x, tok = blockIdx.y, d = threadIdx.x;
  const int NH = A.n_heads, KVH = A.kv.n_kv;
  const int pos = *A.d_pos + tok;
  if (pos < 0 || pos >= A.kv.max_ctx || (A.rd > 0 && pos >= A.rope_rows)) return;   // same rule as the append kernel: rows outside the container are dropped
  if (blk >= NH + 2 * KVH) {                       // gate rows (src/q35_kernels.cu:1048): the projection rounded to the 16-bit type
    const size_t e = ((size_t)tok * NH + (blk - NH - 2 * KVH)) * kD + d;
    A.gate16[e] = A.io_bf16 ? f2bf_bits(A.xgate[e]) : __half_as_ushort(__float2half_rn(A.xgate[e]));
    return;
  }
  const bool isq = blk < NH, isk = !isq && blk < NH + KVH;
  const int head = isq ? blk : (isk ? blk - NH : blk - NH - KVH);
  const float* src = isq ? A.xq + ((size_t)tok * NH + head) * kD
                         : (isk ? A.xk : A.xv) + ((size_t)tok * KVH + head) * kD;
  const float y = f16r(src[d]);
  float out;
  if (isq || isk) {
    float ss = __fmul_rn(y, y);
#pragma unroll
    for (int o = 16; o; o >>= 1) ss = __fadd_rn(ss, __shfl_xor(ss, o, 64));
    if ((d & 31) == 0) red[d >> 5] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) tot = __fadd_rn(tot, red[w]);
    // sqrtf, not __fsqrt_rn: only the former is correctly rounded on this target (measured against IEEE on 2^20 inputs)
    const float r = __fdiv_rn(1.f, sqrtf(__fadd_rn(__fdiv_rn(tot, 128.f), A.eps)));
    const float w = h2f_bits((isq ? A.qn_w16 : A.kn_w16)[d]);
    const float xn = f16r(__fmul_rn(__fmul_rn(y, r), __fadd_rn(1.f, w)));
    out = xn;
    const int hr = A.rd >> 1;
    if (hr > 0) {
      buf[d] = xn;
      __syncthreads();
      if (d < A.rd) {
        const int i = d < hr ? d : d - hr;
        const float2 cs = reinterpret_cast<const float2*>(A.rope)[(size_t)pos * hr + i];
        const float partner = d < hr ? -buf[d + hr] : buf[d - hr];
        out = f16r(__fadd_rn(f16r(__fmul_rn(xn, cs.x)), f16r(__fmul_rn(partner, cs.y))));
      }
    }
    if (A.rot) out = rotate128_fwd(out, buf, isq ? 0.0625f : 0.125f);
  } else {
    out = A.rot ? rotate128_fwd(y, buf, 0.125f) : y;
  }
  asm volatile("" : "+v"(out));                    // as in f16r: the rotation's last multiply is rounded to fp32 first
  const __half o16 = __float2half_rn(out);
  if (isq) A.q16[((size_t)tok * NH + head) * kD + d] = A.io_bf16 ? f2bf_bits(out) : __half_as_ushort(o16);
  else quant_store_value(A.kv, head, pos, !isk, __half2float(o16), d);
}

void launch_attn_post(const PostArgs& A, hipStream_t st) {
  hipLaunchKernelGGL(attn_post_kernel, dim3(A.n_heads + 2 * A.kv.n_kv + (A.gate16 ? A.n_heads : 0), A.M), dim3(128), 0, st, A);
}

}  // namespace yka
