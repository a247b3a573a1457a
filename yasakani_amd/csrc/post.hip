// The step between the QKV projection and the cache for 128-channel heads, fused with quantize-on-append:
// per-head RMS normalisation, partial rotary embedding, optional signed Walsh-Hadamard rotation; Q rows leave as fp16,
// K and V rows go straight into the int4 cache without a round trip through HBM as fp16.
// Follows q35_attn_post_kernel (src/q35_kernels.cu:1013-1065) with fp16 in the place of the reference's bf16 roundings.
// Two deliberate differences from that kernel, so this step is the reference's ALGORITHM, not its bit pattern (which
// its rsqrtf puts out of reach anyway: parity with the reference's own outputs for this step is unpinned, the kernel is
// pinned bit for bit against a CPU restatement of the sequence below, kept with the tests):
//   * the reference first rounds the projected value to its 16-bit type (y = rbf(buf[tid]), :1030) and forms V, the sum
//     of squares and xn from that; here the projection's fp32 value is used unrounded (one rounding fewer);
//   * the reference sums squares by a 32-lane butterfly and then folds its 8 warp sums in sequence (:1050-1056); here the
//     butterfly runs over 64 lanes and the two wave sums are added.
// Compiled with -ffp-contract=off; every value is a fixed sequence of single IEEE operations:
//   ss = sum y^2: butterfly a += a[lane ^ o], o = 32..1, inside each wave (= 64-channel half), then half 0 + half 1
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
  __shared__ float red[2];
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
  const float y = src[d];
  float out;
  if (isq || isk) {
    float ss = __fmul_rn(y, y);
#pragma unroll
    for (int o = 32; o; o >>= 1) ss = __fadd_rn(ss, __shfl_xor(ss, o, 64));
    if ((d & 63) == 0) red[d >> 6] = ss;
    __syncthreads();
    const float tot = __fadd_rn(red[0], red[1]);
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
