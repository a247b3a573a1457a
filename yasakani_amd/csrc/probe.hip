// Machine probe: what this GPU sustains on the instruction mixes the attention kernels are made of.  gfx950.
//
// The reference measures its machine inside its bench hooks (src/kvx_probe.cu:322-449); this is the same idea for the
// figures the kernels here are designed around: dense MFMA rate, plain vector rate, how far matrix and vector
// instructions overlap (inside one wave and between two waves of one SIMD), the shader clock under load, and the
// streaming read rate.  Every loop body is a fixed instruction sequence (inline asm), so the numbers do not depend on
// the compiler's scheduling.  Waves time themselves with the shader clock and with the constant-rate wall clock.
#include "yka_internal.h"

namespace yka {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

namespace {

struct WaveClock { unsigned long long c0, w0; };
__device__ __forceinline__ WaveClock tick() { return WaveClock{(unsigned long long)clock64(), (unsigned long long)wall_clock64()}; }
__device__ __forceinline__ void tock(const WaveClock& t, unsigned long long* rec, int wave_id) {
  const unsigned long long c1 = (unsigned long long)clock64(), w1 = (unsigned long long)wall_clock64();
  if ((threadIdx.x & 63) == 0) { rec[2 * wave_id] = c1 - t.c0; rec[2 * wave_id + 1] = w1 - t.w0; }
}

// operands: %0-%3 four 32x32 accumulators, %4-%11 eight fp32 chains, %12/%13 MFMA A/B, %14/%15 FMA constants
#define YKA_MF32(n) "v_mfma_f32_32x32x16_f16 %" #n ", %12, %13, %" #n "\n\t"
#define YKA_FM(n) "v_fma_f32 %" #n ", %" #n ", %14, %15\n\t"
#define YKA_OPS                                                                                                      \
  : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3), "+v"(x4), "+v"(x5), "+v"(x6), "+v"(x7) \
  : "v"(fa), "v"(fb), "v"(c1), "v"(c2)

// NV vector FMAs behind every MFMA (0, 2, 4, 6 or 8); MF = false leaves the MFMAs out (the vector work alone)
template <int NV, bool MF>
__device__ __forceinline__ void body(f16v& a0, f16v& a1, f16v& a2, f16v& a3, float& x0, float& x1, float& x2, float& x3, float& x4,
                                     float& x5, float& x6, float& x7, h8 fa, h8 fb, float c1, float c2) {
  if constexpr (MF && NV == 0) asm volatile(YKA_MF32(0) YKA_MF32(1) YKA_MF32(2) YKA_MF32(3) YKA_OPS);
  if constexpr (MF && NV == 2) asm volatile(YKA_MF32(0) YKA_FM(4) YKA_FM(5) YKA_MF32(1) YKA_FM(6) YKA_FM(7) YKA_MF32(2) YKA_FM(8) YKA_FM(9) YKA_MF32(3) YKA_FM(10) YKA_FM(11) YKA_OPS);
  if constexpr (MF && NV == 4)
    asm volatile(YKA_MF32(0) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_MF32(1) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11)
                 YKA_MF32(2) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_MF32(3) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_OPS);
  if constexpr (MF && NV == 6)
    asm volatile(YKA_MF32(0) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_MF32(1) YKA_FM(10) YKA_FM(11) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7)
                 YKA_MF32(2) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_FM(4) YKA_FM(5) YKA_MF32(3) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_OPS);
  if constexpr (MF && NV == 8)
    asm volatile(YKA_MF32(0) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_MF32(1) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11)
                 YKA_MF32(2) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_MF32(3) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_OPS);
  if constexpr (!MF)   // 32 FMAs
    asm volatile(YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11)
                 YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_FM(4) YKA_FM(5) YKA_FM(6) YKA_FM(7) YKA_FM(8) YKA_FM(9) YKA_FM(10) YKA_FM(11) YKA_OPS);
}

// the matrix results are read by ordinary instructions after the loop: the asm blocks hide their MFMAs from the
// compiler's hazard handling, so the distance is kept by hand
#define YKA_SETTLE asm volatile("s_nop 15\n\ts_nop 15" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3))

// role of a wave: 0 = MFMA + NV FMAs interleaved, 1 = FMAs alone.  split != 0: waves 4.. of a 512-thread workgroup take
// role 1 with iters_b iterations (two waves per SIMD, one of each role); otherwise every wave takes role 0 (or 1 if !MF).
template <int NV, bool MF>
__global__ void __launch_bounds__(512) mix_kernel(float* sink, unsigned long long* rec, int iters, int iters_b, int split) {
  const int wave = threadIdx.x >> 6, wave_id = blockIdx.x * (blockDim.x >> 6) + wave;
  f16v a0{}, a1{}, a2{}, a3{};
  float x0 = 0.001f * threadIdx.x, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3, x4 = x0 + 4, x5 = x0 + 5, x6 = x0 + 6, x7 = x0 + 7;
  const h8 fa = {1, 1, 1, 1, 1, 1, 1, 1}, fb = {1, 1, 1, 1, 1, 1, 1, 1};
  const float c1 = 0.999f, c2 = 0.001f;
  __syncthreads();
  const WaveClock t = tick();
  if (split && wave >= 4) {
    for (int it = 0; it < iters_b; ++it) body<0, false>(a0, a1, a2, a3, x0, x1, x2, x3, x4, x5, x6, x7, fa, fb, c1, c2);
  } else {
    for (int it = 0; it < iters; ++it) body<NV, MF>(a0, a1, a2, a3, x0, x1, x2, x3, x4, x5, x6, x7, fa, fb, c1, c2);
  }
  YKA_SETTLE;
  tock(t, rec, wave_id);
  const float s = a0[0] + a1[1] + a2[2] + a3[3] + x0 + x1 + x2 + x3 + x4 + x5 + x6 + x7;
  if (s == 12345.678f) sink[wave_id] = s;
}

__global__ void __launch_bounds__(256) mfma16_kernel(float* sink, unsigned long long* rec, int iters) {
  const int wave_id = blockIdx.x * 4 + (threadIdx.x >> 6);
  f4 b0{}, b1{}, b2{}, b3{}, b4{}, b5{}, b6{}, b7{};
  const h8 fa = {1, 1, 1, 1, 1, 1, 1, 1}, fb = {1, 1, 1, 1, 1, 1, 1, 1};
  const WaveClock t = tick();
#define YKA_MF16(n) "v_mfma_f32_16x16x32_f16 %" #n ", %8, %9, %" #n "\n\t"
  for (int it = 0; it < iters; ++it)
    asm volatile(YKA_MF16(0) YKA_MF16(1) YKA_MF16(2) YKA_MF16(3) YKA_MF16(4) YKA_MF16(5) YKA_MF16(6) YKA_MF16(7)
                 : "+v"(b0), "+v"(b1), "+v"(b2), "+v"(b3), "+v"(b4), "+v"(b5), "+v"(b6), "+v"(b7) : "v"(fa), "v"(fb));
#undef YKA_MF16
  asm volatile("s_nop 15\n\ts_nop 15" : "+v"(b0), "+v"(b1), "+v"(b2), "+v"(b3), "+v"(b4), "+v"(b5), "+v"(b6), "+v"(b7));
  tock(t, rec, wave_id);
  const float s = b0[0] + b1[1] + b2[2] + b3[3] + b4[0] + b5[1] + b6[2] + b7[3];
  if (s == 12345.678f) sink[wave_id] = s;
}

// vector opcodes alone: 32 instructions per iteration over 8 independent chains
template <int OP>
__global__ void __launch_bounds__(512) valu_kernel(float* sink, unsigned long long* rec, int iters) {
  const int wave_id = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  float x[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = -0.001f * (threadIdx.x + i);
  const WaveClock t = tick();
  for (int it = 0; it < iters; ++it)
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (OP == 0) asm volatile("v_exp_f32 %0, %0" : "+v"(x[i]));
        if (OP == 1) asm volatile("v_pk_mul_f16 %0, %0, %0" : "+v"(x[i]));
        if (OP == 2) asm volatile("v_cvt_pk_f16_f32 %0, %0, %0" : "+v"(x[i]));
        if (OP == 3) asm volatile("v_max3_f32 %0, %0, %0, %0" : "+v"(x[i]));
        if (OP == 4) asm volatile("v_and_or_b32 %0, %0, %0, %0" : "+v"(x[i]));
        if (OP == 5) asm volatile("v_pk_add_f16 %0, %0, %0" : "+v"(x[i]));
        if (OP == 6) asm volatile("v_perm_b32 %0, %0, %0, %0" : "+v"(x[i]));
        if (OP == 7) asm volatile("v_mul_f32 %0, %0, %0" : "+v"(x[i]));
      }
  tock(t, rec, wave_id);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += x[i];
  if (s == 12345.678f) sink[wave_id] = s;
}

// streaming read: every thread reads 16-byte pieces, a workgroup a contiguous 64 KiB block at a time
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// One wave of MFMAs and one wave of a given vector opcode on every SIMD (waves 0-3 / 4-7 of a 512-thread workgroup): how
// far the matrix pipe and that opcode's pipe run side by side when the instructions come from different waves.
template <int OP>
__global__ void __launch_bounds__(512) cross_kernel(float* sink, unsigned long long* rec, int iters, int iters_b) {
  const int wave = threadIdx.x >> 6, wave_id = blockIdx.x * (blockDim.x >> 6) + wave;
  f16v a0{}, a1{}, a2{}, a3{};
  float x0 = 0.001f * threadIdx.x, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3, x4 = x0 + 4, x5 = x0 + 5, x6 = x0 + 6, x7 = x0 + 7;
  const h8 fa = {1, 1, 1, 1, 1, 1, 1, 1}, fb = {1, 1, 1, 1, 1, 1, 1, 1};
  const float c1 = 0.999f, c2 = 0.001f;
  float x[8] = {x0, x1, x2, x3, x4, x5, x6, x7};
  __syncthreads();
  const WaveClock t = tick();
  if (wave >= 4) {
    for (int it = 0; it < iters_b; ++it) {
#pragma unroll
      for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (OP == 0) asm volatile("v_exp_f32 %0, %0" : "+v"(x[i]));
          if (OP == 1) asm volatile("v_pk_mul_f16 %0, %0, %0" : "+v"(x[i]));
          if (OP == 2) asm volatile("v_cvt_pk_f16_f32 %0, %0, %0" : "+v"(x[i]));
          if (OP == 3) asm volatile("v_max3_f32 %0, %0, %0, %0" : "+v"(x[i]));
          if (OP == 4) asm volatile("v_and_or_b32 %0, %0, %0, %0" : "+v"(x[i]));
          if (OP == 5) asm volatile("v_pk_add_f16 %0, %0, %0" : "+v"(x[i]));
          if (OP == 6) asm volatile("v_perm_b32 %0, %0, %0, %0" : "+v"(x[i]));
          if (OP == 7) asm volatile("v_mul_f32 %0, %0, %0" : "+v"(x[i]));
        }
    }
  } else {
    for (int it = 0; it < iters; ++it) body<0, true>(a0, a1, a2, a3, x0, x1, x2, x3, x4, x5, x6, x7, fa, fb, c1, c2);
  }
  YKA_SETTLE;
  tock(t, rec, wave_id);
  const float s = a0[0] + a1[1] + a2[2] + a3[3] + x[0] + x[1] + x[2] + x[3] + x[4] + x[5] + x[6] + x[7];
  if (s == 12345.678f) sink[wave_id] = s;
}

template <bool NT>
__global__ void __launch_bounds__(256) read_kernel(const u32x4* src, size_t n16, float* sink) {
  uint32_t acc = 0;
  const size_t per_block = 4096;                                  // 16-byte pieces per workgroup step (64 KiB)
  for (size_t base = (size_t)blockIdx.x * per_block; base < n16; base += (size_t)gridDim.x * per_block) {
    u32x4 v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const size_t i = base + (size_t)k * 256 + threadIdx.x;
      const u32x4* p = src + (i < n16 ? i : 0);
      v[k] = NT ? __builtin_nontemporal_load(p) : *p;
    }
#pragma unroll
    for (int k = 0; k < 16; ++k) acc ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
  }
  if (acc == 0x12345679u) sink[blockIdx.x * 256 + threadIdx.x] = (float)acc;
}

}  // namespace

void launch_probe_mix(int nv, bool mfma, float* sink, unsigned long long* rec, int iters, int iters_b, int split, int blocks, int threads, hipStream_t st) {
#define YKA_MIX(NV, MF) hipLaunchKernelGGL((mix_kernel<NV, MF>), dim3(blocks), dim3(threads), 0, st, sink, rec, iters, iters_b, split)
  if (!mfma) YKA_MIX(0, false);
  else if (nv == 0) YKA_MIX(0, true);
  else if (nv == 2) YKA_MIX(2, true);
  else if (nv == 4) YKA_MIX(4, true);
  else if (nv == 6) YKA_MIX(6, true);
  else YKA_MIX(8, true);
#undef YKA_MIX
}
void launch_probe_mfma16(float* sink, unsigned long long* rec, int iters, int blocks, hipStream_t st) {
  hipLaunchKernelGGL(mfma16_kernel, dim3(blocks), dim3(256), 0, st, sink, rec, iters);
}
void launch_probe_valu(int op, float* sink, unsigned long long* rec, int iters, int blocks, int threads, hipStream_t st) {
#define YKA_V(OP) hipLaunchKernelGGL(valu_kernel<OP>, dim3(blocks), dim3(threads), 0, st, sink, rec, iters)
  switch (op) {
    case 0: YKA_V(0); break; case 1: YKA_V(1); break; case 2: YKA_V(2); break; case 3: YKA_V(3); break;
    case 4: YKA_V(4); break; case 5: YKA_V(5); break; case 6: YKA_V(6); break; default: YKA_V(7); break;
  }
#undef YKA_V
}
void launch_probe_cross(int op, float* sink, unsigned long long* rec, int iters, int iters_b, int blocks, hipStream_t st) {
#define YKA_X(OP) hipLaunchKernelGGL(cross_kernel<OP>, dim3(blocks), dim3(512), 0, st, sink, rec, iters, iters_b)
  switch (op) {
    case 0: YKA_X(0); break; case 1: YKA_X(1); break; case 2: YKA_X(2); break; case 3: YKA_X(3); break;
    case 4: YKA_X(4); break; case 5: YKA_X(5); break; case 6: YKA_X(6); break; default: YKA_X(7); break;
  }
#undef YKA_X
}
void launch_probe_read(bool nt, const void* src, size_t bytes, float* sink, int blocks, hipStream_t st) {
  if (nt) hipLaunchKernelGGL(read_kernel<true>, dim3(blocks), dim3(256), 0, st, (const u32x4*)src, bytes / 16, sink);
  else hipLaunchKernelGGL(read_kernel<false>, dim3(blocks), dim3(256), 0, st, (const u32x4*)src, bytes / 16, sink);
}

}  // namespace yka
