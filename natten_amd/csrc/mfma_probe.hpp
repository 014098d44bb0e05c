// Sustained matrix-core rate probe for gfx950: every SIMD runs nothing but 32x32x16 bf16 MFMAs
// (plus a fixed number of independent vector FMAs per MFMA) on operands read once from memory.
// With random operands the chip settles at the clock its power limit allows, so the result is
// the matrix rate a real kernel can hope for, as opposed to the data-sheet peak at the maximum
// clock.  Diagnostic only: it has no counterpart in SHI-Labs/NATTEN.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace natten_amd {

constexpr int kProbeBlocks = 256;        // one workgroup per CU
constexpr int kProbeThreads = 256;       // one wave per SIMD
constexpr int kProbeMfmaPerIter = 16;

// operands: kProbeBlocks * kProbeThreads * 8 vectors of 8 bf16 (16 bytes each)
// sink:     kProbeBlocks * kProbeThreads floats (keeps the results alive)
// clocks:   2 * kProbeBlocks uint64: shader cycles and 100 MHz ticks spent in the loop
template <int FMA_PER_MFMA>
__global__ void __launch_bounds__(kProbeThreads) mfma_probe_kernel(const void* operands, float* sink,
                                                                    unsigned long long* clocks, int iters) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  typedef float f32x16 __attribute__((ext_vector_type(16)));
  const bf16x8* src = static_cast<const bf16x8*>(operands) + (size_t(blockIdx.x) * kProbeThreads + threadIdx.x) * 8;
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = src[i];
    b[i] = src[4 + i];
  }
  f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = 1.0f + float(i) + float(threadIdx.x);
  const float c0 = 1.0001f, c1 = 0.5f;
  const unsigned long long t0 = __builtin_amdgcn_s_memtime(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < kProbeMfmaPerIter; ++u) {
      // four independent accumulators; inline assembly keeps the instruction mix as written
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[u & 3]) : "v"(a[u & 3]), "v"(b[(u >> 2) & 3]));
#pragma unroll
      for (int n = 0; n < FMA_PER_MFMA; ++n)
        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[(u * FMA_PER_MFMA + n) & 7]) : "v"(c0), "v"(c1));
    }
  }
  // the matrix pipe must drain before its results are read: the compiler cannot see the
  // MFMAs inside the assembly statements (two 16-wait-state no-ops cover the last one)
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  const unsigned long long t1 = __builtin_amdgcn_s_memtime(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
#pragma unroll
  for (int i = 0; i < 8; ++i) s += v[i];
  sink[size_t(blockIdx.x) * kProbeThreads + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = t1 - t0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

}  // namespace natten_amd
