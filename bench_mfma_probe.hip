// Measurement aid, not part of the fused GEMM path: a register-only MFMA loop
// (no LDS, no memory traffic inside the loop) whose operand registers are filled
// from a caller-supplied buffer.  It answers one question for the benchmark:
// what do the matrix cores of this part sustain, and at which shader clock, when
// the operands carry the same kind of data as the benchmark's tensors?  On
// MI355X the answer depends on the data: with all-zero or constant operands the
// loop runs at the nominal clock, with N(0,1) halves the part's power management
// lowers the clock by about 30 %.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kChunks = 8192;   // 16-byte operand chunks each buffer holds (128 KiB)

typedef float f32x4 __attribute__((ext_vector_type(4)));

// VARIANT 0: v_mfma_f32_32x32x16_f16 (the instruction of the fused kernels), 1: v_mfma_f32_16x16x32_f16
// (half the output block, twice the depth: twice the operand bytes per flop).  Both count 32768 flop per
// "step" below: one 32x32x16 or two 16x16x32.
template <int VARIANT>
__global__ __launch_bounds__(512) void mfma_loop(const u32x4* srca, const u32x4* srcb, float* sink, uint64_t* clk, int iters) {
#if __HIP_DEVICE_COMPILE__
  u32x4 a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    a[i] = srca[(threadIdx.x * 8 + i) & (kChunks - 1)];
    b[i] = srcb[(threadIdx.x * 8 + i) & (kChunks - 1)];
  }
  float s = 0.f;
  uint64_t c0, r0, c1, r1;
  if constexpr (VARIANT == 0) {
    f32x16 acc[8];
    for (int j = 0; j < 8; ++j)
      for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    c0 = __builtin_amdgcn_s_memtime(); r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[j]),
                                                        __builtin_bit_cast(f16x8, b[(j + it) & 7]), acc[j], 0, 0, 0);
    }
    c1 = __builtin_amdgcn_s_memtime(); r1 = __builtin_amdgcn_s_memrealtime();
    for (int j = 0; j < 8; ++j)
      for (int e = 0; e < 16; ++e) s += acc[j][e];
  } else {
    f32x4 acc[16];
    for (int j = 0; j < 16; ++j)
      for (int e = 0; e < 4; ++e) acc[j][e] = 0.f;
    c0 = __builtin_amdgcn_s_memtime(); r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 16; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a[j & 7]),
                                                        __builtin_bit_cast(f16x8, b[(j + it) & 7]), acc[j], 0, 0, 0);
    }
    c1 = __builtin_amdgcn_s_memtime(); r1 = __builtin_amdgcn_s_memrealtime();
    for (int j = 0; j < 16; ++j)
      for (int e = 0; e < 4; ++e) s += acc[j][e];
  }
  if (s == 12345.678f) sink[threadIdx.x] = s;   // keeps the loop alive, practically never taken
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clk[0] = c1 - c0;   // shader cycles
    clk[1] = r1 - r0;   // 100 MHz ticks
  }
#endif
}

}  // namespace

// a_operands, b_operands: 128 KiB of fp16 data each on the device (the A-side and B-side registers are filled
// from them; pass one buffer twice for a single distribution); sink: >= 2 KiB; clk: two uint64.
// One launch = workgroups x 8 waves x iters x 8 steps of 32768 flop (variant 0: one 32x32x16 MFMA per step,
// variant 1: two 16x16x32).
extern "C" int evt_mfma_probe_launch(const void* a_operands, const void* b_operands, void* sink, void* clk,
                                     int workgroups, int iters, int variant, void* stream) {
  if (!a_operands || !b_operands || !sink || !clk || workgroups <= 0 || iters <= 0 || variant < 0 || variant > 1) return -1;
  if (variant == 0)
    hipLaunchKernelGGL(mfma_loop<0>, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream,
                       (const u32x4*)a_operands, (const u32x4*)b_operands, (float*)sink, (uint64_t*)clk, iters);
  else
    hipLaunchKernelGGL(mfma_loop<1>, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream,
                       (const u32x4*)a_operands, (const u32x4*)b_operands, (float*)sink, (uint64_t*)clk, iters);
  return (int)hipGetLastError();
}
