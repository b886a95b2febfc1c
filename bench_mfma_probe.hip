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

// The same 32x32x16 loop with LDS reads and global -> LDS transfers between the MFMAs, in the proportions of a GEMM
// main loop: per 8 MFMAs a wave issues R ds_read_b128 (1 KiB each over the wave) and D buffer_load ... lds of 16
// bytes per lane (1 KiB each).  What the reads and transfers fetch is the operand data again (it is not used by the
// MFMAs, whose operands stay in registers: the loop measures what the traffic costs next to the MFMAs, on this
// data).  From the rates of a few (R, D) pairs the caller fits the cost of a KiB of either kind in units of one
// MFMA -- the part settles at the clock where the mix fits its power budget.
template <int R, int D>
__global__ __launch_bounds__(512) void mix_loop(const u32x4* srca, const u32x4* srcb, const char* gsrc, float* sink,
                                                uint64_t* clk, int iters) {
#if __HIP_DEVICE_COMPILE__
  __shared__ __attribute__((aligned(1024))) char lds[64 * 1024];      // 32 KiB that is read, 32 KiB transfers land in
  for (int i = threadIdx.x; i < 2048; i += 512) ((u32x4*)lds)[i] = srca[i & (kChunks - 1)];
  __syncthreads();
  u32x4 a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    a[i] = srca[(threadIdx.x * 8 + i) & (kChunks - 1)];
    b[i] = srcb[(threadIdx.x * 8 + i) & (kChunks - 1)];
  }
  f32x16 acc[8];
  for (int j = 0; j < 8; ++j)
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t rbase = (uint32_t)(uintptr_t)lds + (uint32_t)lane * 16u;
  char* land = lds + 32 * 1024 + wave * 4096;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)gsrc, 0, 128 * 1024, 0x00020000u);
  u32x4 got[R > 0 ? R : 1];
  const uint64_t c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[j]),
                                                      __builtin_bit_cast(f16x8, b[(j + it) & 7]), acc[j], 0, 0, 0);
#pragma unroll
      for (int r = 0; r < R; ++r)
        if ((r * 8) / R == j)
          asm volatile("ds_read_b128 %0, %1" : "=v"(got[r]) : "v"(rbase + (uint32_t)(((it * R + r) & 31) * 1024)));
#pragma unroll
      for (int d = 0; d < D; ++d)
        if ((d * 8) / D == j)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(land + d * 1024), 16,
                                                   (uint32_t)lane * 16u, (uint32_t)(((it * D + d) & 127) * 1024), 0, 0);
    }
    if constexpr (R > 0) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int r = 0; r < R; ++r) asm volatile("" : "+v"(got[r]));
    }
    if constexpr (D > 0) __builtin_amdgcn_s_waitcnt(0x0f70 | D);      // vmcnt(D): the previous iteration's have landed
  }
  __builtin_amdgcn_s_waitcnt(0);
  const uint64_t c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
  for (int j = 0; j < 8; ++j)
    for (int e = 0; e < 16; ++e) s += acc[j][e];
  if (s == 12345.678f) sink[threadIdx.x] = s + (R > 0 ? (float)got[0].x : 0.f);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clk[0] = c1 - c0;
    clk[1] = r1 - r0;
  }
#endif
}

}  // namespace

// As evt_mfma_probe_launch (variant 0), with `lds_reads` ds_read_b128 and `transfers` global -> LDS transfers of
// 1 KiB per wave between every 8 MFMAs; traffic_source: 128 KiB on the device that the transfers read.  Supported
// pairs: (0,0) (4,0) (6,0) (8,0) (0,2) (0,3) (6,3) (8,3).  Returns -2 for any other.
extern "C" int evt_mfma_probe_launch_mix(const void* a_operands, const void* b_operands, const void* traffic_source, void* sink,
                                         void* clk, int workgroups, int iters, int lds_reads, int transfers, void* stream) {
  if (!a_operands || !b_operands || !traffic_source || !sink || !clk || workgroups <= 0 || iters <= 0) return -1;
#define EVT_MIX(R_, D_)                                                                                              \
  if (lds_reads == R_ && transfers == D_) {                                                                          \
    hipLaunchKernelGGL((mix_loop<R_, D_>), dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream,            \
                       (const u32x4*)a_operands, (const u32x4*)b_operands, (const char*)traffic_source, (float*)sink, \
                       (uint64_t*)clk, iters);                                                                       \
    return (int)hipGetLastError();                                                                                   \
  }
  EVT_MIX(0, 0) EVT_MIX(4, 0) EVT_MIX(6, 0) EVT_MIX(8, 0) EVT_MIX(0, 2) EVT_MIX(0, 3) EVT_MIX(6, 3) EVT_MIX(8, 3)
#undef EVT_MIX
  return -2;
}

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
