// Measurement aid: what the matrix pipes of this chip sustain when they do nothing else.
//
// A register-resident loop of v_mfma_f32_32x32x16_bf16 (16 per pass over eight A and eight B operand
// registers and four accumulators), eight waves per workgroup, two per SIMD like the forward attention
// kernel: no LDS, no memory traffic, no vector work.  The operands come from the caller, so that the same
// loop can be timed on constant and on random data: the clock the chip holds under this load, and with it
// the rate, depends on how much the multipliers' inputs toggle.
#include "common.h"

namespace moba {

__global__ __launch_bounds__(512, 2) void mfma_probe_kernel(const u32x4* __restrict__ operands, float* sink, int iters) {
  const int lane = threadIdx.x & 63;
  u32x4 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = operands[i * 64 + lane];
    b[i] = operands[(8 + i) * 64 + lane];
  }
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      acc[i & 3] = mfma32(__builtin_bit_cast(bf16x8, a[i & 7]), __builtin_bit_cast(bf16x8, b[(i + (i >> 3)) & 7]), acc[i & 3]);
    // (the operands are not loop constants to the compiler: the sixteen instructions stay sixteen)
#pragma unroll
    for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(a[i]), "+v"(b[i]));
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[j][e];
  if (s == 12345.678f) sink[0] = s;  // (keeps the loop alive; practically never true)
}

}  // namespace moba

using namespace moba;

// operands: 16 KiB of bf16 on the device (sixteen operand registers of 64 lanes x 16 bytes); sink: one float.
// Launches `workgroups` workgroups of eight waves (0: one per compute unit), each wave issuing iters * 16
// matrix instructions = iters * 16 * 32768 flops.  The caller times the launch on `stream`.
extern "C" int moba_mfma_probe(const void* operands, float* sink, int iters, int workgroups, void* stream) {
  LaunchCheck launch_check;
  if (!operands || !sink || iters <= 0 || workgroups < 0 || ((uintptr_t)operands & 15)) return MOBA_ERR_ARG;
  if (workgroups == 0) workgroups = compute_units();
  if (workgroups <= 0) return MOBA_ERR_LAUNCH;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream,
                     (const u32x4*)operands, sink, iters);
  return launch_check.result();
}
