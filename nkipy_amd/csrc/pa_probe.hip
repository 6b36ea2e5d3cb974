// Matrix-core ceiling probe: v_mfma_f32_32x32x16_bf16 back to back from registers, no memory
// traffic at all, operands taken from a caller-supplied buffer.  What this loop reaches is
// what the chip sustains on the matrix cores at its power limit; it depends on the operand
// DATA (constant operands toggle few wires and run near the nominal clock, N(0,1) values
// measured about 30 % lower), so benchmarks quote it for the same data distribution as
// their inputs next to the nominal peak.
//
// Built into libpa_bench.so, a library of its own that only the benchmark loads: the
// product library exports nothing that exists for measurements alone.
#include "pa_common.h"

namespace pa {

__global__ __launch_bounds__(512) void mfma_probe_kernel(const uint4* operands, float* sink, int iters) {
  f32x16_t acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  bf16x8_t a[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) a[j] = __builtin_bit_cast(bf16x8_t, operands[((long)blockIdx.x * 512 + threadIdx.x) * 8 + j]);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j)
      acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j & 7], a[(j + 3) & 7], acc[j & 3], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[c][i];
  sink[(long)blockIdx.x * 512 + threadIdx.x] = s;
}

}  // namespace pa

// Runs `iters` x 16 back-to-back v_mfma_f32_32x32x16_bf16 per wavefront on `blocks` workgroups of 8
// wavefronts, operands taken once from `operands` (blocks * 65536 bytes of bf16 values, device memory),
// nothing else in the loop; `sink` receives blocks * 512 floats.  Synchronous; *ms is the kernel time.
// FLOP = blocks * 8 * iters * 16 * 32768.  Returns 0, -1 for bad arguments, or the hipError_t.
extern "C" int pa_bench_probe_mfma(const void* operands, void* sink, int blocks, int iters, float* ms, void* stream) {
  if (!operands || !sink || !ms || blocks <= 0 || iters <= 0 || ((uintptr_t)operands & 15u)) return -1;
  hipStream_t s = (hipStream_t)stream;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return (int)hipGetLastError();
  if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return (int)hipGetLastError(); }
  (void)hipEventRecord(e0, s);
  hipLaunchKernelGGL(pa::mfma_probe_kernel, dim3(blocks), dim3(512), 0, s, (const uint4*)operands, (float*)sink, iters);
  hipError_t e = hipGetLastError();
  (void)hipEventRecord(e1, s);
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  if (e == hipSuccess) e = hipEventElapsedTime(ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return (int)e;
}
