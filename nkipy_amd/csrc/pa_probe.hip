// Matrix-core ceiling probe: v_mfma_f32_32x32x16_bf16 back to back from registers, no memory
// traffic at all, operands taken from a caller-supplied buffer.  What this loop reaches is
// what the chip sustains on the matrix cores at its power limit; it depends on the operand
// DATA (constant operands toggle few wires and run near the nominal clock, N(0,1) values
// measured about 30 % lower), so benchmarks quote it for the same data distribution as
// their inputs next to the nominal peak.
#include "pa_common.h"

namespace pa {
namespace {

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

}  // namespace

hipError_t launch_mfma_probe(const void* operands, void* sink, int blocks, int iters, hipStream_t s) {
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(blocks), dim3(512), 0, s, (const uint4*)operands, (float*)sink, iters);
  return hipGetLastError();
}

}  // namespace pa
