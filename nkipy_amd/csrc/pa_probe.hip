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


// ---- tile-loop probes -------------------------------------------------------------------------------------
// Stand-alone loops with the instruction mix of the tiled prefill kernel's key loop and none of its bookkeeping
// (no masks, tables or lengths): per 64-key tile and 256 query rows 256 v_mfma_f32_32x32x16_bf16, the K / V^T
// fragment reads from LDS, an exponential, a conversion and a row-sum term per score, the K / V tile copied
// HBM/L2 -> LDS into a ring of four stages, one barrier.  Two forms of the same work per workgroup and tile:
//   tile_loop_32rows_kernel: 8 waves x 32 query rows, two waves per SIMD, scores -> softmax -> PV in turn (the
//                            shipped kernel's structure);
//   tile_loop_64rows_kernel: 4 waves x 64 query rows, one wave per SIMD with the whole register file (512), every
//                            K and V^T fragment feeds two matrix instructions, software pipeline over units of
//                            32 keys x 32 rows: step(u) = matrix QK(u+1) + PV(u-1), vector softmax(u).
// Each workgroup stamps shader cycles (s_memtime) and wall time (s_memrealtime, 100 MHz) around its loop, so the
// benchmark reports cycles per tile and the clock the chip ran at.  `src` holds the operands (bf16 values).
typedef short probe_s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) char probe_lds_char;

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void tile_loop_64rows_kernel(float* out, long long* stamps, const char* src, int iters) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 131072 / 4; i += blockDim.x) ((uint32_t*)smem)[i] = ((const uint32_t*)src)[i + (blockIdx.x & 63) * 1024];
  __syncthreads();
  f32x16_t acc[2][4];
  for (int b = 0; b < 2; ++b) for (int c = 0; c < 4; ++c) for (int i = 0; i < 16; ++i) acc[b][c][i] = 0.f;
  bf16x8_t q[2][8];
  for (int b = 0; b < 2; ++b)
    for (int j = 0; j < 8; ++j) { uint4 av = *(const uint4*)(src + ((size_t)threadIdx.x * 16 + b * 8 + j) * 16 + (size_t)(blockIdx.x & 255) * 65536); q[b][j] = __builtin_bit_cast(bf16x8_t, av); }
  const int n = lane & 31, h = lane >> 5;
  int k_off[8], v_off[4];
  for (int s = 0; s < 8; ++s) k_off[s] = n * 256 + (((2 * s + h) ^ (n & 15)) << 4);
  { const int g = lane >> 4, sl = lane & 15; const int row = 4 * h + (sl >> 2); const int y = 2 * (g & 1) + ((sl & 3) >> 1);
    for (int c = 0; c < 4; ++c) v_off[c] = row * 256 + (((4 * c + y) ^ (4 * (row & 3))) << 4) + (sl & 1) * 8; }
  float l[2] = {0.f, 0.f}, m[2] = {0.f, 0.f};
  f32x16_t cinit[2];
  for (int b = 0; b < 2; ++b) for (int i = 0; i < 16; ++i) cinit[b][i] = 0.f;
  const uint32_t smem_base = (uint32_t)(uintptr_t)(probe_lds_char*)smem;
  const int rr = lane >> 4, pos = lane & 15;
  const char* gsrc = src + (size_t)((blockIdx.x >> 3) % 8) * (6144 * 2048) + (blockIdx.x & 7) * 256 + rr * 2048 + pos * 16;
  auto dma = [&](int tile, int st) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int u = wave * 8 + j;
      uint32_t dst = smem_base + st * 32768 + u * 1024;
      const char* a = gsrc + (size_t)((tile * 64) % 6144 + 4 * (u & 15)) * 2048 + (u >> 4) * (size_t)(8 * 6144 * 2048);
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(a), "s"(dst) : "memory", "m0");
    }
  };
  auto ldk = [&](int stage, int tt, int s) __attribute__((always_inline)) -> bf16x8_t {
    return *(const bf16x8_t*)(smem + stage * 32768 + tt * 8192 + k_off[s]);
  };
  auto ldv = [&](int stage, int g, int c) __attribute__((always_inline)) -> bf16x8_t {
    const probe_lds_char* sp = (const probe_lds_char*)(smem + stage * 32768 + 16384 + g * 4096 + v_off[c]);
    probe_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) probe_s16x4*)sp);
    probe_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) probe_s16x4*)(sp + 2048));
    struct { probe_s16x4 a, b; } pr = {lo, hi};
    return __builtin_bit_cast(bf16x8_t, pr);
  };
  constexpr float LIMIT = 0x1p+64f;

  // one pipeline step: VALU softmax of (Sc, qb_c) -> Pc; MFMA QK of the next unit (kf, qb_n) -> Sn; MFMA PV of the
  // previous unit (vf groups ga, ga+1 with Pp, qb_p)
  auto step = [&](f32x16_t& Sc, uint32_t (&Pc)[8], int qb_c, f32x16_t& Sn, const bf16x8_t (&kf)[8], int qb_n,
                  const uint32_t (&Pp)[8], const bf16x8_t (&vf)[2][4], int qb_p) __attribute__((always_inline)) {
    float psum = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      Sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s], q[qb_n][s], s == 0 ? cinit[qb_n] : Sn, 0, 0, 0);
      {
        const int i = 2 * s;
        const float e0 = __builtin_amdgcn_exp2f(Sc[i]), e1 = __builtin_amdgcn_exp2f(Sc[i + 1]);
        psum += e0 + e1;
        Pc[s] = pack_bf16x2(e0, e1);
      }
      {
        const int g = s >> 2, c = s & 3;
        uint4 pv = make_uint4(Pp[4 * g], Pp[4 * g + 1], Pp[4 * g + 2], Pp[4 * g + 3]);
        acc[qb_p][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[g][c], __builtin_bit_cast(bf16x8_t, pv), acc[qb_p][c], 0, 0, 0);
      }
    }
    // output accumulators and the scores' start values stay in the accumulation registers (without these pins the
    // compiler moves whole tiles between the two halves of the register file at every step)
#pragma unroll
    for (int c = 0; c < 4; ++c) asm volatile("" : "+a"(acc[qb_p][c]));
    asm volatile("" : "+a"(cinit[qb_n]));
    if (__builtin_amdgcn_ballot_w64(!(psum < LIMIT)) != 0) {
      m[qb_c] += 1.f; l[qb_c] *= 0.5f;
      const float nm = -m[qb_c];
      for (int i = 0; i < 16; ++i) asm volatile("v_accvgpr_write_b32 %0, %1" : "+a"(cinit[qb_c][i]) : "v"(nm));
    }
    l[qb_c] += psum;
  };

  dma(0, 0); dma(1, 1); dma(2, 2);
  asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  const long long c0 = clock64(), w0 = wall_clock64();

  f32x16_t S0, S1;                 // scores: unit being exponentiated / unit being formed (roles alternate)
  uint32_t Pa[8], Pb[8];
  bf16x8_t kf0[8], kf1[8];         // K fragments: sub-tile 0 (of the next tile) / sub-tile 1 (of this tile)
  bf16x8_t vfA[2][4], vfB[2][4];   // V^T fragments: key groups 0,1 / 2,3
  for (int i = 0; i < 8; ++i) { Pa[i] = 0; Pb[i] = 0; }
  // prologue: K sub-tile 0 of tile 0, scores of unit (0, qb 0); V fragments hold something
#pragma unroll
  for (int s = 0; s < 8; ++s) kf0[s] = ldk(0, 0, s);
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int c = 0; c < 4; ++c) { vfA[g][c] = ldv(0, g, c); vfB[g][c] = ldv(0, 2 + g, c); }
  S0 = cinit[0];
#pragma unroll
  for (int s = 0; s < 8; ++s) S0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf0[s], q[0][s], S0, 0, 0, 0);

  int stage = 0;
  for (int it = 0; it < iters; ++it) {
    const int sn = (stage + 1) & 3;
    // u0 = (tt0, qb0): softmax S0 -> Pa; QK (tt0, qb1) with kf0 -> S1; PV of (tt1, qb1) of the previous tile: vfB, Pb
    // loads during u0: kf1 (K sub-tile 1 of this tile), vfA (V groups 0,1 of this tile)
#pragma unroll
    for (int s = 0; s < 8; ++s) kf1[s] = ldk(stage, 1, s);
    step(S0, Pa, 0, S1, kf0, 1, Pb, vfB, 1);
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int c = 0; c < 4; ++c) vfA[g][c] = ldv(stage, g, c);
    // u1 = (tt0, qb1): softmax S1 -> Pb; QK (tt1, qb0) with kf1 -> S0; PV of (tt0, qb0): vfA, Pa
    step(S1, Pb, 1, S0, kf1, 0, Pa, vfA, 0);
    // tile boundary work: the next tile's copies have landed everywhere, the stage of the previous tile is free
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    dma(it + 3, (stage + 3) & 3);
    // u2 = (tt1, qb0): softmax S0 -> Pa; QK (tt1, qb1) with kf1 -> S1; PV of (tt0, qb1): vfA, Pb
    // loads during u2: kf0 (K sub-tile 0 of the next tile), vfB (V groups 2,3 of this tile)
#pragma unroll
    for (int s = 0; s < 8; ++s) kf0[s] = ldk(sn, 0, s);
    step(S0, Pa, 0, S1, kf1, 1, Pb, vfA, 1);
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int c = 0; c < 4; ++c) vfB[g][c] = ldv(stage, 2 + g, c);
    // u3 = (tt1, qb1): softmax S1 -> Pb; QK (tt0 of the next tile, qb0) with kf0 -> S0; PV of (tt1, qb0): vfB, Pa
    step(S1, Pb, 1, S0, kf0, 0, Pa, vfB, 0);
    stage = sn;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  const long long c1 = clock64(), w1 = wall_clock64();
  if (threadIdx.x == 0) { stamps[2 * blockIdx.x] = c1 - c0; stamps[2 * blockIdx.x + 1] = w1 - w0; }
  float s = l[0] + l[1] + m[0] + m[1] + S0[0] + S1[1];
  for (int b = 0; b < 2; ++b) for (int c = 0; c < 4; ++c) for (int i = 0; i < 16; i++) s += acc[b][c][i];
  out[(long)blockIdx.x * blockDim.x + threadIdx.x] = s;
}


__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void tile_loop_32rows_kernel(float* out, long long* stamps, const char* src, int iters) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 131072 / 4; i += blockDim.x) ((uint32_t*)smem)[i] = ((const uint32_t*)src)[i + (blockIdx.x & 63) * 1024];
  __syncthreads();
  f32x16_t acc[4];
  for (int c = 0; c < 4; ++c) for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  bf16x8_t q[8];
  for (int j = 0; j < 8; ++j) { uint4 av = *(const uint4*)(src + ((size_t)threadIdx.x * 8 + j) * 16 + (size_t)(blockIdx.x & 255) * 65536); q[j] = __builtin_bit_cast(bf16x8_t, av); }
  const int n = lane & 31, h = lane >> 5;
  int k_off[8], v_off[4];
  for (int s = 0; s < 8; ++s) k_off[s] = n * 256 + (((2 * s + h) ^ (n & 15)) << 4);
  { const int g = lane >> 4, sl = lane & 15; const int row = 4 * h + (sl >> 2); const int y = 2 * (g & 1) + ((sl & 3) >> 1);
    for (int c = 0; c < 4; ++c) v_off[c] = row * 256 + (((4 * c + y) ^ (4 * (row & 3))) << 4) + (sl & 1) * 8; }
  float l = 0.f, m = 0.f;
  f32x16_t cinit;
  for (int i = 0; i < 16; ++i) cinit[i] = 0.f;
  const uint32_t smem_base = (uint32_t)(uintptr_t)(probe_lds_char*)smem;
  const int rr = lane >> 4, pos = lane & 15;
  const char* gsrc = src + (size_t)((blockIdx.x >> 3) % 8) * (6144 * 2048) + (blockIdx.x & 7) * 256 + rr * 2048 + pos * 16;
  auto dma = [&](int tile, int st) __attribute__((always_inline)) {
    for (int j = 0; j < 4; ++j) {
      uint32_t dst = smem_base + st * 32768 + (wave * 4 + j) * 1024;
      const char* a = gsrc + (size_t)((tile * 64) % 6144 + 4 * ((wave * 4 + j) & 15)) * 2048 + ((wave * 4 + j) >> 4) * (size_t)(8 * 6144 * 2048);
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(a), "s"(dst) : "memory", "m0");
    }
  };
  auto ldk = [&](int stage, int tt, int s) __attribute__((always_inline)) -> bf16x8_t {
    return *(const bf16x8_t*)(smem + stage * 32768 + tt * 8192 + k_off[s]);
  };
  auto ldv = [&](int stage, int g, int c) __attribute__((always_inline)) -> bf16x8_t {
    const probe_lds_char* sp = (const probe_lds_char*)(smem + stage * 32768 + 16384 + g * 4096 + v_off[c]);
    probe_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) probe_s16x4*)sp);
    probe_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) probe_s16x4*)(sp + 2048));
    struct { probe_s16x4 a, b; } pr = {lo, hi};
    return __builtin_bit_cast(bf16x8_t, pr);
  };
  for (int st = 0; st < 3; ++st) dma(st, st);
  const long long c0 = clock64(), w0 = wall_clock64();
  constexpr float LIMIT = 0x1p+64f;
  int stage = 0;
  for (int it = 0; it < iters; ++it) {
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    dma(it + 3, (stage + 3) & 3);
    f32x16_t S[2];
    uint32_t pw[16];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      bf16x8_t kf[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) kf[s] = ldk(stage, tt, s);
      S[tt] = cinit;
#pragma unroll
      for (int s = 0; s < 8; ++s) S[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s], q[s], S[tt], 0, 0, 0);
    }
    float psum = 0.f;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        float e0 = __builtin_amdgcn_exp2f(S[tt][i]), e1 = __builtin_amdgcn_exp2f(S[tt][i + 1]);
        psum += e0 + e1;
        pw[8 * tt + i / 2] = pack_bf16x2(e0, e1);
      }
    if (__builtin_amdgcn_ballot_w64(!(psum < LIMIT)) != 0) {
      m += 1.f; l *= 0.5f;
      for (int c = 0; c < 4; ++c) acc[c] *= 0.5f;
      for (int i = 0; i < 16; ++i) cinit[i] = -m;
    }
    l += psum;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x8_t vf[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) vf[c] = ldv(stage, g, c);
      uint4 pv = make_uint4(pw[4 * g], pw[4 * g + 1], pw[4 * g + 2], pw[4 * g + 3]);
      bf16x8_t pf = __builtin_bit_cast(bf16x8_t, pv);
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[c], pf, acc[c], 0, 0, 0);
    }
    stage = (stage + 1) & 3;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  const long long c1 = clock64(), w1 = wall_clock64();
  if (threadIdx.x == 0) { stamps[2 * blockIdx.x] = c1 - c0; stamps[2 * blockIdx.x + 1] = w1 - w0; }
  float s = l + m;
  for (int c = 0; c < 4; ++c) for (int i = 0; i < 16; i++) s += acc[c][i];
  out[(long)blockIdx.x * blockDim.x + threadIdx.x] = s;
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

// form 0: 8 waves x 32 rows; form 1: 4 waves x 64 rows.  src: at least 2 * 8 * 6144 * 2048 + 2^20 bytes of bf16 values;
// sink: blocks * 512 floats; stamps: blocks * 2 int64 (shader cycles, 100 MHz ticks per workgroup).  Synchronous; *ms is
// the kernel time.  FLOP = blocks * iters * 256 * 32768.  Returns 0, -1 for bad arguments, or the hipError_t.
extern "C" int pa_bench_probe_tile_loop(int form, const void* src, void* sink, void* stamps, int blocks, int iters, float* ms, void* stream) {
  if (!src || !sink || !stamps || !ms || blocks <= 0 || iters <= 0 || (form != 0 && form != 1) || ((uintptr_t)src & 15u)) return -1;
  hipStream_t s = (hipStream_t)stream;
  constexpr int lds = 131072;
  hipError_t e = form == 0 ? hipFuncSetAttribute((const void*)pa::tile_loop_32rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds)
                           : hipFuncSetAttribute((const void*)pa::tile_loop_64rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return (int)e;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return (int)hipGetLastError();
  if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return (int)hipGetLastError(); }
  (void)hipEventRecord(e0, s);
  if (form == 0) hipLaunchKernelGGL(pa::tile_loop_32rows_kernel, dim3(blocks), dim3(512), lds, s, (float*)sink, (long long*)stamps, (const char*)src, iters);
  else hipLaunchKernelGGL(pa::tile_loop_64rows_kernel, dim3(blocks), dim3(256), lds, s, (float*)sink, (long long*)stamps, (const char*)src, iters);
  e = hipGetLastError();
  (void)hipEventRecord(e1, s);
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  if (e == hipSuccess) e = hipEventElapsedTime(ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return (int)e;
}
