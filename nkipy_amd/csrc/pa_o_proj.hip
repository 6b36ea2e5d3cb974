// Post-attention output projection on the gfx950 matrix cores:
//   out[m, :] = x[m, :] @ w (+ bias),   x [M, K] = the attention output viewed as [tokens, Hq * D],
//   w [K, N] row-major (the reference stores o_proj.weight transposed: examples/models/qwen3/
//   tensor_preparation.py:148-156), bias [N] (examples/models/gpt_oss/kernels/attention.py:155-163).
// Reference lines: examples/models/qwen3/kernels/attention.py:143-147.  bf16 in, float32 accumulate,
// one rounding to bf16 on the way out.
//
// One workgroup of 8 wavefronts owns a 256 x 256 tile of out; wavefront (wm, wn) owns rows
// 64 wm .. +63 and columns 128 wn .. +127 of it (two 32-row blocks x four 32-column chunks = eight
// 32 x 32 accumulators).  K is walked in steps of 64.  The product is formed transposed,
// out^T[n, m] += w^T[n, k] x^T[k, m] on v_mfma_f32_32x32x16_bf16: the A operand (w^T, 32 n x 16 k)
// comes from the w tile, stored row-major [k][n] exactly as in memory, through the transposing LDS
// read ds_read_b64_tr_b16; the B operand (x^T, 16 k x 32 m) is a plain 16-byte read of a row of the
// x tile.  A lane's accumulator column is one row m of out, as in the attention kernels, so the
// store path is theirs too.
//
// Both tiles travel HBM/L2 -> LDS with global_load_lds_dwordx4 (no registers) into a ring of two
// 64 KB stages: the copies of k-step j + 1 are in flight while step j is multiplied.
//   stage = x tile [256 m][128 B]  +  w tile, columns 0-127 [64 k][256 B]  +  w tile, columns 128-255
// 16-byte chunk g of x row r sits at position g ^ ((r >> 1) & 7) (two 128-byte rows fill the 64 banks once,
// so sixteen consecutive rows must land on sixteen different 16-byte slots); chunk g of w row r at g ^ 4 (r & 3): the
// reads of both kinds then spread over the banks (the copy lane fetches whatever chunk belongs in
// its fixed LDS slot, so the swizzle costs nothing).
#include <atomic>

#include "pa_common.h"

namespace pa {
namespace {

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) char lds_char;

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int XT_B = BM * BK * 2;          // x tile bytes (32 KB)
constexpr int WH_B = BK * 128 * 2;         // half a w tile: 64 k x 128 n (16 KB)
constexpr int STAGE_B = XT_B + 2 * WH_B;   // 64 KB
constexpr int LDS_B = 2 * STAGE_B;

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// lane i's 16 bytes land at lds_base + 16 i; issued as inline assembly so that the waits are placed by hand
__device__ __forceinline__ void dma16(const char* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(lane_off), "s"(base), "s"(lds_base) : "memory", "m0");
}

template <bool BIAS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void o_proj_kernel(OProjParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int wm = wave & 3, wn = wave >> 2;

  // tile of this workgroup: consecutive workgroup ids go to consecutive XCDs; an XCD owns row tiles xcd,
  // xcd + 8, ... and walks its tiles in groups of (all its row tiles) x (4 column tiles), so that the
  // workgroups resident on it at one time (32 on MI355X) share x slabs four ways and w slabs eight ways
  // through that XCD's L2 instead of streaming all of w once per pair of row tiles
  const int MT = (p.M + BM - 1) / BM, NT = (p.N + BN - 1) / BN;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int mtx = (MT + 7) / 8;                       // row tiles per XCD (the last ones may not exist)
  const int grp = slot / (4 * mtx), rem = slot % (4 * mtx);
  const int mt = xcd + 8 * (rem >> 2), nt = 4 * grp + (rem & 3);
  if (mt >= MT || nt >= NT) return;
  const int m0 = mt * BM, n0 = nt * BN;

  // ---- copy maps ---------------------------------------------------------------------------------
  // x tile: 32 units of 1 KB = 8 rows x 128 B; lane i fills (row 8u + i/8, position i%8) with chunk
  // (i%8) ^ ((row >> 1) & 7).  w half tile: 16 units of 4 rows x 256 B; lane i fills (row 4u + i/16, position
  // i%16) with chunk (i%16) ^ 4 (row & 3).  Wave w issues x units w, w+8, w+16, w+24 and w units w,
  // w+8 of both halves.  Rows past M and columns past N are clamped to the last valid ones (their
  // products are never stored).
  const uint32_t smem_base = (uint32_t)(uintptr_t)(lds_char*)smem;
  const long x_row_b = (long)p.K * 2, w_row_b = (long)p.N * 2;
  uint32_t xoff[4], woff[2][2];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = min(8 * (wave + 8 * j) + (lane >> 3), p.M - 1 - m0);
    const int lrow = 8 * (wave + 8 * j) + (lane >> 3);          // row of the tile this lane's LDS slot belongs to
    xoff[j] = (uint32_t)(r * x_row_b) + (uint32_t)(((lane & 7) ^ ((lrow >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int r = 4 * (wave + 8 * j) + (lane >> 4);
      const int chunk = (lane & 15) ^ (4 * ((lane >> 4) & 3));
      const int col = min(n0 + 128 * hf + 8 * chunk, p.N - 8);
      woff[hf][j] = (uint32_t)(r * w_row_b) + (uint32_t)(col * 2);
    }
  const char* xbase = (const char*)p.x + (long)m0 * x_row_b;      // advanced by 128 B per k-step
  const char* wbase = (const char*)p.w;                           // advanced by 64 rows per k-step
  auto request = [&](int stage) __attribute__((always_inline)) {
    const uint32_t sb = smem_base + stage * STAGE_B;
#pragma unroll
    for (int j = 0; j < 4; ++j) dma16(xbase, xoff[j], sb + (wave + 8 * j) * 1024);
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int j = 0; j < 2; ++j) dma16(wbase, woff[hf][j], sb + XT_B + hf * WH_B + (wave + 8 * j) * 1024);
    xbase += BK * 2;
    wbase += (long)BK * w_row_b;
  };

  // ---- fragment read maps (lane constants) ---------------------------------------------------------
  int x_off[4];                       // x^T fragment of k16-step s: row n of a 32-row block, chunk 2s + h
#pragma unroll
  for (int s = 0; s < 4; ++s) x_off[s] = (64 * wm + n) * 128 + (((2 * s + h) ^ ((n >> 1) & 7)) << 4);
  // w^T fragment of 32-column chunk c.  ds_read_b64_tr_b16, per group of 16 lanes: lane i receives, for
  // j = 0..3, the (i%4)-th 16-bit element of the 8 bytes addressed by lane (i/4) + 4j.  Source lane sl
  // therefore points at k row (sl/4) of its half-wave's eight rows (8h .. 8h+3 for the first read, 4 rows
  // further for the second: k-slot 8h + j of the operand is k row 8h + j, the same order as the x^T
  // fragment) and at columns 4 (sl%4) .. +3 of the group's 16-column window.
  int w_off[4];
  {
    const int g = lane >> 4, sl = lane & 15;
    const int row = 8 * h + (sl >> 2);
    const int y = 2 * (g & 1) + ((sl & 3) >> 1);
#pragma unroll
    for (int c = 0; c < 4; ++c) w_off[c] = XT_B + wn * WH_B + row * 256 + (((4 * c + y) ^ (4 * (row & 3))) << 4) + (sl & 1) * 8;
  }

  f32x16_t acc[2][4];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][c][i] = 0.f;

  auto load_x = [&](bf16x8_t (&xf)[2], int stage, int s) __attribute__((always_inline)) {
    const char* b = smem + stage * STAGE_B + x_off[s];
    xf[0] = *(const bf16x8_t*)b;
    xf[1] = *(const bf16x8_t*)(b + 32 * 128);
  };
  auto load_w = [&](bf16x8_t (&wf)[4], int stage, int s) __attribute__((always_inline)) {
    const char* b = smem + stage * STAGE_B + 16 * s * 256;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const lds_char* src = (const lds_char*)(b + w_off[c]);
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)src);
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(src + 4 * 256));
      struct { s16x4_t a, b; } pair = {lo, hi};
      wf[c] = __builtin_bit_cast(bf16x8_t, pair);
    }
  };
  auto mma = [&](const bf16x8_t (&wf)[4], const bf16x8_t (&xf)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        acc[mb][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[c], xf[mb], acc[mb][c], 0, 0, 0);
  };

  // The loop is rotated by one k16-step: the products of a k-step's last k16-step are issued behind the barrier
  // that opens the next k-step, between that step's copy requests, so that the matrix pipeline has work while
  // the requests and the first fragment reads of the new stage are issued.
  auto request_part = [&](int stage, int part) __attribute__((always_inline)) {     // a quarter of request()
    const uint32_t sb = smem_base + stage * STAGE_B;
    dma16(xbase, xoff[part], sb + (wave + 8 * part) * 1024);
    dma16(wbase, woff[part >> 1][part & 1], sb + XT_B + (part >> 1) * WH_B + (wave + 8 * (part & 1)) * 1024);
  };
  const int ktiles = p.K / BK;
  bf16x8_t wa[4], wb[4], xa[2], xb[2];
  request(0);
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  if (ktiles > 1) request(1);
  load_w(wa, 0, 0); load_x(xa, 0, 0);
  for (int kt = 0; kt + 1 < ktiles; ++kt) {
    const int stage = kt & 1;
    load_w(wb, stage, 1); load_x(xb, stage, 1);
    mma(wa, xa);
    load_w(wa, stage, 2); load_x(xa, stage, 2);
    mma(wb, xb);
    load_w(wb, stage, 3); load_x(xb, stage, 3);
    mma(wa, xa);
    wait_vmcnt<0>();                       // this wave's part of step kt + 1 has landed
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // ... and its reads of this stage are done
    __builtin_amdgcn_s_barrier();          // everyone's; the stage of step kt is free
    load_w(wa, stage ^ 1, 0); load_x(xa, stage ^ 1, 0);
    const bool more = kt + 2 < ktiles;
#define OPROJ_TAIL_PART(part, mb)                                                                              \
    __builtin_amdgcn_sched_barrier(0);                                                                         \
    acc[mb][2 * ((part) & 1)] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[2 * ((part) & 1)], xb[mb], acc[mb][2 * ((part) & 1)], 0, 0, 0);             \
    acc[mb][2 * ((part) & 1) + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[2 * ((part) & 1) + 1], xb[mb], acc[mb][2 * ((part) & 1) + 1], 0, 0, 0); \
    __builtin_amdgcn_sched_barrier(0);                                                                         \
    if (more) request_part(stage, part);
    OPROJ_TAIL_PART(0, 0)
    OPROJ_TAIL_PART(1, 0)
    OPROJ_TAIL_PART(2, 1)
    OPROJ_TAIL_PART(3, 1)
#undef OPROJ_TAIL_PART
    xbase += BK * 2;
    wbase += (long)BK * w_row_b;
  }
  {
    const int stage = (ktiles - 1) & 1;
    load_w(wb, stage, 1); load_x(xb, stage, 1);
    mma(wa, xa);
    load_w(wa, stage, 2); load_x(xa, stage, 2);
    mma(wb, xb);
    load_w(wb, stage, 3); load_x(xb, stage, 3);
    mma(wa, xa);
    mma(wb, xb);
  }

  // ---- bias, rounding, store: rows go out through a wave-private patch of the (now idle) ring so that
  // they leave as whole 256-byte pieces, 16 bytes a lane --------------------------------------------------
  __builtin_amdgcn_s_barrier();            // every wave is done reading the ring
  uint16_t* out = (uint16_t*)p.out;
  constexpr int PROW_B = 256 + 8;          // patch row pitch: the 8 bytes spread a column of rows over the banks
  char* patch = smem + wave * (32 * PROW_B);
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int col = 32 * c + 8 * i4 + 4 * h;           // column inside the wave's 128
        float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
        if (BIAS) {
          const int gc = min(n0 + 128 * wn + col, p.N - 4);
          const uint2 bw = *(const uint2*)((const uint16_t*)p.bias + gc);
          b0 = bf16_bits_to_float(bw.x & 0xffffu); b1 = bf16_bits_to_float(bw.x >> 16);
          b2 = bf16_bits_to_float(bw.y & 0xffffu); b3 = bf16_bits_to_float(bw.y >> 16);
        }
        const uint32_t w0 = pack_bf16x2(acc[mb][c][4 * i4] + b0, acc[mb][c][4 * i4 + 1] + b1);
        const uint32_t w1 = pack_bf16x2(acc[mb][c][4 * i4 + 2] + b2, acc[mb][c][4 * i4 + 3] + b3);
        *(uint2*)(patch + n * PROW_B + 2 * col) = make_uint2(w0, w1);
      }
    // the wave reads back what its own lanes wrote: no barrier, the compiler orders the LDS accesses
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = 4 * j + (lane >> 4), ch = lane & 15;
      const uint2 lo = *(const uint2*)(patch + r * PROW_B + 16 * ch), hi = *(const uint2*)(patch + r * PROW_B + 16 * ch + 8);
      const int m = m0 + 64 * wm + 32 * mb + r, col = n0 + 128 * wn + 8 * ch;
      if (m < p.M && col < p.N) store_stream(out + (long)m * p.N + col, make_uint4(lo.x, lo.y, hi.x, hi.y));
    }
  }
}

// Between the two: a few hundred to a few thousand rows (a prefill chunk of a small batch) give fewer 256 x 256 tiles
// than the device has CUs.  Same product, operand layouts and copy scheme on 128 x 128 tiles: a workgroup of 4
// wavefronts, wavefront (wm, wn) owning rows 64 wm .. +63 and columns 64 wn .. +63 (two 32-row blocks x two
// 32-column chunks), stages of 32 KB (x tile [128 m][128 B] + w tile [64 k][256 B]), two workgroups per CU.
constexpr int MBM = 128, MBN = 128;
constexpr int MXT_B = MBM * BK * 2;        // 16 KB
constexpr int MWT_B = BK * MBN * 2;        // 16 KB
constexpr int MSTAGE_B = MXT_B + MWT_B;

// MNST: ring stages.  2 (64 KB: two workgroups per CU) when there are more tiles than CUs; 4 (128 KB, copies three
// k-steps ahead) when every CU holds at most one workgroup anyway and nothing else hides the copies' latency.
template <bool BIAS, int MNST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void o_proj_mid_kernel(OProjParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int wm = wave & 1, wn = wave >> 1;

  // tile order as in the large form: an XCD owns row tiles xcd, xcd + 8, ... and walks them in groups of 4 column tiles
  const int MT = (p.M + MBM - 1) / MBM, NT = (p.N + MBN - 1) / MBN;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int mtx = (MT + 7) / 8;
  const int grp = slot / (4 * mtx), rem = slot % (4 * mtx);
  const int mt = xcd + 8 * (rem >> 2), nt = 4 * grp + (rem & 3);
  if (mt >= MT || nt >= NT) return;
  const int m0 = mt * MBM, n0 = nt * MBN;

  // copy maps: x tile = 16 units of 8 rows x 128 B, w tile = 16 units of 4 rows x 256 B; wave w issues units w, w + 4,
  // w + 8, w + 12 of each; swizzles as in the large form
  const uint32_t smem_base = (uint32_t)(uintptr_t)(lds_char*)smem;
  const long x_row_b = (long)p.K * 2, w_row_b = (long)p.N * 2;
  uint32_t xoff[4], woff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int lrow = 8 * (wave + 4 * j) + (lane >> 3);
    const int r = min(lrow, p.M - 1 - m0);
    xoff[j] = (uint32_t)(r * x_row_b) + (uint32_t)(((lane & 7) ^ ((lrow >> 1) & 7)) << 4);
    const int wr = 4 * (wave + 4 * j) + (lane >> 4);
    const int chunk = (lane & 15) ^ (4 * ((lane >> 4) & 3));
    const int col = min(n0 + 8 * chunk, p.N - 8);
    woff[j] = (uint32_t)(wr * w_row_b) + (uint32_t)(col * 2);
  }
  const char* xbase = (const char*)p.x + (long)m0 * x_row_b;
  const char* wbase = (const char*)p.w;
  const int ktiles = p.K / BK;
  int kt_req = 0, stage_req = 0;
  auto request = [&]() __attribute__((always_inline)) {
    // (requests past the end repeat the last step into a stage nobody reads any more: the wait counts stay exact)
    const uint32_t sb = smem_base + stage_req * MSTAGE_B;
#pragma unroll
    for (int j = 0; j < 4; ++j) dma16(xbase, xoff[j], sb + (wave + 4 * j) * 1024);
#pragma unroll
    for (int j = 0; j < 4; ++j) dma16(wbase, woff[j], sb + MXT_B + (wave + 4 * j) * 1024);
    if (++kt_req < ktiles) {
      xbase += BK * 2;
      wbase += (long)BK * w_row_b;
    }
    stage_req = stage_req + 1 == MNST ? 0 : stage_req + 1;
  };

  int x_off[4], w_off[2];
#pragma unroll
  for (int s = 0; s < 4; ++s) x_off[s] = (64 * wm + n) * 128 + (((2 * s + h) ^ ((n >> 1) & 7)) << 4);
  {
    const int g = lane >> 4, sl = lane & 15;
    const int row = 8 * h + (sl >> 2);
    const int y = 2 * (g & 1) + ((sl & 3) >> 1);
#pragma unroll
    for (int c = 0; c < 2; ++c) w_off[c] = MXT_B + row * 256 + (((4 * (2 * wn + c) + y) ^ (4 * (row & 3))) << 4) + (sl & 1) * 8;
  }

  f32x16_t acc[2][2];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][c][i] = 0.f;

  auto load_x = [&](bf16x8_t (&xf)[2], int stage, int s) __attribute__((always_inline)) {
    const char* b = smem + stage * MSTAGE_B + x_off[s];
    xf[0] = *(const bf16x8_t*)b;
    xf[1] = *(const bf16x8_t*)(b + 32 * 128);
  };
  auto load_w = [&](bf16x8_t (&wf)[2], int stage, int s) __attribute__((always_inline)) {
    const char* b = smem + stage * MSTAGE_B + 16 * s * 256;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const lds_char* src = (const lds_char*)(b + w_off[c]);
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)src);
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(src + 4 * 256));
      struct { s16x4_t a, b; } pair = {lo, hi};
      wf[c] = __builtin_bit_cast(bf16x8_t, pair);
    }
  };
  auto mma = [&](const bf16x8_t (&wf)[2], const bf16x8_t (&xf)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int c = 0; c < 2; ++c)
        acc[mb][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[c], xf[mb], acc[mb][c], 0, 0, 0);
  };

#pragma unroll
  for (int s = 0; s < MNST - 1; ++s) request();
  int stage = 0;
  for (int kt = 0; kt < ktiles; ++kt) {
    wait_vmcnt<(MNST - 2) * 8>();          // this wave's part of step kt has landed (8 copies per wave and step)
    __builtin_amdgcn_s_barrier();          // ... and everyone's; all waves are done with step kt - 1
    request();
    bf16x8_t wa[2], wb[2], xa[2], xb[2];
    load_w(wa, stage, 0); load_x(xa, stage, 0);
    load_w(wb, stage, 1); load_x(xb, stage, 1);
    mma(wa, xa);
    load_w(wa, stage, 2); load_x(xa, stage, 2);
    mma(wb, xb);
    load_w(wb, stage, 3); load_x(xb, stage, 3);
    mma(wa, xa);
    mma(wb, xb);
    stage = stage + 1 == MNST ? 0 : stage + 1;
  }
  wait_vmcnt<0>();                         // nothing may still be landing in LDS

  __builtin_amdgcn_s_barrier();            // every wave is done reading the ring
  uint16_t* out = (uint16_t*)p.out;
  constexpr int PROW_B = 128 + 8;
  char* patch = smem + wave * (32 * PROW_B);
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int col = 32 * c + 8 * i4 + 4 * h;           // column inside the wave's 64
        float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
        if (BIAS) {
          const int gc = min(n0 + 64 * wn + col, p.N - 4);
          const uint2 bw = *(const uint2*)((const uint16_t*)p.bias + gc);
          b0 = bf16_bits_to_float(bw.x & 0xffffu); b1 = bf16_bits_to_float(bw.x >> 16);
          b2 = bf16_bits_to_float(bw.y & 0xffffu); b3 = bf16_bits_to_float(bw.y >> 16);
        }
        const uint32_t w0 = pack_bf16x2(acc[mb][c][4 * i4] + b0, acc[mb][c][4 * i4 + 1] + b1);
        const uint32_t w1 = pack_bf16x2(acc[mb][c][4 * i4 + 2] + b2, acc[mb][c][4 * i4 + 3] + b3);
        *(uint2*)(patch + n * PROW_B + 2 * col) = make_uint2(w0, w1);
      }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = 8 * j + (lane >> 3), ch = lane & 7;
      const uint2 lo = *(const uint2*)(patch + r * PROW_B + 16 * ch), hi = *(const uint2*)(patch + r * PROW_B + 16 * ch + 8);
      const int m = m0 + 64 * wm + 32 * mb + r, col = n0 + 64 * wn + 8 * ch;
      if (m < p.M && col < p.N) store_stream(out + (long)m * p.N + col, make_uint4(lo.x, lo.y, hi.x, hi.y));
    }
  }
}

// Few rows (decode: M = batch, or a verify step): the work is w's bytes, once.  One workgroup of 4 waves per
// 64 output columns owns ALL rows (BM = 32 MBT of them) and streams its 128-byte-wide column slab of w through
// a deep ring of small stages (K step 64: w tile [64 k][128 B] + x tile [BM][128 B]), so that N / 64
// workgroups keep the memory system busy instead of N / 256.  Same operand layouts and product as above; wave w
// takes the 32-column block w & 1 and the 32-row blocks of parity w >> 1.
template <int MBT, bool BIAS>
__global__ __launch_bounds__(256) void o_proj_skinny_kernel(OProjParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int SBM = 32 * MBT;
  constexpr int SX_B = SBM * 128, SW_B = 64 * 128, SSTAGE_B = SX_B + SW_B;
  constexpr int NST = MBT == 2 ? 8 : (MBT == 4 ? 5 : 3);
  constexpr int XU = SBM / 8, UPW = (XU + 8) / 4;       // 1 KB copy units of the x tile; copy instructions per wave and stage
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int nb = wave & 1, mpar = wave >> 1;
  const int n0 = blockIdx.x * 64;
  const int m0 = blockIdx.y * SBM;         // (more rows than one workgroup owns: a second grid dimension of row blocks)

  const uint32_t smem_base = (uint32_t)(uintptr_t)(lds_char*)smem;
  const long x_row_b = (long)p.K * 2, w_row_b = (long)p.N * 2;
  // copy maps: units of 8 rows x 128 B for both tiles; lane i fills (row 8u + i/8, position i%8).  x chunk g of
  // row r sits at g ^ ((r >> 1) & 7), w chunk g of row r at g ^ 4 ((r >> 1) & 1) (two 128-byte rows per bank cycle)
  uint32_t xoff[XU / 4], woff[2];
#pragma unroll
  for (int j = 0; j < XU / 4; ++j) {
    const int lrow = 8 * (wave + 4 * j) + (lane >> 3);
    xoff[j] = (uint32_t)(min(m0 + lrow, p.M - 1) * x_row_b) + (uint32_t)(((lane & 7) ^ ((lrow >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int lrow = 8 * (wave + 4 * j) + (lane >> 3);
    const int chunk = (lane & 7) ^ (4 * ((lrow >> 1) & 1));
    woff[j] = (uint32_t)(lrow * w_row_b) + (uint32_t)(min(n0 + 8 * chunk, p.N - 8) * 2);
  }
  // split form: the workgroups of a column slab along the third grid dimension take equal ranges of K and leave
  // float32 partial tiles for o_proj_split_reduce_kernel (few rows: N / 64 workgroups alone leave most CUs idle)
  const int kt_total = p.K / BK;
  const int kt_begin = (int)((long)kt_total * blockIdx.z / gridDim.z);
  const int ktiles = (int)((long)kt_total * (blockIdx.z + 1) / gridDim.z) - kt_begin;
  int kt_req = 0, stage_req = 0;
  auto request = [&]() __attribute__((always_inline)) {
    // requests past the end repeat the first step (into a stage nobody reads any more): the wait counts stay exact
    const int kt = kt_begin + (kt_req < ktiles ? kt_req : 0);
    const char* xb = (const char*)p.x + (long)kt * (BK * 2);
    const char* wb = (const char*)p.w + (long)kt * BK * w_row_b;
    const uint32_t sb = smem_base + stage_req * SSTAGE_B;
#pragma unroll
    for (int j = 0; j < XU / 4; ++j) dma16(xb, xoff[j], sb + (wave + 4 * j) * 1024);
#pragma unroll
    for (int j = 0; j < 2; ++j) dma16(wb, woff[j], sb + SX_B + (wave + 4 * j) * 1024);
    ++kt_req;
    stage_req = stage_req + 1 == NST ? 0 : stage_req + 1;
  };

  int x_off[4], w_off;
#pragma unroll
  for (int s = 0; s < 4; ++s) x_off[s] = n * 128 + (((2 * s + h) ^ ((n >> 1) & 7)) << 4);
  {
    const int g = lane >> 4, sl = lane & 15;
    const int row = 8 * h + (sl >> 2);
    const int y = 2 * (g & 1) + ((sl & 3) >> 1);
    w_off = SX_B + row * 128 + (((4 * nb + y) ^ (4 * ((row >> 1) & 1))) << 4) + (sl & 1) * 8;
  }
  f32x16_t acc[MBT / 2];
#pragma unroll
  for (int i = 0; i < MBT / 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;

#pragma unroll
  for (int s = 0; s < NST - 1; ++s) request();
  int stage = 0;
  for (int kt = 0; kt < ktiles; ++kt) {
    wait_vmcnt<(NST - 2) * UPW>();
    __builtin_amdgcn_s_barrier();
    request();
    const char* sb = smem + stage * SSTAGE_B;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const lds_char* src = (const lds_char*)(sb + 16 * s * 128 + w_off);
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)src);
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(src + 4 * 128));
      struct { s16x4_t a, b; } pair = {lo, hi};
      const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, pair);
#pragma unroll
      for (int i = 0; i < MBT / 2; ++i) {
        const bf16x8_t xf = *(const bf16x8_t*)(sb + (2 * i + mpar) * (32 * 128) + x_off[s]);
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf, acc[i], 0, 0, 0);
      }
    }
    stage = stage + 1 == NST ? 0 : stage + 1;
  }
  wait_vmcnt<0>();     // nothing may still be landing in LDS when the workgroup retires

  // a lane holds, for its row, 4 consecutive columns at 4 places: 8-byte stores (the output is small here)
  uint16_t* out = (uint16_t*)p.out;
#pragma unroll
  for (int i = 0; i < MBT / 2; ++i) {
    const int m = m0 + 32 * (2 * i + mpar) + n;
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int col = n0 + 32 * nb + 8 * i4 + 4 * h;
      float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
      if (BIAS) {
        const uint2 bw = *(const uint2*)((const uint16_t*)p.bias + min(col, p.N - 4));
        b0 = bf16_bits_to_float(bw.x & 0xffffu); b1 = bf16_bits_to_float(bw.x >> 16);
        b2 = bf16_bits_to_float(bw.y & 0xffffu); b3 = bf16_bits_to_float(bw.y >> 16);
      }
      if (m < p.M && col < p.N) {
        if (p.splits > 1)
          *(float4*)(p.ws + ((long)blockIdx.z * p.M + m) * p.N + col) =
              make_float4(acc[i][4 * i4], acc[i][4 * i4 + 1], acc[i][4 * i4 + 2], acc[i][4 * i4 + 3]);
        else
          *(uint2*)(out + (long)m * p.N + col) = make_uint2(pack_bf16x2(acc[i][4 * i4] + b0, acc[i][4 * i4 + 1] + b1),
                                                             pack_bf16x2(acc[i][4 * i4 + 2] + b2, acc[i][4 * i4 + 3] + b3));
      }
    }
  }
}

// Very few rows (M <= 32: a decode step of a small batch, a verify step of one sequence).  The call is w's bytes
// and a handful of latencies, so nothing is recycled: a workgroup of 4 waves owns 128 output columns and a range
// of at most 8 k-steps of 64, requests ALL of its operands at once -- per k-step the x tile [32 rows][128 B] and the
// w tile [64 k][256 B], 20 KB, up to 160 KB -- and multiplies as the steps land: one memory round trip for the whole
// workgroup instead of a ring that is filled, drained and refilled (the ring form spends a third of its life filling,
// and copies 64 x rows where 8 are live).  (N / 128) x (K / 512) workgroups: 256 at K = N = 4096.  Wave w takes
// the 32-column chunk w; operand layouts, swizzles and the product are those of the kernels above.  The K ranges
// leave float32 partial tiles for o_proj_split_reduce_kernel (one range: bf16 output and bias directly).
constexpr int RS_X = 32 * 128, RS_W = 64 * 256, RS_STAGE = RS_X + RS_W;      // 4 KB + 16 KB per k-step
constexpr int RS_MAX_STEPS = 8;
// MERGE: the x rows are not in memory: row b is the attention output of sequence b, still in the form of the
// per-partition partials a fixed-partition decode launch left (p.part_o, p.part_ml).  The workgroup merges what its
// K range needs (a 16-byte chunk of a row is 8 elements of one q head: the partitions' weights
// l_i 2^(m_i - max m), the weighted sum, one division, one rounding to bf16: decode_reduce_kernel's arithmetic
// in its order, so the bits are those that kernel would have written) and stores the chunks where the copies
// would have put them, while its w tiles are on their way.
template <bool BIAS, bool MERGE = false>
__global__ __launch_bounds__(256) void o_proj_resident_kernel(OProjParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * 128;
  const int kt_total = p.K / BK;
  const int kt_begin = (int)((long)kt_total * blockIdx.y / gridDim.y);
  const int ktiles = (int)((long)kt_total * (blockIdx.y + 1) / gridDim.y) - kt_begin;      // <= RS_MAX_STEPS (host)
  const uint32_t smem_base = (uint32_t)(uintptr_t)(lds_char*)smem;
  const long x_row_b = (long)p.K * 2, w_row_b = (long)p.N * 2;
  // copy maps.  x: 4 units of 8 rows x 128 B, wave w issues unit w; lane i fills (row 8w + i/8, position i%8) with
  // chunk (i%8) ^ ((row >> 1) & 7).  w: 16 units of 4 rows x 256 B, wave w issues units w, w+4, w+8, w+12; lane i
  // fills (row 4u + i/16, position i%16) with chunk (i%16) ^ 4 (row & 3).  Rows past M and columns past N are clamped.
  uint32_t xoff, woff[4];
  {
    const int lrow = 8 * wave + (lane >> 3);
    xoff = (uint32_t)(min(lrow, p.M - 1) * x_row_b) + (uint32_t)(((lane & 7) ^ ((lrow >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = 4 * (wave + 4 * j) + (lane >> 4);
    const int chunk = (lane & 15) ^ (4 * ((lane >> 4) & 3));
    woff[j] = (uint32_t)(r * w_row_b) + (uint32_t)(min(n0 + 8 * chunk, p.N - 8) * 2);
  }
  // MERGE: what the first NE items of this thread need (an item = one 16-byte chunk of an x row, see below) is
  // requested here, ahead of the w tiles, by hand-placed loads whose arrival is awaited by hand too: memory answers in
  // the order of the requests, so these are back long before the tiles, and the merge arithmetic runs while the tiles
  // stream in.  (Loads the compiler places itself would be waited for with everything in flight, tiles included.)
  constexpr int NPRE = 4, NE = 2;
  typedef float f2_t __attribute__((ext_vector_type(2)));
  typedef float f4_t __attribute__((ext_vector_type(4)));
  f2_t e_ml[NE][NPRE];
  f4_t e_oa[NE][NPRE], e_ob[NE][NPRE];
  int e_len[NE], e_qlen[NE];
  float e_sink[NE];
  const int m_items = MERGE ? ktiles * 8 * p.M : 0;
  // x row m is query token m % T of sequence m / T; its q head `head` is row hk n_rep T + t n_rep + j of the sequence's
  // partials, the decode kernels' numbering of (token, head) pairs (T = 1: the q head itself)
  auto item_place = [&](int item, int& kt, int& m, int& c, int& d, long& base, int& b, int& head) __attribute__((always_inline)) {
    const int per_step = 8 * p.M;
    kt = item / per_step;
    const int rem = item - kt * per_step;
    m = rem >> 3; c = rem & 7;
    const int k0 = (kt_begin + kt) * BK + 8 * c;
    head = k0 / p.part_D;
    d = k0 - head * p.part_D;
    const int T = p.part_T, n_rep = p.part_n_rep;
    b = m / T;
    const int t = m - b * T, hk = head / n_rep;
    const int vr = hk * n_rep * T + t * n_rep + (head - hk * n_rep);
    base = ((long)b * (p.K / p.part_D) * T + vr) * p.part_np;
  };
  // the keys the launch gave sequence b: its length, clamped as the launch clamped it; none when a multi-token launch
  // finds no query token for it
  auto context_of = [&](int len, int qlen) __attribute__((always_inline)) -> int {
    int ctx = min(max(len, 0), p.part_max_seq_len);
    if (p.part_query_lens && min(min(max(qlen, 0), p.part_T), ctx) <= 0) ctx = 0;
    return ctx;
  };
  if (MERGE) {
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      int kt, m, c, d, b, head; long base;
      item_place(min(tid + 256 * e, m_items - 1), kt, m, c, d, base, b, head);
      const int32_t* plen = p.part_seq_lens + b;
      asm volatile("global_load_dword %0, %1, off" : "=&v"(e_len[e]) : "v"(plen) : "memory");
      e_sink[e] = 0.f;
      if (p.part_sinks) {
        const float* ps = p.part_sinks + head;
        asm volatile("global_load_dword %0, %1, off" : "=&v"(e_sink[e]) : "v"(ps) : "memory");
      }
      e_qlen[e] = 1;
      if (p.part_query_lens) {
        const int32_t* pq = p.part_query_lens + b;
        asm volatile("global_load_dword %0, %1, off" : "=&v"(e_qlen[e]) : "v"(pq) : "memory");
      }
#pragma unroll
      for (int i = 0; i < NPRE; ++i) {
        const long at = base + min(i, p.part_np - 1);
        const float* pml = p.part_ml + at * 2;
        const float* po = p.part_o + at * p.part_D + d;
        asm volatile("global_load_dwordx2 %0, %1, off" : "=&v"(e_ml[e][i]) : "v"(pml) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(e_oa[e][i]) : "v"(po) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=&v"(e_ob[e][i]) : "v"(po) : "memory");
      }
    }
  }
  {
    const char* xb = (const char*)p.x + (long)kt_begin * (BK * 2);
    const char* wb = (const char*)p.w + (long)kt_begin * BK * w_row_b;
    for (int kt = 0; kt < ktiles; ++kt) {
      const uint32_t sb = smem_base + kt * RS_STAGE;
      if (!MERGE) dma16(xb, xoff, sb + wave * 1024);
#pragma unroll
      for (int j = 0; j < 4; ++j) dma16(wb, woff[j], sb + RS_X + (wave + 4 * j) * 1024);
      xb += BK * 2;
      wb += (long)BK * w_row_b;
    }
  }
  if (MERGE) {
#pragma clang fp contract(off)      // round where decode_reduce_kernel rounds: products and sums as written
    // item = (k-step kt, row m < M, chunk c): elements k0 .. k0 + 7 of x row m, k0 = (kt_begin + kt) * 64 + 8 c, all of
    // one q head.  Up to NPRE partitions' values are requested before any is used (slots past a sequence's own
    // partition count exist and are loaded, not used).
    const int Dh = p.part_D, np_max = p.part_np;
    auto finish = [&](int kt, int m, int c, int d, long base, int ctx, float sink, const f2_t (&ml)[NPRE], const f4_t (&oa)[NPRE],
                      const f4_t (&ob)[NPRE]) __attribute__((always_inline)) {
      const int np = min((ctx + p.part_size - 1) / p.part_size, np_max);
      float mt = -INFINITY;
#pragma unroll
      for (int i = 0; i < NPRE; ++i)
        if (i < np) mt = fmaxf(mt, ml[i].x);
      for (int i = NPRE; i < np; ++i) mt = fmaxf(mt, p.part_ml[(base + i) * 2]);
      const float m_ref = mt == -INFINITY ? 0.f : mt;
      float lt = 0.f, ot[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) ot[j] = 0.f;
      auto add = [&](float mi, float li, const f4_t& a, const f4_t& b) __attribute__((always_inline)) {
        const float wgt = li * exp2f(mi - m_ref);
        lt += wgt;
        ot[0] = __builtin_fmaf(wgt, a.x, ot[0]); ot[1] = __builtin_fmaf(wgt, a.y, ot[1]);
        ot[2] = __builtin_fmaf(wgt, a.z, ot[2]); ot[3] = __builtin_fmaf(wgt, a.w, ot[3]);
        ot[4] = __builtin_fmaf(wgt, b.x, ot[4]); ot[5] = __builtin_fmaf(wgt, b.y, ot[5]);
        ot[6] = __builtin_fmaf(wgt, b.z, ot[6]); ot[7] = __builtin_fmaf(wgt, b.w, ot[7]);
      };
#pragma unroll
      for (int i = 0; i < NPRE; ++i)
        if (i < np) add(ml[i].x, ml[i].y, oa[i], ob[i]);
      for (int i = NPRE; i < np; ++i) {
        const f4_t a = *(const f4_t*)(p.part_o + (base + i) * Dh + d), b = *(const f4_t*)(p.part_o + (base + i) * Dh + d + 4);
        add(p.part_ml[(base + i) * 2], p.part_ml[(base + i) * 2 + 1], a, b);
      }
      // attention sink: one more term of the denominator (decode_reduce_kernel's expression)
      const float sink_w = p.part_sinks ? exp2f(sink * kLog2e - m_ref) : 0.f;
      const float den = p.part_sinks ? lt + sink_w : lt;
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = lt > 0.f ? ot[j] / den : 0.f;
      *(uint4*)(smem + kt * RS_STAGE + m * 128 + ((c ^ ((m >> 1) & 7)) << 4)) =
          make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
    };
    // the early requests: back when at most the wave's tile copies are still out (four per k-step)
    if (ktiles == RS_MAX_STEPS) wait_vmcnt<4 * RS_MAX_STEPS>();
    else wait_vmcnt<0>();
#pragma unroll
    for (int e = 0; e < NE; ++e) {
#pragma unroll
      for (int i = 0; i < NPRE; ++i) asm volatile("" : "+v"(e_ml[e][i]), "+v"(e_oa[e][i]), "+v"(e_ob[e][i]));
      asm volatile("" : "+v"(e_len[e]), "+v"(e_qlen[e]), "+v"(e_sink[e]));
      const int item = tid + 256 * e;
      if (item < m_items) {
        int kt, m, c, d, b, head; long base;
        item_place(item, kt, m, c, d, base, b, head);
        finish(kt, m, c, d, base, context_of(e_len[e], e_qlen[e]), e_sink[e], e_ml[e], e_oa[e], e_ob[e]);
      }
    }
    // more than NE items per thread (more than 8 rows): the rest by ordinary loads
    for (int item = tid + 256 * NE; item < m_items; item += 256) {
      int kt, m, c, d, b, head; long base;
      item_place(item, kt, m, c, d, base, b, head);
      f2_t ml[NPRE];
      f4_t oa[NPRE], ob[NPRE];
#pragma unroll
      for (int i = 0; i < NPRE; ++i) {
        const long at = base + min(i, np_max - 1);
        ml[i] = *(const f2_t*)(p.part_ml + at * 2);
        oa[i] = *(const f4_t*)(p.part_o + at * Dh + d);
        ob[i] = *(const f4_t*)(p.part_o + at * Dh + d + 4);
      }
      finish(kt, m, c, d, base, context_of(p.part_seq_lens[b], p.part_query_lens ? p.part_query_lens[b] : 1),
             p.part_sinks ? p.part_sinks[head] : 0.f, ml, oa, ob);
    }
  }
  int x_off[4], w_off;
#pragma unroll
  for (int s = 0; s < 4; ++s) x_off[s] = n * 128 + (((2 * s + h) ^ ((n >> 1) & 7)) << 4);
  {
    const int g = lane >> 4, sl = lane & 15;
    const int row = 8 * h + (sl >> 2);
    const int y = 2 * (g & 1) + ((sl & 3) >> 1);
    w_off = RS_X + row * 256 + (((4 * wave + y) ^ (4 * (row & 3))) << 4) + (sl & 1) * 8;
  }
  f32x16_t acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  auto step = [&](int kt) __attribute__((always_inline)) {
    const char* sb = smem + kt * RS_STAGE;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const lds_char* src = (const lds_char*)(sb + 16 * s * 256 + w_off);
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)src);
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(src + 4 * 256));
      struct { s16x4_t a, b; } pair = {lo, hi};
      const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, pair);
      const bf16x8_t xf = *(const bf16x8_t*)(sb + x_off[s]);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf, acc, 0, 0, 0);
    }
  };
  if (ktiles == RS_MAX_STEPS) {
    // a full range: the steps are multiplied as they land (5 copy instructions per wave and step; 4 when the x tile
    // is merged here, and then the first barrier also publishes the merged chunks, ordinary LDS stores of other waves)
    constexpr int CPS = MERGE ? 4 : 5;
    wait_vmcnt<CPS * (RS_MAX_STEPS - 1)>();
    if (MERGE) __syncthreads();
    else __builtin_amdgcn_s_barrier();
    step(0);
#define RS_STEP(kt) wait_vmcnt<CPS * (RS_MAX_STEPS - 1 - (kt))>(); __builtin_amdgcn_s_barrier(); step(kt);
    RS_STEP(1) RS_STEP(2) RS_STEP(3) RS_STEP(4) RS_STEP(5) RS_STEP(6) RS_STEP(7)
#undef RS_STEP
  } else {
    wait_vmcnt<0>();
    if (MERGE) __syncthreads();          // the merged x chunks are ordinary LDS stores of other waves
    else __builtin_amdgcn_s_barrier();
    for (int kt = 0; kt < ktiles; ++kt) step(kt);
  }
  // a lane holds, for its row, 4 consecutive columns at 4 places
  const int m = n;
#pragma unroll
  for (int i4 = 0; i4 < 4; ++i4) {
    const int col = n0 + 32 * wave + 8 * i4 + 4 * h;
    if (m < p.M && col < p.N) {
      if (p.splits > 1) {
        *(float4*)(p.ws + ((long)blockIdx.y * p.M + m) * p.N + col) =
            make_float4(acc[4 * i4], acc[4 * i4 + 1], acc[4 * i4 + 2], acc[4 * i4 + 3]);
      } else {
        float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
        if (BIAS) {
          const uint2 bw = *(const uint2*)((const uint16_t*)p.bias + col);
          b0 = bf16_bits_to_float(bw.x & 0xffffu); b1 = bf16_bits_to_float(bw.x >> 16);
          b2 = bf16_bits_to_float(bw.y & 0xffffu); b3 = bf16_bits_to_float(bw.y >> 16);
        }
        *(uint2*)((uint16_t*)p.out + (long)m * p.N + col) = make_uint2(pack_bf16x2(acc[4 * i4] + b0, acc[4 * i4 + 1] + b1),
                                                                        pack_bf16x2(acc[4 * i4 + 2] + b2, acc[4 * i4 + 3] + b3));
      }
    }
  }
}

// Sum of the split form's partial tiles, always in the order of the K ranges, plus the bias; one rounding to bf16.
// A thread owns four consecutive columns of a row (N is a multiple of 8, so they never straddle rows).
template <bool BIAS>
__global__ __launch_bounds__(256) void o_proj_split_reduce_kernel(OProjParams p) {
  const long total = (long)p.M * p.N / 4;
  const long item = (long)blockIdx.x * 256 + threadIdx.x;
  if (item >= total) return;
  const float4* src = (const float4*)p.ws + item;
  // all ranges requested at once (at most eight exist: o_proj_splits), added in their order
  float4 part[8];
#pragma unroll
  for (int z = 0; z < 8; ++z) part[z] = z < p.splits ? src[(long)z * total] : make_float4(0.f, 0.f, 0.f, 0.f);
  float4 a = part[0];
#pragma unroll
  for (int z = 1; z < 8; ++z)
    if (z < p.splits) { a.x += part[z].x; a.y += part[z].y; a.z += part[z].z; a.w += part[z].w; }
  if (BIAS) {
    const uint2 bw = *(const uint2*)((const uint16_t*)p.bias + (item * 4) % p.N);
    a.x += bf16_bits_to_float(bw.x & 0xffffu); a.y += bf16_bits_to_float(bw.x >> 16);
    a.z += bf16_bits_to_float(bw.y & 0xffffu); a.w += bf16_bits_to_float(bw.y >> 16);
  }
  *(uint2*)((uint16_t*)p.out + item * 4) = make_uint2(pack_bf16x2(a.x, a.y), pack_bf16x2(a.z, a.w));
}

template <int MBT>
hipError_t launch_skinny(const OProjParams& p, hipStream_t s) {
  constexpr int NST = MBT == 2 ? 8 : (MBT == 4 ? 5 : 3);
  constexpr int lds = NST * (32 * MBT * 128 + 64 * 128);
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)o_proj_skinny_kernel<MBT, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_skinny_kernel<MBT, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured.store(1, std::memory_order_release);
  }
  const bool split = p.splits > 1 && p.ws && p.M <= 32 * MBT;
  OProjParams q = p;
  if (!split) q.splits = 1;
  const dim3 grid((unsigned)((p.N + 63) / 64), (unsigned)((p.M + 32 * MBT - 1) / (32 * MBT)), (unsigned)q.splits);
  if (p.bias && !split) hipLaunchKernelGGL((o_proj_skinny_kernel<MBT, true>), grid, dim3(256), lds, s, q);
  else hipLaunchKernelGGL((o_proj_skinny_kernel<MBT, false>), grid, dim3(256), lds, s, q);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !split) return e;
  const unsigned blocks = (unsigned)(((long)p.M * p.N / 4 + 255) / 256);
  if (p.bias) hipLaunchKernelGGL((o_proj_split_reduce_kernel<true>), dim3(blocks), dim3(256), 0, s, q);
  else hipLaunchKernelGGL((o_proj_split_reduce_kernel<false>), dim3(blocks), dim3(256), 0, s, q);
  return hipGetLastError();
}

}  // namespace

// Up to 128 rows the call streams w once through N / 64 workgroups; with a workspace up to four K ranges per column
// slab bring that towards the CU count (K = N = 4096, kernel time without the merge: 16.9 -> 9.9 us at 64 rows with
// four ranges, 12.4 with eight), each at least 8 steps of 64 long.
// M <= 32: the resident form, ranges of at most 8 k-steps (then K / 512 of them, up to eight); 0 when K is longer
static int o_proj_resident_splits(int M, int K) {
  if (M <= 0 || M > 32) return 0;
  const int s = (K / BK + RS_MAX_STEPS - 1) / RS_MAX_STEPS;
  return s <= 8 ? s : 0;
}

static hipError_t launch_resident(const OProjParams& p, hipStream_t s) {
  static std::atomic<int> configured{0};
  constexpr int lds = RS_MAX_STEPS * RS_STAGE;
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)o_proj_resident_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_resident_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_resident_kernel<false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_resident_kernel<true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured.store(1, std::memory_order_release);
  }
  const int ktiles = (p.K / BK + p.splits - 1) / p.splits;
  const dim3 grid((unsigned)((p.N + 127) / 128), (unsigned)p.splits);
  const int bytes = ktiles * RS_STAGE;
  if (p.part_o) {
    if (p.bias && p.splits == 1) hipLaunchKernelGGL((o_proj_resident_kernel<true, true>), grid, dim3(256), bytes, s, p);
    else hipLaunchKernelGGL((o_proj_resident_kernel<false, true>), grid, dim3(256), bytes, s, p);
  } else if (p.bias && p.splits == 1) hipLaunchKernelGGL((o_proj_resident_kernel<true>), grid, dim3(256), bytes, s, p);
  else hipLaunchKernelGGL((o_proj_resident_kernel<false>), grid, dim3(256), bytes, s, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || p.splits == 1) return e;
  const unsigned blocks = (unsigned)(((long)p.M * p.N / 4 + 255) / 256);
  if (p.bias) hipLaunchKernelGGL((o_proj_split_reduce_kernel<true>), dim3(blocks), dim3(256), 0, s, p);
  else hipLaunchKernelGGL((o_proj_split_reduce_kernel<false>), dim3(blocks), dim3(256), 0, s, p);
  return hipGetLastError();
}

int o_proj_splits(int M, int K, int N) {
  if (M <= 0 || M > 128) return 1;
  if (const int r = o_proj_resident_splits(M, K)) return r;
  const long slabs = (N + 63) / 64;
  long s = 256 / slabs;
  if (s > 4) s = 4;
  if (s > K / BK / 8) s = K / BK / 8;
  return s < 2 ? 1 : (int)s;
}

// Worth it while a thread has at most the two items whose loads go out ahead of the weight tiles (8 rows at 8 k-steps
// per range: a verify step of 32 rows took 41 us per layer with the merge here, 35 with the merge launch)
bool o_proj_takes_partials(int M, int K, int D, int splits, bool have_ws) {
  const int r = o_proj_resident_splits(M, K);
  if (!(r > 0 && splits == r && (r == 1 || have_ws) && (D == 64 || D == 128) && K % D == 0)) return false;
  const int ktiles = (K / BK + r - 1) / r;
  return (long)M * 8 * ktiles <= 512;
}

static std::atomic<int> g_o_proj_force_large{0};
void o_proj_debug_force_large(int on) { g_o_proj_force_large = on; }

hipError_t launch_o_proj(const OProjParams& p, hipStream_t s) {
  // up to 32 rows with the workspace for its K ranges (or K <= 512): everything resident, one round trip
  if (const int r = o_proj_resident_splits(p.M, p.K); r > 0 && p.splits == r && (r == 1 || p.ws)) return launch_resident(p, s);
  if (p.part_o) return hipErrorInvalidValue;      // only the resident form merges partials (o_proj_takes_partials)
  // up to 256 rows: one workgroup per 64 columns owns every row (the call is bound by w's bytes)
  if (p.M <= 64) return launch_skinny<2>(p, s);
  if (p.M <= 128) return launch_skinny<4>(p, s);
  // a few hundred rows: the 128-row form over several row blocks as long as its workgroups (N / 64 per block) fit
  // the device in one go; measured against the other forms at K = N = 4096.  With a longer K two of them per CU
  // are still ahead of the 128 x 128 form, whose one wave per SIMD pays a latency per k-step (us few rows / 128 x 128:
  // K = 8 192 N = 5 120 M = 512 111.8 / 146.9, M = 768 115.1 / 150.0; K = N = 5 120 M = 512 72.0 / 96.5; K = N = 8 192 M = 384
  // 113.3 / 150.0; at K = 4 096 it is the other way round: N = 4 096 M = 640 48.6 / 41.5, N = 2 880 M = 768 51.3 / 34.8)
  const long few_rows_wgs = p.K >= 5120 ? 512 : 256;
  if (!g_o_proj_force_large && (long)((p.M + 127) / 128) * ((p.N + 63) / 64) <= few_rows_wgs && (long)p.M * p.K * 2 < 0x7fffffffL)
    return launch_skinny<4>(p, s);
  if (p.M <= 256) return launch_skinny<8>(p, s);
  {
    // fewer large tiles than CUs (256 on this part): the 128 x 128 form fills the device better, as long as its
    // workgroups are all resident at once (two per CU); a third of them on some CUs costs a whole further round
    // (K = N = 4096, us: M = 2 304 107 against 92 with the large tiles, M = 3 328 125 against 109; M = 2 048 72 against 82)
    const long big_tiles = (long)((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    const long MTm = (p.M + MBM - 1) / MBM, NTm = (p.N + MBN - 1) / MBN;
    if (big_tiles < 224 && MTm * NTm <= 512 && !g_o_proj_force_large) {
      const long total_m = 8 * ((MTm + 7) / 8) * 4 * ((NTm + 3) / 4);
      if (total_m > 0x7fffffffL) return hipErrorInvalidValue;
      const bool deep = MTm * NTm <= 256;
      static std::atomic<int> configured_mid{0};
      if (!configured_mid.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void*)o_proj_mid_kernel<false, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * MSTAGE_B);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_mid_kernel<true, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * MSTAGE_B);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_mid_kernel<false, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, 4 * MSTAGE_B);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_mid_kernel<true, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, 4 * MSTAGE_B);
        if (e != hipSuccess) return e;
        configured_mid.store(1, std::memory_order_release);
      }
      const dim3 grid((unsigned)total_m), wg(256);
      if (deep) {
        if (p.bias) hipLaunchKernelGGL((o_proj_mid_kernel<true, 4>), grid, wg, 4 * MSTAGE_B, s, p);
        else hipLaunchKernelGGL((o_proj_mid_kernel<false, 4>), grid, wg, 4 * MSTAGE_B, s, p);
      } else {
        if (p.bias) hipLaunchKernelGGL((o_proj_mid_kernel<true, 2>), grid, wg, 2 * MSTAGE_B, s, p);
        else hipLaunchKernelGGL((o_proj_mid_kernel<false, 2>), grid, wg, 2 * MSTAGE_B, s, p);
      }
      return hipGetLastError();
    }
  }
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)o_proj_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_B);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)o_proj_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_B);
    if (e != hipSuccess) return e;
    configured.store(1, std::memory_order_release);
  }
  const long MT = (p.M + BM - 1) / BM, NT = (p.N + BN - 1) / BN;
  const long total = 8 * ((MT + 7) / 8) * 4 * ((NT + 3) / 4);
  if (total > 0x7fffffffL) return hipErrorInvalidValue;
  if (p.bias) hipLaunchKernelGGL(o_proj_kernel<true>, dim3((unsigned)total), dim3(512), LDS_B, s, p);
  else hipLaunchKernelGGL(o_proj_kernel<false>, dim3((unsigned)total), dim3(512), LDS_B, s, p);
  return hipGetLastError();
}

}  // namespace pa
