// Paged KV-cache write: the new tokens' K and V rows are scattered into the block pool
// before attention runs.  The reference updates a dense cache with
// `cache_k[:, query_pos] = xk`, query_pos = start_pos + arange(seq_len)
// (examples/models/gpt_oss/kernels/attention.py:85,92-100; qwen3/kernels/attention.py:100-106);
// here token t < query_lens[b] of sequence b sits at position seq_lens[b] - query_lens[b] + t
// and goes to pool row (block_tables[b, pos / block_size], pos % block_size).
//
// bf16 and fp32 pools receive the rows bit for bit.  fp8 (OCP e4m3fn) pools are quantised on
// the way in with one float32 scale per (block, kv head), kept as the running maximum of
// absmax / 448 over the tokens the block holds: when a write raises the scale, the block's
// earlier rows are re-encoded under the new one.  A block whose first row is part of the write
// is fresh (its old scale and contents are ignored).
//
// One workgroup per (sequence, touched block, kv head, K or V): the (block, head) slab is
// private to it, so scale maintenance needs no atomics.  Pure streaming work, HBM bound.
#include "pa_common.h"

namespace pa {
namespace {

constexpr int WG = 256;

__device__ __forceinline__ float block_max(float v, float* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < WG / 64; ++w) r = fmaxf(r, red[w]);
  return r;
}

// two floats -> two e4m3fn codes in the low or high half of `old`; round to nearest even,
// saturating (the inputs are clamped: the conversion's own overflow behaviour is mode dependent)
__device__ __forceinline__ uint32_t pack_fp8x2(float a, float b, uint32_t old, bool high) {
  a = __builtin_amdgcn_fmed3f(a, -448.f, 448.f);
  b = __builtin_amdgcn_fmed3f(b, -448.f, 448.f);
  return high ? (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true)
              : (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
}

// ESZ: bytes per stored element (4 fp32 copy, 2 bf16 copy, 1 fp8 quantise from bf16 rows)
template <int ESZ>
__global__ __launch_bounds__(WG) void kv_write_kernel(KvWriteParams p) {
  __shared__ float red[WG / 64];
  const int which = blockIdx.x & 1;            // 0: K, 1: V
  const int jj = blockIdx.x >> 1;              // touched block of the sequence
  const int h = blockIdx.y, b = blockIdx.z;
  int tq = p.query_lens[b];
  tq = min(max(tq, 0), p.T);
  const int seq = min(p.seq_lens[b], p.max_blocks * p.block_size);
  const int start = seq - tq;
  if (tq == 0 || start < 0) return;            // nothing to write / inconsistent lengths: leave the pool alone
  const int bs = p.block_size;
  const int jb = start / bs + jj;
  if ((long)jb * bs >= seq) return;
  const int blk = p.block_tables[(long)b * p.max_blocks + jb];
  if (blk < 0 || blk >= p.num_blocks) return;  // a bad table entry must not redirect the write
  const int lo = max(start, jb * bs) - jb * bs;
  const int hi = min(seq, (jb + 1) * bs) - jb * bs;
  const int n = hi - lo;
  const int t0 = jb * bs + lo - start;

  const int D = p.D;
  const long row_elems = (long)p.Hkv * D;
  const char* src = (const char*)(which ? p.v_new : p.k_new);
  char* dst = (char*)(which ? p.v_cache : p.k_cache);

  if (ESZ != 1) {
    // ---- copy: 16 bytes per thread and step
    const int cpr = D * ESZ / 16;               // chunks per row
    const char* s0 = src + (((long)b * p.T + t0) * row_elems + (long)h * D) * ESZ;
    char* d0 = dst + (((long)blk * bs + lo) * row_elems + (long)h * D) * ESZ;
    for (int i = threadIdx.x; i < n * cpr; i += WG) {
      const int r = i / cpr, c = i - r * cpr;
      *(uint4*)(d0 + (long)r * row_elems * ESZ + c * 16) = *(const uint4*)(s0 + (long)r * row_elems * ESZ + c * 16);
    }
    return;
  }

  // ---- fp8: source rows are bf16, 8 elements (16 B in, 8 B out) per thread and step
  float* scale_tbl = which ? p.v_scale : p.k_scale;
  const int cpr = D / 8;
  const uint16_t* s0 = (const uint16_t*)src + ((long)b * p.T + t0) * row_elems + (long)h * D;
  uint8_t* d_blk = (uint8_t*)dst + (long)blk * bs * row_elems + (long)h * D;
  const float s_old = lo > 0 ? scale_tbl[(long)blk * p.Hkv + h] : 0.f;   // read before anyone rewrites it

  // The first HOLD chunks of a thread stay in registers between the absmax pass and the encode
  // pass (a 64-row block of D = 128 is exactly 4 chunks per thread); anything beyond is read twice.
  constexpr int HOLD = 4;
  uint4 held[HOLD];
  float amax = 0.f;
  auto chunk_absmax = [&](const uint4& v) __attribute__((always_inline)) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      amax = fmaxf(amax, fabsf(bf16_bits_to_float(w[j] & 0xffffu)));
      amax = fmaxf(amax, fabsf(bf16_bits_to_float(w[j] >> 16)));
    }
  };
#pragma unroll
  for (int k = 0; k < HOLD; ++k) {
    const int i = threadIdx.x + k * WG;
    held[k] = make_uint4(0, 0, 0, 0);
    if (i < n * cpr) {
      const int r = i / cpr, c = i - r * cpr;
      held[k] = *(const uint4*)(s0 + (long)r * row_elems + c * 8);
    }
    chunk_absmax(held[k]);
  }
  for (int i = threadIdx.x + HOLD * WG; i < n * cpr; i += WG) {
    const int r = i / cpr, c = i - r * cpr;
    chunk_absmax(*(const uint4*)(s0 + (long)r * row_elems + c * 8));
  }
  amax = block_max(amax, red);
  float s_new = fmaxf(s_old, __fdiv_rn(amax, 448.f));
  if (s_new == 0.f) s_new = 1.f;

  if (lo > 0 && s_new != s_old) {
    // the scale grew: earlier rows of the block are re-encoded under it
    for (int i = threadIdx.x; i < lo * cpr; i += WG) {
      const int r = i / cpr, c = i - r * cpr;
      uint2* q = (uint2*)(d_blk + (long)r * row_elems + c * 8);
      const uint2 codes = *q;
      float f[8];
      fp8x4_to_float(codes.x, f);
      fp8x4_to_float(codes.y, f + 4);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = __fdiv_rn(f[j] * s_old, s_new);
      uint2 o;
      o.x = pack_fp8x2(f[0], f[1], 0u, false); o.x = pack_fp8x2(f[2], f[3], o.x, true);
      o.y = pack_fp8x2(f[4], f[5], 0u, false); o.y = pack_fp8x2(f[6], f[7], o.y, true);
      *q = o;
    }
  }
  auto encode_store = [&](const uint4& v, int i) __attribute__((always_inline)) {
    const int r = i / cpr, c = i - r * cpr;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = __fdiv_rn(bf16_bits_to_float(w[j] & 0xffffu), s_new);
      f[2 * j + 1] = __fdiv_rn(bf16_bits_to_float(w[j] >> 16), s_new);
    }
    uint2 o;
    o.x = pack_fp8x2(f[0], f[1], 0u, false); o.x = pack_fp8x2(f[2], f[3], o.x, true);
    o.y = pack_fp8x2(f[4], f[5], 0u, false); o.y = pack_fp8x2(f[6], f[7], o.y, true);
    *(uint2*)(d_blk + (long)(lo + r) * row_elems + c * 8) = o;
  };
#pragma unroll
  for (int k = 0; k < HOLD; ++k) {
    const int i = threadIdx.x + k * WG;
    if (i < n * cpr) encode_store(held[k], i);
  }
  for (int i = threadIdx.x + HOLD * WG; i < n * cpr; i += WG) {
    const int r = i / cpr, c = i - r * cpr;
    encode_store(*(const uint4*)(s0 + (long)r * row_elems + c * 8), i);
  }
  if (threadIdx.x == 0) scale_tbl[(long)blk * p.Hkv + h] = s_new;
}

}  // namespace

hipError_t launch_kv_write(const KvWriteParams& p, hipStream_t s) {
  const int touched = (p.T + p.block_size - 1) / p.block_size + 1;   // a chunk of T rows spans at most this many blocks
  const dim3 grid(2 * touched, p.Hkv, p.B);
  if (p.kv_dtype == PA_FP8_E4M3FN) hipLaunchKernelGGL(kv_write_kernel<1>, grid, dim3(WG), 0, s, p);
  else if (p.kv_dtype == PA_BF16) hipLaunchKernelGGL(kv_write_kernel<2>, grid, dim3(WG), 0, s, p);
  else hipLaunchKernelGGL(kv_write_kernel<4>, grid, dim3(WG), 0, s, p);
  return hipGetLastError();
}

}  // namespace pa
