// Scalar-ALU paged decode attention, split-K reduce and block-table gather.
//
// This is the any-shape path: fp32 storage (where bf16 matrix cores cannot be
// used without losing the 1e-5 tolerance) and bf16 / fp8 shapes the MFMA
// kernel does not take.  One workgroup per (partition, q head, sequence); a
// row of D elements is spread over D/4 adjacent lanes (4 elements each), so a
// wavefront streams 64/(D/4) token rows per step with fully coalesced loads.
// Online softmax (running max / sum) per row group, merged through LDS.
//
// Math restated: examples/models/qwen3/kernels/attention.py:112-144 with
// softmax.py:4-6, evaluated in float32 in a single pass.
#include "pa_common.h"

namespace pa {
namespace {

template <typename T> struct Load4;
template <> struct Load4<float> {
  static __device__ __forceinline__ void get(const void* base, long idx, float* f) {
    float4 v = *(const float4*)((const float*)base + idx);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
  }
};
template <> struct Load4<uint16_t> {  // bf16 bits
  static __device__ __forceinline__ void get(const void* base, long idx, float* f) {
    uint2 v = *(const uint2*)((const uint16_t*)base + idx);
    f[0] = bf16_bits_to_float(v.x & 0xffffu); f[1] = bf16_bits_to_float(v.x >> 16);
    f[2] = bf16_bits_to_float(v.y & 0xffffu); f[3] = bf16_bits_to_float(v.y >> 16);
  }
};
template <> struct Load4<uint8_t> {  // e4m3fn codes
  static __device__ __forceinline__ void get(const void* base, long idx, float* f) {
    uint32_t v = *(const uint32_t*)((const uint8_t*)base + idx);
    fp8x4_to_float(v, f);
  }
};

constexpr int kGenericThreads = 256;

template <typename QT, typename KVT, int D>
__global__ __launch_bounds__(kGenericThreads) void decode_generic_kernel(DecodeParams p) {
  constexpr int LPR = D / 4;                  // lanes per row
  constexpr int GROUPS = kGenericThreads / LPR;  // row groups per workgroup
  constexpr bool kScaled = sizeof(KVT) == 1;
  const int part = blockIdx.x, hq = blockIdx.y, b = blockIdx.z;
  const int n_rep = p.Hq / p.Hkv;
  const int hk = hq / n_rep;
  int ctx = p.seq_lens[b];
  ctx = min(max(ctx, 0), p.max_seq_len);
  const int t_begin = part * p.partition_size;
  const int tid = threadIdx.x;
  if (t_begin >= ctx) {
    if (ctx == 0 && part == 0 && p.num_partitions == 1) {
      for (int d = tid; d < D; d += kGenericThreads)
        Store<QT>::put(p.out, ((long)b * p.Hq + hq) * D + d, 0.f);
    }
    return;
  }
  const int t_end = min(ctx, t_begin + p.partition_size);
  const int group = tid / LPR;
  const int dl = (tid % LPR) * 4;

  float qv[4];
  Load4<QT>::get(p.q, ((long)b * p.Hq + hq) * D + dl, qv);
  const int32_t* table = p.block_tables + (long)b * p.max_blocks;

  float m = -INFINITY, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int t = t_begin + group; t < t_end; t += GROUPS) {
    int blk = table[t / p.block_size];
    blk = min(max(blk, 0), p.num_blocks - 1);
    const long row = ((long)blk * p.block_size + (t % p.block_size)) * p.Hkv + hk;
    float kv[4], vv[4];
    Load4<KVT>::get(p.k_cache, row * D + dl, kv);
    Load4<KVT>::get(p.v_cache, row * D + dl, vv);
    float s = qv[0] * kv[0] + qv[1] * kv[1] + qv[2] * kv[2] + qv[3] * kv[3];
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    s *= p.scale_log2e;
    float vs = 1.f;
    if (kScaled) {
      s *= p.k_scale[(long)blk * p.Hkv + hk];
      vs = p.v_scale[(long)blk * p.Hkv + hk];
    }
    const float m_new = fmaxf(m, s);
    const float alpha = exp2f(m - m_new);
    const float pr = exp2f(s - m_new);
    l = l * alpha + pr;
    const float pv = pr * vs;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = acc[i] * alpha + pv * vv[i];
    m = m_new;
  }

  __shared__ float sm_m[GROUPS];
  __shared__ float sm_l[GROUPS];
  __shared__ float sm_o[GROUPS][D];
  if ((tid % LPR) == 0) { sm_m[group] = m; sm_l[group] = l; }
#pragma unroll
  for (int i = 0; i < 4; ++i) sm_o[group][dl + i] = acc[i];
  __syncthreads();
  for (int d = tid; d < D; d += kGenericThreads) {
    float mt = -INFINITY;
    for (int g = 0; g < GROUPS; ++g) mt = fmaxf(mt, sm_m[g]);
    float lt = 0.f, ot = 0.f;
    for (int g = 0; g < GROUPS; ++g) {
      const float w = exp2f(sm_m[g] - mt);   // empty groups: exp2(-inf) = 0
      lt += sm_l[g] * w;
      ot += sm_o[g][d] * w;
    }
    const float o = ot / lt;
    if (p.num_partitions == 1) {
      Store<QT>::put(p.out, ((long)b * p.Hq + hq) * D + d, o);
    } else {
      const long slot = ((long)b * p.Hq + hq) * p.num_partitions + part;
      p.ws_out[slot * D + d] = o;
      if (d == 0) { p.ws_ml[slot * 2] = mt; p.ws_ml[slot * 2 + 1] = lt; }
    }
  }
}

// Merge of split-K partials: m = max m_i, w_i = l_i 2^(m_i - m),
// out = sum w_i o_i / sum w_i.   One workgroup per (row, sequence); a row is a q head, or, for a
// launch with several query tokens per sequence (p.query_lens), a (token, head) pair of a kv head, token-major:
// such a row may have seen no key in a partition (m = -inf, l = 0) or be padding (zeros).
template <typename QT>
__global__ void decode_reduce_kernel(DecodeParams p) {
  // no contraction of the sums below into multiply-adds of the compiler's choosing: the projection's merge-on-load
  // (o_proj_resident_kernel) repeats this arithmetic and must round where this kernel rounds
#pragma clang fp contract(off)
  const int vr = blockIdx.x, b = blockIdx.y;
  const bool multi = p.query_lens != nullptr;
  const int rows_total = p.Hq * (multi ? p.T : 1);
  const long base = ((long)b * rows_total + vr) * p.num_partitions;
  // The kernel is a chain of dependent loads (length -> partition count -> maxima -> partials), each a trip to
  // memory, around a few additions.  The first PRE partitions' values are therefore requested at once and before the
  // length is known (their slots exist whatever the length; what a partition past the context holds is not used).
  constexpr int PRE = 4;
  const int npre = min(PRE, p.num_partitions);
  const int d0 = threadIdx.x;
  float m_[PRE], l_[PRE], o_[PRE];
#pragma unroll
  for (int i = 0; i < PRE; ++i) {
    m_[i] = -INFINITY; l_[i] = 0.f; o_[i] = 0.f;
    if (i < npre) {
      m_[i] = p.ws_ml[(base + i) * 2];
      l_[i] = p.ws_ml[(base + i) * 2 + 1];
      if (d0 < p.D) o_[i] = p.ws_out[(base + i) * p.D + d0];
    }
  }
  int ctx = p.seq_lens[b];
  ctx = min(max(ctx, 0), p.max_seq_len);
  long out_at = ((long)b * p.Hq + vr) * p.D;
  int tq_rows = 1, head = vr;
  if (multi) {
    // context and rows of this launch as the streaming kernel takes them (query tokens [t0, t0 + T) of T_stride)
    const int qfull = min(min(max(p.query_lens[b], 0), p.T_stride), ctx);
    const int tq = min(max(qfull - p.t0, 0), p.T);
    ctx = tq > 0 ? ctx - qfull + p.t0 + tq : 0;
    tq_rows = tq;
    const int n_rep = p.Hq / p.Hkv, n_rows = n_rep * p.T;
    const int hk = vr / n_rows, j = vr - hk * n_rows, t = j / n_rep;
    head = hk * n_rep + (j - t * n_rep);
    out_at = (((long)b * p.T_stride + p.t0 + t) * p.Hq + head) * p.D;
  }
  // partitions count from the first tile the launch's rows see (a sliding window skips what lies before it)
  int span = ctx;
  if (p.window > 0) span -= (max(ctx - tq_rows + 1 - p.window, 0) >> 5) << 5;
  const int np = (span + p.partition_size - 1) / p.partition_size;
  float mt = -INFINITY;
#pragma unroll
  for (int i = 0; i < PRE; ++i)
    if (i < np) mt = fmaxf(mt, m_[i]);
  for (int i = PRE; i < np; ++i) mt = fmaxf(mt, p.ws_ml[(base + i) * 2]);
  const float m_ref = mt == -INFINITY ? 0.f : mt;
  // attention sink: one more term of the denominator, no value
  const float sink_w = p.sinks ? exp2f(p.sinks[head] * kLog2e - m_ref) : 0.f;
  for (int d = d0; d < p.D; d += blockDim.x) {
    float lt = 0.f, ot = 0.f;
#pragma unroll
    for (int i = 0; i < PRE; ++i)
      if (i < np) {
        const float w = l_[i] * exp2f(m_[i] - m_ref);
        lt += w;
        ot = __builtin_fmaf(w, d == d0 ? o_[i] : p.ws_out[(base + i) * p.D + d], ot);
      }
    for (int i = PRE; i < np; ++i) {
      const float w = p.ws_ml[(base + i) * 2 + 1] * exp2f(p.ws_ml[(base + i) * 2] - m_ref);
      lt += w;
      ot = __builtin_fmaf(w, p.ws_out[(base + i) * p.D + d], ot);    // (the projection's merge-on-load repeats this arithmetic)
    }
    Store<QT>::put(p.out, out_at + d, lt > 0.f ? ot / (p.sinks ? lt + sink_w : lt) : 0.f);
  }
}

// out[b, t, :] = pool[table[b, t / bs], t % bs, :] for t < seq_len, zero after.
// Rows are copied in 16-byte pieces when the row size allows, else bytewise.
template <typename V>
__global__ void gather_kernel(const V* __restrict__ cache, const int32_t* __restrict__ tables,
                              const int32_t* __restrict__ seq_lens, V* __restrict__ out,
                              int row_vecs, int block_size, int max_blocks, int num_blocks,
                              int max_seq_len) {
  const int b = blockIdx.y;
  const int ctx = min(max(seq_lens[b], 0), max_seq_len);
  const long total = (long)max_seq_len * row_vecs;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const int t = (int)(i / row_vecs);
    const int c = (int)(i % row_vecs);
    V val = V();
    if (t < ctx) {
      int blk = tables[(long)b * max_blocks + t / block_size];
      blk = min(max(blk, 0), num_blocks - 1);
      val = cache[((long)blk * block_size + (t % block_size)) * row_vecs + c];
    }
    out[(long)b * total + i] = val;
  }
}

template <typename QT, typename KVT>
hipError_t launch_generic_typed(const DecodeParams& p, hipStream_t s) {
  dim3 grid(p.num_partitions, p.Hq, p.B), block(kGenericThreads);
  switch (p.D) {
    case 32:  hipLaunchKernelGGL((decode_generic_kernel<QT, KVT, 32>), grid, block, 0, s, p); break;
    case 64:  hipLaunchKernelGGL((decode_generic_kernel<QT, KVT, 64>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((decode_generic_kernel<QT, KVT, 128>), grid, block, 0, s, p); break;
    case 256: hipLaunchKernelGGL((decode_generic_kernel<QT, KVT, 256>), grid, block, 0, s, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_decode_generic(const DecodeParams& p, int q_dtype, int kv_dtype, hipStream_t s) {
  if (q_dtype == PA_F32 && kv_dtype == PA_F32) return launch_generic_typed<float, float>(p, s);
  if (q_dtype == PA_BF16 && kv_dtype == PA_BF16) return launch_generic_typed<uint16_t, uint16_t>(p, s);
  if (q_dtype == PA_BF16 && kv_dtype == PA_FP8_E4M3FN) return launch_generic_typed<uint16_t, uint8_t>(p, s);
  return hipErrorInvalidValue;
}

hipError_t launch_decode_reduce(const DecodeParams& p, int q_dtype, hipStream_t s) {
  dim3 grid(p.Hq * (p.query_lens ? p.T : 1), p.B), block(p.D <= 64 ? 64 : 128);
  if (q_dtype == PA_F32) hipLaunchKernelGGL(decode_reduce_kernel<float>, grid, block, 0, s, p);
  else hipLaunchKernelGGL(decode_reduce_kernel<uint16_t>, grid, block, 0, s, p);
  return hipGetLastError();
}

hipError_t launch_gather(const void* cache, const int32_t* tables, const int32_t* seq_lens, void* out,
                         int B, int row_bytes, int block_size, int max_blocks, int num_blocks,
                         int max_seq_len, hipStream_t s) {
  if (B == 0 || max_seq_len == 0) return hipSuccess;
  const bool vec16 = (row_bytes % 16) == 0 && ((uintptr_t)cache % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int row_vecs = vec16 ? row_bytes / 16 : row_bytes;
  const long total = (long)max_seq_len * row_vecs;
  int gx = (int)((total + 255) / 256);
  if (gx > 4096) gx = 4096;
  dim3 grid(gx, B), block(256);
  if (vec16)
    hipLaunchKernelGGL(gather_kernel<uint4>, grid, block, 0, s, (const uint4*)cache, tables, seq_lens,
                       (uint4*)out, row_vecs, block_size, max_blocks, num_blocks, max_seq_len);
  else
    hipLaunchKernelGGL(gather_kernel<uint8_t>, grid, block, 0, s, (const uint8_t*)cache, tables, seq_lens,
                       (uint8_t*)out, row_vecs, block_size, max_blocks, num_blocks, max_seq_len);
  return hipGetLastError();
}

}  // namespace pa
