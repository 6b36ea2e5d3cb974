// GQA-aware paged decode attention on the gfx950 matrix cores.
//
// One workgroup per (partition, kv head [x 16-head chunk], sequence); each of
// its NW wavefronts streams 32-token tiles of K and V straight from HBM into
// registers (no LDS on the streaming path) and keeps an online-softmax state
// for up to 16 query heads of the group at once, so one read of a K/V row
// serves the whole GQA group (examples/models/qwen3/kernels/attention.py:15-22
// never materialised).
//
// v_mfma_f32_16x16x32_bf16 operand layout (lane = 16*g + r, g = 0..3, r = 0..15):
//   A[16 x 32]: lane holds row r, k-slots 8g .. 8g+7
//   B[32 x 16]: lane holds column r, k-slots 8g .. 8g+7
//   C/D[16x16]: lane holds column r, rows 4g .. 4g+3
//
// Scores:  S^T[token, head] = K[token, :] . Q^T[:, head]
//   A = K rows: lane (g, r) loads row  t0 + 16u + 4(r%4) + r/4  (u = 16-token
//   sub-tile) in 16-byte pieces; the k-slot -> d assignment is the same
//   arbitrary bijection for K and Q, chosen so that one load instruction reads
//   64 contiguous bytes of each row.  With that row order the result lane
//   (g, head) holds tokens t0 + 16u + 4i + g (i = 0..3).
// Output:  O^T[d, head] += V^T[d, token] . P^T[token, head]
//   B = P^T comes straight from the score registers: k-slot 8g + j  <->  token
//   t0 + 4j + g (j = 4u + i) — no data movement, only f32 -> bf16 packing.
//   A = V^T must list, per lane, 8 tokens for one d.  Lane (g, c) loads, for
//   j = 0..7, the VEC = D/16 consecutive d's  VEC*c .. of token t0 + 4j + g
//   (so one load instruction reads 4 whole rows), then an in-register 8 x VEC
//   transpose (v_perm_b32) yields for each e < VEC the vector "tokens j = 0..7
//   at d = VEC*c + e".  MFMA e therefore produces output rows c <-> d = VEC*c+e.
// The per-head softmax state (max, sum) lives in the lane's own registers
// because a lane's column (head) never changes; only the tile max crosses
// lanes (two xor-shuffles over g).
//
// fp8 (OCP e4m3fn) KV: bytes are expanded to bf16 exactly (every e4m3 value is
// a bf16 value) right after the load; the per-(block, kv head) scales are
// applied to the fp32 scores (K) and folded into P (V), so the dequantised
// cache is never written anywhere.
//
// Math restated: attention.py:112-144 + softmax.py:4-6 in one pass; the merge
// of partitions is  m = max m_i, l = sum l_i 2^(m_i-m), o = sum o_i l_i 2^(m_i-m)/l.
#include "pa_common.h"

namespace pa {
namespace {

template <int N> struct VecLoad;
template <> struct VecLoad<1> {
  static __device__ __forceinline__ void get(const void* p, uint32_t* r) { r[0] = *(const uint32_t*)p; }
};
template <> struct VecLoad<2> {
  static __device__ __forceinline__ void get(const void* p, uint32_t* r) {
    uint2 v = *(const uint2*)p; r[0] = v.x; r[1] = v.y;
  }
};
template <> struct VecLoad<4> {
  static __device__ __forceinline__ void get(const void* p, uint32_t* r) {
    uint4 v = *(const uint4*)p; r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
  }
};

__device__ __forceinline__ bf16x8_t as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  uint4 v = make_uint4(a, b, c, d);
  return __builtin_bit_cast(bf16x8_t, v);
}

// One 32-token tile as loaded (raw bits).
template <int D, bool FP8>
struct Tile {
  static constexpr int VEC = D / 16;                       // d's per lane for V
  static constexpr int KLD = FP8 ? D / 64 : D / 32;        // 16-byte K loads per 16-token sub-tile
  static constexpr int VW = (VEC * (FP8 ? 1 : 2)) / 4;     // dwords per V load
  uint32_t k[2][KLD][4];
  uint32_t v[8][VW];
  float ksc[2], vsc[2];     // fp8 only: scales of the two 16-token halves
};

template <int D, bool FP8, int NW>
__global__ __launch_bounds__(NW * 64) void decode_mfma_kernel(DecodeParams p) {
  using T = Tile<D, FP8>;
  constexpr int VEC = T::VEC, KLD = T::KLD, VW = T::VW;
  constexpr int KSTEPS = D / 32;
  constexpr int ESZ = FP8 ? 1 : 2;
  constexpr int OSTRIDE = D + 16;   // LDS row stride (floats) for the merge

  const int part = blockIdx.x, b = blockIdx.z;
  const int n_rep = p.Hq / p.Hkv;
  const int gchunks = (n_rep + 15) / 16;
  const int hk = blockIdx.y / gchunks;
  const int hbase = hk * n_rep + (blockIdx.y % gchunks) * 16;       // first q head of this chunk
  const int nheads = min(16, n_rep - (blockIdx.y % gchunks) * 16);  // valid columns

  int ctx = p.seq_lens[b];
  ctx = min(max(ctx, 0), p.max_seq_len);
  const int t_begin = part * p.partition_size;
  const int tid = threadIdx.x;
  if (t_begin >= ctx) {
    if (ctx == 0 && part == 0 && p.num_partitions == 1) {
      for (int i = tid; i < nheads * D; i += NW * 64)
        ((uint16_t*)p.out)[((long)b * p.Hq + hbase) * D + i] = 0;
    }
    return;
  }
  const int t_end = min(ctx, t_begin + p.partition_size);
  const int ntiles = (t_end - t_begin + 31) >> 5;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;

  // ---- Q^T fragments (B operand), zero for padded head columns --------------
  bf16x8_t qf[KSTEPS];
  {
    const uint16_t* qrow = (const uint16_t*)p.q + ((long)b * p.Hq + hbase + r) * D;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      // d range of k-slots 8g..8g+7 in step s (must mirror the K loads below)
      const int d0 = FP8 ? ((4 * (s >> 1) + g) * 16 + (s & 1) * 8) : ((4 * s + g) * 8);
      uint4 v = make_uint4(0, 0, 0, 0);
      if (r < nheads) v = *(const uint4*)(qrow + d0);
      qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
  }

  const int32_t* table = p.block_tables + (long)b * p.max_blocks;
  const long row_stride = (long)p.Hkv * D * ESZ;   // bytes between consecutive tokens of a block
  const char* kbase = (const char*)p.k_cache + (long)hk * D * ESZ;
  const char* vbase = (const char*)p.v_cache + (long)hk * D * ESZ;
  const int krow = 4 * (r & 3) + (r >> 2);         // row order of the K sub-tile
  const int last = ctx - 1;

  // Issue the loads of tile `ti` (tokens t0 .. t0+31).  Rows past the context
  // are redirected to the last valid token so that no stale pool bytes (which
  // could be NaN patterns) ever reach the matrix cores.
  auto load_tile = [&](T& tl, int ti) {
    const int t0 = t_begin + (ti << 5);
    // the two 16-token halves each lie inside one block (block_size is a power
    // of two >= 16 and t0 is a multiple of 32)
    const int t1 = min(t0 + 16, last);             // wave-uniform
    int blk0 = table[t0 >> p.block_shift];
    int blk1 = table[t1 >> p.block_shift];
    blk0 = min(max(blk0, 0), p.num_blocks - 1);
    blk1 = min(max(blk1, 0), p.num_blocks - 1);
    const int bmask = p.block_size - 1;
    const long row0 = (long)blk0 * p.block_size + (t0 & bmask);          // pool row of token t0
    const long row1 = (long)blk1 * p.block_size + ((t0 + 16) & bmask);   // pool row of token t0+16
    if (FP8) {
      tl.ksc[0] = p.k_scale[(long)blk0 * p.Hkv + hk];
      tl.ksc[1] = p.k_scale[(long)blk1 * p.Hkv + hk];
      tl.vsc[0] = p.v_scale[(long)blk0 * p.Hkv + hk];
      tl.vsc[1] = p.v_scale[(long)blk1 * p.Hkv + hk];
    }
    const int lmax = last - t0;                    // largest valid local index (>= 0)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int tl_ = min(16 * u + krow, lmax);
      const long row = (tl_ < 16) ? row0 + tl_ : row1 + (tl_ - 16);
      const char* rowp = kbase + row * row_stride;
#pragma unroll
      for (int s = 0; s < KLD; ++s) VecLoad<4>::get(rowp + (4 * s + g) * 16, tl.k[u][s]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int tl_ = min(4 * j + g, lmax);
      const long row = (tl_ < 16) ? row0 + tl_ : row1 + (tl_ - 16);
      const char* rowp = vbase + row * row_stride;
      VecLoad<VW>::get(rowp + r * (VEC * ESZ), tl.v[j]);
    }
  };

  f32x4_t oacc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) oacc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  auto compute_tile = [&](const T& tl, int ti) {
    const int t0 = t_begin + (ti << 5);
    // ---- scores ----
    f32x4_t sacc[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      sacc[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (!FP8) {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          sacc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              as_bf16x8(tl.k[u][s][0], tl.k[u][s][1], tl.k[u][s][2], tl.k[u][s][3]), qf[s], sacc[u], 0, 0, 0);
      } else {
#pragma unroll
        for (int s = 0; s < KLD; ++s) {
          uint32_t w[8];
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            float f[4];
            fp8x4_to_float(tl.k[u][s][d], f);
            w[2 * d] = pack_hi16(f[0], f[1]);
            w[2 * d + 1] = pack_hi16(f[2], f[3]);
          }
          sacc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[0], w[1], w[2], w[3]), qf[2 * s], sacc[u], 0, 0, 0);
          sacc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[4], w[5], w[6], w[7]), qf[2 * s + 1], sacc[u], 0, 0, 0);
        }
      }
    }
    // ---- online softmax for this lane's head column ----
    float sv[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const float sc = FP8 ? p.scale_log2e * tl.ksc[u] : p.scale_log2e;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tok = t0 + 16 * u + 4 * i + g;
        const float x = sacc[u][i] * sc;
        sv[4 * u + i] = tok < t_end ? x : -INFINITY;
        tmax = fmaxf(tmax, sv[4 * u + i]);
      }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float pr[8], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pr[i] = __builtin_amdgcn_exp2f(sv[i] - m_new);
      psum += pr[i];
    }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int e = 0; e < VEC; ++e) oacc[e] *= alpha;
    if (FP8) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { pr[i] *= tl.vsc[0]; pr[4 + i] *= tl.vsc[1]; }
    }
    const bf16x8_t pf = as_bf16x8(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]),
                                  pack_bf16x2(pr[4], pr[5]), pack_bf16x2(pr[6], pr[7]));
    // ---- V^T fragments: in-register transpose, then O^T += V^T P^T ----
    if (!FP8) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
        uint32_t w[4];
#pragma unroll
        for (int jp = 0; jp < 4; ++jp)
          w[jp] = __builtin_amdgcn_perm(tl.v[2 * jp + 1][e >> 1], tl.v[2 * jp][e >> 1], sel);
        oacc[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[0], w[1], w[2], w[3]), pf, oacc[e], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int dw = 0; dw < VW; ++dw) {
        float f[8][4];
#pragma unroll
        for (int j = 0; j < 8; ++j) fp8x4_to_float(tl.v[j][dw], f[j]);
#pragma unroll
        for (int eb = 0; eb < 4; ++eb) {
          const int e = 4 * dw + eb;
          uint32_t w[4];
#pragma unroll
          for (int jp = 0; jp < 4; ++jp) w[jp] = pack_hi16(f[2 * jp][eb], f[2 * jp + 1][eb]);
          oacc[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[0], w[1], w[2], w[3]), pf, oacc[e], 0, 0, 0);
        }
      }
    }
  };

  // ---- stream this wave's tiles, next tile's loads in flight during compute ----
  {
    T ta, tb;
    int ti = wave;
    if (ti < ntiles) {
      load_tile(ta, ti);
      while (true) {
        if (ti + NW < ntiles) load_tile(tb, ti + NW);
        compute_tile(ta, ti);
        ti += NW;
        if (ti >= ntiles) break;
        if (ti + NW < ntiles) load_tile(ta, ti + NW);
        compute_tile(tb, ti);
        ti += NW;
        if (ti >= ntiles) break;
      }
    }
  }

  // ---- merge the NW wave states through LDS ----
  __shared__ float sm_m[NW][16];
  __shared__ float sm_l[NW][16];
  __shared__ __attribute__((aligned(16))) float sm_o[NW][16][OSTRIDE];
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (g == 0) { sm_m[wave][r] = m_run; sm_l[wave][r] = l_run; }
  if (r < nheads) {
#pragma unroll
    for (int e = 0; e < VEC; ++e)   // value for d = VEC*(4g+i) + e stored at e*16 + 4g + i
      *(f32x4_t*)&sm_o[wave][r][e * 16 + 4 * g] = oacc[e];
  }
  __syncthreads();
  for (int idx = tid; idx < nheads * D; idx += NW * 64) {
    const int h = idx / D, d = idx % D;
    const int pos = (d % VEC) * 16 + d / VEC;
    float mt = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) mt = fmaxf(mt, sm_m[w][h]);
    float lt = 0.f, ot = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float wt = __builtin_amdgcn_exp2f(sm_m[w][h] - mt);   // idle waves: 2^-inf = 0
      lt += sm_l[w][h] * wt;
      ot += sm_o[w][h][pos] * wt;
    }
    const float o = ot / lt;
    const int hq = hbase + h;
    if (p.num_partitions == 1) {
      ((uint16_t*)p.out)[((long)b * p.Hq + hq) * D + d] = float_to_bf16_bits(o);
    } else {
      const long slot = ((long)b * p.Hq + hq) * p.num_partitions + part;
      p.ws_out[slot * D + d] = o;
      if (d == 0) { p.ws_ml[slot * 2] = mt; p.ws_ml[slot * 2 + 1] = lt; }
    }
  }
}

template <int D, bool FP8>
hipError_t launch_typed(const DecodeParams& p, int waves, hipStream_t s) {
  const int n_rep = p.Hq / p.Hkv;
  dim3 grid(p.num_partitions, p.Hkv * ((n_rep + 15) / 16), p.B);
  switch (waves) {
    case 1: hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 1>), grid, dim3(64), 0, s, p); break;
    case 2: hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 2>), grid, dim3(128), 0, s, p); break;
    default: hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 4>), grid, dim3(256), 0, s, p); break;
  }
  return hipGetLastError();
}

}  // namespace

bool decode_mfma_supported(const DecodeParams& p, int q_dtype, int kv_dtype) {
  if (q_dtype != PA_BF16) return false;
  if (kv_dtype != PA_BF16 && kv_dtype != PA_FP8_E4M3FN) return false;
  if (p.D != 64 && p.D != 128) return false;
  if (p.block_shift < 4) return false;   // power-of-two block size >= 16
  if (p.partition_size % 32 != 0) return false;
  return true;
}

hipError_t launch_decode_mfma(const DecodeParams& p, int kv_dtype, int waves, hipStream_t s) {
  const bool fp8 = kv_dtype == PA_FP8_E4M3FN;
  if (p.D == 128) return fp8 ? launch_typed<128, true>(p, waves, s) : launch_typed<128, false>(p, waves, s);
  if (p.D == 64) return fp8 ? launch_typed<64, true>(p, waves, s) : launch_typed<64, false>(p, waves, s);
  return hipErrorInvalidValue;
}

}  // namespace pa
