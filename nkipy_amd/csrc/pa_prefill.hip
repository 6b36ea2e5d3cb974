// Causal flash-attention prefill on the gfx950 matrix cores: paged chunked
// prefill against a cached prefix, and block-sparse prefill over dense K/V.
//
// One workgroup (4 wavefronts) owns 128 query rows of one (sequence, q head);
// each wavefront owns 32 of them.  Keys are walked in tiles of 64; a tile of K
// and V is staged through LDS once per workgroup and read by all four waves.
//
// v_mfma_f32_32x32x16_bf16 operand layout (lane = 32*h + n, h = 0..1, n = 0..31):
//   A[32 x 16]: lane holds row n, k-slots 8h .. 8h+7
//   B[16 x 32]: lane holds column n, k-slots 8h .. 8h+7
//   C/D[32x32]: lane holds column n, rows 8*(i/4) + 4h + (i%4) for i = 0..15
//
// Scores are computed transposed, S^T[key, q] = K[key, :] . Q^T[:, q], so that a
// lane's column is one query row: the running max / sum of the online softmax
// are per-lane scalars and need one cross-lane exchange (h = 0 <-> 1) per tile.
// The probabilities then feed the second product O^T[d, q] += V^T[d, key] P^T[key, q]
// as its B operand straight from the accumulator registers: MFMA kk of a
// 32-key sub-tile takes i = 8kk .. 8kk+7, i.e. k-slot 8h+j <-> key
// 16kk + 8(j/4) + 4h + (j%4).  V^T (A operand) must present those 8 keys
// contiguously for one d: V is transposed on its way into LDS (4 keys x 8 d per
// thread, v_perm_b32, 8-byte stores) into Vt[d][slot] with the slot order
// slot = 32tt + 16kk + 8h + 4a + b  for key = 32tt + 16kk + 8a + 4h + b.
//
// Masking follows examples/models/gpt_oss/kernels/attention.py:85,127-135: query
// i of a chunk that starts at `prefix` sees keys j <= prefix + i (additive
// -100000 there; an exact zero weight here, which is the same number in fp32).
// The block-sparse form adds the block predicate to the same loop: inactive key
// tiles are never loaded.
#include <atomic>

#include "pa_common.h"

namespace pa {
namespace {

constexpr int BM = 128;              // query rows per workgroup
constexpr int BN = 64;               // keys per tile
constexpr int HD = 128;              // head dim
constexpr int K_ROW_BYTES = HD * 2 + 16;   // LDS K row: 256 B + 16 B pad (bank spread for b128 reads)
constexpr int VT_ROW_BYTES = BN * 2 + 16;  // LDS V^T row: 64 slots + pad
constexpr int VT_BYTES = HD * VT_ROW_BYTES + (HD / 8) * 16;

__device__ __forceinline__ bf16x8_t as_bf16x8_prefill(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  uint4 v = make_uint4(a, b, c, d);
  return __builtin_bit_cast(bf16x8_t, v);
}

__device__ __forceinline__ int vt_row_offset(int d) { return d * VT_ROW_BYTES + (d >> 3) * 16; }

__device__ __forceinline__ bool block_active(int i, int j, int head, int local, int stride) {
  return j <= i && ((i - j) < local || ((j + head % stride) % stride) == 0);
}

// MODE: 0 = dense K/V [B, S, Hkv, D]; 1 = paged, block size a power of two >= 16
// (one table entry per 16-key group, looked up once per wave on the scalar unit);
// 2 = paged, any block size (every staged key resolves its own table entry).
// FP8 (paged only): the pool holds e4m3fn codes with one float32 scale per (block, kv head); a
// thread fetches 8 codes where it would fetch 8 bf16 values and expands them, times the scale of
// their block, to bf16 on the way into LDS, so the dequantised cache exists only there.
template <bool SPARSE, int MODE, bool FP8>
__global__ __launch_bounds__(256, 2) void prefill_kernel(PrefillParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // two stages, each: K tile [64][272 B] then V^T tile
  constexpr int STAGE_BYTES = BN * K_ROW_BYTES + VT_BYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int nqt = (p.T + BM - 1) / BM;
  const int qt = nqt - 1 - (int)blockIdx.x;       // heavy (late) query tiles first
  const int hq = blockIdx.y, b = blockIdx.z;
  const int hk = hq / (p.Hq / p.Hkv);

  int tq = p.query_lens ? p.query_lens[b] : p.T;
  int ctx = p.seq_lens ? p.seq_lens[b] : p.S;
  tq = min(max(tq, 0), p.T);
  if (MODE != 0) ctx = min(ctx, p.max_blocks * p.block_size);
  ctx = max(ctx, 0);
  tq = min(tq, ctx);          // more query tokens than context: the first ctx of them count, without a prefix (as pa_verify)
  const int prefix = ctx - tq;
  const int q0 = qt * BM;
  uint16_t* out = (uint16_t*)p.out;
  const long q_row_stride = (long)p.Hq * HD;

  if (q0 >= tq) {   // only padding rows here: zeros
    for (int i = tid; i < BM * (HD / 8); i += 256) {
      const int row = q0 + i / (HD / 8);
      if (row < p.T) *(uint4*)(out + ((long)b * p.T + row) * q_row_stride + (long)hq * HD + (i % (HD / 8)) * 8) = make_uint4(0, 0, 0, 0);
    }
    return;
  }

  // ---- this lane's query row and its Q^T fragments --------------------------
  const int qrow = q0 + wave * 32 + n;
  const bool qvalid = qrow < tq;
  const int qlim = prefix + min(qrow, tq - 1);     // last visible key of this lane's row
  bf16x8_t qf[HD / 16];
  {
    const uint16_t* qp = (const uint16_t*)p.q + ((long)b * p.T + qrow) * q_row_stride + (long)hq * HD;
#pragma unroll
    for (int s = 0; s < HD / 16; ++s) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (qvalid) v = *(const uint4*)(qp + 16 * s + 8 * h);
      qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
  }
  const int wq_lo = q0 + wave * 32;                               // first row of this wave
  const int wq_hi = min(wq_lo + 31, tq - 1);                      // last valid row (may be < wq_lo)
  const bool wave_has_rows = wq_lo < tq;
  const int k_end = prefix + min(q0 + BM, tq);                    // keys the workgroup needs: [0, k_end)
  const int ntiles = (k_end + BN - 1) / BN;

  // ---- global -> LDS staging maps ----------------------------------------------
  // K: piece i (0..3) of a thread = key 16 i + tid/16, 16-byte chunk tid%16.
  // V: a thread owns 4 keys of one slot group and one 8-d chunk.
  const int kchunk = tid & 15, kkey = tid >> 4;
  const int vg = tid >> 4;                                       // slot group: slots 4vg .. 4vg+3
  const int vkey0 = 32 * (vg >> 3) + 16 * ((vg >> 2) & 1) + 8 * (vg & 1) + 4 * ((vg >> 1) & 1);
  const int32_t* table = MODE != 0 ? p.block_tables + (long)b * p.max_blocks : nullptr;
  constexpr int ESZ = FP8 ? 1 : 2;                               // bytes per pool element
  const long kv_row_stride = (long)p.Hkv * HD * ESZ;             // bytes between consecutive tokens
  const char* kbase = (const char*)p.k + (long)hk * HD * ESZ;
  const char* vbase = (const char*)p.v + (long)hk * HD * ESZ;

  // generic: row of key `key` (clamped into the context), one table lookup per lane
  auto pool_row = [&](int key, int* blk_out) __attribute__((always_inline)) -> long {
    key = min(key, ctx - 1);
    if (MODE == 0) return (long)b * p.S + key;
    int blk, off;
    if (p.block_shift >= 0) { blk = table[key >> p.block_shift]; off = key & (p.block_size - 1); }
    else { blk = table[key / p.block_size]; off = key % p.block_size; }
    blk = min(max(blk, 0), p.num_blocks - 1);
    *blk_out = blk;
    return (long)blk * p.block_size + off;
  };
  // fast: first pool row of the 16-key group that starts at the wave-uniform key kb
  // (the group lies inside one block and inside the context)
  auto group_row = [&](int kb, int* blk_out) __attribute__((always_inline)) -> long {
    if (MODE == 0) return (long)b * p.S + kb;
    int blk = table[kb >> p.block_shift];
    blk = min(max(blk, 0), p.num_blocks - 1);
    *blk_out = blk;
    return (long)blk * p.block_size + (kb & (p.block_size - 1));
  };
  // per-lane byte offsets inside a 16-key group (constant over the whole loop): 8 elements per piece
  const int k_lane_off = (int)((kkey & 3) * kv_row_stride) + kchunk * 8 * ESZ;
  const int v_lane_off = (int)((vkey0 & 15) * kv_row_stride) + kchunk * 8 * ESZ;

  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  u32x4_t kreg[4], vreg[4];          // FP8: raw codes in .xy until store_tile expands them
  float kss[4], vss[4];              // FP8: scale of each piece's block
  auto fetch8 = [&](const char* src) __attribute__((always_inline)) -> u32x4_t {
    if (FP8) { const uint2 v = *(const uint2*)src; return u32x4_t{v.x, v.y, 0u, 0u}; }
    return *(const u32x4_t*)src;
  };
  auto load_tile = [&](int kt) __attribute__((always_inline)) {
    const int key0 = kt * BN;
    int blk = 0;
    if (MODE != 2 && key0 + BN <= ctx) {         // whole tile inside the context: uniform addressing
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const char* g = kbase + group_row(key0 + 16 * i + 4 * wave, &blk) * kv_row_stride;
        kreg[i] = fetch8(g + k_lane_off);
        if (FP8) kss[i] = p.k_scale[(long)blk * p.Hkv + hk];
      }
      const char* g = vbase + group_row(key0 + 32 * (wave >> 1) + 16 * (wave & 1), &blk) * kv_row_stride;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        vreg[i] = fetch8(g + v_lane_off + i * kv_row_stride);
        if (FP8) vss[i] = p.v_scale[(long)blk * p.Hkv + hk];
      }
    } else {                                      // last tile of a context, or odd block sizes
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        kreg[i] = fetch8(kbase + pool_row(key0 + 16 * i + kkey, &blk) * kv_row_stride + kchunk * 8 * ESZ);
        if (FP8) kss[i] = p.k_scale[(long)blk * p.Hkv + hk];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + vkey0 + i;
        vreg[i] = fetch8(vbase + pool_row(key, &blk) * kv_row_stride + kchunk * 8 * ESZ);
        if (FP8) vss[i] = p.v_scale[(long)blk * p.Hkv + hk];
        // rows past the context may hold anything (NaN patterns too); their weight is an
        // exact zero, which only helps if the value is finite
        if (key >= ctx) vreg[i] = u32x4_t{0u, 0u, 0u, 0u};
      }
    }
  };
  // FP8: 8 codes -> 8 bf16 values times the block's scale (rounded to nearest even)
  auto expand = [&](u32x4_t& r, float sc8) __attribute__((always_inline)) {
    float f[8];
    fp8x4_to_float(r[0], f);
    fp8x4_to_float(r[1], f + 4);
    r = u32x4_t{pack_bf16x2(f[0] * sc8, f[1] * sc8), pack_bf16x2(f[2] * sc8, f[3] * sc8),
                pack_bf16x2(f[4] * sc8, f[5] * sc8), pack_bf16x2(f[6] * sc8, f[7] * sc8)};
  };
  auto store_tile = [&](char* ks, char* vts) __attribute__((always_inline)) {
    if (FP8) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { expand(kreg[i], kss[i]); expand(vreg[i], vss[i]); }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) *(u32x4_t*)(ks + (16 * i + kkey) * K_ROW_BYTES + kchunk * 16) = kreg[i];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
      const uint32_t w0 = __builtin_amdgcn_perm(vreg[1][e >> 1], vreg[0][e >> 1], sel);   // keys 0,1 at d = 8c + e
      const uint32_t w1 = __builtin_amdgcn_perm(vreg[3][e >> 1], vreg[2][e >> 1], sel);   // keys 2,3
      *(uint2*)(vts + vt_row_offset(8 * kchunk + e) + vg * 8) = make_uint2(w0, w1);
    }
  };

  // ---- accumulators ------------------------------------------------------------
  f32x16_t oacc[HD / 32];
#pragma unroll
  for (int c = 0; c < HD / 32; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[c][i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float sc = p.scale_log2e;

  const int qblk = wq_lo / BN;                    // sparse: q block of this wave
  const int wg_blk_lo = q0 / BN, wg_blk_hi = (min(q0 + BM, tq) - 1) / BN;
  auto tile_needed = [&](int kt) __attribute__((always_inline)) -> bool {   // does any wave need key tile kt?
    if (!SPARSE) return true;
    for (int i = wg_blk_lo; i <= wg_blk_hi; ++i)
      if (block_active(i, kt, hq, p.sparse_local, p.sparse_stride)) return true;
    return false;
  };
  auto next_tile = [&](int kt) __attribute__((always_inline)) -> int {      // first needed tile >= kt
    while (kt < ntiles && !tile_needed(kt)) ++kt;
    return kt;
  };

  // lane-constant LDS read offsets
  const int k_rd_off = n * K_ROW_BYTES + 16 * h;
  const int v_rd_off = vt_row_offset(n) + 16 * h;   // + vt_row_offset(32 c) - vt_row_offset(0) per d chunk

  // Software pipeline over the needed tiles, one barrier per tile: tile j is computed from
  // LDS stage j%2; tile j+1, loaded into registers during tile j-1, is parked in the other
  // stage first, and tile j+2's global loads are in flight during the math.
  int kt = next_tile(0);
  int stage = 0;
  if (kt < ntiles) {
    load_tile(kt);
    store_tile(smem, smem + BN * K_ROW_BYTES);
  }
  int kt_next = kt < ntiles ? next_tile(kt + 1) : ntiles;
  if (kt_next < ntiles) load_tile(kt_next);
  __syncthreads();
  while (kt < ntiles) {
    char* ks = smem + stage * STAGE_BYTES;
    char* vts = ks + BN * K_ROW_BYTES;
    // registers hold tile kt_next: park it in the other stage (last read two tiles ago,
    // every wave has passed the barrier since), then request the tile after it
    const int kt_next2 = kt_next < ntiles ? next_tile(kt_next + 1) : ntiles;
    if (kt_next < ntiles) {
      char* ks2 = smem + (stage ^ 1) * STAGE_BYTES;
      store_tile(ks2, ks2 + BN * K_ROW_BYTES);
      if (kt_next2 < ntiles) load_tile(kt_next2);
    }

    const int key0 = kt * BN;
    bool active = wave_has_rows && key0 <= prefix + wq_hi;
    if (SPARSE) active = active && block_active(qblk, kt, hq, p.sparse_local, p.sparse_stride);
    if (active) {
      // ---- S^T = K Q^T ----
      f32x16_t sacc[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[tt][i] = 0.f;
#pragma unroll
        for (int s = 0; s < HD / 16; ++s) {
          const bf16x8_t kf = *(const bf16x8_t*)(ks + k_rd_off + 32 * tt * K_ROW_BYTES + 32 * s);
          sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], sacc[tt], 0, 0, 0);
        }
      }
      // ---- online softmax on this lane's column ----
      const bool need_mask = key0 + BN - 1 > prefix + wq_lo;    // tile reaches past the first row's diagonal
      float tmax = -INFINITY;
      if (need_mask) {
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = key0 + 32 * tt + 8 * (i >> 2) + 4 * h + (i & 3);
            sacc[tt][i] = key <= qlim ? sacc[tt][i] : -INFINITY;
          }
      }
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, sacc[tt][i]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64)) * sc;        // sc > 0: max commutes with the scale
      // a row whose visible keys all lie in later tiles keeps m = -inf for now
      const float m_new = fmaxf(m_run, tmax);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
      float psum = 0.f;
      uint32_t pw[2][8];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[tt][i], sc, -m_use));
          const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[tt][i + 1], sc, -m_use));
          psum += p0 + p1;
          pw[tt][i >> 1] = pack_bf16x2(p0, p1);
        }
      l_run = l_run * alpha + psum;
      if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {   // rescale only when some row's max moved
#pragma unroll
        for (int c = 0; c < HD / 32; ++c) oacc[c] *= alpha;
      }
      m_run = m_new;
      // ---- O^T += V^T P^T ----
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const bf16x8_t pf = as_bf16x8_prefill(pw[tt][4 * kk], pw[tt][4 * kk + 1], pw[tt][4 * kk + 2], pw[tt][4 * kk + 3]);
#pragma unroll
          for (int c = 0; c < HD / 32; ++c) {
            const bf16x8_t vf = *(const bf16x8_t*)(vts + v_rd_off + c * (32 * VT_ROW_BYTES + 4 * 16) + 16 * (4 * tt + 2 * kk));
            oacc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, oacc[c], 0, 0, 0);
          }
        }
    }
    __syncthreads();       // stage^1 is complete, stage is free
    kt = kt_next;
    kt_next = kt_next2;
    stage ^= 1;
  }

  // ---- normalise and write this lane's query row ---------------------------------
  l_run += __shfl_xor(l_run, 32, 64);
  // attention sink: a per-head logit that joins the softmax as one more column with no value
  if (p.sinks && l_run > 0.f) l_run += __builtin_amdgcn_exp2f(p.sinks[hq] * kLog2e - m_run);
  if (qrow < p.T && wq_lo < p.T) {
    uint16_t* op = out + ((long)b * p.T + qrow) * q_row_stride + (long)hq * HD;
    const float inv = (qvalid && l_run > 0.f) ? 1.f / l_run : 0.f;
#pragma unroll
    for (int c = 0; c < HD / 32; ++c)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d = 32 * c + 8 * i4 + 4 * h;
        const uint32_t w0 = qvalid ? pack_bf16x2(oacc[c][4 * i4] * inv, oacc[c][4 * i4 + 1] * inv) : 0u;
        const uint32_t w1 = qvalid ? pack_bf16x2(oacc[c][4 * i4 + 2] * inv, oacc[c][4 * i4 + 3] * inv) : 0u;
        *(uint2*)(op + d) = make_uint2(w0, w1);
      }
  }
}

constexpr int kPrefillLdsBytes = 2 * (BN * K_ROW_BYTES + VT_BYTES);

template <bool SPARSE, int MODE, bool FP8 = false>
hipError_t launch_prefill_typed(const PrefillParams& p, dim3 grid, hipStream_t s) {
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)prefill_kernel<SPARSE, MODE, FP8>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kPrefillLdsBytes);
    if (e != hipSuccess) return e;
    configured.store(1, std::memory_order_release);
  }
  hipLaunchKernelGGL((prefill_kernel<SPARSE, MODE, FP8>), grid, dim3(256), kPrefillLdsBytes, s, p);
  return hipGetLastError();
}

}  // namespace

bool prefill_supported(const PrefillParams& p) {
  if (p.D != HD) return false;
  if (p.block_tables && p.block_size <= 0) return false;
  return true;
}

hipError_t launch_prefill(const PrefillParams& p, hipStream_t s) {
  if (p.impl != 1 && prefill_async_supported(p))
    return launch_prefill_async(p, p.impl == 4 || p.impl == 8 ? p.impl : 0, s);
  const int nqt = (p.T + BM - 1) / BM;
  if (nqt > 65535 * 32 || p.Hq > 65535 || p.B > 65535) return hipErrorInvalidValue;
  dim3 grid(nqt, p.Hq, p.B);
  if (p.kv_fp8) {      // fp8 pools: the register-staged kernel expands the codes on their way into LDS
    if (!p.block_tables || p.sparse_stride > 0 || !p.k_scale || !p.v_scale) return hipErrorInvalidValue;
    if (p.block_shift >= 4) return launch_prefill_typed<false, 1, true>(p, grid, s);
    return launch_prefill_typed<false, 2, true>(p, grid, s);
  }
  if (p.sparse_stride > 0) return launch_prefill_typed<true, 0>(p, grid, s);
  if (!p.block_tables) return launch_prefill_typed<false, 0>(p, grid, s);
  if (p.block_shift >= 4) return launch_prefill_typed<false, 1>(p, grid, s);
  return launch_prefill_typed<false, 2>(p, grid, s);
}

}  // namespace pa
