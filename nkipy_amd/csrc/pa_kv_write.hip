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
//
// Optionally the reference's pre-attention step runs on the way (XFORM): QK RMSNorm
// (examples/models/qwen3/kernels/rmsnorm.py:4-21) and RoPE at the token's absolute position
// (rope.py:23-48; call sites qwen3/kernels/attention.py:78-97) are applied to the K rows before
// they are stored, and a second kernel does the same to Q in place.  A row of D elements is
// held by D/8 consecutive lanes, 8 elements each; the mean of squares is a butterfly over
// those lanes and the rotation partner (element i <-> i + D/2) sits D/16 lanes away.
#include <type_traits>

#include "pa_common.h"

#define PA_HD __device__ __forceinline__
#include "pa_div.h"

namespace pa {
namespace {

// What these kernels write (pool rows, transformed Q rows) goes out through streaming stores (pre-attention workload
// 0.085 -> 0.074 ms, plain write 21.9 -> 20.9 us); streaming the loads as well measured slower: the new rows come out
// of the kernel before this one.

constexpr int WG = 256;
// Waves per SIMD the write kernels are compiled for: their workgroups are short chains of dependent loads, so
// residency counts, but a register budget that makes the compiler spill costs more (a reload from scratch waits
// for every outstanding store as well).  6 (70 registers) for the plain forms, 4 (109) for the transforming fp8
// form, which holds four fetched chunks with their cos / sin pieces.  Measured on the KV-write and pre-attention
// workloads: (8, 8) 25.9 / 118.8 us per step, (6, 4) 20.0 / 85.6, (4, 4) 21.1 / 85.1.
constexpr int KVW_MIN_WAVES = 6, KVW_MIN_WAVES_XFORM = 4;
// The Q kernel: threads per workgroup and rows a thread has in flight (128 x 4 and 64 x 8 measured the same).
constexpr int QWG = 256, QUNR = 2;

// RMSNorm (if w) and RoPE of 8-element chunks of rows held by `cpr` consecutive lanes each.
// Arithmetic as the reference's bf16 tensors give it: the norm in float32 rounded once to bf16,
// every product and sum of the rotation rounded to bf16.

// value of lane ^ MASK (MASK a power of two below 32) without a trip through LDS memory
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
  if (MASK == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128 /* row_ror:8 */, 0xf, 0xf, true));
  return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (MASK << 10) | 0x1f));   // bit mode: and 0x1f, or 0, xor MASK
}
// Step MASK of a butterfly sum over aligned groups of lanes, steps taken in the order 1, 2, 4, ...: v + the value
// of a lane of the other half of the 2 MASK group.  Before step MASK all lanes of a MASK group hold the same
// partial sum, so any lane of the other half serves, and the data-parallel-primitive forms of the adds reach one:
// the quad permutations for 1 and 2, the mirror of 8 lanes for 4, of 16 lanes for 8.
template <int MASK>
__device__ __forceinline__ float butterfly_add(float v) {
  constexpr int ctrl = MASK == 1 ? 0xB1 /* quad_perm [1,0,3,2] */ : MASK == 2 ? 0x4E /* quad_perm [2,3,0,1] */
                     : MASK == 4 ? 0x141 /* row_half_mirror */ : 0x140 /* row_mirror */;
  if (MASK <= 8) return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xf, 0xf, true));
  return v + lane_xor<MASK>(v);
}
// two float32 -> two bf16 (round to nearest even) in one instruction, as one opaque operation: written as two
// scalar conversions the compiler takes the pair apart again where the halves are used separately
__device__ __forceinline__ uint32_t round2_bf16(float lo, float hi) {
  uint32_t w;
  asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w) : "v"(lo), "v"(hi));
  return w;
}
__device__ __forceinline__ void unpack_bf16x8(const uint4& v, float (&x)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    x[2 * j] = __uint_as_float(w[j] << 16);
    x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
  }
}

// What chunk c of a row needs of the position's cos / sin rows: 8 cosines and 8 sines as float32, the sines
// negated in the first half of the row.  First half: x0 c - x1 s with x0 = own; second half: x0 s + x1 c with
// x1 = own.  Both are round(round(own c) + round(other s')) with s' = -s in the first half: rounding to nearest
// even is symmetric in sign and the sum commutes, so the bits are those of the two written-out forms.
template <int CPR>
struct RopeCoeffs {
  float cs[8], sn[8];
  // the 16 bytes of each table row that chunk c needs, as they lie in memory
  static __device__ __forceinline__ void fetch(int c, const uint16_t* cos_row, const uint16_t* sin_row, uint4& cw, uint4& sw) {
    constexpr int hc = CPR / 2;
    const int fi = 8 * (c < hc ? c : c - hc);
    cw = *(const uint4*)(cos_row + fi);
    sw = *(const uint4*)(sin_row + fi);
  }
  __device__ __forceinline__ void set(int c, const uint4& cw, uint4 sw) {
    const uint32_t flip = c < CPR / 2 ? 0x80008000u : 0u;      // the sign, two elements per instruction
    sw.x ^= flip; sw.y ^= flip; sw.z ^= flip; sw.w ^= flip;
    unpack_bf16x8(cw, cs);
    unpack_bf16x8(sw, sn);
  }
  __device__ __forceinline__ void load(int c, const uint16_t* cos_row, const uint16_t* sin_row) {
    uint4 cw, sw;
    fetch(c, cos_row, sin_row, cw, sw);
    set(c, cw, sw);
  }
};

// CPR: lanes (8-element chunks) per row = D / 8, a compile-time power of two.  x: the chunk's values; all
// lanes of the row call this together.  wf: the chunk's norm weights (used if `norm`).  Returns the chunk
// as it is stored.
template <int CPR>
__device__ __forceinline__ uint4 norm_rope_chunk(float (&x)[8], bool norm, const float (&wf)[8], float eps, const RopeCoeffs<CPR>& rc) {
  constexpr int D = 8 * CPR;
  if (norm) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += x[j] * x[j];
    if (CPR > 1) ss = butterfly_add<1>(ss);
    if (CPR > 2) ss = butterfly_add<2>(ss);
    if (CPR > 4) ss = butterfly_add<4>(ss);
    if (CPR > 8) ss = butterfly_add<8>(ss);
    if (CPR > 16) ss = butterfly_add<16>(ss);
    // x / sqrt(mean + eps) as x * rsq(...): within 2 float32 ulp of the divided form, far below
    // the bf16 rounding that follows
    const float inv = __builtin_amdgcn_rsqf(__fdiv_rn(ss, (float)D) + eps);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t r = round2_bf16((x[2 * j] * inv) * wf[2 * j], (x[2 * j + 1] * inv) * wf[2 * j + 1]);
      x[2 * j] = __uint_as_float(r << 16);
      x[2 * j + 1] = __uint_as_float(r & 0xffff0000u);
    }
  }
  constexpr int hc = CPR / 2;
  uint32_t o[4];
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    const uint32_t a = round2_bf16(x[j] * rc.cs[j], x[j + 1] * rc.cs[j + 1]);
    const uint32_t b = round2_bf16(lane_xor<hc>(x[j]) * rc.sn[j], lane_xor<hc>(x[j + 1]) * rc.sn[j + 1]);
    o[j / 2] = round2_bf16(__uint_as_float(a << 16) + __uint_as_float(b << 16),
                           __uint_as_float(a & 0xffff0000u) + __uint_as_float(b & 0xffff0000u));
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}
__device__ __forceinline__ void load_norm_weights(const uint16_t* w, int c, float (&wf)[8]) {
  if (w) {
    unpack_bf16x8(*(const uint4*)(w + 8 * c), wf);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) wf[j] = 1.f;
  }
}

__device__ __forceinline__ void unpack8(const uint4& v, float (&x)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    x[2 * j] = bf16_bits_to_float(w[j] & 0xffffu);
    x[2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
  }
}
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
template <int ESZ, int XCPR>      // XCPR: D / 8 of a transforming write, 0 for a plain one
__global__ __launch_bounds__(WG) __attribute__((amdgpu_waves_per_eu(XCPR != 0 && ESZ == 1 ? KVW_MIN_WAVES_XFORM : KVW_MIN_WAVES, 8))) void kv_write_kernel(KvWriteParams p) {
  constexpr bool XFORM = XCPR != 0;
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

  // K rows of a transforming write: RMSNorm + RoPE at the row's absolute position
  const bool xf = XFORM && which == 0;
  // A chunk is fetched (the row's 16 bytes and, for a transforming write, the 16 bytes of the position's
  // cos and sin rows) and then finished (transformed): callers with several chunks fetch them all first.
  using Rope = RopeCoeffs<XFORM ? XCPR : 2>;
  struct RawChunk { uint4 v, cw, sw; };
  float k_wf[8];                                  // the lane's norm weights: its chunk index is the same for all its rows
  auto fetch_chunk = [&](const uint16_t* s0, int r, int c) __attribute__((always_inline)) -> RawChunk {
    RawChunk raw;
    raw.v = *(const uint4*)(s0 + (long)r * row_elems + c * 8);
    if (xf) {
      const int pos = min(jb * bs + lo + r, p.rope_max_pos - 1);
      Rope::fetch(c, p.rope_cos + (long)pos * (D / 2), p.rope_sin + (long)pos * (D / 2), raw.cw, raw.sw);
    }
    return raw;
  };
  auto finish_chunk = [&](const RawChunk& raw, int c) __attribute__((always_inline)) -> uint4 {
    if (!xf) return raw.v;
    float x[8];
    unpack8(raw.v, x);
    Rope rc;
    rc.set(c, raw.cw, raw.sw);
    return norm_rope_chunk<XFORM ? XCPR : 2>(x, p.k_norm_weight != nullptr, k_wf, p.norm_eps, rc);
  };
  auto load_row_chunk = [&](const uint16_t* s0, int r, int c) __attribute__((always_inline)) -> uint4 {
    return finish_chunk(fetch_chunk(s0, r, c), c);
  };

  // Chunk i = threadIdx.x + k WG of the slab is chunk c of row r; (r, c) walk along with i without divisions
  // (`cpr` is a run-time number for the plain kernels).
  const int cpr = XFORM ? XCPR : D * ESZ / (ESZ == 1 ? 8 : 16);   // chunks per row
  const int total = n * cpr;
  const int r_first = threadIdx.x / cpr, c_first = threadIdx.x - r_first * cpr;
  const int dr = WG / cpr, dc = WG - dr * cpr;
  auto advance = [&](int& r, int& c) __attribute__((always_inline)) {
    r += dr; c += dc;
    if (c >= cpr) { c -= cpr; ++r; }
  };
  if (xf) load_norm_weights(p.k_norm_weight, c_first, k_wf);   // (XCPR divides WG: c stays c_first)

  if (ESZ != 1) {
    // ---- copy: 16 bytes per thread and step
    const char* s0 = src + (((long)b * p.T + t0) * row_elems + (long)h * D) * ESZ;
    char* d0 = dst + (((long)blk * bs + lo) * row_elems + (long)h * D) * ESZ;
    int r = r_first, c = c_first;
    for (int i = threadIdx.x; i < total; i += WG, advance(r, c)) {
      uint4 v;
      if (ESZ == 2 && XFORM) v = load_row_chunk((const uint16_t*)s0, r, c);
      else v = *(const uint4*)(s0 + (long)r * row_elems * ESZ + c * 16);
      store_stream(d0 + (long)r * row_elems * ESZ + c * 16, v);
    }
    return;
  }

  // ---- fp8: source rows are bf16, 8 elements (16 B in, 8 B out) per thread and step
  float* scale_tbl = which ? p.v_scale : p.k_scale;
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
  {
    // all HOLD fetches go out before the first is used; a chunk past the slab's end reads row 0 instead (the
    // slab has one) and counts as zeros
    int r = r_first, c = c_first, i = threadIdx.x;
    RawChunk raw[HOLD];
    int ck[HOLD];
#pragma unroll
    for (int k = 0; k < HOLD; ++k, i += WG, advance(r, c)) {
      ck[k] = c;
      raw[k] = fetch_chunk(s0, i < total ? r : 0, c);
    }
#pragma unroll
    for (int k = 0; k < HOLD; ++k) {
      const uint4 v = finish_chunk(raw[k], ck[k]);
      held[k] = threadIdx.x + k * WG < total ? v : make_uint4(0, 0, 0, 0);
      chunk_absmax(held[k]);
    }
    for (; i < total; i += WG, advance(r, c)) chunk_absmax(load_row_chunk(s0, r, c));
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
  // x / s_new of the bf16 values x: the same bits from a product with the reciprocal and one correction
  // (pa_div.h) wherever s_new allows it, which is everywhere but at the far ends of the float32 range
  const float r_new = pa_refine_rcp(s_new, __builtin_amdgcn_rcpf(s_new));
  auto encode_store = [&](auto fast, const uint4& v, int r, int c) __attribute__((always_inline)) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float x0 = bf16_bits_to_float(w[j] & 0xffffu), x1 = bf16_bits_to_float(w[j] >> 16);
      f[2 * j] = decltype(fast)::value ? pa_div_by(x0, s_new, r_new) : __fdiv_rn(x0, s_new);
      f[2 * j + 1] = decltype(fast)::value ? pa_div_by(x1, s_new, r_new) : __fdiv_rn(x1, s_new);
    }
    uint2 o;
    o.x = pack_fp8x2(f[0], f[1], 0u, false); o.x = pack_fp8x2(f[2], f[3], o.x, true);
    o.y = pack_fp8x2(f[4], f[5], 0u, false); o.y = pack_fp8x2(f[6], f[7], o.y, true);
    store_stream(d_blk + (long)(lo + r) * row_elems + c * 8, o);
  };
  auto encode_all = [&](auto fast) __attribute__((always_inline)) {
    int r = r_first, c = c_first, i = threadIdx.x;
#pragma unroll
    for (int k = 0; k < HOLD; ++k, i += WG, advance(r, c))
      if (i < total) encode_store(fast, held[k], r, c);
    for (; i < total; i += WG, advance(r, c)) encode_store(fast, load_row_chunk(s0, r, c), r, c);
  };
  if (pa_div_by_ok(s_new, __float_as_uint(s_new))) encode_all(std::true_type{});
  else encode_all(std::false_type{});
  if (threadIdx.x == 0) scale_tbl[(long)blk * p.Hkv + h] = s_new;
}

// Q rows: RMSNorm + RoPE in place (or into q_out); rows t >= query_lens[b] become zeros.
// One workgroup per token (b, t): its Hq rows share the position, so no index arithmetic
// beyond the head stride is done per row.  A thread asks for UNR of its rows before it looks
// at the lengths (q_in holds all B * T tokens, so the addresses are valid for dead tokens too):
// the row loads do not wait behind the lengths -> position -> table-row chain, and UNR of them
// are in flight per lane.
template <int CPR, int WGQ, int UNR>
__global__ __launch_bounds__(WGQ) void q_norm_rope_kernel(KvWriteParams p) {
  constexpr int D = 8 * CPR, cpr = CPR, hstep = WGQ / cpr;
  const int t = blockIdx.x, b = blockIdx.y;
  const int c = threadIdx.x % cpr, h0 = threadIdx.x / cpr;
  const long tok = ((long)b * p.T + t) * p.Hq;
  if (h0 >= p.Hq) return;
  uint4 v[UNR];
  auto load_rows = [&](int hb) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      v[u] = make_uint4(0, 0, 0, 0);
      if (hb + u * hstep < p.Hq) v[u] = *(const uint4*)((const uint16_t*)p.q_in + (tok + hb + u * hstep) * D + c * 8);
    }
  };
  load_rows(h0);
  int tq = p.query_lens[b];
  tq = min(max(tq, 0), p.T);
  const int start = p.seq_lens[b] - tq;
  const bool live = t < tq && start >= 0;
  const int pos = min(max(start + t, 0), p.rope_max_pos - 1);
  RopeCoeffs<CPR> rc;      // the token's position and the lane's chunk are the same for all its rows
  float wf[8];
  if (live) {
    rc.load(c, p.rope_cos + (long)pos * (D / 2), p.rope_sin + (long)pos * (D / 2));
    load_norm_weights(p.q_norm_weight, c, wf);
  }
  for (int hb = h0;;) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      if (hb + u * hstep >= p.Hq) break;
      if (live) {
        float x[8];
        unpack8(v[u], x);
        v[u] = norm_rope_chunk<CPR>(x, p.q_norm_weight != nullptr, wf, p.norm_eps, rc);
      } else {
        v[u] = make_uint4(0, 0, 0, 0);
      }
      store_stream((uint16_t*)p.q_out + (tok + hb + u * hstep) * D + c * 8, v[u]);
    }
    hb += UNR * hstep;
    if (hb >= p.Hq) break;
    load_rows(hb);
  }
}

template <int CPR>
void launch_xform(const KvWriteParams& p, dim3 grid, hipStream_t s) {
  if (p.q_in) hipLaunchKernelGGL((q_norm_rope_kernel<CPR, QWG, QUNR>), dim3(p.T, p.B), dim3(QWG), 0, s, p);
  if (p.kv_dtype == PA_FP8_E4M3FN) hipLaunchKernelGGL((kv_write_kernel<1, CPR>), grid, dim3(WG), 0, s, p);
  else hipLaunchKernelGGL((kv_write_kernel<2, CPR>), grid, dim3(WG), 0, s, p);
}

}  // namespace

bool kv_write_xform_supported(int D) { return D == 64 || D == 128 || D == 256; }

hipError_t launch_kv_write(const KvWriteParams& p, hipStream_t s) {
  const int touched = (p.T + p.block_size - 1) / p.block_size + 1;   // a chunk of T rows spans at most this many blocks
  const dim3 grid(2 * touched, p.Hkv, p.B);
  if (p.rope_cos != nullptr) {
    if (p.D == 64) launch_xform<8>(p, grid, s);
    else if (p.D == 128) launch_xform<16>(p, grid, s);
    else if (p.D == 256) launch_xform<32>(p, grid, s);
    else return hipErrorInvalidValue;
    return hipGetLastError();
  }
  if (p.kv_dtype == PA_FP8_E4M3FN) hipLaunchKernelGGL((kv_write_kernel<1, 0>), grid, dim3(WG), 0, s, p);
  else if (p.kv_dtype == PA_BF16) hipLaunchKernelGGL((kv_write_kernel<2, 0>), grid, dim3(WG), 0, s, p);
  else hipLaunchKernelGGL((kv_write_kernel<4, 0>), grid, dim3(WG), 0, s, p);
  return hipGetLastError();
}

}  // namespace pa
