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
#include "pa_common.h"

namespace pa {
namespace {

constexpr int WG = 256;

// RMSNorm (if w) and RoPE of one 8-element chunk c of a row held by `cpr` consecutive lanes.
// x: the chunk's values; all lanes of the row call this together.  Arithmetic as the
// reference's bf16 tensors give it: the norm in float32 rounded once to bf16, every product
// and sum of the rotation rounded to bf16.
// value of lane ^ MASK (MASK a power of two below 32) without a trip through LDS memory
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
  if (MASK == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128 /* row_ror:8 */, 0xf, 0xf, true));
  return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (MASK << 10) | 0x1f));   // bit mode: and 0x1f, or 0, xor MASK
}
// CPR: lanes (8-element chunks) per row = D / 8, a compile-time power of two
template <int CPR>
__device__ __forceinline__ void norm_rope_chunk(float (&x)[8], int c, const uint16_t* w, float eps,
                                                const uint16_t* cos_row, const uint16_t* sin_row) {
  constexpr int D = 8 * CPR;
  // (roundings to bf16 go through the conversion instruction, round to nearest even, two values at a time)
  if (w) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += x[j] * x[j];
    if (CPR > 1) ss += lane_xor<1>(ss);
    if (CPR > 2) ss += lane_xor<2>(ss);
    if (CPR > 4) ss += lane_xor<4>(ss);
    if (CPR > 8) ss += lane_xor<8>(ss);
    if (CPR > 16) ss += lane_xor<16>(ss);
    // x / sqrt(mean + eps) as x * rsq(...): within 2 float32 ulp of the divided form, far below
    // the bf16 rounding that follows
    const float inv = __builtin_amdgcn_rsqf(__fdiv_rn(ss, (float)D) + eps);
    const uint4 ww = *(const uint4*)(w + 8 * c);
    const uint32_t wv[4] = {ww.x, ww.y, ww.z, ww.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t r = pack_bf16x2((x[2 * j] * inv) * bf16_bits_to_float(wv[j] & 0xffffu), (x[2 * j + 1] * inv) * bf16_bits_to_float(wv[j] >> 16));
      x[2 * j] = __uint_as_float(r << 16);
      x[2 * j + 1] = __uint_as_float(r & 0xffff0000u);
    }
  }
  constexpr int hc = CPR / 2;
  const bool first = c < hc;
  const int fi = 8 * (first ? c : c - hc);
  const uint4 cw = *(const uint4*)(cos_row + fi);
  uint4 sw = *(const uint4*)(sin_row + fi);
  // first half: x0 c - x1 s with x0 = own; second half: x0 s + x1 c with x1 = own.  Both are
  // round(round(own c) + round(other s')) with s' = -s in the first half: rounding to nearest even is
  // symmetric in sign and the sum commutes, so the bits are those of the two written-out forms.  The sign
  // goes into the packed sine words, two elements per instruction.
  const uint32_t flip = first ? 0x80008000u : 0u;
  sw.x ^= flip; sw.y ^= flip; sw.z ^= flip; sw.w ^= flip;
  float cs[8], sn[8];
  {
    const uint32_t a[4] = {cw.x, cw.y, cw.z, cw.w}, b[4] = {sw.x, sw.y, sw.z, sw.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      cs[2 * j] = bf16_bits_to_float(a[j] & 0xffffu); cs[2 * j + 1] = bf16_bits_to_float(a[j] >> 16);
      sn[2 * j] = bf16_bits_to_float(b[j] & 0xffffu); sn[2 * j + 1] = bf16_bits_to_float(b[j] >> 16);
    }
  }
  // two roundings per conversion instruction
  auto r16x2 = [](float& f0, float& f1) __attribute__((always_inline)) {
    const uint32_t w = pack_bf16x2(f0, f1);
    f0 = __uint_as_float(w << 16);
    f1 = __uint_as_float(w & 0xffff0000u);
  };
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    float a0 = x[j] * cs[j], a1 = x[j + 1] * cs[j + 1];
    float b0 = lane_xor<hc>(x[j]) * sn[j], b1 = lane_xor<hc>(x[j + 1]) * sn[j + 1];
    r16x2(a0, a1);
    r16x2(b0, b1);
    float s0 = a0 + b0, s1 = a1 + b1;
    r16x2(s0, s1);
    x[j] = s0; x[j + 1] = s1;
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
__device__ __forceinline__ uint4 pack8(const float (&x)[8]) {   // values already bf16-representable or to be rounded
  return make_uint4(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]), pack_bf16x2(x[6], x[7]));
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
// (eight waves per SIMD: the workgroups are short chains of dependent loads, and more of them resident measured 2-3 % faster
// than the 96 registers the compiler takes when left alone)
__global__ __launch_bounds__(WG) __attribute__((amdgpu_waves_per_eu(8, 8))) void kv_write_kernel(KvWriteParams p) {
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
  auto load_row_chunk = [&](const uint16_t* s0, int r, int c, int cpr) __attribute__((always_inline)) -> uint4 {
    uint4 v = *(const uint4*)(s0 + (long)r * row_elems + c * 8);
    if (xf) {
      const int pos = min(jb * bs + lo + r, p.rope_max_pos - 1);
      float x[8];
      unpack8(v, x);
      norm_rope_chunk<XFORM ? XCPR : 2>(x, c, p.k_norm_weight, p.norm_eps, p.rope_cos + (long)pos * (D / 2), p.rope_sin + (long)pos * (D / 2));
      v = pack8(x);
    }
    return v;
  };

  if (ESZ != 1) {
    // ---- copy: 16 bytes per thread and step
    const int cpr = D * ESZ / 16;               // chunks per row
    const char* s0 = src + (((long)b * p.T + t0) * row_elems + (long)h * D) * ESZ;
    char* d0 = dst + (((long)blk * bs + lo) * row_elems + (long)h * D) * ESZ;
    for (int i = threadIdx.x; i < n * cpr; i += WG) {
      const int r = i / cpr, c = i - r * cpr;
      uint4 v;
      if (ESZ == 2 && XFORM) v = load_row_chunk((const uint16_t*)s0, r, c, cpr);
      else v = *(const uint4*)(s0 + (long)r * row_elems * ESZ + c * 16);
      *(uint4*)(d0 + (long)r * row_elems * ESZ + c * 16) = v;
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
      held[k] = load_row_chunk(s0, r, c, cpr);
    }
    chunk_absmax(held[k]);
  }
  for (int i = threadIdx.x + HOLD * WG; i < n * cpr; i += WG) {
    const int r = i / cpr, c = i - r * cpr;
    chunk_absmax(load_row_chunk(s0, r, c, cpr));
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
    encode_store(load_row_chunk(s0, r, c, cpr), i);
  }
  if (threadIdx.x == 0) scale_tbl[(long)blk * p.Hkv + h] = s_new;
}

// Q rows: RMSNorm + RoPE in place (or into q_out); rows t >= query_lens[b] become zeros.
// One workgroup per token (b, t): its Hq rows share the position, so no index arithmetic
// beyond the head stride is done per row.
template <int CPR>
__global__ __launch_bounds__(WG) void q_norm_rope_kernel(KvWriteParams p) {
  constexpr int D = 8 * CPR, cpr = CPR;
  const int t = blockIdx.x, b = blockIdx.y;
  const int c = threadIdx.x % cpr, h0 = threadIdx.x / cpr, hstep = WG / cpr;
  int tq = p.query_lens[b];
  tq = min(max(tq, 0), p.T);
  const int start = p.seq_lens[b] - tq;
  const bool live = t < tq && start >= 0;
  const int pos = min(max(start + t, 0), p.rope_max_pos - 1);
  const long tok = ((long)b * p.T + t) * p.Hq;
  for (int hq = h0; hq < p.Hq; hq += hstep) {
    const long off = (tok + hq) * D + c * 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (live) {
      v = *(const uint4*)((const uint16_t*)p.q_in + off);
      float x[8];
      unpack8(v, x);
      norm_rope_chunk<CPR>(x, c, p.q_norm_weight, p.norm_eps, p.rope_cos + (long)pos * (D / 2), p.rope_sin + (long)pos * (D / 2));
      v = pack8(x);
    }
    *(uint4*)((uint16_t*)p.q_out + off) = v;
  }
}

template <int CPR>
void launch_xform(const KvWriteParams& p, dim3 grid, hipStream_t s) {
  if (p.q_in) hipLaunchKernelGGL(q_norm_rope_kernel<CPR>, dim3(p.T, p.B), dim3(WG), 0, s, p);
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
