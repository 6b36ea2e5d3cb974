// Shared device helpers and launch parameter blocks for the paged attention
// kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/paged_attn.h"

namespace pa {

constexpr float kLog2e = 1.4426950408889634f;

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// ---- host-side error text (thread local) -----------------------------------
void set_error(const char* fmt, ...);
int fail_arg(const char* fmt, ...);     // records the text, returns -1
int check_hip(hipError_t e, const char* what);

// ---- profiling hooks ----------------------------------------------------------
void profile_begin(hipStream_t s);
void profile_end(hipStream_t s);

// ---- storage helpers ------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// two floats -> packed bf16 pair (lo = a, hi = b), round-to-nearest-even
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  bf16x2_t v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}

// Stores of data that is written once and read by a later kernel (attention and projection outputs, pool rows,
// transformed Q rows): as streaming (non-temporal) stores they do not displace what the running kernels reuse.
// Measured per kernel where they are used; 1-2 % on the matrix-core kernels, 5-15 % on the write kernels.
__device__ __forceinline__ void store_stream(void* p, const uint4& v) {
  typedef uint32_t stream_u32x4 __attribute__((ext_vector_type(4)));
  const stream_u32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, (stream_u32x4*)p);
}
__device__ __forceinline__ void store_stream(void* p, const uint2& v) {
  typedef uint32_t stream_u32x2 __attribute__((ext_vector_type(2)));
  const stream_u32x2 w = {v.x, v.y};
  __builtin_nontemporal_store(w, (stream_u32x2*)p);
}

// four OCP e4m3fn bytes of one dword -> four floats (exact)
__device__ __forceinline__ void fp8x4_to_float(uint32_t w, float* f) {
  f32x2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
  f32x2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
  f[0] = lo.x; f[1] = lo.y; f[2] = hi.x; f[3] = hi.y;
}

// two OCP e4m3fn bytes (the low or the high half of w) -> a bf16 pair, exact, in one instruction: the scaled
// conversion takes its scale's exponent only, and 1.0 leaves the values as they are (every e4m3 value is a bf16 value)
template <bool HIGH_HALF>
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t w) {
  typedef __bf16 bf16_pair_t __attribute__((ext_vector_type(2)));
  const bf16_pair_t v = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, 1.0f, HIGH_HALF);
  return __builtin_bit_cast(uint32_t, v);
}

// high halves of two floats packed as a bf16 pair (exact when both values are
// representable in bf16, as every e4m3 value is): lo = a, hi = b
__device__ __forceinline__ uint32_t pack_hi16(float a, float b) {
  return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}

template <typename T> struct Store;
template <> struct Store<float> {
  static __device__ __forceinline__ void put(void* base, long idx, float v) { ((float*)base)[idx] = v; }
};
template <> struct Store<uint16_t> {
  static __device__ __forceinline__ void put(void* base, long idx, float v) {
    ((uint16_t*)base)[idx] = float_to_bf16_bits(v);
  }
};

// ---- Q transform on load ---------------------------------------------------------
// The reference's pre-attention step on Q (QK RMSNorm, examples/models/qwen3/kernels/rmsnorm.py:4-21;
// RoPE at the token's absolute position, rope.py:23-48) applied by the attention kernel to the Q
// rows as it loads them, instead of by a kernel of its own that reads and rewrites Q.
struct QTransform {
  const uint16_t* norm_weight;  // [D] bf16 or null (no norm)
  const uint16_t* cos;          // [max_pos, D/2] bf16; null: no transform at all
  const uint16_t* sin;
  int max_pos;
  float eps;
};

// A lane holds NS chunks of 8 consecutive elements of one row of 8 * CPR elements; the other
// chunks of the row are held by lanes whose number differs in bits of L's choosing.  L says
// where chunk index bit `bit` lives: in the lane's slot number s (L::slot_xor(bit) != 0) or in
// the lane number (L::lane_xor(bit) != 0), and L::chunk(s, part) numbers the chunk held in slot
// s by a lane whose part number is `part`.  The arithmetic and its order are those of the
// stand-alone transform kernel (mean of squares as a butterfly over the chunk index, norm in
// float32 rounded once to bf16, every product and sum of the rotation rounded to bf16), so
// the two give the same bits.
// The transform comes in two halves so that a caller can put other memory requests between them: the loads of
// what it needs from the tables (norm weights, the position's cos and sin rows), and the arithmetic.
template <int NS>
struct NormRopeCoeffs {
  uint4 w[NS], cs[NS], sn[NS];
};
template <int CPR, int NS, class L>
__device__ __forceinline__ void norm_rope_fetch(const QTransform& t, int pos, int part, NormRopeCoeffs<NS>& c) {
  constexpr int D = 8 * CPR;
  constexpr int hc = CPR / 2;
  const uint16_t* cos_row = t.cos + (long)pos * (D / 2);
  const uint16_t* sin_row = t.sin + (long)pos * (D / 2);
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int ch = L::chunk(s, part);
    const int fi = 8 * (ch < hc ? ch : ch - hc);
    c.cs[s] = *(const uint4*)(cos_row + fi);
    c.sn[s] = *(const uint4*)(sin_row + fi);
    c.w[s] = make_uint4(0, 0, 0, 0);
    if (t.norm_weight) c.w[s] = *(const uint4*)(t.norm_weight + 8 * ch);
  }
}
template <int CPR, int NS, class L>
__device__ __forceinline__ void norm_rope_apply(float (&x)[NS][8], const QTransform& t, int part, const NormRopeCoeffs<NS>& c) {
  constexpr int D = 8 * CPR;
  auto r16 = [](float f) __attribute__((always_inline)) { return __uint_as_float(pack_bf16x2(f, 0.f) << 16); };
  auto unpack = [](const uint4& v, float (&f)[8]) __attribute__((always_inline)) {
    const uint32_t a[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = bf16_bits_to_float(a[j] & 0xffffu);
      f[2 * j + 1] = bf16_bits_to_float(a[j] >> 16);
    }
  };
  if (t.norm_weight) {
    float ss[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      ss[s] = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss[s] += x[s][j] * x[s][j];
    }
#pragma unroll
    for (int bit = 1; bit < CPR; bit <<= 1) {
      float nx[NS];
#pragma unroll
      for (int s = 0; s < NS; ++s)
        nx[s] = ss[s] + (L::slot_xor(bit) ? ss[s ^ L::slot_xor(bit)] : __shfl_xor(ss[s], L::lane_xor(bit)));
#pragma unroll
      for (int s = 0; s < NS; ++s) ss[s] = nx[s];
    }
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const float inv = __builtin_amdgcn_rsqf(__fdiv_rn(ss[s], (float)D) + t.eps);
      float w[8];
      unpack(c.w[s], w);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[s][j] = r16((x[s][j] * inv) * w[j]);
    }
  }
  constexpr int hc = CPR / 2;
  float y[NS][8];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int ch = L::chunk(s, part);
    const bool first = ch < hc;
    float cs[8], sn[8];
    unpack(c.cs[s], cs);
    unpack(c.sn[s], sn);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float other = L::slot_xor(hc) ? x[s ^ L::slot_xor(hc)][j] : __shfl_xor(x[s][j], L::lane_xor(hc));
      y[s][j] = first ? r16(r16(x[s][j] * cs[j]) - r16(other * sn[j])) : r16(r16(other * sn[j]) + r16(x[s][j] * cs[j]));
    }
  }
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int j = 0; j < 8; ++j) x[s][j] = y[s][j];
}
template <int CPR, int NS, class L>
__device__ __forceinline__ void q_norm_rope_lane(float (&x)[NS][8], const QTransform& t, int pos, int part) {
  NormRopeCoeffs<NS> c;
  norm_rope_fetch<CPR, NS, L>(t, pos, part, c);
  norm_rope_apply<CPR, NS, L>(x, t, part, c);
}

// ---- decode ------------------------------------------------------------------------
struct DecodeParams {
  const void* q;            // [B, Hq, D]; [B, T, Hq, D] for a multi-token call
  const void* k_cache;      // [num_blocks, block_size, Hkv, D]
  const void* v_cache;
  const float* k_scale;     // [num_blocks, Hkv] or null
  const float* v_scale;
  const int32_t* block_tables;  // [B, max_blocks]
  const int32_t* seq_lens;      // [B]
  const int32_t* query_lens;    // [B] for a multi-token call (balanced schedule only), else null
  void* out;                // shaped like q
  float* ws_out;            // [B, Hq, P, D]
  float* ws_ml;             // [B, Hq, P, 2]
  int32_t* ws_start;        // balanced schedule: [B + 1] tiles before each sequence, and the total
  int B, Hq, Hkv, D;
  int T;                    // query tokens per sequence in this launch (1: decode)
  int T_stride, t0;         // multi-token launches: tokens per sequence in q / out, and the first one this launch covers
  int window;               // sliding window in tokens (balanced schedule only), 0 = none
  const float* sinks;       // [Hq] per-head sink logits (balanced schedule only) or null
  int rows_per_wave;        // query rows of a kv head carried by one wavefront: 16, or 32 (multi-token calls only)
  int block_size, max_blocks, num_blocks;
  int block_shift;          // log2(block_size), or -1 when not a power of two
  int partition_size, num_partitions, max_seq_len;
  float scale_log2e;
  int head_major;           // fixed-partition grid order: kv head fastest (1) or partition fastest (0)
  int bal_hsw, bal_ns, bal_gv;  // balanced schedule: head slots and chunks per workgroup, total chunks
  int bal_lockstep;         // keep the head waves of a workgroup on the same tile with a barrier
  QTransform qt;            // balanced schedule only: Q rows are normed and rotated as they are loaded
  // Fixed-partition kernels, bf16 pools: the step's new token handed over with the call instead of written to the
  // pool by a launch of its own.  Row (b, kv head) of new_k / new_v [B, Hkv, D] bf16 is token seq_lens[b] - 1 of
  // sequence b (the reference's cache update, examples/models/qwen3/kernels/attention.py:100-106): the wave that
  // reaches that token attends to it from registers, and one wave per (sequence, kv head) stores it in the pool.
  // new_kt is the K half of the pre-attention transform (its norm weight is K's; cos null: rows go in as given).
  // Sequences with new_lens[b] == 0 take no new token (null: every sequence takes one).
  const void* new_k;
  const void* new_v;
  const int32_t* new_lens;
  QTransform new_kt;
};

hipError_t launch_decode_generic(const DecodeParams& p, int q_dtype, int kv_dtype, hipStream_t s);
hipError_t launch_decode_mfma(const DecodeParams& p, int kv_dtype, int waves, hipStream_t s);
bool decode_new_row_supported(const DecodeParams& p, int q_dtype, int kv_dtype);   // shapes whose fixed-partition kernels take p.new_k
bool decode_mfma_supported(const DecodeParams& p, int q_dtype, int kv_dtype);
hipError_t launch_decode_reduce(const DecodeParams& p, int q_dtype, hipStream_t s);
void plan_decode_balanced(DecodeParams& p, int num_cus);
size_t decode_balanced_workspace_bytes(int B, int Hq, int D, int gv);
hipError_t launch_decode_balanced(const DecodeParams& p, int kv_dtype, hipStream_t s);
hipError_t launch_decode_balanced_reduce(const DecodeParams& p, hipStream_t s);

// ---- prefill -----------------------------------------------------------------------
struct PrefillParams {
  const void* q;            // [B, T, Hq, D] bf16
  const void* k;            // paged: pool [num_blocks, block_size, Hkv, D]; dense: [B, S, Hkv, D]
  const void* v;
  const int32_t* block_tables;  // null for the dense (blocksparse) form
  const int32_t* seq_lens;      // null for the dense form (then every sequence has S keys)
  const int32_t* query_lens;    // null for the dense form (then T queries)
  void* out;
  int B, T, Hq, Hkv, D;
  int block_size, max_blocks, num_blocks;
  int block_shift;          // log2(block_size), or -1 when not a power of two
  int S;                    // dense form: keys per sequence
  int sparse_local, sparse_stride;  // blocksparse pattern; sparse_stride == 0 -> plain causal
  float scale_log2e;
  int impl;                 // 0 automatic, 1 register-staged, 4 / 8 asynchronous (waves per workgroup), 5 asynchronous with packed rows,
                            // 6 asynchronous, head dim 64 with one q head per wave
  int window;               // paged form, asynchronous kernel only: sliding window in tokens, 0 = none
  const float* sinks;       // same: [Hq] per-head sink logits or null
  int kv_fp8;               // paged form: the pool holds e4m3fn codes (register-staged kernel only)
  const float* k_scale;     // kv_fp8: [num_blocks, Hkv] scales
  const float* v_scale;
  int splits;               // same: workgroups sharing the key tiles of one query tile (1: no split)
  float* ws_o;              // splits > 1: [B * T * Hq, splits, D] partial outputs
  float* ws_ml;             // splits > 1: [B * T * Hq, splits, 2] partial (max, sum)
  QTransform qt;            // asynchronous kernel only: Q rows are normed and rotated as they are loaded
  int num_cus;              // CUs of the device the call runs on (0: unknown, taken as 256); steers the workgroup shape
  int len_bound;            // the caller's bound on the sequence lengths (0: none); steers the workgroup shape as well
};

hipError_t launch_prefill(const PrefillParams& p, hipStream_t s);
int prefill_async_splits(const PrefillParams& p, int num_cus, int max_seq_len = 0);   // split the launcher would like for this call (max_seq_len: the caller's bound on the lengths, 0 = none)
bool prefill_supported(const PrefillParams& p);
hipError_t launch_prefill_async(const PrefillParams& p, int waves, hipStream_t s);
bool prefill_async_supported(const PrefillParams& p);

// ---- gather ------------------------------------------------------------------------
// ---- paged KV write --------------------------------------------------------------
struct KvWriteParams {
  const void* k_new;        // [B, T, Hkv, D] bf16 (fp32 for an fp32 pool)
  const void* v_new;
  void* k_cache;            // [num_blocks, block_size, Hkv, D]
  void* v_cache;
  float* k_scale;           // [num_blocks, Hkv] (fp8 pools) or null
  float* v_scale;
  const int32_t* block_tables;
  const int32_t* seq_lens;
  const int32_t* query_lens;
  int B, T, Hkv, D, block_size, max_blocks, num_blocks, kv_dtype;
  // pre-attention transform (all null / zero for a plain write): RMSNorm weights [D] bf16 (null: no
  // norm), RoPE tables [rope_max_pos, D/2] bf16, Q rows [B, T, Hq, D] bf16 transformed into q_out
  const void* q_in;
  void* q_out;
  const uint16_t* q_norm_weight;
  const uint16_t* k_norm_weight;
  const uint16_t* rope_cos;
  const uint16_t* rope_sin;
  float norm_eps;
  int Hq, rope_max_pos;
};
hipError_t launch_kv_write(const KvWriteParams& p, hipStream_t s);
bool kv_write_xform_supported(int D);   // head dims the fused RMSNorm + RoPE write is built for

// ---- post-attention output projection ---------------------------------------------------
struct OProjParams {
  const void* x;            // [M, K] bf16: attention output, tokens x (Hq * D)
  const void* w;            // [K, N] bf16, row-major
  const void* bias;         // [N] bf16 or null
  void* out;                // [M, N] bf16
  int M, K, N;
  float* ws;                // split form: [splits, M, N] float32 partial products, or null
  int splits;               // K ranges summed by a second kernel (1: none); o_proj_splits() or less
  // The resident few-rows form can take its x rows from the split-K partials of a fixed-partition decode launch
  // instead of from memory (x null): row m of x is the attention output [Hq * D] of one (sequence, query token),
  // merged from the sequence's partitions while the tile is formed, with the arithmetic of decode_reduce_kernel.
  const float* part_o;      // [B, Hq * T rows, np, D] normalised partial outputs (rows numbered as the decode kernels do)
  const float* part_ml;     // [B, Hq * T rows, np, 2] (max, sum) of each partial
  const int32_t* part_seq_lens;   // [B] context lengths (clamped to part_max_seq_len as the decode launch did)
  const int32_t* part_query_lens; // multi-token launch: [B] query tokens per sequence; null for decode
  const float* part_sinks;        // [Hq] sink logits of the attention call (one more term of each row's denominator), or null
  int part_np, part_size, part_max_seq_len, part_D;
  int part_T, part_n_rep;         // tokens per sequence in the launch (x row m is token m % T of sequence m / T), q heads per kv head
};
hipError_t launch_o_proj(const OProjParams& p, hipStream_t s);
int o_proj_splits(int M, int K, int N);     // K ranges the few-rows forms would like to spread over more workgroups
bool o_proj_takes_partials(int M, int K, int D, int splits, bool have_ws);   // launch_o_proj can merge decode partials on its x load
void o_proj_debug_force_large(int on);      // debug: 256 x 256 tiles also where the 128 x 128 form would be taken

hipError_t launch_gather(const void* cache, const int32_t* tables, const int32_t* seq_lens, void* out,
                         int B, int row_bytes, int block_size, int max_blocks, int num_blocks,
                         int max_seq_len, hipStream_t s);

}  // namespace pa
