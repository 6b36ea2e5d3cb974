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

// N dwords per lane; NT: a streaming (non-temporal) load, for bytes that are read once
template <int N, bool NT = false> struct VecLoad;
template <bool NT> struct VecLoad<1, NT> {
  static __device__ __forceinline__ void get(const void* p, uint32_t* r) { r[0] = *(const uint32_t*)p; }
};
template <bool NT> struct VecLoad<2, NT> {
  static __device__ __forceinline__ void get(const void* p, uint32_t* r) {
    typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
    const u2_t v = NT ? __builtin_nontemporal_load((const u2_t*)p) : *(const u2_t*)p;
    r[0] = v.x; r[1] = v.y;
  }
};
template <bool NT> struct VecLoad<4, NT> {
  static __device__ __forceinline__ void get(const void* p, uint32_t* r) {
    typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
    const u4_t v = NT ? __builtin_nontemporal_load((const u4_t*)p) : *(const u4_t*)p;
    r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
  }
};
// V rows are read whole by one instruction and never again: streamed, they stop displacing what is reused.  K in
// its operand order is fetched in 64-byte pieces, two instructions per 128-byte line: streaming that as well (or
// instead) measured slower; DecodeWave::load_k has a second form that fetches whole lines and can be streamed.
// Paged decode (64 sequences, 512-8192 tokens), kernel us, K / V plain-plain, streamed-streamed, streamed-plain,
// plain-streamed: bf16 187.2, 175.9, 181.1, 169.2; fp8 (twice the sequences) 403.2, 415.4, 425.9, 384.4; the
// four-token verify 197.4, 190.2, 193.6, 179.8.
// V is streamed only by the wave that is the rows' one reader: with more than one 16 R-row group per kv head the
// other groups' waves read the same rows again and should find them in the cache (verify with 32 rows per kv head on
// two waves: 229 us cached, 257 us streamed), hence the SV template argument, chosen per launch.  (A run-time choice
// puts the loads into a conditional, which costs the decode kernel 4 %.)
constexpr bool kStreamK = false;

__device__ __forceinline__ bf16x8_t as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  uint4 v = make_uint4(a, b, c, d);
  return __builtin_bit_cast(bf16x8_t, v);
}

// One 32-token tile as loaded (raw bits), K and V halves separately so that
// their register lifetimes can interleave (K of tile n dies after the scores,
// which frees its registers for V of tile n+1).
template <int D, bool FP8>
struct KTile {
  static constexpr int KLD = FP8 ? D / 64 : D / 32;        // 16-byte K loads per 16-token sub-tile
  uint32_t k[2][KLD][4];
  float ksc[2];             // fp8 only: scales of the two 16-token halves
};
template <int D, bool FP8>
struct VTile {
  static constexpr int VEC = D / 16;                       // d's per lane for V
  static constexpr int VW = (VEC * (FP8 ? 1 : 2)) / 4;     // dwords per V load
  uint32_t v[8][VW];
  float vsc[2];
};

// Per-wavefront streaming state: Q fragments, online-softmax state and output
// accumulators for R groups of up to 16 query rows of one kv head of one sequence.
//
// MULTI = false: one query token per sequence; the rows are the q heads of the
// kv group.  MULTI = true: p.T query tokens per sequence (the last query_lens[b]
// tokens of the context, K/V already in the pool); the rows of a kv group are
// its n_rep * T (token, head) pairs, token-major, numbered as "virtual heads"
// hk * n_rep * T + t * n_rep + head.  Row (t, .) sees keys
// < ctx - tq + t + 1, so the causal mask is one more per-lane bound on the token
// index; a row may then see no key at all in a tile or in a whole chunk, which the
// softmax update and the stores allow for (state m = -inf, l = 0, o = 0).
// R = 2 (MULTI only): the wave carries two 16-row operands, rows jbase + 16 rg + r,
// against the same K and V registers, so a kv group of up to 32 rows streams its
// context once through one wave.  LEAN (for R = 2 at D = 128, which would not fit
// 256 registers otherwise): the Q fragments live in LDS, each lane reading back
// the 16-byte pieces it wrote itself (no conflicts, no barrier), and V is single-
// buffered: the next tile's V is requested right after the current P.V.
// Where the 8-element chunks of a Q row sit in the Q^T operand: lane (g, r) holds, in k-step s,
// chunk 4 s + g (bf16 pools) or 8 (s >> 1) + 2 g + (s & 1) (fp8 pools, whose K loads cover 16
// elements of a row per lane).  g is lane >> 4.
template <bool FP8>
struct QOperandLayout {
  static __device__ __forceinline__ int chunk(int s, int g) { return FP8 ? 8 * (s >> 1) + 2 * g + (s & 1) : 4 * s + g; }
  static constexpr int slot_xor(int bit) { return FP8 ? (bit == 1 ? 1 : bit == 8 ? 2 : 0) : (bit >> 2); }
  static constexpr int lane_xor(int bit) { return FP8 ? (bit == 2 ? 16 : bit == 4 ? 32 : 0) : (bit == 1 ? 16 : bit == 2 ? 32 : 0); }
};

// NEWROW (decode, bf16 pools, fixed partitions): the sequence's newest token is not in the pool yet but comes with
// the call (p.new_k / p.new_v).  The wave whose tile holds it (`take_new_row`) keeps the lane's pieces of the row in
// registers and puts them in the place of what the tile loads brought for that token (and for the rows behind it,
// which the loads redirect to it), so the scores and the output are those of a pool that already held the row; the
// same wave stores the row in the pool for the steps to come.
template <int D, bool FP8, bool MULTI = false, int R = 1, bool LEAN = false, bool SV = false, bool NEWROW = false>
struct DecodeWave {
  static_assert(!NEWROW || (!FP8 && R == 1 && !LEAN && !SV), "the new-row forms are bf16, one 16-row operand per wave");
  using KT = KTile<D, FP8>;
  using VT = VTile<D, FP8>;
  static constexpr int VEC = VT::VEC, KLD = KT::KLD, VW = VT::VW;
  static constexpr int KSTEPS = D / 32;
  static constexpr int ESZ = FP8 ? 1 : 2;
  // K streamed too (with V), for bf16 pools: config 2 kernel 169.3 -> 166.4 us, verify 180.0 -> 178.0; on the fp8
  // pool, whose expansion already costs vector instructions, the rearrangement costs more than it brings (375.5 -> 379.5)
  static constexpr bool SK = SV && !FP8 && D * ESZ >= 128;

  const DecodeParams& p;
  int hk, hbase, nheads;     // kv head, first (virtual) q head, valid rows of this wave
  int r, g, krow;            // lane = 16 g + r; row order of the K sub-tile
  const int32_t* table;
  const char* kbase;
  const char* vbase;
  long row_stride;           // bytes between consecutive tokens of a block
  int last;                  // ctx - 1 of the current sequence
  int jbase;                 // first row of this wave inside its kv group
  // SK: K travels as whole 128-byte lines (see load_k); where this lane's chunk of steps with even / odd s sits
  // after the load (byte address of the source lane for ds_bpermute), and in which of the two loads of a line
  int kperm_addr[2];
  bool k_first_half;
  int row_end[R];            // MULTI: keys [0, row_end) are visible to this lane's row (0: padding row)
  bf16x8_t qf[LEAN ? 1 : R][LEAN ? 1 : KSTEPS];
  uint4* qlds;               // LEAN: this wave's [R][KSTEPS][64] fragment store in LDS
  int qlane;                 // LEAN: lane index into it, re-made opaque per tile so the reads stay in the loop
  bf16x8_t pf[R];            // P^T fragments of the current tile
  f32x4_t oacc[R][VEC];
  float m_run[R], l_run[R];
  // NEWROW: chunk 4 s + g of the new K row (the lane's operand piece in k-step s, as transformed), the lane's
  // VEC elements of the new V row, the tile that holds the token (-1: none for this wave) and, while that tile is
  // worked on, the token's index in it (tile rows from there on are the new row)
  uint4 knew[NEWROW ? KSTEPS : 1];
  uint32_t vnew[NEWROW ? VW : 1];
  int new_t0, new_from;
  // NEWROW with MULTI (a few new tokens per sequence): the workgroup keeps the tokens' rows in LDS, row t of
  // new_k_lds / new_v_lds [T][D] bf16 being token first_new + t of the sequence (K as transformed); patch_new_rows
  // puts them into the tiles that hold those tokens.  first_new: a position no tile reaches when nothing is to patch.
  const char* new_k_lds;
  const char* new_v_lds;
  int first_new;

  __device__ __forceinline__ DecodeWave(const DecodeParams& p_, int head_slot, int lane, uint4* qlds_ = nullptr)
      : p(p_), qlds(qlds_), qlane(lane) {
    const int n_rows = (p.Hq / p.Hkv) * (MULTI ? p.T : 1);
    const int gchunks = (n_rows + 16 * R - 1) / (16 * R);
    hk = head_slot / gchunks;
    jbase = (head_slot % gchunks) * (16 * R);
    hbase = hk * n_rows + jbase;
    nheads = min(16 * R, n_rows - jbase);
    r = lane & 15;
    g = lane >> 4;
    krow = 4 * (r & 3) + (r >> 2);
    k_first_half = krow < 8;
    kperm_addr[0] = 4 * (8 * (krow & 7) + g);
    kperm_addr[1] = 4 * (8 * (krow & 7) + 4 + g);
    row_stride = (long)p.Hkv * D * ESZ;
    kbase = (const char*)p.k_cache + (long)hk * D * ESZ;
    vbase = (const char*)p.v_cache + (long)hk * D * ESZ;
    new_t0 = -1;
    new_from = 64;
    new_k_lds = new_v_lds = nullptr;
    first_new = 0x7fffffff;
  }

  // NEWROW with MULTI: tile rows of [t0, t0 + 32) that are new tokens (or are redirected to the last one, which is
  // new) take their K chunks and V elements from the workgroup's LDS copy instead of what the loads brought
  __device__ __forceinline__ void patch_new_rows(KT& k, VT& v, int t0) const {
    if constexpr (NEWROW && MULTI) {
      if (t0 + 31 < first_new) return;                 // wave-uniform: no new token in this tile
      const int lmax = last - t0;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int tn = t0 + min(16 * u + krow, lmax) - first_new;
        if (tn >= 0) {
#pragma unroll
          for (int s = 0; s < KLD; ++s) {
            const uint4 c = *(const uint4*)(new_k_lds + ((long)tn * D + (4 * s + g) * 8) * 2);
            k.k[u][s][0] = c.x; k.k[u][s][1] = c.y; k.k[u][s][2] = c.z; k.k[u][s][3] = c.w;
          }
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int tn = t0 + min(4 * j + g, lmax) - first_new;
        if (tn >= 0) {
          const uint32_t* src = (const uint32_t*)(new_v_lds + ((long)tn * D + r * VEC) * 2);
#pragma unroll
          for (int dw = 0; dw < VW; ++dw) v.v[j][dw] = src[dw];
        }
      }
    }
  }

  // NEWROW: this wave is the one whose tiles include token `pos` (= ctx - 1, the step's new token, whose rows begin()
  // has put into knew / vnew): from now on the tile that holds it is patched.  The same wave, if it is the first
  // of the kv head's rows, stores both rows in the pool when its tiles are done (store_new_row: K by the lanes
  // r = 0, chunks 4 s + g; V by the lanes g = 0, elements VEC r ..) -- not before: on this target loads and stores
  // share one counter and may complete out of order, so with a store pending the compiler waits for every load in
  // flight wherever it waits for one, and the tile loop would lose its prefetch.
  __device__ __forceinline__ void adopt_new_row(int pos) { new_t0 = pos & ~31; }
  __device__ __forceinline__ void store_new_row(int b, int pos) {
    if (jbase != 0) return;
    const int blk = p.block_tables[(long)b * p.max_blocks + (pos >> p.block_shift)];
    if (blk < 0 || blk >= p.num_blocks) return;      // a bad table entry must not redirect the write
    const long row = (long)blk * p.block_size + (pos & (p.block_size - 1));
    char* kdst = const_cast<char*>(kbase) + row * row_stride;
    char* vdst = const_cast<char*>(vbase) + row * row_stride;
    if (r == 0) {
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) *(uint4*)(kdst + (4 * s + g) * 16) = knew[NEWROW ? s : 0];
    }
    if (g == 0) {
      constexpr int NV = NEWROW ? VW : 1;
      if (VW == 4) *(uint4*)(vdst + r * (VEC * ESZ)) = make_uint4(vnew[0], vnew[1 % NV], vnew[2 % NV], vnew[3 % NV]);
      else *(uint2*)(vdst + r * (VEC * ESZ)) = make_uint2(vnew[0], vnew[1 % NV]);
    }
  }
  // NEWROW, a context clamped below its new token (the length bound of the call is shorter than the sequence): the
  // token is not attended to, only stored, with K transformed at its own position
  __device__ __forceinline__ void retransform_new_k(int b, int pos) {
    const uint16_t* krow = (const uint16_t*)p.new_k + ((long)b * p.Hkv + hk) * D;
    uint4 kraw[NEWROW ? KSTEPS : 1];
#pragma unroll
    for (int s = 0; s < (NEWROW ? KSTEPS : 1); ++s) kraw[s] = *(const uint4*)(krow + (4 * s + g) * 8);
    transform_new_k(kraw, pos);
  }

  // MULTI: element offset in q / out of row group rg's row of this lane, its query token and q head
  __device__ __forceinline__ long row_offset(int b, int rg, int* t_out, int* head_out) const {
    const int n_rep = p.Hq / p.Hkv;
    const int j = jbase + 16 * rg + r;
    const int t = j / n_rep;
    *t_out = t;
    *head_out = hk * n_rep + (j - t * n_rep);
    return (((long)b * p.T_stride + p.t0 + t) * p.Hq + *head_out) * D;
  }

  // Start on sequence b (context ctx >= 1, of which the last tq tokens are the
  // queries): load Q^T fragments (B operand, zero for padded columns) and reset
  // the softmax state.  In two halves, so that a caller can request its first tile
  // between them: issue_q sends every load the start needs (Q rows, what their
  // transform takes from the tables, with NEWROW the new token's rows), finish_q does
  // the arithmetic.  begin() is the two in a row.
  struct QPending {
    uint4 qraw[R][KSTEPS];
    NormRopeCoeffs<KSTEPS> qc[R];
    uint4 kraw[NEWROW ? KSTEPS : 1];
    NormRopeCoeffs<KSTEPS> kc;
  };
  __device__ __forceinline__ void begin(int b, int ctx, int tq = 1) {
    QPending q;
    issue_q(q, b, ctx, tq);
    finish_q(q);
  }
  __device__ __forceinline__ void issue_q(QPending& q, int b, int ctx, int tq = 1) {
    table = p.block_tables + (long)b * p.max_blocks;
    last = ctx - 1;
    // NEWROW: the new token's rows are requested here, with the Q rows, by every wave (one round trip for all of
    // them; the wave that turns out to hold the token adopts them, see adopt_new_row), and K is transformed behind Q
    if constexpr (NEWROW && !MULTI) {
      const uint16_t* krow = (const uint16_t*)p.new_k + ((long)b * p.Hkv + hk) * D;
      const uint16_t* vrow = (const uint16_t*)p.new_v + ((long)b * p.Hkv + hk) * D;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) q.kraw[s] = *(const uint4*)(krow + (4 * s + g) * 8);
      VecLoad<VW>::get(vrow + r * VEC, vnew);
      if (p.new_kt.cos)
        norm_rope_fetch<D / 8, KSTEPS, QOperandLayout<false>>(p.new_kt, min(max(last, 0), p.new_kt.max_pos - 1), g, q.kc);
    }
#pragma unroll
    for (int rg = 0; rg < R; ++rg) {
      bool row_valid = 16 * rg + r < nheads;
      const uint16_t* qrow;
      if (MULTI) {
        int t, head;
        qrow = (const uint16_t*)p.q + row_offset(b, rg, &t, &head);
        row_valid = row_valid && t < tq;
        row_end[rg] = row_valid ? ctx - tq + t + 1 : 0;
      } else {
        qrow = (const uint16_t*)p.q + ((long)b * p.Hq + hbase + r) * D;
      }
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        // d range of k-slots 8g..8g+7 in step s (must mirror the K loads below)
        const int d0 = FP8 ? ((4 * (s >> 1) + g) * 16 + (s & 1) * 8) : ((4 * s + g) * 8);
        q.qraw[rg][s] = make_uint4(0, 0, 0, 0);
        if (row_valid) q.qraw[rg][s] = *(const uint4*)(qrow + d0);
      }
      if (p.qt.cos) {
        const int qpos = MULTI ? row_end[rg] - 1 : last;
        norm_rope_fetch<D / 8, KSTEPS, QOperandLayout<FP8>>(p.qt, min(max(qpos, 0), p.qt.max_pos - 1), g, q.qc[rg]);
      }
    }
  }
  __device__ __forceinline__ void finish_q(QPending& q) {
#pragma unroll
    for (int rg = 0; rg < R; ++rg) {
      uint4 (&qraw)[KSTEPS] = q.qraw[rg];
      if (p.qt.cos) {
        // norm and rotation of the row on the way in; every lane takes part (a row is spread
        // over the four lanes r, r + 16, r + 32, r + 48), padded rows carry zeros
        float x[KSTEPS][8];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const uint32_t w[4] = {qraw[s].x, qraw[s].y, qraw[s].z, qraw[s].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            x[s][2 * j] = bf16_bits_to_float(w[j] & 0xffffu);
            x[s][2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
          }
        }
        norm_rope_apply<D / 8, KSTEPS, QOperandLayout<FP8>>(x, p.qt, g, q.qc[rg]);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          qraw[s].x = pack_bf16x2(x[s][0], x[s][1]); qraw[s].y = pack_bf16x2(x[s][2], x[s][3]);
          qraw[s].z = pack_bf16x2(x[s][4], x[s][5]); qraw[s].w = pack_bf16x2(x[s][6], x[s][7]);
        }
      }
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        if (LEAN) qlds[(rg * KSTEPS + s) * 64 + qlane] = qraw[s];
        else qf[rg][s] = __builtin_bit_cast(bf16x8_t, qraw[s]);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) oacc[rg][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      m_run[rg] = -INFINITY;
      l_run[rg] = 0.f;
    }
    if constexpr (NEWROW && !MULTI) {
      // the raw K row -> knew, normed and rotated at position ctx - 1 as the write kernel would (same arithmetic,
      // same bits; new_kt.cos null: stored as given)
      if (p.new_kt.cos) {
        float x[KSTEPS][8];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const uint32_t w[4] = {q.kraw[s].x, q.kraw[s].y, q.kraw[s].z, q.kraw[s].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            x[s][2 * j] = bf16_bits_to_float(w[j] & 0xffffu);
            x[s][2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
          }
        }
        norm_rope_apply<D / 8, KSTEPS, QOperandLayout<false>>(x, p.new_kt, g, q.kc);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          q.kraw[s] = make_uint4(pack_bf16x2(x[s][0], x[s][1]), pack_bf16x2(x[s][2], x[s][3]),
                                 pack_bf16x2(x[s][4], x[s][5]), pack_bf16x2(x[s][6], x[s][7]));
      }
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) knew[s] = q.kraw[s];
    }
  }

  // NEWROW: the raw K row -> knew, normed and rotated at position pos (the slow path of a token the call's length
  // bound hides: see retransform_new_k)
  __device__ __forceinline__ void transform_new_k(uint4 (&kraw)[NEWROW ? KSTEPS : 1], int pos) {
    if constexpr (NEWROW) {
      if (p.new_kt.cos) {
        float x[KSTEPS][8];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const uint32_t w[4] = {kraw[s].x, kraw[s].y, kraw[s].z, kraw[s].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            x[s][2 * j] = bf16_bits_to_float(w[j] & 0xffffu);
            x[s][2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
          }
        }
        q_norm_rope_lane<D / 8, KSTEPS, QOperandLayout<false>>(x, p.new_kt, min(max(pos, 0), p.new_kt.max_pos - 1), g);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          kraw[s] = make_uint4(pack_bf16x2(x[s][0], x[s][1]), pack_bf16x2(x[s][2], x[s][3]),
                               pack_bf16x2(x[s][4], x[s][5]), pack_bf16x2(x[s][6], x[s][7]));
      }
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) knew[s] = kraw[s];
    }
  }

  // Pool rows of tokens t0 and t0+16 (the two 16-token halves of a tile each lie
  // inside one block: block_size is a power of two >= 16, t0 a multiple of 32).
  struct TileRows { long row0, row1; int blk0, blk1, lmax; };
  __device__ __forceinline__ TileRows tile_rows(int t0) const {
    TileRows tr;
    const int t1 = min(t0 + 16, last);             // wave-uniform
    const int blk0 = table[t0 >> p.block_shift];
    const int blk1 = table[t1 >> p.block_shift];
    tr.blk0 = min(max(blk0, 0), p.num_blocks - 1);
    tr.blk1 = min(max(blk1, 0), p.num_blocks - 1);
    const int bmask = p.block_size - 1;
    tr.row0 = (long)tr.blk0 * p.block_size + (t0 & bmask);
    tr.row1 = (long)tr.blk1 * p.block_size + ((t0 + 16) & bmask);
    tr.lmax = last - t0;                           // largest valid local index (>= 0)
    return tr;
  }

  // Loads of the tile starting at token t0.  Rows past the context are
  // redirected to the last valid token so that no stale pool bytes (which could
  // be NaN patterns) ever reach the matrix cores.
  __device__ __forceinline__ void load_k(KT& tl, int t0) const {
    const TileRows tr = tile_rows(t0);
    if (FP8) {
      tl.ksc[0] = p.k_scale[(long)tr.blk0 * p.Hkv + hk];
      tl.ksc[1] = p.k_scale[(long)tr.blk1 * p.Hkv + hk];
    }
    if (SK) {
      // One instruction = 8 rows x one whole 128-byte line (lane: row 8 hf + lane / 8 of the sub-tile in tile
      // order, 16-byte chunk lane % 8), so that a streamed line is used up by the instruction that fetches it; slot
      // [2 ln + hf] holds line ln of rows 8 hf .. 8 hf + 7.  k_chunk() below hands the matrix instructions their
      // operand order back.
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          const int tl_ = min(16 * u + 8 * hf + 2 * g + (r >> 3), tr.lmax);
          const long row = (tl_ < 16) ? tr.row0 + tl_ : tr.row1 + (tl_ - 16);
          const char* rowp = kbase + row * row_stride + (r & 7) * 16;
#pragma unroll
          for (int ln = 0; ln < KLD / 2; ++ln) VecLoad<4, true>::get(rowp + ln * 128, tl.k[u][2 * ln + hf]);
        }
      return;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int tl_ = min(16 * u + krow, tr.lmax);
      const long row = (tl_ < 16) ? tr.row0 + tl_ : tr.row1 + (tl_ - 16);
      const char* rowp = kbase + row * row_stride;
#pragma unroll
      for (int s = 0; s < KLD; ++s) VecLoad<4, kStreamK>::get(rowp + (4 * s + g) * 16, tl.k[u][s]);
    }
  }
  // The 16 bytes lane (g, r) feeds to the matrix instruction in step s of sub-tile u: chunk 4 s + g of tile row
  // krow(r).  As loaded by the plain form they are tl.k[u][s]; as loaded by the streamed form they sit in line
  // s / 2, in the load of the row's half, in lane 8 (krow % 8) + (4 s + g) % 8: one cross-lane read (LDS pipeline,
  // no LDS memory) from each half's registers and a select.
  __device__ __forceinline__ void k_chunk(const KT& tl, int u, int s, uint32_t (&out)[4]) const {
    if (!SK) {
#pragma unroll
      for (int d = 0; d < 4; ++d) out[d] = tl.k[u][s][d];
      if (NEWROW) {
        const bool nw = 16 * u + krow >= new_from;     // the new token's row, or one redirected to it
        const uint32_t kn[4] = {knew[NEWROW ? s : 0].x, knew[NEWROW ? s : 0].y, knew[NEWROW ? s : 0].z, knew[NEWROW ? s : 0].w};
#pragma unroll
        for (int d = 0; d < 4; ++d) out[d] = nw ? kn[d] : out[d];
      }
      return;
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t a = (uint32_t)__builtin_amdgcn_ds_bpermute(kperm_addr[s & 1], (int)tl.k[u][2 * (s >> 1)][d]);
      const uint32_t b = (uint32_t)__builtin_amdgcn_ds_bpermute(kperm_addr[s & 1], (int)tl.k[u][2 * (s >> 1) + 1][d]);
      out[d] = k_first_half ? a : b;
    }
  }
  __device__ __forceinline__ void load_v(VT& tl, int t0) const {
    const TileRows tr = tile_rows(t0);
    if (FP8) {
      tl.vsc[0] = p.v_scale[(long)tr.blk0 * p.Hkv + hk];
      tl.vsc[1] = p.v_scale[(long)tr.blk1 * p.Hkv + hk];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int tl_ = min(4 * j + g, tr.lmax);
      const long row = (tl_ < 16) ? tr.row0 + tl_ : tr.row1 + (tl_ - 16);
      const char* rowp = vbase + row * row_stride;
      VecLoad<VW, SV>::get(rowp + r * (VEC * ESZ), tl.v[j]);
    }
  }

  // Scores of the tile at t0 (tokens >= t_end masked), online softmax update,
  // rescale of the accumulators, P^T fragments.
  __device__ __forceinline__ bf16x8_t q_frag(int rg, int s) const {
    if (LEAN) return __builtin_bit_cast(bf16x8_t, qlds[(rg * KSTEPS + s) * 64 + qlane]);
    return qf[LEAN ? 0 : rg][LEAN ? 0 : s];
  }

  __device__ __forceinline__ void scores_softmax(const KT& tl, const VT& vt, int t0, int t_end) {
    f32x4_t sacc[R][2];
    if (LEAN) asm volatile("" : "+v"(qlane));
    if (NEWROW) new_from = t0 == new_t0 ? last - t0 : 64;
#pragma unroll
    for (int rg = 0; rg < R; ++rg) sacc[rg][0] = sacc[rg][1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    // each Q fragment is fetched once and used for both 16-token halves
    if (!FP8) {
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
        for (int rg = 0; rg < R; ++rg) {
          const bf16x8_t q = q_frag(rg, s);
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            uint32_t kc[4];
            k_chunk(tl, u, s, kc);
            sacc[rg][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kc[0], kc[1], kc[2], kc[3]), q, sacc[rg][u], 0, 0, 0);
          }
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < KLD; ++s) {
        uint32_t w[2][8];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          uint32_t kc[4];
          k_chunk(tl, u, s, kc);
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            w[u][2 * d] = fp8x2_to_bf16x2<false>(kc[d]);
            w[u][2 * d + 1] = fp8x2_to_bf16x2<true>(kc[d]);
          }
        }
#pragma unroll
        for (int rg = 0; rg < R; ++rg) {
          const bf16x8_t q0 = q_frag(rg, 2 * s), q1 = q_frag(rg, 2 * s + 1);
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            sacc[rg][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[u][0], w[u][1], w[u][2], w[u][3]), q0, sacc[rg][u], 0, 0, 0);
            sacc[rg][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[u][4], w[u][5], w[u][6], w[u][7]), q1, sacc[rg][u], 0, 0, 0);
          }
        }
      }
    }
#pragma unroll
    for (int rg = 0; rg < R; ++rg) {
      float sv[8];
      float tmax = -INFINITY;
      const int lim = MULTI ? min(t_end, row_end[rg]) : t_end;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float sc = FP8 ? p.scale_log2e * tl.ksc[u] : p.scale_log2e;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int tok = t0 + 16 * u + 4 * i + g;
          const float x = sacc[rg][u][i] * sc;
          sv[4 * u + i] = tok < lim ? x : -INFINITY;
        }
      }
      // sliding window: keys more than window - 1 tokens behind the row's own position are
      // hidden; only the first tiles of a sequence's span reach below the newest row's bound
      if (p.window > 0 && t0 < last + 1 - p.window) {
        const int lo = (MULTI ? row_end[rg] : last + 1) - p.window;
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (t0 + 16 * (i >> 2) + 4 * (i & 3) + g < lo) sv[i] = -INFINITY;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) tmax = fmaxf(tmax, sv[i]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run[rg], tmax);
      // MULTI: a row that has seen no key yet keeps m = -inf; exponents are then taken against 0
      const float m_ref = (MULTI && m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run[rg] - m_ref);
      m_run[rg] = m_new;
      float pr[8], psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        pr[i] = __builtin_amdgcn_exp2f(sv[i] - m_ref);
        psum += pr[i];
      }
      l_run[rg] = l_run[rg] * alpha + psum;
#pragma unroll
      for (int e = 0; e < VEC; ++e) oacc[rg][e] *= alpha;
      if (FP8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { pr[i] *= vt.vsc[0]; pr[4 + i] *= vt.vsc[1]; }
      }
      pf[rg] = as_bf16x8(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]),
                         pack_bf16x2(pr[4], pr[5]), pack_bf16x2(pr[6], pr[7]));
    }
  }

  // V^T fragments by in-register transpose, then O^T += V^T P^T.
  __device__ __forceinline__ void accumulate_pv(const VT& tl) {
    if (!FP8) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
        uint32_t w[4];
#pragma unroll
        for (int jp = 0; jp < 4; ++jp) {
          uint32_t hi = tl.v[2 * jp + 1][e >> 1], lo = tl.v[2 * jp][e >> 1];
          if (NEWROW) {      // tile rows 4 j + g from the new token's on are the new row
            hi = 4 * (2 * jp + 1) + g >= new_from ? vnew[NEWROW ? e >> 1 : 0] : hi;
            lo = 4 * (2 * jp) + g >= new_from ? vnew[NEWROW ? e >> 1 : 0] : lo;
          }
          w[jp] = __builtin_amdgcn_perm(hi, lo, sel);
        }
#pragma unroll
        for (int rg = 0; rg < R; ++rg)
          oacc[rg][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[0], w[1], w[2], w[3]), pf[rg], oacc[rg][e], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int dw = 0; dw < VW; ++dw) {
        // codes of token pairs side by side first (bytes a0 b0 a1 b1 | a2 b2 a3 b3 of rows a = 2 jp, b = 2 jp + 1),
        // then one conversion per pair gives the operand's (token 2 jp, token 2 jp + 1) word for a column
        uint32_t t[4][2];
#pragma unroll
        for (int jp = 0; jp < 4; ++jp) {
          t[jp][0] = __builtin_amdgcn_perm(tl.v[2 * jp + 1][dw], tl.v[2 * jp][dw], 0x05010400u);
          t[jp][1] = __builtin_amdgcn_perm(tl.v[2 * jp + 1][dw], tl.v[2 * jp][dw], 0x07030602u);
        }
#pragma unroll
        for (int eb = 0; eb < 4; ++eb) {
          const int e = 4 * dw + eb;
          uint32_t w[4];
#pragma unroll
          for (int jp = 0; jp < 4; ++jp) w[jp] = (eb & 1) ? fp8x2_to_bf16x2<true>(t[jp][eb >> 1]) : fp8x2_to_bf16x2<false>(t[jp][eb >> 1]);
#pragma unroll
          for (int rg = 0; rg < R; ++rg)
            oacc[rg][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w[0], w[1], w[2], w[3]), pf[rg], oacc[rg][e], 0, 0, 0);
        }
      }
    }
  }

  // Stream n tiles starting at tokens t_first, t_first + t_step, ...; the next
  // tile's K is requested before the scores of the current one, its V before the
  // current P.V.  Loads inside the loop are unconditional (the remainder is
  // peeled) so that the wait counters stay exact and a wait for tile i never
  // includes the loads of tile i+1.
  __device__ __forceinline__ void stream(int t_first, int t_step, int n, int t_end, bool lockstep = false) {
    if (n <= 0) return;
    KT ka;
    VT va;
    load_k(ka, t_first);
    load_v(va, t_first);
    stream_from(ka, va, t_first, t_step, n, t_end, lockstep);
  }
  // ... with the first tile's loads (into ka, va) already requested by the caller
  __device__ __forceinline__ void stream_from(KT& ka, VT& va, int t_first, int t_step, int n, int t_end, bool lockstep = false) {
    if (n <= 0) return;
    KT kb;
    int t = t_first;
    int i = 0;
    if (LEAN) {
      while (i + 2 < n) {
        if (lockstep) __builtin_amdgcn_s_barrier();
        load_k(kb, t + t_step);
        scores_softmax(ka, va, t, t_end);
        accumulate_pv(va);
        load_v(va, t + t_step);
        if (lockstep) __builtin_amdgcn_s_barrier();
        load_k(ka, t + 2 * t_step);
        scores_softmax(kb, va, t + t_step, t_end);
        accumulate_pv(va);
        load_v(va, t + 2 * t_step);
        i += 2;
        t += 2 * t_step;
      }
      if (i + 1 < n) {
        load_k(kb, t + t_step);
        scores_softmax(ka, va, t, t_end);
        accumulate_pv(va);
        load_v(va, t + t_step);
        scores_softmax(kb, va, t + t_step, t_end);
        accumulate_pv(va);
      } else {
        scores_softmax(ka, va, t, t_end);
        accumulate_pv(va);
      }
      return;
    }
    VT vb;
    while (i + 2 < n) {
      if (lockstep) __builtin_amdgcn_s_barrier();
      load_k(kb, t + t_step);
      patch_new_rows(ka, va, t);
      scores_softmax(ka, va, t, t_end);
      load_v(vb, t + t_step);
      accumulate_pv(va);
      if (lockstep) __builtin_amdgcn_s_barrier();
      load_k(ka, t + 2 * t_step);
      patch_new_rows(kb, vb, t + t_step);
      scores_softmax(kb, vb, t + t_step, t_end);
      load_v(va, t + 2 * t_step);
      accumulate_pv(vb);
      i += 2;
      t += 2 * t_step;
    }
    if (i + 1 < n) {
      load_k(kb, t + t_step);
      patch_new_rows(ka, va, t);
      scores_softmax(ka, va, t, t_end);
      load_v(vb, t + t_step);
      accumulate_pv(va);
      patch_new_rows(kb, vb, t + t_step);
      scores_softmax(kb, vb, t + t_step, t_end);
      accumulate_pv(vb);
    } else {
      patch_new_rows(ka, va, t);
      scores_softmax(ka, va, t, t_end);
      accumulate_pv(va);
    }
  }

  // Sum of exponentials over the whole tile stream (all lanes of a row).
  __device__ __forceinline__ float total_l(int rg = 0) const {
    float l = l_run[rg];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    return l;
  }

  // Write this wave's normalised result for its rows: lane (g, r) holds, for
  // i = 0..3, the VEC consecutive d's starting at VEC * (4g + i).
  __device__ __forceinline__ void store_final(int b) const {
#pragma unroll
    for (int rg = 0; rg < R; ++rg) {
      float l = total_l(rg);
      if (16 * rg + r >= nheads) continue;
      int t, head = hbase + r;
      uint16_t* dst = MULTI ? (uint16_t*)p.out + row_offset(b, rg, &t, &head)
                            : (uint16_t*)p.out + ((long)b * p.Hq + hbase + r) * D;
      // attention sink: one more term of the denominator, no value
      if (p.sinks && l > 0.f) l += __builtin_amdgcn_exp2f(p.sinks[head] * kLog2e - m_run[rg]);
      const float inv = (MULTI && l == 0.f) ? 0.f : 1.f / l;    // padding rows: zeros
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t w[VEC / 2];
#pragma unroll
        for (int e = 0; e < VEC; e += 2)
          w[e / 2] = (uint32_t)float_to_bf16_bits(oacc[rg][e][i] * inv) |
                     ((uint32_t)float_to_bf16_bits(oacc[rg][e + 1][i] * inv) << 16);
        uint32_t* o = (uint32_t*)(dst + VEC * (4 * g + i));
        if (VEC == 8) *(uint4*)o = make_uint4(w[0], w[1], w[2], w[3]);
        else *(uint2*)o = make_uint2(w[0], w[1 % (VEC / 2)]);
      }
    }
  }
  // Split-K partials of this wave's rows for piece slot `piece`.  The workspace holds, per piece slot, the
  // rows (virtual q heads) in order; the floats of a 16-row group are laid out as the lanes hold them, not row
  // by row: float4 number ((j * 4 + g) * nh + r) of the group is what lane (g, r) stores with its j-th
  // instruction (nh = rows of the group, j = i * VEC / 4 + e / 4, covering d = VEC (4 g + i) + e .. + 3).  An
  // instruction then writes one contiguous run of 64 nh bytes instead of 16-byte pieces 128 bytes apart, and
  // the merge kernel, whose threads walk the float4s of a group in order, reads contiguously as well.  The
  // multi-token form, with four times decode's partial bytes, stores them as streaming writes (nothing in
  // this kernel reads them back and most are issued as the kernel ends); for decode's few megabytes the
  // merge kernel finding them in the cache is worth more.
  __device__ __forceinline__ void store_partial(long piece) const {
    typedef float f4_t __attribute__((ext_vector_type(4)));
    const long rows_total = (long)p.Hq * (MULTI ? p.T : 1);
#pragma unroll
    for (int rg = 0; rg < R; ++rg) {
      const float l = total_l(rg);
      if (16 * rg + r >= nheads) continue;
      const int nh = min(16, nheads - 16 * rg);
      const long row0 = piece * rows_total + hbase + 16 * rg;
      const float inv = (MULTI && l == 0.f) ? 0.f : 1.f / l;
      f4_t* dst = (f4_t*)(p.ws_out + row0 * D);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int e = 0; e < VEC; e += 4) {
          const f4_t val = {oacc[rg][e][i] * inv, oacc[rg][e + 1][i] * inv, oacc[rg][e + 2][i] * inv, oacc[rg][e + 3][i] * inv};
          f4_t* at = dst + ((i * (VEC / 4) + e / 4) * 4 + g) * nh + r;
          if (MULTI) __builtin_nontemporal_store(val, at);
          else *at = val;
        }
      }
      if (g == 0) *(float2*)(p.ws_ml + (row0 + r) * 2) = make_float2(m_run[rg], l);
    }
  }
};

// Keys and query rows of sequence b in this launch.  Decode: the whole context and one row.  A
// multi-token launch covers query tokens [t0, t0 + T) of the T_stride tokens per sequence in q:
// its rows are the tq of them that lie below the sequence's query length, and its context ends
// with the last of those (a launch none of whose tokens the sequence has streams nothing).
struct SeqSpan { int ctx, tq; };
__device__ __forceinline__ SeqSpan seq_span(const DecodeParams& p, int b) {
  const int c = min(max(p.seq_lens[b], 0), p.max_seq_len);
  if (!p.query_lens) return {c, 1};
  const int qfull = min(min(max(p.query_lens[b], 0), p.T_stride), c);
  const int tq = min(max(qfull - p.t0, 0), p.T);
  return {tq > 0 ? c - qfull + p.t0 + tq : 0, tq};
}
__device__ __forceinline__ int clamp_ctx(const DecodeParams& p, int b) { return seq_span(p, b).ctx; }

// Query tokens of sequence b in this launch (decode: 1)
__device__ __forceinline__ int query_len(const DecodeParams& p, int b, int ctx) {
  (void)ctx;
  return seq_span(p, b).tq;
}
// First 32-token tile that any query row of sequence b sees (0 without a sliding window)
__device__ __forceinline__ int first_tile(const DecodeParams& p, int b, int ctx) {
  if (p.window <= 0) return 0;
  return max(ctx - query_len(p, b, ctx) + 1 - p.window, 0) >> 5;
}

// Waves' worth of rows over all kv heads: rows of a kv head = its q heads x query tokens,
// p.rows_per_wave (16 or 32) of them per wave
__host__ __device__ __forceinline__ int head_slots_of(const DecodeParams& p) {
  return p.Hkv * (((p.Hq / p.Hkv) * p.T + p.rows_per_wave - 1) / p.rows_per_wave);
}

// ---------------------------------------------------------------------------
// Fixed partitions: one workgroup per (partition, head slot, sequence), NW waves
// interleave the partition's tiles and merge through LDS.
// ---------------------------------------------------------------------------
// MULTI (a few query tokens per sequence, small calls of pa_verify): the rows of a kv head are its (query token, q
// head) pairs, token-major, 16 per wave as in the balanced kernel; a row may see no key in a partition (its causal
// bound lies before it), which leaves an empty partial (m = -inf, l = 0); rows past the query length come out as zeros.
// NEWROW: the step's new K / V row comes with the call (see DecodeWave); the workgroup of the partition that holds
// token ctx - 1 attends to it from registers and stores it.
template <int D, bool FP8, int NW, bool MULTI = false, bool NEWROW = false>
__global__ __launch_bounds__(NW * 64, NW > 4 ? 1 : 2) void decode_mfma_kernel(DecodeParams p) {
  using W = DecodeWave<D, FP8, MULTI, 1, false, false, NEWROW>;
  constexpr int VEC = W::VEC;
  constexpr int OSTRIDE = D + 16;   // LDS row stride (floats) for the merge

  const int part = p.head_major ? blockIdx.y : blockIdx.x, b = blockIdx.z;
  const int hidx = p.head_major ? blockIdx.x : blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  W w(p, hidx, lane);
  const SeqSpan sp = seq_span(p, b);
  const int ctx = sp.ctx;
  int new_len = 0;
  bool takes_new = false;
  if constexpr (NEWROW && !MULTI) {
    new_len = min(p.seq_lens[b], p.max_blocks * p.block_size);
    takes_new = new_len >= 1 && (!p.new_lens || p.new_lens[b] >= 1);
  }
  // NEWROW with MULTI: the step's new tokens of this sequence, as the write kernel places them: new_n of them from
  // position new_start on (lengths beyond the table count as its capacity; nothing to write when the lengths are
  // inconsistent).  The call attends to them only if its own view of the sequence ends with them (no length bound
  // below the sequence, query tokens = new tokens); otherwise they are stored and the pool rows are read as they are.
  int new_n = 0, new_start = 0;
  bool new_seen = false;
  if constexpr (NEWROW && MULTI) {
    const int len = min(p.seq_lens[b], p.max_blocks * p.block_size);
    new_n = min(max(p.new_lens[b], 0), p.T);
    new_start = len - new_n;
    if (new_start < 0) new_n = 0;
    new_seen = new_n > 0 && len == ctx && new_n == sp.tq;
  }
  // where virtual row vr (q head, or (token, head) pair) of sequence b lies in out
  const int n_rep = p.Hq / p.Hkv;
  auto out_row = [&](int vr) __attribute__((always_inline)) -> uint16_t* {
    if (!MULTI) return (uint16_t*)p.out + ((long)b * p.Hq + vr) * D;
    const int n_rows = n_rep * p.T;
    const int hk = vr / n_rows, j = vr - hk * n_rows, t = j / n_rep;
    return (uint16_t*)p.out + (((long)b * p.T_stride + p.t0 + t) * p.Hq + hk * n_rep + (j - t * n_rep)) * D;
  };
  // partitions count from the first tile any query row sees (the start of the context, or what a sliding window leaves)
  const int t_begin = (first_tile(p, b, ctx) << 5) + part * p.partition_size;
  if (t_begin >= ctx) {
    if (ctx == 0 && part == 0 && p.num_partitions == 1) {
      for (int i = tid; i < w.nheads * D; i += NW * 64) out_row(w.hbase + i / D)[i % D] = 0;
    }
    return;
  }
  const int t_end = min(ctx, t_begin + p.partition_size);
  const int ntiles = (t_end - t_begin + 31) >> 5;
  // NEWROW with MULTI: the workgroup whose partition ends the context (the first one, for tokens the call does not
  // see) stores the new rows when its tiles are done; it and every workgroup whose partition holds one of the
  // tokens keep the rows in LDS: K normed and rotated at each token's position by wave 0 (lane (g, r): token r,
  // chunks 4 s + g; the write kernel's arithmetic, hence its bits), V as given.
  __shared__ __attribute__((aligned(16))) char sm_new[(NEWROW && MULTI) ? 2 * 16 * D * 2 : 16];
  bool new_storer = false, new_rows = false;
  uint4 nk_raw[(NEWROW && MULTI) ? W::KSTEPS : 1], nv_raw = make_uint4(0, 0, 0, 0);
  NormRopeCoeffs<W::KSTEPS> nk_c;
  constexpr int CPRW = D / 8;                                // 16-byte chunks per row
  if constexpr (NEWROW && MULTI) {
    new_storer = new_n > 0 && w.jbase == 0 && (new_seen ? t_end == ctx : part == 0);
    const bool new_here = new_seen && new_start < t_end;        // (the tokens end the context: they begin before t_end or not at all)
    new_rows = new_storer || new_here;
    if (new_rows) {
      // the loads first (wave 0: token r's K chunks 4 s + g and what their transform takes from the tables; every
      // thread: one 16-byte chunk of the V rows, 16 tokens x D / 8 chunks at most); the arithmetic follows behind
      // the requests of the Q rows and of the first tile
      if (wave == 0) {
        const int t = min(w.r, new_n - 1);
        const uint16_t* krow = (const uint16_t*)p.new_k + (((long)b * p.T + t) * p.Hkv + w.hk) * D;
#pragma unroll
        for (int s = 0; s < W::KSTEPS; ++s) nk_raw[s] = *(const uint4*)(krow + (4 * s + w.g) * 8);
        if (p.new_kt.cos)
          norm_rope_fetch<D / 8, W::KSTEPS, QOperandLayout<false>>(p.new_kt, min(max(new_start + t, 0), p.new_kt.max_pos - 1), w.g, nk_c);
      }
      if (tid < new_n * CPRW) {
        const int t = tid / CPRW, ch = tid - t * CPRW;
        nv_raw = *(const uint4*)((const uint16_t*)p.new_v + (((long)b * p.T + t) * p.Hkv + w.hk) * D + ch * 8);
      }
      if (new_here) w.first_new = new_start;
      w.new_k_lds = sm_new;
      w.new_v_lds = sm_new + 16 * D * 2;
    }
  }
  // every load the start needs, then this wave's first tile, then the arithmetic of the start: the first tile is on
  // its way while Q is normed and rotated (one trip to memory less on the path of every workgroup)
  const int t_first = t_begin + 32 * wave, n_mine = (ntiles - wave + NW - 1) / NW;
  typename W::QPending qp;
  typename W::KT k_first;
  typename W::VT v_first;
  w.issue_q(qp, b, ctx, sp.tq);
  if (n_mine > 0) {
    w.load_k(k_first, t_first);
    w.load_v(v_first, t_first);
  }
  if constexpr (NEWROW && MULTI) {
    if (new_rows) {
      if (wave == 0) {
        float x[W::KSTEPS][8];
#pragma unroll
        for (int s = 0; s < W::KSTEPS; ++s) {
          const uint32_t wd[4] = {nk_raw[s].x, nk_raw[s].y, nk_raw[s].z, nk_raw[s].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            x[s][2 * j] = bf16_bits_to_float(wd[j] & 0xffffu);
            x[s][2 * j + 1] = bf16_bits_to_float(wd[j] >> 16);
          }
        }
        if (p.new_kt.cos) norm_rope_apply<D / 8, W::KSTEPS, QOperandLayout<false>>(x, p.new_kt, w.g, nk_c);
        if (w.r < new_n) {
#pragma unroll
          for (int s = 0; s < W::KSTEPS; ++s)
            *(uint4*)(sm_new + ((long)w.r * D + (4 * s + w.g) * 8) * 2) =
                make_uint4(pack_bf16x2(x[s][0], x[s][1]), pack_bf16x2(x[s][2], x[s][3]),
                           pack_bf16x2(x[s][4], x[s][5]), pack_bf16x2(x[s][6], x[s][7]));
        }
      }
      if (tid < new_n * CPRW) *(uint4*)(sm_new + 16 * D * 2 + (long)tid * 16) = nv_raw;
      __syncthreads();
    }
  }
  w.finish_q(qp);
  int store_pos = -1;       // NEWROW: this wave stores the new token's rows at this position when its tiles are done
  if constexpr (NEWROW && !MULTI) {
    // the new token is number seq_lens[b] - 1, as the write kernel places it (lengths beyond the table count as
    // its capacity); a sequence that takes none this step (new_lens[b] == 0) or is empty is streamed as it is
    if (takes_new) {
      const int pos = new_len - 1;
      if (pos == ctx - 1) {
        // seen by this call: the wave that streams its tile patches that tile and stores the row
        if (pos >= t_begin && pos < t_end && ((pos - t_begin) >> 5) % NW == wave) {
          w.adopt_new_row(pos);
          store_pos = pos;
        }
      } else if (part == 0 && wave == 0) {
        store_pos = pos;                    // a length bound below the new token: stored, not attended to
      }
    }
  }
  w.stream_from(k_first, v_first, t_first, 32 * NW, n_mine, t_end);
  if constexpr (NEWROW && !MULTI) {
    if (store_pos >= 0) {
      if (store_pos != ctx - 1) w.retransform_new_k(b, store_pos);     // K was rotated for position ctx - 1
      w.store_new_row(b, store_pos);
    }
  }
  if constexpr (NEWROW && MULTI) {
    if (new_storer) {
      // behind the tile loop, not in front of it: a pending store would make every wait in the loop a wait for all
      for (int i = tid; i < 2 * new_n * CPRW; i += NW * 64) {
        const int which = i >= new_n * CPRW, ii = i - which * new_n * CPRW;
        const int t = ii / CPRW, ch = ii - t * CPRW, pos = new_start + t;
        const int blk = p.block_tables[(long)b * p.max_blocks + (pos >> p.block_shift)];
        if (blk < 0 || blk >= p.num_blocks) continue;             // a bad table entry must not redirect the write
        const long row = (long)blk * p.block_size + (pos & (p.block_size - 1));
        char* dst = const_cast<char*>(which ? w.vbase : w.kbase) + row * w.row_stride + ch * 16;
        *(uint4*)dst = *(const uint4*)(sm_new + which * 16 * D * 2 + ((long)t * D + ch * 8) * 2);
      }
    }
  }

  // ---- merge the NW wave states through LDS ----
  // (eight waves keep rows for at most 8 q heads per kv head: 16 rows of 8 waves would not fit the static 64 KB)
  constexpr int MROWS = NW > 4 ? 8 : 16;
  __shared__ float sm_m[NW][16];
  __shared__ float sm_l[NW][16];
  __shared__ __attribute__((aligned(16))) float sm_o[NW][MROWS][OSTRIDE];
  const float l_tot = w.total_l();
  const int r = w.r, g = w.g, nheads = w.nheads;
  if (g == 0) { sm_m[wave][r] = w.m_run[0]; sm_l[wave][r] = l_tot; }
  if (r < nheads) {
#pragma unroll
    for (int e = 0; e < VEC; ++e)   // value for d = VEC*(4g+i) + e stored at e*16 + 4g + i
      *(f32x4_t*)&sm_o[wave][r][e * 16 + 4 * g] = w.oacc[0][e];
  }
  __syncthreads();
  const long rows_total = (long)p.Hq * (MULTI ? p.T : 1);
  for (int idx = tid; idx < nheads * D; idx += NW * 64) {
    const int h = idx / D, d = idx % D;
    const int pos = (d % VEC) * 16 + d / VEC;
    float mt = -INFINITY;
#pragma unroll
    for (int x = 0; x < NW; ++x) mt = fmaxf(mt, sm_m[x][h]);
    const float m_ref = (MULTI && mt == -INFINITY) ? 0.f : mt;      // a row that saw no key here: every weight 0
    float lt = 0.f, ot = 0.f;
#pragma unroll
    for (int x = 0; x < NW; ++x) {
      const float wt = __builtin_amdgcn_exp2f(sm_m[x][h] - m_ref);   // idle waves: 2^-inf = 0
      lt += sm_l[x][h] * wt;
      ot += sm_o[x][h][pos] * wt;
    }
    const int vr = w.hbase + h;
    if (p.num_partitions == 1) {
      // attention sink: one more term of the denominator, no value (as the balanced kernel's store_final)
      float den = lt;
      if (p.sinks && lt > 0.f) {
        int head = vr;
        if (MULTI) {
          const int n_rows = n_rep * p.T, hk = vr / n_rows, j = vr - hk * n_rows;
          head = hk * n_rep + j % n_rep;
        }
        den += __builtin_amdgcn_exp2f(p.sinks[head] * kLog2e - mt);
      }
      out_row(vr)[d] = float_to_bf16_bits((MULTI && lt == 0.f) ? 0.f : ot / den);
    } else {
      const float o = (MULTI && lt == 0.f) ? 0.f : ot / lt;
      const long slot = ((long)b * rows_total + vr) * p.num_partitions + part;
      p.ws_out[slot * D + d] = o;
      if (d == 0) { p.ws_ml[slot * 2] = mt; p.ws_ml[slot * 2 + 1] = lt; }
    }
  }
}

// ---------------------------------------------------------------------------
// Balanced schedule.  The 32-token tiles of all sequences form one flattened
// stream of N tiles; it is cut into gv equal chunks of L = ceil(N / gv) tiles,
// one per resident group of wavefronts, so every group streams the same number
// of bytes whatever the mix of context lengths.  A workgroup holds `hsw` head
// slots x `ns` chunks: the waves of one chunk read the same token rows for
// different kv heads at the same time, which makes each 64 KB block of the pool
// one contiguous DRAM stream; a barrier per tile keeps them on the same rows (worth 3 % of
// bandwidth: requests for the eight 256-byte pieces of a 2 KB token row arrive together).
// A chunk may cover the tail of one sequence, whole sequences, and the head of
// another; each (sequence, chunk) piece yields either the final output (when
// the sequence lies inside one chunk) or a split-K partial in slot
// [q head][b + chunk], merged by decode_balanced_reduce_kernel.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int tiles_of(int ctx) { return (ctx + 31) >> 5; }

// Inclusive prefix sum over the 64 lanes of a wave on DPP adds: shifts by 1, 2, 4 and 8 inside each row of 16 lanes
// (a lane without a source adds 0), then lane 15 of rows 0 and 2 into rows 1 and 3, then lane 31 into rows 2 and 3.
__device__ __forceinline__ int wave_inclusive_sum(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0x111 /* row_shr:1 */, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, 0x112 /* row_shr:2 */, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, 0x114 /* row_shr:4 */, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, 0x118 /* row_shr:8 */, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, 0x142 /* row_bcast:15 */, 0xa, 0xf, false);
  x += __builtin_amdgcn_update_dpp(0, x, 0x143 /* row_bcast:31 */, 0xc, 0xf, false);
  return x;
}
// Tiles of sequence b that the schedule streams: all of them, or those the window reaches
__device__ __forceinline__ int span_tiles(const DecodeParams& p, int b) {
  const int ctx = clamp_ctx(p, b);
  return tiles_of(ctx) - first_tile(p, b, ctx);
}

// Calls of more than kScanInRegs sequences: the tiles before each sequence (and the total) are laid down in
// p.ws_start by this one-workgroup launch ahead of the streaming kernel, whose waves then find their first sequence
// by search instead of each scanning every length (a scan is a chain of a load and six cross-lane steps per 64
// sequences: at 8 192 sequences of one to three tiles the scans were half of the streaming kernel's time).
constexpr int kScanInRegs = 512;
__global__ __launch_bounds__(1024) void decode_tile_prefix_kernel(DecodeParams p) {
  __shared__ int wave_total[16];
  __shared__ int carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < p.B; base += 4096) {
    const int b0 = base + 4 * tid;
    int t[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      t[i] = b0 + i < p.B ? span_tiles(p, b0 + i) : 0;
      sum += t[i];
    }
    const int incl = wave_inclusive_sum(sum);
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before += wave_total[w];
    int run = before + incl - sum;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (b0 + i < p.B) p.ws_start[b0 + i] = run;
      run += t[i];
    }
    __syncthreads();
    if (tid == 1023) carry = run;
    __syncthreads();
  }
  if (tid == 0) p.ws_start[p.B] = carry;
}

// Wave-wide: the sequence that holds flattened tile f (0 <= f < ws_start[B]) and the tiles before it, from the
// prefix sums: 64 probes per round, the last probe not above f wins (equal sums, i.e. sequences without tiles, are
// thereby skipped)
__device__ __forceinline__ void find_tile(const DecodeParams& p, int lane, int f, int* b_out, int* start_out) {
  int lo = 0, hi = p.B, start = 0;
  while (true) {
    const int step = (hi - lo + 63) >> 6;
    const int pos = lo + lane * step;
    const int v = pos < hi ? p.ws_start[pos] : 0x7fffffff;
    const unsigned long long m = __ballot(v <= f);
    const int c = __popcll(m) - 1;                   // lane 0 probes lo, whose sum is not above f
    start = __shfl(v, c, 64);
    lo += c * step;
    hi = min(hi, lo + step);
    if (step == 1) break;
  }
  *b_out = lo;
  *start_out = start;
}

template <int D, bool FP8, bool MULTI, int R, bool SV>
__global__ __launch_bounds__(512, 2) void decode_balanced_kernel(DecodeParams p) {
  constexpr bool LEAN = R == 2 && D == 128;
  using W = DecodeWave<D, FP8, MULTI, R, LEAN, SV>;
  __shared__ uint4 q_store[LEAN ? 8 * R * W::KSTEPS * 64 : 1];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int head_slots = head_slots_of(p);
  const int hs = blockIdx.y * p.bal_hsw + wave % p.bal_hsw;
  if (hs >= head_slots) return;
  const int cv = blockIdx.x * p.bal_ns + wave / p.bal_hsw;   // chunk of this wave
  const int gv = p.bal_gv;

  // Total number of tiles and the sequence that holds this wave's first tile.  Up to 512 sequences
  // the lengths are fetched once, all loads in flight together, and scanned in registers; beyond
  // that the prefix sums are there already (decode_tile_prefix_kernel).
  constexpr int SCAN_STEPS = kScanInRegs / 64;
  const bool scan_in_regs = p.B <= kScanInRegs;
  int N = 0, tl[SCAN_STEPS], incl[SCAN_STEPS];
  if (scan_in_regs) {
#pragma unroll
    for (int i = 0; i < SCAN_STEPS; ++i) tl[i] = (64 * i + lane < p.B) ? span_tiles(p, 64 * i + lane) : 0;
#pragma unroll
    for (int i = 0; i < SCAN_STEPS; ++i) {
      incl[i] = 0;
      if (64 * i < p.B) {                    // (wave-uniform: steps past the last sequence cost nothing)
        incl[i] = wave_inclusive_sum(tl[i]);
        N += __builtin_amdgcn_readlane(incl[i], 63);
      }
    }
  } else {
    N = p.ws_start[p.B];
  }
  if (scan_in_regs && blockIdx.x == 0 && blockIdx.y == 0 && wave == 0) {
    // tiles before each sequence (and the total), for the merge kernel: it then needs no scan of its own
    int base = 0;
#pragma unroll
    for (int i = 0; i < SCAN_STEPS; ++i) {
      if (64 * i + lane < p.B) p.ws_start[64 * i + lane] = base + incl[i] - tl[i];
      base += __builtin_amdgcn_readlane(incl[i], 63);
    }
    if (lane == 0) p.ws_start[p.B] = base;
  }
  if (N == 0) return;
  const int L = (N + gv - 1) / gv;
  int f = cv * L;
  if (f >= N) return;
  const int f_end = min(N, f + L);
  int b = 0, start = 0;
  if (scan_in_regs) {
    int base = 0;
    bool found = false;
#pragma unroll
    for (int i = 0; i < SCAN_STEPS; ++i) {
      const int total = __builtin_amdgcn_readlane(incl[i], 63);
      if (!found && f < base + total) {
        const unsigned long long m = __ballot(base + incl[i] > f);
        const int idx = __ffsll((long long)m) - 1;
        b = 64 * i + idx;
        start = base + __builtin_amdgcn_readlane(incl[i] - tl[i], idx);
        found = true;
      }
      base += total;
    }
  } else {
    find_tile(p, lane, f, &b, &start);
  }
  b = __builtin_amdgcn_readfirstlane(b);
  start = __builtin_amdgcn_readfirstlane(start);

  W w(p, hs, lane, LEAN ? q_store + wave * (R * W::KSTEPS * 64) : nullptr);
  while (f < f_end) {
    const int ctx = clamp_ctx(p, b);
    const int T = span_tiles(p, b);
    if (T == 0) { ++b; continue; }
    const int ti = f - start + first_tile(p, b, ctx);
    const int n = min(T - (f - start), f_end - f);
    w.begin(b, ctx, MULTI ? query_len(p, b, ctx) : 1);
    w.stream(ti << 5, 32, n, ctx, p.bal_lockstep != 0);
    const int c_first = start / L, c_last = (start + T - 1) / L;
    if (c_first == c_last) w.store_final(b);
    else w.store_partial(b + cv);
    f += n;
    start += T;
    ++b;
  }
}

// Merge of the balanced schedule's partials: one thread per (q head, 4 consecutive d) of a
// sequence, a single pass with online rescaling so that the loads of all chunks can be in
// flight together.  Sequences that were written as final output are skipped, empty ones
// are zero-filled.
// G consecutive lanes share one item and take every G-th piece of the sequence; their partial
// merges are combined with a butterfly.  G = 1 when there are many sequences (each spans a few
// chunks), 8 or 32 when a sequence spans many.
template <int D, int G, bool FOLD = false>
__global__ __launch_bounds__(256) void decode_balanced_reduce_kernel(DecodeParams p) {
  const int b = blockIdx.x;
  const int start = p.ws_start[b];                   // tiles before this sequence (streaming kernel, or prefix launch)
  const int T = p.ws_start[b + 1] - start;
  const int N = p.ws_start[p.B];
  constexpr int QUADS = D / 4, VEC = D / 16;
  const int rows_total = p.Hq * p.T;                  // virtual heads (p.T = 1 for decode)
  const int gv = p.bal_gv;
  const int L = (N + gv - 1) / gv;
  const int c_first = T ? start / L : 0, c_last = T ? (start + T - 1) / L : 0;
  if (T != 0 && c_first == c_last) return;            // single piece: written by the streaming kernel
  // the items of a sequence are spread over gridDim.y workgroups, or (FOLD) all taken by one: for calls of thousands
  // of sequences, nearly all of which return above, that is a fourth of the workgroups to start
  const int ny = (rows_total * QUADS * G + 255) / 256;
  for (int by = FOLD ? 0 : blockIdx.y; by < (FOLD ? ny : (int)blockIdx.y + 1); ++by) {
  const int item = by * (256 / G) + threadIdx.x / G;
  const int g = threadIdx.x % G;
  const bool mine = item < rows_total * QUADS;
  // item = number of a float4 within a piece slot, in the order the streaming kernel lays them out
  // (store_partial): which row and which four d's it is
  const int n_rep = p.Hq / p.Hkv, n_rows = n_rep * p.T;
  const int row_f = min(item / QUADS, rows_total - 1);
  const int hk = row_f / n_rows, grp = (row_f - hk * n_rows) & ~15;      // kv head, first row of the 16-row group
  const int nh = min(16, n_rows - grp);
  const int within = item - (hk * n_rows + grp) * QUADS;                // float4 number inside the group
  const int jg = within / nh, r = within - jg * nh;
  const int gq = jg & 3, j = jg >> 2;
  const int d0 = VEC * (4 * gq + j / (VEC / 4)) + 4 * (j % (VEC / 4));
  const int hq = hk * n_rows + grp + r;               // virtual head
  uint16_t* dst = (uint16_t*)p.out + ((long)b * p.Hq + hq) * D + d0;
  int head = hq;                                      // the real q head of this item
  if (p.query_lens) {
    const int jrow = grp + r, t = jrow / n_rep;
    head = hk * n_rep + (jrow - t * n_rep);
    dst = (uint16_t*)p.out + (((long)b * p.T_stride + p.t0 + t) * p.Hq + head) * D + d0;
  }
  if (T == 0) {
    if (mine && g == 0) *(uint2*)dst = make_uint2(0u, 0u);
    continue;
  }
  if (!mine) continue;                      // (a whole group of G lanes: the butterfly below stays among takers)
  float m = -INFINITY, l = 0.f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
  for (int c = c_first + g; c <= c_last; c += G) {
    const long slot = (long)(b + c) * rows_total;
    const float2 ml = *(const float2*)(p.ws_ml + (slot + hq) * 2);
    const float4 o = *((const float4*)(p.ws_out + slot * D) + item);
    const float m_new = fmaxf(m, ml.x);
    const float m_ref = m_new == -INFINITY ? 0.f : m_new;   // pieces in which a row saw no key carry m = -inf, l = 0
    const float a = exp2f(m - m_ref);
    const float wt = ml.y * exp2f(ml.x - m_ref);
    l = l * a + wt;
    acc.x = acc.x * a + wt * o.x; acc.y = acc.y * a + wt * o.y;
    acc.z = acc.z * a + wt * o.z; acc.w = acc.w * a + wt * o.w;
    m = m_new;
  }
#pragma unroll
  for (int off = 1; off < G; off <<= 1) {      // lanes without a piece carry m = -inf, l = 0
    const float m2 = __shfl_xor(m, off, 64), l2 = __shfl_xor(l, off, 64);
    const float4 a2 = make_float4(__shfl_xor(acc.x, off, 64), __shfl_xor(acc.y, off, 64),
                                  __shfl_xor(acc.z, off, 64), __shfl_xor(acc.w, off, 64));
    const float m_new = fmaxf(m, m2);
    const float a = m == -INFINITY ? 0.f : exp2f(m - m_new), b2 = m2 == -INFINITY ? 0.f : exp2f(m2 - m_new);
    l = l * a + l2 * b2;
    acc.x = acc.x * a + a2.x * b2; acc.y = acc.y * a + a2.y * b2;
    acc.z = acc.z * a + a2.z * b2; acc.w = acc.w * a + a2.w * b2;
    m = m_new;
  }
  if (g != 0) continue;
  if (p.sinks && l > 0.f) l += exp2f(p.sinks[head] * kLog2e - m);    // attention sink: denominator only
  const float inv = l == 0.f ? 0.f : 1.f / l;     // padding rows of a multi-token call: zeros
  *(uint2*)dst =
      make_uint2(pack_bf16x2(acc.x * inv, acc.y * inv), pack_bf16x2(acc.z * inv, acc.w * inv));
  }
}

template <int D, bool FP8>
hipError_t launch_typed(const DecodeParams& p, int waves, hipStream_t s) {
  const int n_rep = p.Hq / p.Hkv;
  const int slots = head_slots_of(p);                  // Hkv x 16-row groups of a kv head's rows
  dim3 grid(p.num_partitions, slots, p.B);
  if (p.head_major) grid = dim3(slots, p.num_partitions, p.B);
  if (p.query_lens) {      // multi-token rows: the four-wave form
    if (p.rows_per_wave != 16) return hipErrorInvalidValue;
    if (p.new_k) {
      if constexpr (FP8) return hipErrorInvalidValue;
      else {
        if (slots != p.Hkv || p.T > 16 || !p.new_lens) return hipErrorInvalidValue;     // one 16-row wave per kv head holds all its rows
        hipLaunchKernelGGL((decode_mfma_kernel<D, false, 4, true, true>), grid, dim3(256), 0, s, p);
        return hipGetLastError();
      }
    }
    hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 4, true>), grid, dim3(256), 0, s, p);
    return hipGetLastError();
  }
  if (p.new_k) {
    if constexpr (FP8) {
      return hipErrorInvalidValue;
    } else {
      if (waves == 8) {
        if (n_rep > 8) return hipErrorInvalidValue;
        hipLaunchKernelGGL((decode_mfma_kernel<D, false, 8, false, true>), grid, dim3(512), 0, s, p);
      } else {
        hipLaunchKernelGGL((decode_mfma_kernel<D, false, 4, false, true>), grid, dim3(256), 0, s, p);
      }
      return hipGetLastError();
    }
  }
  switch (waves) {
    case 1: hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 1>), grid, dim3(64), 0, s, p); break;
    case 2: hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 2>), grid, dim3(128), 0, s, p); break;
    case 8:
      if (n_rep > 8) return hipErrorInvalidValue;      // its merge area holds 8 rows per wave
      hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 8>), grid, dim3(512), 0, s, p);
      break;
    default: hipLaunchKernelGGL((decode_mfma_kernel<D, FP8, 4>), grid, dim3(256), 0, s, p); break;
  }
  return hipGetLastError();
}

template <int D, bool FP8>
hipError_t launch_balanced_typed(const DecodeParams& p, hipStream_t s) {
  const int head_slots = head_slots_of(p);
  dim3 grid(p.bal_gv / p.bal_ns, (head_slots + p.bal_hsw - 1) / p.bal_hsw);
  const dim3 wg(64 * p.bal_hsw * p.bal_ns);
  const bool one_reader = head_slots == p.Hkv;         // one wave per kv head: it alone reads that head's V rows
  if (p.B > kScanInRegs) hipLaunchKernelGGL(decode_tile_prefix_kernel, dim3(1), dim3(1024), 0, s, p);
  if (p.query_lens && p.rows_per_wave == 32) {
    if (one_reader) hipLaunchKernelGGL((decode_balanced_kernel<D, FP8, true, 2, true>), grid, wg, 0, s, p);
    else hipLaunchKernelGGL((decode_balanced_kernel<D, FP8, true, 2, false>), grid, wg, 0, s, p);
  } else if (p.query_lens) {
    if (one_reader) hipLaunchKernelGGL((decode_balanced_kernel<D, FP8, true, 1, true>), grid, wg, 0, s, p);
    else hipLaunchKernelGGL((decode_balanced_kernel<D, FP8, true, 1, false>), grid, wg, 0, s, p);
  } else {
    if (one_reader) hipLaunchKernelGGL((decode_balanced_kernel<D, FP8, false, 1, true>), grid, wg, 0, s, p);
    else hipLaunchKernelGGL((decode_balanced_kernel<D, FP8, false, 1, false>), grid, wg, 0, s, p);
  }
  return hipGetLastError();
}

}  // namespace

bool decode_mfma_supported(const DecodeParams& p, int q_dtype, int kv_dtype) {
  if (q_dtype != PA_BF16) return false;
  if (kv_dtype != PA_BF16 && kv_dtype != PA_FP8_E4M3FN) return false;
  if (p.D != 64 && p.D != 128) return false;
  if (p.block_shift < 4) return false;   // power-of-two block size >= 16
  return true;
}

bool decode_new_row_supported(const DecodeParams& p, int q_dtype, int kv_dtype) {
  if (!decode_mfma_supported(p, q_dtype, kv_dtype) || kv_dtype != PA_BF16) return false;
  if (!p.query_lens) return p.T == 1;
  // multi-token rows: all rows of a kv head on one 16-row wave, at most 16 tokens
  return p.rows_per_wave == 16 && (p.Hq / p.Hkv) * p.T <= 16 && p.T <= 16;
}

hipError_t launch_decode_mfma(const DecodeParams& p, int kv_dtype, int waves, hipStream_t s) {
  const bool fp8 = kv_dtype == PA_FP8_E4M3FN;
  if (p.D == 128) return fp8 ? launch_typed<128, true>(p, waves, s) : launch_typed<128, false>(p, waves, s);
  if (p.D == 64) return fp8 ? launch_typed<64, true>(p, waves, s) : launch_typed<64, false>(p, waves, s);
  return hipErrorInvalidValue;
}

void plan_decode_balanced(DecodeParams& p, int num_cus) {
  const int head_slots = head_slots_of(p);
  constexpr int kWavesPerCu = 8;                       // two per SIMD at this register footprint
  p.bal_hsw = head_slots < kWavesPerCu ? head_slots : kWavesPerCu;
  p.bal_ns = kWavesPerCu / p.bal_hsw;
  const int head_groups = (head_slots + p.bal_hsw - 1) / p.bal_hsw;
  int wgs = num_cus / head_groups;                     // workgroups per head group: one per CU in total
  if (wgs < 1) wgs = 1;
  p.bal_gv = wgs * p.bal_ns;
}

size_t decode_balanced_workspace_bytes(int B, int Hq, int D, int gv) {
  // partials [B + gv piece slots][Hq rows][D + 2] floats, then B + 1 tile prefix sums
  return (size_t)Hq * ((size_t)B + gv) * ((size_t)D + 2) * sizeof(float) + ((size_t)B + 1) * sizeof(int32_t);
}

hipError_t launch_decode_balanced(const DecodeParams& p, int kv_dtype, hipStream_t s) {
  const bool fp8 = kv_dtype == PA_FP8_E4M3FN;
  if (p.D == 128) return fp8 ? launch_balanced_typed<128, true>(p, s) : launch_balanced_typed<128, false>(p, s);
  if (p.D == 64) return fp8 ? launch_balanced_typed<64, true>(p, s) : launch_balanced_typed<64, false>(p, s);
  return hipErrorInvalidValue;
}

template <int G>
static hipError_t launch_reduce_g(const DecodeParams& p, hipStream_t s) {
  const int items = p.Hq * p.T * (p.D / 4);
  if (G == 1 && p.B >= 2048) {
    if (p.D == 128) hipLaunchKernelGGL((decode_balanced_reduce_kernel<128, 1, true>), dim3(p.B), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((decode_balanced_reduce_kernel<64, 1, true>), dim3(p.B), dim3(256), 0, s, p);
    return hipGetLastError();
  }
  dim3 grid(p.B, (items * G + 255) / 256);
  if (p.D == 128) hipLaunchKernelGGL((decode_balanced_reduce_kernel<128, G>), grid, dim3(256), 0, s, p);
  else hipLaunchKernelGGL((decode_balanced_reduce_kernel<64, G>), grid, dim3(256), 0, s, p);
  return hipGetLastError();
}

hipError_t launch_decode_balanced_reduce(const DecodeParams& p, hipStream_t s) {
  // lanes per item by the number of pieces a sequence is cut into on average: a sequence spans
  // about gv / B chunks (few sequences, or few kv heads and hence several chunks per workgroup)
  const int pieces = p.bal_gv / p.B;
  if (pieces >= 64) return launch_reduce_g<32>(p, s);
  if (pieces >= 8) return launch_reduce_g<8>(p, s);
  return launch_reduce_g<1>(p, s);
}

}  // namespace pa
