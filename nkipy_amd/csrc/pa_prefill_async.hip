// Causal flash-attention prefill on the gfx950 matrix cores, asynchronous form:
// K and V tiles travel HBM/L2 -> LDS with global_load_lds_dwordx4 (no registers,
// several tiles in flight in a ring of LDS stages) and V^T fragments are read with
// the transposing LDS load ds_read_b64_tr_b16, so nothing is transposed by hand.
//
// One workgroup of NW wavefronts owns 32*NW query rows of one (sequence, q head);
// each wavefront owns 32 of them.  Keys are walked in tiles of 64.
//
// v_mfma_f32_32x32x16_bf16 operand layout (lane = 32*h + n, h = 0..1, n = 0..31):
//   A[32 x 16]: lane holds row n, k-slots 8h .. 8h+7
//   B[16 x 32]: lane holds column n, k-slots 8h .. 8h+7
//   C/D[32x32]: lane holds column n, rows 8*(i/4) + 4h + (i%4) for i = 0..15
// Scores are computed transposed, S^T[key, q] = K[key, :] . Q^T[:, q]: a lane's
// column is one query row, so the online-softmax state is per-lane scalars and
// the probabilities are already the B operand of O^T[d, q] += V^T[d, key] P^T[key, q]
// (MFMA kk of a 32-key sub-tile takes accumulator registers 8kk .. 8kk+7, i.e.
// k-slot 8h+j <-> key 16kk + 8(j/4) + 4h + (j%4)).
//
// LDS stage = K tile [64 keys][256 B] + V tile [64 keys][256 B], both row-major
// exactly as in the pool; the 16-byte chunk index of a row is XORed with
// (row & 15) for K and 4 * (row & 3) for V so that the b128 reads of K (32 rows,
// same chunk: 16 consecutive lanes must hit 16 different chunk positions) and the
// transposing reads of V (8 rows, a 64-byte window each: 4 rows must hit 4 different
// windows) run at the full LDS rate; narrower swizzles measured 65 % of it.  The
// swizzle costs nothing: a DMA lane may fetch any global chunk into its fixed LDS slot.
//
// ds_read_b64_tr_b16, per group of 16 lanes: lane i receives, for j = 0..3, the
// (i%4)-th 16-bit element of the 8 bytes addressed by lane (i/4) + 4j.  Source
// lane s therefore points at key row (s/4) and d columns 4*(s%4) .. +3 of the
// group's 16-column window; lane i ends up with 4 keys at one d.
//
// Masking follows examples/models/gpt_oss/kernels/attention.py:85,127-135: query
// i of a chunk that starts at `prefix` sees keys j <= prefix + i.
#include <atomic>

#include "pa_common.h"



namespace pa {
namespace {

constexpr int HD = 128;                // elements of a 256-byte row: the head dim, or two heads of 64
constexpr int ROW_B = HD * 2;          // bytes per K/V row
// Where the 8-element chunks of a Q row sit: lane (n, h) holds chunk 2 s + h in slot s, so the
// lowest chunk-index bit is the half-wave and the others are the slot number.
struct QRowLayout {
  static __device__ __forceinline__ int chunk(int s, int h) { return 2 * s + h; }
  static constexpr int slot_xor(int bit) { return bit >> 1; }
  static constexpr int lane_xor(int bit) { return bit == 1 ? 32 : 0; }
};

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) char lds_char;

__device__ __forceinline__ bf16x8_t make_frag(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  u32x4_t v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8_t, v);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// 16-byte-per-lane copy HBM/L2 -> LDS without registers: lane i's bytes land at
// lds_base + 16 i.  Issued as inline assembly so that the compiler's wait-count
// insertion does not treat every later LDS read as dependent on every copy still in
// flight (it would drain the whole ring with vmcnt(0)); the waits are placed by hand.
__device__ __forceinline__ void dma16_uniform(const char* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(lane_off), "s"(base), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void dma16_lane(const char* addr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(addr), "s"(lds_base) : "memory", "m0");
}
// The same as streaming (non-temporal) copies, for tiles that no other workgroup reads: a line that is read once
// and not kept in the caches comes from HBM at a higher rate.
__device__ __forceinline__ void dma16_uniform_stream(const char* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
               :: "v"(lane_off), "s"(base), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void dma16_lane_stream(const char* addr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
               :: "v"(addr), "s"(lds_base) : "memory", "m0");
}

// Block-table reads go through the constant address space: wave-uniform indices then
// become scalar loads (their own counter), not vector loads that would have to be
// waited for in order with the copies above.
typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;

// MODE: 0 = dense K/V [B, S, Hkv, D]; 1 = paged, block size a power of two >= 16.
// TT: 32-key sub-tiles per key tile (2: 64-key tiles).
// PACK (short chunks of a GQA model): the query rows of a workgroup are (token, head) pairs of one
// kv head, token-major, instead of 32*NW tokens of one q head: a chunk of T < 32*NW tokens then fills
// the tile with n_rep heads' rows that share every K/V tile, where the plain form would run n_rep
// workgroups with mostly padding rows.
// SPLIT (few workgroups, long contexts): p.splits workgroups share the key tiles of one query tile
// and leave unnormalised partial results (m, l, O) in the workspace for prefill_split_reduce_kernel:
// a lone workgroup walks its tiles at about a microsecond each, whatever the rest of the chip does.
// FP8 (8 waves, paged): the pool holds e4m3fn codes with a float32 scale per (block, kv head).  The
// copies bring raw codes into a ring of four 16 KB stages; every wave then expands the 8 rows it
// copied itself (codes x their block's scale -> bf16, once per workgroup, not once per reader) into one
// of two bf16 stages in exactly the layout the bf16 path copies into, one tile ahead of the
// compute, so everything from the fragment reads on is shared.  Raw rows are private to the wave that
// copies and expands them, so the raw ring needs no barrier; the bf16 stages use the one per tile.
// DH: head dim, 128 or 64.  At 64 a 256-byte piece of a pool row is two adjacent kv heads: the tile
// layout stays that of 256-byte rows and the two halves of the workgroup's waves work for the two heads.
// QH (head dim 64 only): q heads of one kv group per wave, 1 or 2.  With 2 a wave carries the same 32 query
// tokens for two adjacent q heads: every K and V tile then serves twice the matrix work (at head dim 64 a tile
// otherwise has half the matrix work of head dim 128 against the same copies and barrier), and between two
// barriers the waves of a SIMD have twice as many matrix and vector phases to slide under one another.
template <bool SPARSE, int MODE, int NW, int TT, bool WIN, bool PACK, bool SPLIT, bool FP8, int DH, int QH>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void prefill_async_kernel(PrefillParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int BN = 32 * TT;                // keys per tile
  constexpr int TILE_B = BN * ROW_B;         // one tensor's tile in LDS
  constexpr int STAGE_B = 2 * TILE_B;        // K then V
  constexpr int UK = BN / 4;                 // 1 KB copy units per tensor tile
  constexpr int BMW = 32 * NW;               // query rows per workgroup
  // Head dim 64 (PAIR): a 256-byte row of the pool then holds two adjacent kv heads, and the LDS tile
  // layout, the copies and the fragment maps stay those of 256-byte rows.  The first half of the waves
  // works for a q head of the even kv head on the rows' first 128 bytes, the second half for the q head
  // at the same place in the odd kv head's group on the other 128 bytes; both halves take the same
  // TOKW query tokens, so every byte copied is used.  An odd number of kv heads leaves the last head without
  // a partner: its workgroups take the 256 bytes that end with it (the pair one head earlier), the second half
  // of the waves works for it and the first half only copies (`idle_half`).
  constexpr bool PAIR = DH == 64;
  static_assert(DH == HD || (PAIR && NW == 8 && MODE == 1 && !SPARSE && !PACK), "head dim 64: 8-wave paged dense form only");
  static_assert(QH == 1 || (QH == 2 && PAIR), "two q heads per wave: head dim 64 only");
  constexpr int KS = DH / 16;                // k-steps of the score product
  constexpr int VC = DH / 32;                // 32-wide d chunks of the output
  constexpr int TOKW = PAIR ? BMW / 2 : BMW; // query tokens per workgroup (plain form)
  // Blocksparse with 8 waves (STAG): the workgroup's four 64-row query blocks walk the vertical-stride tiles together
  // and then the local band STAGGERED: at band step s the q block j works on key tile (its own block) - local + 1 + s,
  // so all four are busy on four different resident tiles for exactly `local` steps and one new tile is requested per
  // step (four resident stages + one in flight).
  constexpr bool STAG = SPARSE && NW == 8;
  constexpr int NST = STAG ? 5 : NW == 8 ? 4 : 2;   // LDS stages the copies land in
  constexpr int UPW = FP8 ? 2 : 2 * UK / NW; // copy units per wave per tile (FP8: 8 raw rows of K, 8 of V)
  static_assert(!FP8 || (NW == 8 && MODE == 1 && !SPARSE && !PACK && TT == 2), "fp8 pools: 8-wave paged dense form only");
  constexpr int EB = FP8 ? 1 : 2;            // bytes per pool element
  constexpr int RAW_TILE_B = BN * HD;        // FP8: one tensor's raw tile
  constexpr int RAW_STAGE_B = 2 * RAW_TILE_B;
  constexpr int BFS = FP8 ? 2 : NST;         // stages that hold bf16 tiles (FP8: the raw ring lies behind them)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  // ---- which (sequence, head, query tile): kv-head groups are spread over the 8 XCDs
  // (consecutive workgroup ids go to consecutive XCDs), and all query tiles and q heads
  // that share one kv head run on one XCD, back to back, heavy tiles first: their K/V
  // stays in that XCD's L2.
  const int n_rep = p.Hq / p.Hkv;
  const int nqt = PACK ? (p.T * n_rep + BMW - 1) / BMW : (p.T + TOKW - 1) / TOKW;
  const int kvg = PAIR ? (p.Hkv + 1) / 2 : p.Hkv;    // K/V row groups: kv heads, or pairs of them
  const int hpg = n_rep / QH;                  // workgroups (per query tile) that cover the q heads of a kv head
  const int per_group = PACK ? nqt : nqt * hpg;
  // PACK with one row tile per kv head: this workgroup is the only reader of its keys and values
  const bool stream_kv = PACK && nqt == 1;
  const int groups = p.B * kvg;
  const int xcd = blockIdx.x & 7;
  const int part = SPLIT ? (int)(blockIdx.x >> 3) % p.splits : 0;      // which share of the key tiles
  const int slot = SPLIT ? (int)(blockIdx.x >> 3) / p.splits : (int)(blockIdx.x >> 3);
  const int grp = xcd + 8 * (slot / per_group);
  if (grp >= groups) return;
  const int rr_ = slot % per_group;
  const int b = grp / kvg, hk = grp % kvg;     // PAIR: hk numbers the pair
  const int qt = PACK ? nqt - 1 - rr_ : nqt - 1 - rr_ / hpg;
  const int kv0 = PAIR ? min(2 * hk, p.Hkv - 2) : hk;    // first kv head of the rows' 256 bytes (PAIR: Hkv >= 2, checked on the host)
  const int hq = PACK ? hk * n_rep : kv0 * n_rep + QH * (rr_ % hpg);     // PACK: first head of the group; PAIR: the first kv head's; QH 2: and hq + 1
  // row r of the workgroup (0 .. BMW-1) -> query token and q head
  const int v0 = qt * TOKW;
  auto row_token = [&](int r) __attribute__((always_inline)) { return PACK ? (v0 + r) / n_rep : v0 + (PAIR ? (r & (TOKW - 1)) : r); };
  auto row_head = [&](int r) __attribute__((always_inline)) { return PACK ? hq + (v0 + r) % n_rep : hq + (PAIR && r >= TOKW ? n_rep : 0); };
  const int par = PAIR ? wave / (NW / 2) : 0;   // which 128 bytes of the rows this wave works on
  const bool lone = PAIR && 2 * hk + 1 >= p.Hkv;          // the unpaired last head of an odd Hkv
  const bool idle_half = lone && par == 0;                // these waves' head belongs to the pair before: copies only

  int tq = p.query_lens ? p.query_lens[b] : p.T;
  int ctx = p.seq_lens ? p.seq_lens[b] : p.S;
  tq = min(max(tq, 0), p.T);
  if (MODE != 0) ctx = min(ctx, p.max_blocks * p.block_size);
  ctx = max(ctx, 0);
  tq = min(tq, ctx);          // more query tokens than context: the first ctx of them count, without a prefix (as pa_verify)
  const int prefix = ctx - tq;
  const int q0 = row_token(0);                                    // first query token of the workgroup
  uint16_t* out = (uint16_t*)p.out;
  const long q_row_stride = (long)p.Hq * DH;

  if (q0 >= tq) {   // only padding rows here: zeros (written by the reduce kernel when splitting)
    if (SPLIT) return;
    for (int i = tid; i < BMW * (DH / 8); i += NW * 64) {
      const int r = i / (DH / 8);
      const int row = row_token(r);
      if (row < p.T && !(lone && r < TOKW)) {
#pragma unroll
        for (int j = 0; j < QH; ++j)
          *(uint4*)(out + ((long)b * p.T + row) * q_row_stride + (long)(row_head(r) + j) * DH + (i % (DH / 8)) * 8) = make_uint4(0, 0, 0, 0);
      }
    }
    return;
  }

  // ---- this lane's query row (token index qrow, head hq_l; QH 2: also head hq_l + 1) and its Q^T fragments ----
  const int qrow = row_token(wave * 32 + n);
  const int hq_l = row_head(wave * 32 + n);
  const bool qvalid = qrow < tq && !idle_half;
  const int qlim = prefix + min(qrow, tq - 1);     // last visible key of this lane's row
  const float sc = p.scale_log2e;
  bf16x8_t qf[QH][KS];            // loaded below, between the first copy requests
  const int wq_lo = row_token(wave * 32);                         // first token of this wave
  const int wq_hi = min(row_token(wave * 32 + 31), tq - 1);       // last valid token (may be < wq_lo)
  const bool wave_has_rows = wq_lo < tq && !idle_half;
  const int k_end = prefix + min(row_token(BMW - 1) + 1, tq);     // keys the workgroup needs: [0, k_end)
  // sliding window (its own instantiation, so that the plain form carries none of its scalar
  // work): the row at position pos sees keys (pos - win, pos]
  const int win = WIN ? p.window : 0;
  // key tiles of this workgroup: [kt_begin, ntiles)
  int kt_begin = win > 0 ? max(prefix + q0 - win + 1, 0) / BN : 0;   // first tile the first row sees
  int ntiles = (k_end + BN - 1) / BN;
  const long row_g = ((long)b * p.T + qrow) * p.Hq + hq_l;            // this lane's (first) row among all B * T * Hq
  if (SPLIT) {
    const int n_all = ntiles - kt_begin;
    const int lo = kt_begin + (int)((long)part * n_all / p.splits);
    ntiles = kt_begin + (int)((long)(part + 1) * n_all / p.splits);
    kt_begin = lo;
    if (kt_begin >= ntiles) {                  // nothing for this share: an empty partial
#pragma unroll
      for (int j = 0; j < QH; ++j)
        if (qvalid && h == 0) *(float2*)(p.ws_ml + ((row_g + j) * p.splits + part) * 2) = make_float2(-INFINITY, 0.f);
      return;
    }
  }

  // ---- DMA maps ---------------------------------------------------------------------
  // A tile is 2 UK units of 1 KB (4 rows): the first UK are K, the rest V.  Wave w issues
  // units w, w + NW, ...  In a unit lane i fills LDS slot (row 4u + i/16, position i%16)
  // with the global chunk  position ^ (row & 7).
  const const_i32_ptr table = MODE != 0 ? (const_i32_ptr)(uintptr_t)(p.block_tables + (long)b * p.max_blocks) : nullptr;
  const uint32_t smem_base = (uint32_t)(uintptr_t)(lds_char*)smem;
  const long kv_row_bytes = (long)p.Hkv * DH * EB;
  const char* kbase = (const char*)p.k + (long)kv0 * DH * EB;    // PAIR: 256 bytes from kv head kv0 on
  const char* vbase = (const char*)p.v + (long)kv0 * DH * EB;
  const int dma_rr = lane >> 4, dma_pos = lane & 15;
  // every unit of a wave starts at the same row modulo 16 (NW is a multiple of 4), hence the
  // same swizzle: K rows use row & 15, V rows 4 * (row & 3) (what their read patterns want)
  const int dma_chunk_k = dma_pos ^ ((4 * (wave & 3) + dma_rr) & 15);
  const int dma_chunk_v = dma_pos ^ (4 * dma_rr);
  const uint32_t kv_row_bytes_u = (uint32_t)kv_row_bytes;
  const uint32_t block_bytes_u = MODE != 0 ? (uint32_t)p.block_size * kv_row_bytes_u : 0u;
  const int dma_lane_off_k = (int)(dma_rr * kv_row_bytes) + dma_chunk_k * 16;
  const int dma_lane_off_v = (int)(dma_rr * kv_row_bytes) + dma_chunk_v * 16;
  // FP8: a unit is 8 raw rows of 128 B, copied as they lie: lane i -> row i / 8, 16-byte piece i % 8
  const int dma_lane_off_raw = (int)((lane >> 3) * kv_row_bytes) + (lane & 7) * 16;

  auto lane_row = [&](int key) __attribute__((always_inline)) -> long {   // same, per lane, clamped
    key = min(key, ctx - 1);
    if (MODE == 0) return (long)b * p.S + key;
    int blk = table[key >> p.block_shift];
    blk = min(max(blk, 0), p.num_blocks - 1);
    return (long)blk * p.block_size + (key & (p.block_size - 1));
  };
  // Block-table entries of the tile that will be requested next, fetched one request early:
  // the scalar loads then complete under a whole tile of compute instead of in front of the
  // copies that need them.  K and V units of a wave share their rows, hence UPW/2 entries.
  int blk_pf[UPW / 2];
  auto prefetch_table = [&](int kt) __attribute__((always_inline)) {
    if (MODE == 0) return;
#pragma unroll
    for (int i = 0; i < UPW / 2; ++i) {
      const int r0 = FP8 ? 8 * wave : 4 * ((wave + NW * i) & (UK - 1));
      blk_pf[i] = table[min((kt * BN + r0) >> p.block_shift, p.max_blocks - 1)];
    }
  };
  // The UPW copy units of this wave for tile kt, K first: unit j covers rows 4u .. 4u+3 of
  // the K (j < UPW/2) or V tile, u = (wave + NW j) mod UK.
  auto issue_tile = [&](int kt, int stage) __attribute__((always_inline)) {
    const int key0 = kt * BN;
    if (FP8) {       // this wave's 8 rows of K and of V, raw, into its own 1 KB of the raw stage
      const uint32_t rbase = smem_base + BFS * STAGE_B + stage * RAW_STAGE_B + wave * 1024;
      if (key0 + BN <= ctx) {
        const uint32_t blk = (uint32_t)min(max(blk_pf[0], 0), p.num_blocks - 1);
        const uint64_t off = (uint64_t)blk * block_bytes_u + (uint32_t)((key0 + 8 * wave) & (p.block_size - 1)) * kv_row_bytes_u;
        dma16_uniform(kbase + off, dma_lane_off_raw, rbase);
        dma16_uniform(vbase + off, dma_lane_off_raw, rbase + RAW_TILE_B);
      } else {
        const long src = lane_row(key0 + 8 * wave + (lane >> 3)) * kv_row_bytes + (lane & 7) * 16;
        dma16_lane(kbase + src, rbase);
        dma16_lane(vbase + src, rbase + RAW_TILE_B);
      }
      return;
    }
    const uint32_t sbase = smem_base + stage * STAGE_B;
    if (key0 + BN <= ctx) {                       // whole tile inside the context: one row base per unit
      // byte offset of a unit's first row = block * (block bytes) + in-block row * (row bytes):
      // one 32x32->64 multiply and one 32-bit multiply on the scalar ALU (both factors fit 32
      // bits, checked on the host); K and V units of a wave share it
#pragma unroll
      for (int j = 0; j < UPW / 2; ++j) {
        const int u = (wave + NW * j) & (UK - 1);
        uint64_t off;
        if (MODE == 0) {
          off = (uint64_t)(uint32_t)(b * p.S + key0 + 4 * u) * kv_row_bytes_u;
        } else {
          const uint32_t blk = (uint32_t)min(max(blk_pf[j], 0), p.num_blocks - 1);
          off = (uint64_t)blk * block_bytes_u + (uint32_t)((key0 + 4 * u) & (p.block_size - 1)) * kv_row_bytes_u;
        }
        if (PACK && stream_kv) {
          dma16_uniform_stream(kbase + off, dma_lane_off_k, sbase + u * 1024);
          dma16_uniform_stream(vbase + off, dma_lane_off_v, sbase + TILE_B + u * 1024);
        } else {
          dma16_uniform(kbase + off, dma_lane_off_k, sbase + u * 1024);
          dma16_uniform(vbase + off, dma_lane_off_v, sbase + TILE_B + u * 1024);
        }
      }
    } else {                                      // last tile of a context: rows past it re-read its last row
#pragma unroll
      for (int j = 0; j < UPW; ++j) {
        const bool is_k = j < UPW / 2;
        const int u = (wave + NW * j) & (UK - 1);
        const char* src = (is_k ? kbase : vbase) + lane_row(key0 + 4 * u + dma_rr) * kv_row_bytes + (is_k ? dma_chunk_k : dma_chunk_v) * 16;
        if (PACK && stream_kv) dma16_lane_stream(src, sbase + (is_k ? 0 : TILE_B) + u * 1024);
        else dma16_lane(src, sbase + (is_k ? 0 : TILE_B) + u * 1024);
      }
    }
  };

  // ---- LDS read maps (lane constants) -------------------------------------------------
  int k_off[KS];                      // K fragment of k-step s: row n, chunk 2s + h (PAIR: of this wave's half)
#pragma unroll
  for (int s = 0; s < KS; ++s) k_off[s] = n * ROW_B + (((2 * (KS * par + s) + h) ^ (n & 15)) << 4);
  int v_off[VC];                      // V^T fragment source of d-chunk c
  {
    const int g = lane >> 4, sl = lane & 15;
    const int row = 4 * h + (sl >> 2);                       // key row inside a 16-key window (also row & 7)
    const int y = 2 * (g & 1) + ((sl & 3) >> 1);             // 16-byte chunk inside the 64-byte d window
#pragma unroll
    for (int c = 0; c < VC; ++c) v_off[c] = row * ROW_B + (((4 * (VC * par + c) + y) ^ (4 * (row & 3))) << 4) + (sl & 1) * 8;
  }

  // ---- accumulators ------------------------------------------------------------
  f32x16_t oacc[QH][VC];
#pragma unroll
  for (int j = 0; j < QH; ++j)
#pragma unroll
    for (int c = 0; c < VC; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[j][c][i] = 0.f;
  // Softmax state of this lane's query row.  Scores come out of the matrix cores already
  // relative to a reference m_ref (the accumulator starts at -m_ref), in log2 units.  The
  // reference is set to the row maximum of the first tile in which the row sees a key and
  // after that moves only when float range is at stake (see softmax below), so in the steady
  // state there is no row maximum, no per-element subtraction and no rescaling of the output
  // accumulators.  When it does move it goes to the tile's maximum.
  constexpr float REF_SLACK = 8.f;
  float m_ref[QH], l_run[QH];
  float slack[QH];                    // -inf until the row has seen a finite score (m_ref is arbitrary till then)
  bool fresh_rows[QH];                // wave-uniform: some row of the wave still has slack == -inf
  f32x16_t cinit[QH];                 // -m_ref in every accumulator slot
#pragma unroll
  for (int j = 0; j < QH; ++j) {
    m_ref[j] = 0.f; l_run[j] = 0.f; slack[j] = -INFINITY; fresh_rows[j] = true;
#pragma unroll
    for (int i = 0; i < 16; ++i) cinit[j][i] = 0.f;
  }

  const int head_phase = SPARSE ? hq % p.sparse_stride : 0;
  const int qblk = wq_lo / 64;                    // sparse: q block of this wave
  const int wg_blk_lo = q0 / 64;
  // Walk over the key tiles the workgroup needs.  Dense: every tile.  Sparse: a tile (= one
  // 64-key sparsity block) is needed if it is a vertical-stride column, (kt + head_phase) %
  // stride == 0, or lies in the local window of some q block of the workgroup, kt >=
  // first_local.  The phase is carried along, so a step costs a few scalar instructions and no
  // integer division however many tiles it skips.
  struct Walk { int kt, ph; };
  const int first_local = wg_blk_lo - p.sparse_local + 1;
  auto walk_settle = [&](Walk& w) __attribute__((always_inline)) {      // to the first needed tile >= w.kt
    if (!SPARSE) return;
    if (w.kt >= first_local || w.ph == 0) return;
    const int jump = p.sparse_stride - w.ph;                             // to the next vertical column
    if (w.kt + jump >= first_local) {
      w.ph += first_local - w.kt;
      if (w.ph == p.sparse_stride) w.ph = 0;
      w.kt = first_local;
    } else {
      w.kt += jump;
      w.ph = 0;
    }
  };
  auto walk_step = [&](Walk& w) __attribute__((always_inline)) {
    ++w.kt;
    if (SPARSE) {
      if (++w.ph == p.sparse_stride) w.ph = 0;
      walk_settle(w);
    }
  };

  // does this wave compute on tile w.kt?
  auto tile_active = [&](const Walk& w) __attribute__((always_inline)) -> bool {
    bool act = wave_has_rows && w.kt * BN <= prefix + wq_hi;
    if (win > 0) act = act && (w.kt + 1) * BN > prefix + wq_lo - win + 1;   // tile ends inside the first row's window
    if (SPARSE) act = act && w.kt <= qblk && (qblk - w.kt < p.sparse_local || w.ph == 0);
    return act;
  };
  // ---- ring of NST stages: tiles are requested NST-1 ahead; requests past the end are
  // repeated on the first tile so that the wait counter stays exact ------------------------
  Walk w_first = {kt_begin, head_phase};
  walk_settle(w_first);
  const int kt_first = w_first.kt;
  Walk w_i = w_first;                 // next tile to request
  int stage_i = 0;                    // ... and the stage it goes to
  // The entries for the following request are fetched in the middle of a tile's work, after
  // its last wait on K fragments and before the softmax, where no LDS read is pending: a
  // scalar load in flight turns every LDS wait into a wait for everything.
  auto prefetch_next = [&]() __attribute__((always_inline)) { prefetch_table(w_i.kt < ntiles ? w_i.kt : kt_first); };
  prefetch_table(kt_first);
  // FP8: scales of this wave's rows in the tiles in flight (its 8 rows lie in one block); a request
  // puts the new pair in slot 3, a shift per tile brings it to slot 0 when the tile is expanded
  typedef const __attribute__((address_space(4))) float* const_f32_ptr;
  float ksq[4] = {0.f, 0.f, 0.f, 0.f}, vsq[4] = {0.f, 0.f, 0.f, 0.f};
  float ksq2[4] = {0.f, 0.f, 0.f, 0.f}, vsq2[4] = {0.f, 0.f, 0.f, 0.f};      // PAIR: the odd kv head's
  // STAG: request r is vertical tile number r (tiles stag_v0 + r * stride, those some q block of the workgroup sees
  // below its local window) for r < stag_nv, then band tile stag_band0 + (r - stag_nv); requests that fall outside
  // [0, ntiles) are clamped into it (they re-read a valid tile and are never consumed, but keep the wait counts exact)
  constexpr int QB = BMW / 64;                  // q blocks per workgroup
  const int stag_v0 = head_phase == 0 ? 0 : p.sparse_stride - head_phase;
  const int stag_vmax = min(wg_blk_lo + QB - 1 - p.sparse_local, ntiles - 1);
  const int stag_nv = STAG && stag_vmax >= stag_v0 ? (stag_vmax - stag_v0) / p.sparse_stride + 1 : 0;
  // band steps in which every q block's tile would lie before tile 0 are left out (a local window longer than the
  // sequence so far)
  const int stag_skip = max(p.sparse_local - wg_blk_lo - QB, 0);
  const int stag_band0 = wg_blk_lo - p.sparse_local + 1 + stag_skip;
  int stag_req = 0;                             // next request
  auto request_next = [&]() __attribute__((always_inline)) {
    if constexpr (STAG) {
      const int t = stag_req < stag_nv ? stag_v0 + stag_req * p.sparse_stride : stag_band0 + (stag_req - stag_nv);
      issue_tile(min(max(t, 0), ntiles - 1), stage_i);
      ++stag_req;
      stage_i = stage_i + 1 == NST ? 0 : stage_i + 1;
      return;
    }
    issue_tile(w_i.kt < ntiles ? w_i.kt : kt_first, stage_i);
    if (FP8) {
      const long si = (long)min(max(blk_pf[0], 0), p.num_blocks - 1) * p.Hkv + kv0;
      ksq[3] = ((const_f32_ptr)(uintptr_t)p.k_scale)[si];
      vsq[3] = ((const_f32_ptr)(uintptr_t)p.v_scale)[si];
      if (PAIR) {
        ksq2[3] = ((const_f32_ptr)(uintptr_t)p.k_scale)[si + 1];
        vsq2[3] = ((const_f32_ptr)(uintptr_t)p.v_scale)[si + 1];
      }
    }
    if (w_i.kt < ntiles) walk_step(w_i);
    stage_i = stage_i + 1 == NST ? 0 : stage_i + 1;
  };
  auto shift_scales = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      ksq[i] = ksq[i + 1]; vsq[i] = vsq[i + 1];
      if (PAIR) { ksq2[i] = ksq2[i + 1]; vsq2[i] = vsq2[i + 1]; }
    }
  };
  // FP8: codes of tile kt in raw stage rs -> bf16 values in stage bs, this wave's 8 rows; rows past the
  // context get the scale 0 (their codes are a copy of the last valid row, their block may not exist)
  // A lane expands one 16-byte chunk (8 codes) of two rows, rows lane / 16 and lane / 16 + 4 of the wave's eight,
  // chunk lane % 16: a store instruction then writes whole rows, 16 consecutive lanes the 16 different chunk
  // positions of one row, and no two of them share a bank.  (With a lane expanding 16 codes of one row into two
  // chunks, the lanes of a row wrote every other chunk position per instruction and collided pairwise.)
  auto expand = [&](int kt, int rs, int bs) __attribute__((always_inline)) {
    const char* raw = smem + BFS * STAGE_B + rs * RAW_STAGE_B + wave * 1024;
    const int ch = lane & 15;
    // PAIR: the first 64 codes of a raw row belong to the even kv head, the others to the odd one
    const float ks = PAIR && ch >= 8 ? ksq2[0] : ksq[0], vs = PAIR && ch >= 8 ? vsq2[0] : vsq[0];
    auto widen = [&](uint2 c, float scl) __attribute__((always_inline)) -> uint4 {
      float f[8];
      fp8x4_to_float(c.x, f);
      fp8x4_to_float(c.y, f + 4);
      return make_uint4(pack_bf16x2(f[0] * scl, f[1] * scl), pack_bf16x2(f[2] * scl, f[3] * scl),
                        pack_bf16x2(f[4] * scl, f[5] * scl), pack_bf16x2(f[6] * scl, f[7] * scl));
    };
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int lrow = (lane >> 4) + 4 * u, row = 8 * wave + lrow;
      const bool live = kt * BN + row < ctx;
      const uint2 rk = *(const uint2*)(raw + lrow * HD + ch * 8), rv = *(const uint2*)(raw + RAW_TILE_B + lrow * HD + ch * 8);
      char* kd = smem + bs * STAGE_B + row * ROW_B;
      *(uint4*)(kd + ((ch ^ (row & 15)) << 4)) = widen(rk, live ? ks : 0.f);
      *(uint4*)(kd + TILE_B + ((ch ^ (4 * (row & 3))) << 4)) = widen(rv, live ? vs : 0.f);
    }
  };

  // ---- fragment loads and matrix steps, one "group" at a time -------------------------
  // A group is the 8 K fragments of a 32-key sub-tile (8 MFMAs) or the 4 V^T fragments of
  // a 16-key slice (4 MFMAs).  The loads of group g+1 are written before the MFMAs of group
  // g; where exactly they issue is left to the compiler's scheduler (pinning the order with
  // scheduling barriers measured 3 % slower).
  auto load_k = [&](bf16x8_t (&kf)[KS], int stage, int tt) __attribute__((always_inline)) {
    const char* ks = smem + stage * STAGE_B + 32 * tt * ROW_B;
#pragma unroll
    for (int s = 0; s < KS; ++s) kf[s] = *(const bf16x8_t*)(ks + k_off[s]);
  };
  auto load_v = [&](bf16x8_t (&vf)[VC], int stage, int g) __attribute__((always_inline)) {   // g = 2 tt + kk
    const char* vs = smem + stage * STAGE_B + TILE_B + 16 * g * ROW_B;
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const lds_char* src = (const lds_char*)(vs + v_off[c]);
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)src);
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(src + 8 * ROW_B));
      struct { s16x4_t a, b; } pair = {lo, hi};
      vf[c] = __builtin_bit_cast(bf16x8_t, pair);
    }
  };
  auto mma_qk = [&](f32x16_t& sacc, const bf16x8_t (&kf)[KS], int j) __attribute__((always_inline)) {
    sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[0], qf[j][0], cinit[j], 0, 0, 0);
#pragma unroll
    for (int s = 1; s < KS; ++s)
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s], qf[j][s], sacc, 0, 0, 0);
  };
  auto mma_pv = [&](const bf16x8_t (&vf)[VC], const uint32_t (&pw)[8], int kk, int j) __attribute__((always_inline)) {
    const bf16x8_t pf = make_frag(pw[4 * kk], pw[4 * kk + 1], pw[4 * kk + 2], pw[4 * kk + 3]);
#pragma unroll
    for (int c = 0; c < VC; ++c)
      oacc[j][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[c], pf, oacc[j][c], 0, 0, 0);
  };
  // S^T = K Q^T of head j for the tile in `stage`; leaves the first V^T group of `vstage` in flight
  auto scores = [&](f32x16_t (&sacc)[TT], int stage, bf16x8_t (&v0)[VC], int vstage, int j) __attribute__((always_inline)) {
    bf16x8_t ka[KS], kb[KS];
    load_k(ka, stage, 0);
    if (TT == 2) {
      load_k(kb, stage, 1);
      mma_qk(sacc[0], ka, j);
      load_v(v0, vstage, 0);
      mma_qk(sacc[TT - 1], kb, j);
    } else {
      load_v(v0, vstage, 0);
      mma_qk(sacc[0], ka, j);
    }
  };
  // O^T += V^T P^T of head j for the tile in `stage`; group 0's fragments were loaded by scores()
  auto accumulate = [&](const uint32_t (&pw)[TT][8], int stage, bf16x8_t (&v0)[VC], int j) __attribute__((always_inline)) {
    bf16x8_t v1[VC];
#pragma unroll
    for (int g = 0; g < 2 * TT; g += 2) {
      load_v(v1, stage, g + 1);
      mma_pv(v0, pw[g >> 1], 0, j);
      if (g + 2 < 2 * TT) load_v(v0, stage, g + 2);
      mma_pv(v1, pw[g >> 1], 1, j);
    }
  };
  // The same with the products of the last two groups left for later: their V^T fragments end up in dv0 / dv1
  // and the probabilities they multiply in dpw.  The tile loop issues them behind the next tile's barrier,
  // where the matrix pipeline would otherwise wait for the copy requests and the first K fragments.
  auto accumulate_but_last = [&](const uint32_t (&pw)[TT][8], int stage, bf16x8_t (&v0)[VC], bf16x8_t (&dv0)[VC],
                                 bf16x8_t (&dv1)[VC], uint32_t (&dpw)[8], int j) __attribute__((always_inline)) {
#pragma unroll
    for (int g = 0; g + 2 < 2 * TT; g += 2) {
      load_v(dv1, stage, g + 1);
      mma_pv(v0, pw[g >> 1], 0, j);
      load_v(g + 4 < 2 * TT ? v0 : dv0, stage, g + 2);
      mma_pv(dv1, pw[g >> 1], 1, j);
    }
    if (TT == 1) {
#pragma unroll
      for (int c = 0; c < VC; ++c) dv0[c] = v0[c];
    }
    load_v(dv1, stage, 2 * TT - 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) dpw[i] = pw[TT - 1][i];
  };

  // online softmax on this lane's column: scores -> packed bf16 probabilities, state update
  // (sacc: NS 32-key sub-tiles that start at key key0; j: which head of the wave)
  auto softmax = [&](auto& sacc, auto& pw, int key0, int j) __attribute__((always_inline)) {
    constexpr int NS = sizeof(sacc) / sizeof(sacc[0]);
    const bool need_mask = key0 + 32 * NS - 1 > prefix + wq_lo;    // reaches past the first row's diagonal
    if (need_mask) {
      int kb = key0;
      // sub-tile form: keeps the key arithmetic and the compares inside the branch (the compiler hoisted them onto
      // every tile); the whole-tile forms do not need it, and with it they run out of registers
      if constexpr (NS == 1) asm volatile("" : "+s"(kb));
#pragma unroll
      for (int tt = 0; tt < NS; ++tt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kb + 32 * tt + 8 * (i >> 2) + 4 * h + (i & 3);
          sacc[tt][i] = key <= qlim ? sacc[tt][i] : -INFINITY;
        }
    }
    if (win > 0 && key0 < prefix + wq_hi - win + 1) {         // tile starts below the last row's window
      const int qlo = qlim - win + 1;
      int kb = key0;
      if constexpr (NS == 1) asm volatile("" : "+s"(kb));       // (as above)
#pragma unroll
      for (int tt = 0; tt < NS; ++tt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kb + 32 * tt + 8 * (i >> 2) + 4 * h + (i & 3);
          sacc[tt][i] = key >= qlo ? sacc[tt][i] : -INFINITY;
        }
    }
    // Steady state: every row of the wave has a reference already (slack is finite), the scores
    // arrive relative to it, and nothing but a float overflow can go wrong with a reference that is
    // too low: bf16 and float32 keep their relative precision whatever the magnitude.  So the
    // probabilities are taken at once and the row maximum is never formed; only if a row's sum
    // comes out beyond 2^OVF_LOG2 (or not a number) is the tile redone the careful way below.
    constexpr float OVF_LIMIT = 0x1p+64f;
    if (!fresh_rows[j]) {
      float psum = 0.f;
#pragma unroll
      for (int tt = 0; tt < NS; ++tt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const float p0 = __builtin_amdgcn_exp2f(sacc[tt][i]);
          const float p1 = __builtin_amdgcn_exp2f(sacc[tt][i + 1]);
          psum += p0 + p1;
          pw[tt][i >> 1] = pack_bf16x2(p0, p1);
        }
      if (__builtin_amdgcn_ballot_w64(!(psum < OVF_LIMIT)) == 0) {
        l_run[j] += psum;
        return;
      }
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int tt = 0; tt < NS; ++tt)
#pragma unroll
      for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, sacc[tt][i]);
    {   // the other half-wave holds the remaining keys of this query row: swap halves in registers
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(tmax), __float_as_uint(tmax), false, false);
      tmax = __builtin_fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    }
    // move the reference for the first finite tile of a row, or when a score lies more than the
    // slack above it
    const bool move = tmax > slack[j];
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      const float shift = move ? tmax : 0.f;
      const float alpha = (move && slack[j] != -INFINITY) ? __builtin_amdgcn_exp2f(-shift) : 1.f;   // a fresh row has nothing to rescale
      m_ref[j] += shift;
      slack[j] = move ? REF_SLACK : slack[j];
      l_run[j] *= alpha;
      // (in-place forms: the accumulators and the reference tuple must come out of this rare branch in the registers
      // they went in with, or the register allocator may pay for the join with copies on the common path)
#pragma unroll
      for (int c = 0; c < VC; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) asm volatile("v_mul_f32 %0, %1, %0" : "+v"(oacc[j][c][i]) : "v"(alpha));
#pragma unroll
      for (int tt = 0; tt < NS; ++tt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[tt][i] -= shift;
      const float neg_ref = -m_ref[j];
#pragma unroll
      for (int i = 0; i < 16; ++i) asm volatile("v_mov_b32 %0, %1" : "+v"(cinit[j][i]) : "v"(neg_ref));
    }
    float psum = 0.f;
#pragma unroll
    for (int tt = 0; tt < NS; ++tt)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = __builtin_amdgcn_exp2f(sacc[tt][i]);
        const float p1 = __builtin_amdgcn_exp2f(sacc[tt][i + 1]);
        psum += p0 + p1;
        pw[tt][i >> 1] = pack_bf16x2(p0, p1);
      }
    l_run[j] += psum;
    fresh_rows[j] = __builtin_amdgcn_ballot_w64(slack[j] == -INFINITY) != 0;
  };
  // ---- prologue: the first tile's copies, then Q, then the rest of the ring: the Q loads and
  // the first tile travel together instead of one memory latency after the other
  request_next();
  prefetch_next();
#pragma unroll
  for (int j = 0; j < QH; ++j) {
    const uint16_t* qp = (const uint16_t*)p.q + ((long)b * p.T + qrow) * q_row_stride + (long)(hq_l + j) * DH;
    uint4 qraw[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      qraw[s] = make_uint4(0, 0, 0, 0);
      if (qvalid) qraw[s] = *(const uint4*)(qp + 16 * s + 8 * h);
    }
    if (!SPARSE && p.qt.cos) {
      // norm and rotation of the row on the way in; every lane takes part (the row's other
      // half sits in lane ^ 32), rows past the query length carry zeros
      float x[KS][8];
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const uint32_t w[4] = {qraw[s].x, qraw[s].y, qraw[s].z, qraw[s].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          x[s][2 * j] = bf16_bits_to_float(w[j] & 0xffffu);
          x[s][2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
        }
      }
      const int pos = min(max(prefix + qrow, 0), p.qt.max_pos - 1);
      q_norm_rope_lane<DH / 8, KS, QRowLayout>(x, p.qt, pos, h);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        qraw[s].x = pack_bf16x2(x[s][0], x[s][1]); qraw[s].y = pack_bf16x2(x[s][2], x[s][3]);
        qraw[s].z = pack_bf16x2(x[s][4], x[s][5]); qraw[s].w = pack_bf16x2(x[s][6], x[s][7]);
      }
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const uint4 v = qraw[s];
      // scale * log2(e) goes into Q once (rounded to bf16 again: a relative 2^-9 per element,
      // below the rounding of the probabilities), so that the scores leave the matrix cores
      // ready for exp2
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      uint32_t r[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        r[j] = pack_bf16x2(bf16_bits_to_float(w[j] & 0xffffu) * sc, bf16_bits_to_float(w[j] >> 16) * sc);
      qf[j][s] = make_frag(r[0], r[1], r[2], r[3]);
    }
    // the Q loads must be complete (and known to the compiler to be) before the loop, or the
    // first use of a fragment inside it would drain the ring with a full wait
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" ::"v"(qf[j][s]));
  }
#pragma unroll
  for (int s = 1; s < NST - 1; ++s) {
    if (FP8) shift_scales();
    request_next();
    prefetch_next();
  }
  if (FP8) {     // the raw ring holds four tiles; the first one is expanded before the loop
    shift_scales();
    request_next();
    prefetch_next();
    wait_vmcnt<3 * UPW>();
    expand(kt_first, 0, 0);
  }

  {
    Walk w_c = w_first;
    int stage_c = 0;
    int rs_n = 1;                                  // FP8: raw stage of the tile after the current one
    // one q head per wave: the last two groups of a tile's O^T += V^T P^T wait here for the next barrier
    constexpr bool DEFER = QH == 1;
    bf16x8_t dv0[DEFER ? VC : 1], dv1[DEFER ? VC : 1];
    uint32_t dpw[8];
    bool pending = false;
    auto flush_pending = [&]() __attribute__((always_inline)) {
      if constexpr (DEFER) {
        if (pending) {
          mma_pv(dv0, dpw, 0, 0);
          mma_pv(dv1, dpw, 1, 0);
          pending = false;
        }
      }
    };
    if constexpr (STAG) {
      const int n_steps = stag_nv + p.sparse_local - stag_skip;
      const int jq = qblk - wg_blk_lo;             // this wave's q block within the workgroup
      int stage_v = 0;                             // stage of the request with the step's number
      for (int g = 0; g < n_steps; ++g) {
        const bool band = g >= stag_nv;
        // vertical steps consume request g (three younger ones may still be in flight); band steps consume
        // requests g .. g + 3, the youngest of them issued one step ago
        if (band) wait_vmcnt<0>(); else wait_vmcnt<(NST - 2) * UPW>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        request_next();                            // request g + 4, into the stage request g - 1 has left
        flush_pending();
        int tile, stage;
        bool act = wave_has_rows;
        if (!band) {
          tile = stag_v0 + g * p.sparse_stride;
          stage = stage_v;
          act = act && tile <= qblk - p.sparse_local;          // strictly below this q block's window
        } else {
          const int sb = g - stag_nv;
          tile = qblk - p.sparse_local + 1 + stag_skip + sb;
          stage = stage_v + jq;
          stage = stage >= NST ? stage - NST : stage;
          act = act && tile >= 0;
        }
        if (act) {
          f32x16_t sacc[TT];
          uint32_t pw[TT][8];
          bf16x8_t v0[VC];
          scores(sacc, stage, v0, stage, 0);
          softmax(sacc, pw, tile * BN, 0);
          accumulate_but_last(pw, stage, v0, dv0, dv1, dpw, 0);
          pending = true;
        }
        stage_v = stage_v + 1 == NST ? 0 : stage_v + 1;
      }
    }
    while (!STAG && w_c.kt < ntiles) {
      if (FP8) {
        wait_vmcnt<2 * UPW>();                     // this wave's raw rows of the next tile have landed
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // ... and its bf16 rows of the current one are written
      } else {
        wait_vmcnt<(NST - 2) * UPW>();             // this wave's part of the current tile has landed
        if (DEFER) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // ... and its reads of the previous one are done
      }
      __builtin_amdgcn_s_barrier();                // ... and everyone's; all waves are done with the previous tile
      if (FP8) shift_scales();
      request_next();
      flush_pending();       // (behind the requests: issued in front of them it measured 0.3 % slower)
      if (FP8) {
        if (w_c.kt + 1 < ntiles) expand(w_c.kt + 1, rs_n, stage_c ^ 1);
        rs_n = (rs_n + 1) & 3;
      }
      if (tile_active(w_c)) {
        if constexpr (QH == 1) {
          f32x16_t sacc[TT];
          uint32_t pw[TT][8];
          bf16x8_t v0[VC];
          scores(sacc, stage_c, v0, stage_c, 0);
          prefetch_next();
          softmax(sacc, pw, w_c.kt * BN, 0);
          accumulate_but_last(pw, stage_c, v0, dv0, dv1, dpw, 0);
          pending = true;
        } else {
          // two heads, one 32-key sub-tile at a time: its K fragments and its two groups of V^T fragments are
          // read once and serve both heads; scores, probabilities and fragments of one sub-tile are all the
          // registers hold besides the accumulators
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            bf16x8_t kf[KS];
            load_k(kf, stage_c, tt);
            f32x16_t sacc[QH][1];
            uint32_t pw[QH][1][8];
#pragma unroll
            for (int j = 0; j < QH; ++j) mma_qk(sacc[j][0], kf, j);
            bf16x8_t va[VC], vb[VC];
            load_v(va, stage_c, 2 * tt);
            load_v(vb, stage_c, 2 * tt + 1);
            if (tt == 0) {
              // the scalar loads must not drift up in front of the wait for the K fragments (LDS reads and scalar
              // loads share a counter: that wait would then sit out the loads' whole latency)
              __builtin_amdgcn_sched_barrier(0);
              prefetch_next();
            }
#pragma unroll
            for (int j = 0; j < QH; ++j) softmax(sacc[j], pw[j], w_c.kt * BN + 32 * tt, j);
#pragma unroll
            for (int j = 0; j < QH; ++j) {
              mma_pv(va, pw[j][0], 0, j);
              mma_pv(vb, pw[j][0], 1, j);
            }
          }
        }
      } else {
        prefetch_next();
      }
      walk_step(w_c);
      stage_c = stage_c + 1 == BFS ? 0 : stage_c + 1;
    }
    flush_pending();
  }
  wait_vmcnt<0>();     // nothing may still be landing in LDS when the workgroup retires

  // ---- normalise and write this lane's query row ---------------------------------
#pragma unroll
  for (int j = 0; j < QH; ++j) {
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run[j]), __float_as_uint(l_run[j]), false, false);
    l_run[j] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  }
  if (SPLIT) {     // partial result relative to m_ref; the sink and the division belong to the merge
    if (qvalid) {
#pragma unroll
      for (int j = 0; j < QH; ++j) {
        float* po = p.ws_o + ((row_g + j) * p.splits + part) * DH;
#pragma unroll
        for (int c = 0; c < VC; ++c)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4)
            *(float4*)(po + 32 * c + 8 * i4 + 4 * h) =
                make_float4(oacc[j][c][4 * i4], oacc[j][c][4 * i4 + 1], oacc[j][c][4 * i4 + 2], oacc[j][c][4 * i4 + 3]);
        if (h == 0)
          *(float2*)(p.ws_ml + ((row_g + j) * p.splits + part) * 2) = make_float2(slack[j] == -INFINITY ? -INFINITY : m_ref[j], l_run[j]);
      }
    }
    return;
  }
  // attention sink: a per-head logit that joins the softmax as one more column with no value
#pragma unroll
  for (int j = 0; j < QH; ++j)
    if (p.sinks && l_run[j] > 0.f) l_run[j] += __builtin_amdgcn_exp2f(p.sinks[hq_l + j] * kLog2e - m_ref[j]);
  // The rows go out through LDS: a lane holds 4 consecutive d of one row at 16 places, which as direct
  // stores would be 8-byte pieces of 64 different rows per instruction; staged row-major in a
  // wave-private patch of the (now idle) tile ring they leave as whole 256-byte rows, 16 bytes a lane.
  __builtin_amdgcn_s_barrier();                  // every wave is done reading the ring
#pragma unroll
  for (int hj = 0; hj < QH; ++hj) {
    constexpr int OROW_B = 2 * DH + 8;           // row pitch: the 8 bytes spread a column of rows over the banks
    constexpr int OCH = DH / 8, ORI = 64 / OCH;  // 16-byte pieces per row; rows a wave stores per instruction
    char* patch = smem + (wave * QH + hj) * (32 * OROW_B);
    const float inv = (qvalid && l_run[hj] > 0.f) ? 1.f / l_run[hj] : 0.f;
#pragma unroll
    for (int c = 0; c < VC; ++c)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d = 32 * c + 8 * i4 + 4 * h;
        const uint32_t w0 = qvalid ? pack_bf16x2(oacc[hj][c][4 * i4] * inv, oacc[hj][c][4 * i4 + 1] * inv) : 0u;
        const uint32_t w1 = qvalid ? pack_bf16x2(oacc[hj][c][4 * i4 + 2] * inv, oacc[hj][c][4 * i4 + 3] * inv) : 0u;
        *(uint2*)(patch + n * OROW_B + 2 * d) = make_uint2(w0, w1);
      }
    // the wave reads back what its own lanes wrote: no barrier, the compiler orders the LDS accesses
#pragma unroll
    for (int j = 0; j < 32 / ORI; ++j) {
      const int r = ORI * j + lane / OCH, ch = lane % OCH;
      const uint2 lo = *(const uint2*)(patch + r * OROW_B + 16 * ch), hi = *(const uint2*)(patch + r * OROW_B + 16 * ch + 8);
      const int tok = row_token(wave * 32 + r);
      if (tok < p.T && !idle_half)
        store_stream(out + ((long)b * p.T + tok) * q_row_stride + (long)(row_head(wave * 32 + r) + hj) * DH + 8 * ch,
                     make_uint4(lo.x, lo.y, hi.x, hi.y));
    }
  }
}

// Merge of the split form: one thread per (query row, 4 consecutive d); rows past query_lens become zeros.
__global__ __launch_bounds__(256) void prefill_split_reduce_kernel(PrefillParams p) {
  const long item = (long)blockIdx.x * 256 + threadIdx.x;
  const int D = p.D;
  const long row = item / (D / 4);
  const int q4 = (int)(item % (D / 4));
  if (row >= (long)p.B * p.T * p.Hq) return;
  const int hq = (int)(row % p.Hq);
  const long bt = row / p.Hq;
  const int t = (int)(bt % p.T), b = (int)(bt / p.T);
  const int ctx = max(min(p.seq_lens[b], p.max_blocks * p.block_size), 0);
  const int tq = min(min(max(p.query_lens[b], 0), p.T), ctx);
  uint16_t* dst = (uint16_t*)p.out + row * D + 4 * q4;
  if (t >= tq) { *(uint2*)dst = make_uint2(0u, 0u); return; }
  float m = -INFINITY, l = 0.f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int c = 0; c < p.splits; ++c) {
    const float2 ml = *(const float2*)(p.ws_ml + (row * p.splits + c) * 2);
    if (ml.y == 0.f) continue;                 // a share in which the row saw no key (its O may be unwritten)
    const float4 o = *(const float4*)(p.ws_o + (row * p.splits + c) * D + 4 * q4);
    const float m_new = fmaxf(m, ml.x);
    const float a = exp2f(m - m_new), w = exp2f(ml.x - m_new);
    l = l * a + ml.y * w;
    acc.x = acc.x * a + o.x * w; acc.y = acc.y * a + o.y * w;
    acc.z = acc.z * a + o.z * w; acc.w = acc.w * a + o.w * w;
    m = m_new;
  }
  if (p.sinks && l > 0.f) l += exp2f(p.sinks[hq] * kLog2e - m);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  *(uint2*)dst = make_uint2(pack_bf16x2(acc.x * inv, acc.y * inv), pack_bf16x2(acc.z * inv, acc.w * inv));
}

template <bool SPARSE, int MODE, int NW, int TT = 2, bool WIN = false, bool PACK = false, bool SPLIT = false, bool FP8 = false, int DH = HD, int QH = 1>
hipError_t launch_typed(const PrefillParams& p, hipStream_t s) {
  constexpr int lds = (SPARSE && NW == 8 ? 5 : NW == 8 ? 4 : 2) * 2 * 32 * TT * ROW_B;
  constexpr int TOKW = DH == 64 ? 16 * NW : 32 * NW;      // query tokens per workgroup (plain form)
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)prefill_async_kernel<SPARSE, MODE, NW, TT, WIN, PACK, SPLIT, FP8, DH, QH>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured.store(1, std::memory_order_release);
  }
  const int n_rep = p.Hq / p.Hkv;
  const long per_group = PACK ? ((long)p.T * n_rep + 32 * NW - 1) / (32 * NW)
                              : (long)((p.T + TOKW - 1) / TOKW) * (n_rep / QH);
  const long groups = (long)p.B * (DH == 64 ? (p.Hkv + 1) / 2 : p.Hkv);
  const long total = 8 * ((groups + 7) / 8) * per_group * (SPLIT ? p.splits : 1);
  if (total > 0x7fffffffL) return hipErrorInvalidValue;
  hipLaunchKernelGGL((prefill_async_kernel<SPARSE, MODE, NW, TT, WIN, PACK, SPLIT, FP8, DH, QH>), dim3((unsigned)total), dim3(NW * 64), lds, s, p);
  if (SPLIT) {
    const long items = (long)p.B * p.T * p.Hq * (DH / 4);
    hipLaunchKernelGGL(prefill_split_reduce_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s, p);
  }
  return hipGetLastError();
}

// head dim 64: q heads per wave (two when the kv group has an even number of them)
int d64_heads_per_wave(const PrefillParams& p) { return (p.Hq / p.Hkv) % 2 == 0 && p.impl != 6 ? 2 : 1; }

// workgroups of the paged dense form for a given choice of waves and packing
long prefill_workgroups(const PrefillParams& p, int waves, bool pack) {
  const int n_rep = p.Hq / p.Hkv;
  if (p.D == 64) return (long)p.B * ((p.Hkv + 1) / 2) * ((p.T + 16 * waves - 1) / (16 * waves)) * (n_rep / d64_heads_per_wave(p));
  const long per_group = pack ? ((long)p.T * n_rep + 32 * waves - 1) / (32 * waves)
                              : (long)((p.T + 32 * waves - 1) / (32 * waves)) * n_rep;
  return (long)p.B * p.Hkv * per_group;
}

}  // namespace

bool prefill_async_supported(const PrefillParams& p) {
  if (p.block_tables && p.block_shift < 4) return false;   // paged: power-of-two block size >= 16
  if (p.D == HD) return true;
  // head dim 64: two adjacent kv heads share the 256-byte rows the kernel is laid out for
  return p.D == 64 && p.Hkv >= 2 && p.block_tables && p.sparse_stride == 0;
}

static bool prefill_packs(const PrefillParams& p) {
  const bool sparse = p.sparse_stride > 0, paged = p.block_tables != nullptr;
  // chunks shorter than a 4-wave tile of a GQA model: rows packed over the heads of a kv group
  return paged && !sparse && !p.kv_fp8 && p.D == HD && p.Hq > p.Hkv && p.T < 128 && (p.impl == 0 || p.impl == 5);
}
static int prefill_waves(const PrefillParams& p, int waves) {
  const bool sparse = p.sparse_stride > 0;
  // waves: 4 (two workgroups of 128 query rows per CU, 2-stage ring) or 8 (one workgroup of
  // 256 rows, 4-stage ring: half the copy requests per FLOP).  Measured within a few per cent of
  // each other; automatic choice: 8 for dense chunks of more than 128 rows that fill the device, 4 for short
  // chunks, small grids and the sparse form.
  if (p.kv_fp8 || p.D == 64) return 8; // fp8 pools and head dim 64: the 8-wave form only
  if (prefill_packs(p)) return 4;
  if (waves == 0) {
    waves = (!sparse && p.T > 128) ? 8 : 4;
    // fewer 256-row workgroups than CUs (one request's chunk of up to a few thousand tokens): the call is bound by
    // its longest workgroup, and twice as many of half the size, two per CU, finish sooner (B = 1: T = 512 behind
    // a 4 K prefix 66 -> 55 us, T = 1 024 37.5 -> 33.5 us; with the device full the 8-wave form is ~7 % ahead)
    const long wgs8 = (long)p.B * p.Hq * ((p.T + 255) / 256), cus = p.num_cus > 0 ? p.num_cus : 256;
    if (waves == 8 && p.block_tables && wgs8 < cus) waves = 4;
    // short contexts by the caller's bound (prompts of a batch with little cached in front: at most 16 key tiles per
    // workgroup) with the device full twice over: a workgroup's start and end weigh as much as its tiles, and the two
    // 4-wave workgroups of a CU overlap them (32 / 8 heads, no prefix, us 8 / 4 waves: 32 x 256 tokens 56.8 / 49.0, 16 x
    // 512 69.7 / 65.6, 8 x 1 024 97.7 / 95.1, 4 x 1 024 57.2 / 52.6; with the device full once the 8-wave form stays: 2 x
    // 1 024 31.5 / 35.3, 4 x 512 21.2 / 22.5)
    if (waves == 8 && p.block_tables && p.len_bound > 0 && p.len_bound <= 1024 && wgs8 >= 2 * cus) waves = 4;
  }
  return waves;
}

int prefill_async_splits(const PrefillParams& p, int num_cus, int max_seq_len) {
  if (p.sparse_stride > 0 || !p.block_tables || !prefill_async_supported(p) || p.impl == 1) return 1;
  // A prompt with little cached in front of it is bound by its causal diagonal: the query tiles differ in work by
  // the tile count, the light ones leave room on the device whatever is done, and the split's partials and merge
  // launch cost more than it gains (one sequence, 32 / 8 heads of 128, us split / unsplit: T = 1 024 alone 34.8 /
  // 25.1, behind 1 024 cached tokens 48.4 / 44.4, behind 2 048 63.5 / 65.0, behind 4 096 93.9 / 100.6; T = 512 behind
  // 512 29.1 / 25.7, behind 1 024 35.1 / 34.7, behind 2 048 40.7 / 56.0).  Known only from the caller's bound on the
  // lengths: the table capacity says nothing about them.
  if (max_seq_len > 0 && (long)max_seq_len < 3L * p.T) return 1;
  const int waves = prefill_waves(p, p.impl == 4 || p.impl == 8 ? p.impl : 0);
  const long wgs = prefill_workgroups(p, waves, prefill_packs(p));
  const long slots = (long)num_cus * (waves == 4 ? 2 : 1);     // workgroups the device holds at once
  if (wgs >= slots) return 1;                         // enough workgroups to fill the chip
  // key tiles a workgroup may have to walk: by the caller's bound, else by the table capacity
  const long tiles = ((max_seq_len > 0 ? (long)max_seq_len : (long)p.max_blocks * p.block_size) + 63) / 64;
  long s = (2L * num_cus + wgs - 1) / wgs;            // aim at two workgroups per CU
  // ... of at least 8 key tiles each; the more workgroups there are to begin with, the longer a share must be to
  // pay for its partials (a float32 row per query row and share) and the merge launch: 16 tiles from one workgroup
  // per two CUs on, 40 from one per CU on (32 / 8 heads of 128, us unsplit / two shares: 2 x 512 tokens behind 1 K
  // 36.6 / 46.7, 4 x 256 behind 1 K 32.1 / 41.4, 2 x 256 behind 1 K 30.2 / 32.7; 1 x 256 behind 1 K 30.0 / 27.3 and
  // 1 x 1 024 behind 4 K 98.2 / 93.1 keep their two)
  const long min_tiles = wgs >= num_cus ? 40 : 2 * wgs >= num_cus ? 16 : 8;
  if (s > tiles / min_tiles) s = tiles / min_tiles;
  if (s > 16) s = 16;
  return s < 2 ? 1 : (int)s;
}

hipError_t launch_prefill_async(const PrefillParams& p, int waves, hipStream_t s) {
  const bool sparse = p.sparse_stride > 0;
  const bool paged = p.block_tables != nullptr;
  const bool pack = prefill_packs(p);
  waves = prefill_waves(p, waves);
  if (p.D == 64) {
    if (sparse || !paged || p.Hkv < 2 || (p.kv_fp8 && (!p.k_scale || !p.v_scale))) return hipErrorInvalidValue;
    if (p.splits > 1 && (!p.ws_o || !p.ws_ml)) return hipErrorInvalidValue;
    // Head dim 64 always takes the instantiation that carries the sliding-window tests (window 0: no row is cut).
    // The one without them, otherwise the same code, leaves the register allocator with spills (two heads per
    // wave) or with some fifty register copies per key tile on the common path (one head per wave).
    const int form = (p.kv_fp8 ? 2 : 0) + (p.splits > 1 ? 1 : 0);
    if (d64_heads_per_wave(p) == 2) {
      switch (form) {
        case 0: return launch_typed<false, 1, 8, 2, true, false, false, false, 64, 2>(p, s);
        case 1: return launch_typed<false, 1, 8, 2, true, false, true, false, 64, 2>(p, s);
        case 2: return launch_typed<false, 1, 8, 2, true, false, false, true, 64, 2>(p, s);
        default: return launch_typed<false, 1, 8, 2, true, false, true, true, 64, 2>(p, s);
      }
    }
    switch (form) {
      case 0: return launch_typed<false, 1, 8, 2, true, false, false, false, 64>(p, s);
      case 1: return launch_typed<false, 1, 8, 2, true, false, true, false, 64>(p, s);
      case 2: return launch_typed<false, 1, 8, 2, true, false, false, true, 64>(p, s);
      default: return launch_typed<false, 1, 8, 2, true, false, true, true, 64>(p, s);
    }
  }
  if (p.kv_fp8) {
    if (sparse || !paged || !p.k_scale || !p.v_scale) return hipErrorInvalidValue;
    if (p.splits > 1) {
      if (!p.ws_o || !p.ws_ml) return hipErrorInvalidValue;
      return p.window > 0 ? launch_typed<false, 1, 8, 2, true, false, true, true>(p, s)
                          : launch_typed<false, 1, 8, 2, false, false, true, true>(p, s);
    }
    return p.window > 0 ? launch_typed<false, 1, 8, 2, true, false, false, true>(p, s)
                        : launch_typed<false, 1, 8, 2, false, false, false, true>(p, s);
  }
  if (p.splits > 1) {
    if (sparse || !paged || !p.ws_o || !p.ws_ml) return hipErrorInvalidValue;
    if (p.window > 0) {
      if (pack) return launch_typed<false, 1, 4, 2, true, true, true>(p, s);
      return waves == 8 ? launch_typed<false, 1, 8, 2, true, false, true>(p, s) : launch_typed<false, 1, 4, 2, true, false, true>(p, s);
    }
    if (pack) return launch_typed<false, 1, 4, 2, false, true, true>(p, s);
    return waves == 8 ? launch_typed<false, 1, 8, 2, false, false, true>(p, s) : launch_typed<false, 1, 4, 2, false, false, true>(p, s);
  }
  if (p.window > 0) {
    if (sparse || !paged) return hipErrorInvalidValue;
    if (pack) return launch_typed<false, 1, 4, 2, true, true>(p, s);
    return waves == 8 ? launch_typed<false, 1, 8, 2, true>(p, s) : launch_typed<false, 1, 4, 2, true>(p, s);
  }
  if (pack) return launch_typed<false, 1, 4, 2, false, true>(p, s);
  if (waves == 8) {
    if (sparse) return launch_typed<true, 0, 8>(p, s);
    return paged ? launch_typed<false, 1, 8>(p, s) : launch_typed<false, 0, 8>(p, s);
  }
  if (sparse) return launch_typed<true, 0, 4>(p, s);
  return paged ? launch_typed<false, 1, 4>(p, s) : launch_typed<false, 0, 4>(p, s);
}

}  // namespace pa
