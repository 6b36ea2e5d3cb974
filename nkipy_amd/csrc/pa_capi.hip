// extern "C" surface of libpaged_attn.so: argument validation on the host,
// kernel selection, launch.  See include/paged_attn.h for the contract.
#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "pa_common.h"

namespace pa {

static thread_local char tl_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(tl_error, sizeof(tl_error), fmt, ap);
  va_end(ap);
}

int fail_arg(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(tl_error, sizeof(tl_error), fmt, ap);
  va_end(ap);
  return -1;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  set_error("%s: %s (%d)", what, hipGetErrorString(e), (int)e);
  return (int)e > 0 ? (int)e : 1;
}

// ---- debug switches ------------------------------------------------------------
static std::atomic<int> g_decode_impl{0};
static std::atomic<int> g_decode_waves{0};
static std::atomic<int> g_head_major{1};
static std::atomic<int> g_prefill_impl{0};
static std::atomic<int> g_lockstep{1};
// The per-tile barrier that keeps the kv-head waves of a balanced decode workgroup on the same tile: debug switch 4,
// 1 = automatic (the default), 0 = never, 2 = always.  Automatic: on for bf16 pools (the heads' rows of a token are one
// contiguous piece of DRAM; config 2 80.4 % of HBM peak with it, 77.5 % without), off for fp8 pools (the waves' expansion
// work makes them arrive apart, and waiting for the last costs more than the drift: config 5 77.6 % with, 79.3 % without).
static int lockstep_for(int kv_dtype, int bal_ns) {
  const int mode = g_lockstep.load();
  if (bal_ns != 1 || mode == 0) return 0;
  return mode == 2 || kv_dtype != PA_FP8_E4M3FN ? 1 : 0;
}
static std::atomic<int> g_verify_rows{0};
static std::atomic<int> g_prefill_split{1};
static std::atomic<int> g_d64_tiled_from{PA_VERIFY_MAX_TOKENS + 1};   // query tokens from which head dim 64 takes the tiled kernel
// Small decode calls whose length bound is at most this many tokens run as ONE partition per sequence on eight waves
// (the waves merge through LDS, so there is no split-K workspace and no merge launch): debug switch 9, 0 = never.
static std::atomic<int> g_decode_single_max{1024};
static std::atomic<int> g_decode_fine{256};     // tokens per partition of the smallest fixed-partition calls (0: the caller's always)
static std::atomic<long> g_small_call_pairs{0};  // debug switch 12: the (sequence, kv head) pair limit of small calls (0: the rule in decode_small_call)
static std::atomic<int> g_step_fusion{0};       // pa_decode_step, debug switch 10
static std::atomic<int> g_d64_wide{1};          // debug switch 13: partitions counted in bytes at head dim 64 (see token_scale)

// ---- profiling: event pairs around the main kernel of each op ----------------
// Events come from a free list that pa_profile_collect refills, so that a timed pass which follows a collected
// pass of the same length creates none: the records are then all the profiling adds to a step.
static std::atomic<int> g_profile{0};
static std::mutex g_prof_mu;
static std::vector<std::pair<hipEvent_t, hipEvent_t>> g_prof_events;
static std::vector<hipEvent_t> g_prof_free;
static thread_local hipEvent_t tl_start = nullptr;

static hipEvent_t profile_event() {
  {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    if (!g_prof_free.empty()) {
      hipEvent_t e = g_prof_free.back();
      g_prof_free.pop_back();
      return e;
    }
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  return e;
}

void profile_begin(hipStream_t s) {
  if (!g_profile.load(std::memory_order_relaxed)) return;
  hipEvent_t a = profile_event();
  if (!a) return;
  (void)hipEventRecord(a, s);
  tl_start = a;
}

void profile_end(hipStream_t s) {
  if (!tl_start) return;
  hipEvent_t b = profile_event();
  std::lock_guard<std::mutex> lk(g_prof_mu);
  if (!b) { g_prof_free.push_back(tl_start); tl_start = nullptr; return; }
  (void)hipEventRecord(b, s);
  g_prof_events.emplace_back(tl_start, b);
  tl_start = nullptr;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// CUs of the current device (256 on MI355X), cached; 256 when no device is visible
// so that size queries work on a build machine.
static int current_num_cus() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return 256; }
  int v = cached[dev].load(std::memory_order_relaxed);
  if (v > 0) return v;
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return 256;
  }
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

static int ilog2_exact(int v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

}  // namespace pa

using namespace pa;

extern "C" {

int pa_version(void) { return 300; }   // 0.3.0: pa_prefill takes max_seq_len; the one-call steps; sinks and windows on small calls

const char* pa_last_error(void) { return tl_error; }

// The switches reroute kernels for every thread of the process, so a server that links the library cannot be
// switched by accident or by another component: they work only when PA_ENABLE_DEBUG=1 was in the environment
// when the first call looked (tests set it), and are refused otherwise.
static bool debug_enabled() {
  static const bool on = [] {
    const char* v = getenv("PA_ENABLE_DEBUG");
    return v && v[0] == '1' && v[1] == 0;
  }();
  return on;
}

int pa_debug_set(int key, int value) {
  tl_error[0] = 0;
  if (!debug_enabled())
    return fail_arg("pa_debug_set: the debug switches are off (set PA_ENABLE_DEBUG=1 in the environment before the "
                    "library's first use)");
  if (key == 0) { g_decode_impl = value; return 0; }
  if (key == 1) { g_decode_waves = value; return 0; }
  if (key == 2) { g_head_major = value; return 0; }
  if (key == 3) { g_prefill_impl = value; return 0; }
  if (key == 4) { g_lockstep = value; return 0; }
  if (key == 5) { g_verify_rows = value; return 0; }
  if (key == 6) { g_prefill_split = value; return 0; }
  if (key == 7) { g_d64_tiled_from = value > 0 ? value : PA_VERIFY_MAX_TOKENS + 1; return 0; }
  if (key == 8) { o_proj_debug_force_large(value); return 0; }
  if (key == 9) { g_decode_single_max = value < 0 ? 0 : value; return 0; }
  if (key == 10) { g_step_fusion = value; return 0; }
  if (key == 11) { g_decode_fine = value < 0 ? 0 : value & ~31; return 0; }
  if (key == 12) { g_small_call_pairs = value < 0 ? 0 : value; return 0; }
  if (key == 13) { g_d64_wide = value != 0; return 0; }
  return fail_arg("pa_debug_set: unknown key %d", key);
}

int pa_profile_enable(int on) {
  g_profile = on ? 1 : 0;
  return 0;
}

int pa_profile_collect(float* ms, int cap) {
  std::vector<std::pair<hipEvent_t, hipEvent_t>> ev;
  {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    ev.swap(g_prof_events);
  }
  int n = 0;
  for (auto& pr : ev) {
    float t = 0.f;
    if (hipEventSynchronize(pr.second) == hipSuccess &&
        hipEventElapsedTime(&t, pr.first, pr.second) == hipSuccess && ms && n < cap)
      ms[n++] = t;
  }
  {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    for (auto& pr : ev) {
      g_prof_free.push_back(pr.first);
      g_prof_free.push_back(pr.second);
    }
  }
  return n;
}

// What an event pair reads around a kernel that does nothing: the part of every pa_profile_collect figure that is
// not the kernel (the events are stamped by the command processor around the dispatch, not by the kernel's first
// and last wave, which is what a kernel trace reports).
__global__ void profile_empty_kernel() {}
int pa_profile_empty_launch(void* stream) {
  hipStream_t s = (hipStream_t)stream;
  profile_begin(s);
  hipLaunchKernelGGL(profile_empty_kernel, dim3(1), dim3(64), 0, s);
  hipError_t e = hipGetLastError();
  profile_end(s);
  return check_hip(e, "pa_profile_empty_launch");
}

// Checks an optional Q transform and copies it into the kernel parameters; returns 0 or -1.
static int take_q_transform(const char* who, const pa_q_transform* qt, bool kernel_ok, QTransform& dst) {
  memset(&dst, 0, sizeof(dst));
  if (!qt) return 0;
  if (!kernel_ok)
    return fail_arg("%s: q_transform needs the matrix-core kernels (bf16 q, head_dim 64 or 128 for decode and verify, "
                    "128 for tiled prefill, block_size a power of two >= 16)", who);
  if (!qt->rope_cos || !qt->rope_sin || qt->rope_max_pos <= 0)
    return fail_arg("%s: q_transform needs rope_cos, rope_sin and rope_max_pos > 0", who);
  if (!aligned16(qt->rope_cos) || !aligned16(qt->rope_sin) || !aligned16(qt->norm_weight))
    return fail_arg("%s: q_transform tables must be 16-byte aligned", who);
  dst.norm_weight = (const uint16_t*)qt->norm_weight;
  dst.cos = (const uint16_t*)qt->rope_cos; dst.sin = (const uint16_t*)qt->rope_sin;
  dst.max_pos = qt->rope_max_pos; dst.eps = qt->norm_eps;
  return 0;
}

static int num_partitions_for(int max_seq_len, int partition_size) {
  if (max_seq_len <= 0) return 1;
  return (max_seq_len + partition_size - 1) / partition_size;
}

size_t pa_decode_workspace_bytes(int B, int Hq, int D, int max_seq_len, int partition_size) {
  if (B <= 0 || Hq <= 0 || D <= 0 || partition_size <= 0) return 0;
  const int np = num_partitions_for(max_seq_len, partition_size);
  const size_t fixed = np <= 1 ? 0 : (size_t)B * Hq * np * ((size_t)D + 2) * sizeof(float);
  // the balanced schedule keeps one partial per (q head, sequence + chunk); at
  // most 8 chunks per CU exist whatever the head layout
  const size_t balanced = decode_balanced_workspace_bytes(B, Hq, D, 8 * current_num_cus());
  return fixed > balanced ? fixed : balanced;
}

// Which kernel pa_decode takes for a shape: 1 scalar-ALU, 2 MFMA with fixed partitions, 3 MFMA balanced;
// -1 when a forced kernel (debug switch 0) does not take the shape.
// The balanced kernel pays a fixed price for its schedule (a scan of the lengths in every workgroup, partials and a
// merge launch whatever the sizes: 11 us for the smallest call), the fixed-partition kernel merges a sequence's
// waves inside the workgroup and needs the merge launch only past one partition, but leaves the device unevenly
// filled at scale.  Measured where it matters, inside a decode step of eight attention layers with a pool each (so
// that every layer's K and V come from HBM, not from a cache the previous call warmed), us per layer with fixed
// partitions of 512 / balanced (B x context, 32 / 8 heads of 128, bf16): 1 x 1 K 25.8 / 29.2, 1 x 4 K 28.3 / 31.7,
// 4 x 2 K 28.5 / 35.9, 8 x 1 K 29.6 / 36.0, 4 x 4 K 33.1 / 38.4, 8 x 2 K 40.1 / 39.6, 8 x 4 K 47.4 / 49.8,
// 16 x 2 K 59.3 / 49.1, 32 x 1 K 61.8 / 49.6, 16 x 4 K 78.6 / 77.6.  (Timed call by call on one pool, which then sits
// in the last-level cache, the fixed partitions stay ahead up to four times these sizes; a serving step is not that.)
// 16 x 1 K 41.2 / 38.8, 8 x 600 29.1 / 30.6, 32 x 600 47.4 / 42.8: what decides is the number of sequences, not the
// bytes.  So calls of at most 80 (sequence, kv head) pairs and at most eight partitions per sequence that can touch at
// most this many bytes of K and V, by the caller's bound on the lengths, take the fixed partitions when nothing
// needs the balanced kernel.
// The most tokens the partitions of one sequence cover: the length bound, or, under a sliding window, what the window
// of the oldest query row reaches back to, rounded out to its 32-token tile (the kernels count partitions from there)
static int span_bound(const DecodeParams& p) {
  if (p.window <= 0) return p.max_seq_len;
  const long reach = (long)p.window + std::max(p.T, 1) - 1 + 31;
  return (int)std::min<long>(p.max_seq_len, reach);
}
// The partition sizes below were found on bf16 pools of head dim 128; what they measure is the bytes a workgroup
// streams, and a token of head dim 64, or of an fp8 pool, is half of them.  Where a limit in tokens would send such a
// call to more partitions than pay (or to the balanced kernel), the partitions are twice the tokens instead: the
// caller's partition_size when it gives more than eight partitions, the finer partitions of a single sequence
// likewise, and the longest partition the sized ones may have.  (us per call replayed, before / after.  64 / 8 heads of
// 64, bf16: B = 1 behind 4 K 12.6 / 11.3, behind 8 K 15.8 / 14.0; B = 2 behind 8 K 17.6 / 14.5; B = 4 behind 6 K 19.6 /
// 18.0; B = 32 behind 2 K 35.3 / 30.5.  64 / 8 heads of 128, fp8: B = 1 behind 8 K 18.4 / 16.5, B = 4 behind 6 K 22.1 /
// 19.2, B = 32 behind 2 K 37.2 / 29.1.  Doubling everything cost where the tokens' count was fine: head dim 64, B = 8
// behind 1 K 9.7 -> 10.6.)
static int token_scale(const DecodeParams& p, int kv_dtype) {
  return g_d64_wide.load() && (p.D <= 64 || kv_dtype == PA_FP8_E4M3FN) ? 2 : 1;
}
constexpr int kDecodeSmallCallPartitions = 8;
static int base_partition(const DecodeParams& p, int kv_dtype) {
  if (num_partitions_for(span_bound(p), p.partition_size) <= kDecodeSmallCallPartitions) return p.partition_size;
  // (not for fp8 pools of head dim 64, which are better off on the balanced kernel there: B = 2 behind 8 K 15.4
  // against 16.6 us, B = 4 behind 6 K 15.6 against 16.4)
  if (p.D <= 64 && kv_dtype == PA_FP8_E4M3FN) return p.partition_size;
  return p.partition_size * token_scale(p, kv_dtype);
}
constexpr long kDecodeSmallCallBytes = 160L << 20;
constexpr long kDecodeSmallCallPairs = 256;     // (80 while every call took partitions of 512; see decode_sized_partition)
// The same comparison on the gpt-oss layer (64 / 8 heads of 64, whose rows are half as long; us per layer, fixed /
// balanced, contexts of 1 K): B = 12 27.4 / 30.3, 16 29.0 / 31.2, 24 31.1 / 35.7, 32 33.5 / 38.2, 64 55.3 / 48.8; B = 16 at
// 4 K 47.2 / 47.9: at head dim 64 the fixed partitions stay ahead up to four times as many pairs.  And a sliding window
// that fits one partition leaves every sequence a handful of tiles, which one workgroup per (sequence, kv head) reads
// in one go, without partials or a merge (window 128: B = 16 17.3 / 26.0, B = 64 23.8 / 31.7).
constexpr long kDecodeSmallCallPairsD64 = 320;
constexpr long kDecodeSmallCallPairsOnePartition = 1024;
static bool decode_small_call(const DecodeParams& p, int kv_dtype, int max_parts = kDecodeSmallCallPartitions) {
  const long esz = kv_dtype == PA_FP8_E4M3FN ? 1 : (kv_dtype == PA_BF16 ? 2 : 4);
  if (p.max_seq_len <= 0 || p.partition_size <= 0 || p.partition_size % 32) return false;
  if (num_partitions_for(span_bound(p), base_partition(p, kv_dtype)) > max_parts) return false;
  long pairs_max = p.D <= 64 ? kDecodeSmallCallPairsD64 : kDecodeSmallCallPairs;
  // ... and so do contexts of at most 768 tokens, which decode reads as one partition on eight waves (head dim 128,
  // contexts of 600, fixed / balanced: B = 16 27.6 / 35.9, 32 31.4 / 42.0, 48 47.4 / 47.9; verify, T = 4: B = 16
  // 39.8 / 46.0, 32 53.0 / 60.2)
  if ((p.window > 0 && span_bound(p) <= p.partition_size) || span_bound(p) <= 768) pairs_max = kDecodeSmallCallPairsOnePartition;
  if (g_small_call_pairs.load() > 0) pairs_max = g_small_call_pairs.load();
  if ((long)p.B * p.Hkv * ((p.Hq / p.Hkv * std::max(p.T, 1) + 15) / 16) > pairs_max) return false;
  const double bytes = 2.0 * p.B * (double)span_bound(p) * p.Hkv * p.D * esz;
  return bytes <= (double)kDecodeSmallCallBytes;
}
// Partitions of 256 tokens instead of the caller's (larger) ones when those would give the device very few
// workgroups (a single sequence, mostly): same units, partitions of 512 / of 256: 1 x 1 K 25.8 / 22.9, 1 x 4 K
// 28.3 / 27.9; with more workgroups to begin with the finer ones cost more than they bring (8 x 1 K 29.6 / 32.4).
static int decode_fine_partition(const DecodeParams& p, int kv_dtype) {
  const int base = base_partition(p, kv_dtype);
  int kFine = g_decode_fine.load();
  if (kFine > 0 && num_partitions_for(span_bound(p), kFine) > 12) kFine *= token_scale(p, kv_dtype);    // (9 of 256 behind 2 K: 9.1 us, 5 of 512: 9.2-9.3)
  if (kFine <= 0 || base <= kFine || span_bound(p) <= kFine) return base;
  const long slots = (long)p.Hkv * ((p.Hq / p.Hkv * std::max(p.T, 1) + 15) / 16);      // workgroups per sequence and partition
  if (p.B * slots * num_partitions_for(span_bound(p), base) > 64) return base;
  if (num_partitions_for(span_bound(p), kFine) > 16) return base;
  return kFine;
}
// Many (sequence, kv head) pairs: partitions sized to the device instead.  Two of these workgroups on one CU slow each
// other by a third (B = 8 / 10 / 11 sequences behind 1 K on partitions of 512, 192-264 workgroups of which a third
// trivial: kernel 15.4 / 16.1 / 16.7 us; B = 12: 21.3), so the context is cut into as many partitions as keep the
// workgroups at one per CU -- not finer than 256 tokens, not longer than 1 152 (twice that at head dim 64, see
// token_scale) -- and, where that cannot be had, at two per CU.  us per layer of a decode step, balanced / partitions of 512 / sized this way, contexts of 1 K: B = 12 35.9 /
// 35.6 / 31.0, 16 38.4 / 37.6 / 33.8, 24 44.5 / 46.2 / 39.2, 32 49.5 / 54.6 / 44.2; of 2 K: B = 16 47.6 / 52.8 / 46.4.
// Returns the partition size, or 0 when the call is too large for the fixed partitions altogether.
static int decode_sized_partition(const DecodeParams& p, int kv_dtype, int num_cus) {
  const long pairs = (long)p.B * p.Hkv * ((p.Hq / p.Hkv * std::max(p.T, 1) + 15) / 16);
  const int reach = span_bound(p), ts = token_scale(p, kv_dtype);
  const int np_min = (reach + 1152 * ts - 1) / (1152 * ts);
  for (int per_cu = 1; per_cu <= 2; ++per_cu) {
    const long room = (long)per_cu * num_cus / pairs;                  // partitions per pair that fit
    if (room < np_min) continue;
    const int finest = num_partitions_for(reach, per_cu == 1 ? 256 : 512);
    const int np = (int)std::max<long>(np_min, std::min<long>(room, finest));
    return (((reach + np - 1) / np) + 31) & ~31;
  }
  return 0;
}
// The partitions of a call made equal: as many as `part` tokens each would give, cut evenly over what a sequence can
// reach (a bound of 1 120 tokens on partitions of 512 is 512 + 512 + 96, the kernel as long as its longest workgroup;
// as 384 + 384 + 352 a decode step of 8 sequences takes 27.5 us per layer instead of 29.4)
static int equal_partitions(int reach, int part) {
  const int np = num_partitions_for(reach, part);
  return np <= 1 ? part : (((reach + np - 1) / np) + 31) & ~31;
}
static int decode_kind(const DecodeParams& p, int q_dtype, int kv_dtype, bool needs_balanced = false) {
  const int impl = g_decode_impl.load();
  const bool mfma_ok = decode_mfma_supported(p, q_dtype, kv_dtype);
  if ((impl == 2 || impl == 3) && !mfma_ok) return -1;
  if (!mfma_ok || impl == 1) return 1;
  if (impl == 0) return !needs_balanced && decode_small_call(p, kv_dtype) ? 2 : 3;
  return impl == 2 ? 2 : 3;
}

size_t pa_decode_workspace_bytes_for(int B, int Hq, int Hkv, int D, int block_size, int max_seq_len,
                                     int partition_size, int q_dtype, int kv_dtype) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || D <= 0 || block_size <= 0 || partition_size <= 0) return 0;
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.D = D; p.T = 1; p.rows_per_wave = 16;
  p.block_size = block_size; p.block_shift = ilog2_exact(block_size);
  p.max_seq_len = max_seq_len; p.partition_size = partition_size;
  const int kind = decode_kind(p, q_dtype, kv_dtype);
  int np = num_partitions_for(max_seq_len, partition_size);
  if (kind == 2 && max_seq_len > 0) np = std::max(np, num_partitions_for(max_seq_len, decode_fine_partition(p, kv_dtype)));
  const size_t fixed = np <= 1 ? 0 : (size_t)B * Hq * np * ((size_t)D + 2) * sizeof(float);
  if (max_seq_len <= 0) {
    // no bound given: pa_decode then takes the table capacity, which this function is not told.  The answer covers
    // every kernel that call can pick: the balanced one, or fixed partitions, which are chosen for at most eight
    // (the scalar kernel's partitions are not bounded that way: its callers give the bound)
    if (kind == 1 || kind < 0) return 0;
    plan_decode_balanced(p, current_num_cus());
    const size_t balanced = decode_balanced_workspace_bytes(B, Hq, D, p.bal_gv);
    const size_t most = (size_t)B * Hq * 16 * ((size_t)D + 2) * sizeof(float);      // (up to sixteen of the finer partitions)
    return most > balanced ? most : balanced;
  }
  if (kind == 1 || kind < 0) return fixed;
  plan_decode_balanced(p, current_num_cus());
  const size_t balanced = decode_balanced_workspace_bytes(B, Hq, D, p.bal_gv);
  if (kind == 3) return balanced;
  // fixed partitions, by choice or by the size of the call: a forced kernel choice can still send the call to the
  // balanced kernel, so the answer covers both
  return fixed > balanced ? fixed : balanced;
}

// pa_decode in two halves, so that pa_decode_step can decide between them what rides on the decode launch:
// plan_decode validates and picks the kernel, run_decode sizes the workspace and launches.
struct DecodePlan {
  DecodeParams p;
  int kind;                 // 1 scalar-ALU, 2 MFMA with fixed partitions, 3 MFMA balanced
  int waves;                // fixed partitions: waves per workgroup (0: the kernel's default)
  int caller_partition;     // the caller's partition size (p.partition_size may be a finer one)
  int q_dtype, kv_dtype;
};

static int plan_decode(const char* who, DecodePlan& pl, const void* q, const void* k_cache, const void* v_cache,
                       const float* k_scale, const float* v_scale, const int32_t* block_tables, const int32_t* seq_lens,
                       void* out, bool out_required, int B, int Hq, int Hkv, int D, int block_size,
                       int max_blocks_per_seq, int num_blocks, int max_seq_len, float scale, int partition_size,
                       int q_dtype, int kv_dtype, const float* sinks, int sliding_window,
                       const pa_q_transform* q_transform) {
  if (sliding_window < 0) return fail_arg("%s: sliding_window=%d must be >= 0 (0 = none)", who, sliding_window);
  if (B < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return fail_arg("%s: bad sizes B=%d Hq=%d Hkv=%d D=%d", who, B, Hq, Hkv, D);
  if (Hq % Hkv) return fail_arg("%s: Hq=%d is not a multiple of Hkv=%d", who, Hq, Hkv);
  if (block_size <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0)
    return fail_arg("%s: bad paging sizes block_size=%d max_blocks_per_seq=%d num_blocks=%d", who,
                    block_size, max_blocks_per_seq, num_blocks);
  if (partition_size <= 0) return fail_arg("%s: partition_size=%d must be positive", who, partition_size);
  if (!(q_dtype == PA_F32 && kv_dtype == PA_F32) && !(q_dtype == PA_BF16 && kv_dtype == PA_BF16) &&
      !(q_dtype == PA_BF16 && kv_dtype == PA_FP8_E4M3FN))
    return fail_arg("%s: unsupported dtype pair q=%d kv=%d", who, q_dtype, kv_dtype);
  if (D != 32 && D != 64 && D != 128 && D != 256) return fail_arg("%s: head_dim %d not in {32,64,128,256}", who, D);
  if (B == 0) return 0;
  if (!q || !k_cache || !v_cache || !block_tables || !seq_lens || (out_required && !out))
    return fail_arg("%s: null pointer argument", who);
  if (kv_dtype == PA_FP8_E4M3FN && (!k_scale || !v_scale)) return fail_arg("%s: fp8 KV needs k_scale and v_scale", who);
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
    return fail_arg("%s: q, k_cache, v_cache and out must be 16-byte aligned", who);
  const long cap = (long)max_blocks_per_seq * block_size;
  if (max_seq_len <= 0 || max_seq_len > cap) max_seq_len = (int)(cap > 0x7fffffffL ? 0x7fffffffL : cap);

  DecodeParams& p = pl.p;
  memset(&p, 0, sizeof(p));
  p.q = q; p.k_cache = k_cache; p.v_cache = v_cache; p.k_scale = k_scale; p.v_scale = v_scale;
  p.block_tables = block_tables; p.seq_lens = seq_lens; p.out = out;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.D = D; p.T = 1; p.rows_per_wave = 16;
  p.block_size = block_size; p.max_blocks = max_blocks_per_seq; p.num_blocks = num_blocks;
  p.block_shift = ilog2_exact(block_size);
  p.partition_size = partition_size;
  p.max_seq_len = max_seq_len;
  p.sinks = sinks; p.window = sliding_window;
  p.num_partitions = num_partitions_for(span_bound(p), partition_size);
  p.scale_log2e = scale * kLog2e;
  p.head_major = g_head_major.load();
  pl.caller_partition = partition_size;
  pl.q_dtype = q_dtype; pl.kv_dtype = kv_dtype;
  if (p.num_partitions > 65535 || B > 65535) return fail_arg("%s: grid too large (partitions=%d B=%d)", who, p.num_partitions, B);
  // kernel choice: 0 automatic, 1 scalar-ALU, 2 MFMA with fixed partitions, 3 MFMA balanced
  // (sinks and a sliding window live in both MFMA kernels; a call forced onto the fixed partitions keeps them)
  const int kind = pl.kind = decode_kind(p, q_dtype, kv_dtype);
  if (kind < 0) return fail_arg("%s: MFMA kernel forced but shape unsupported", who);
  if (kind == 2 && partition_size % 32) return fail_arg("%s: the fixed-partition MFMA kernel needs partition_size %% 32 == 0", who);
  // a small call of short contexts: the whole context as one partition on eight waves, which merge through LDS, so
  // that there is no merge launch.  Per call replayed from a HIP graph (32 / 8 heads of 128, bf16, us, two partitions of
  // 512 + merge against one partition): contexts of 350-700 tokens B = 1 10.1 / 9.7, B = 16 12.3 / 11.1, B = 64
  // 31.3 / 26.6; 512-1024 tokens B = 8 10.4 / 12.0 (the longer chain per wave costs more than the launch), B = 64
  // 36.7 / 34.7.  So: bounds up to three quarters of the limit always, up to the limit when the grid is large anyway.
  pl.waves = g_decode_waves.load();
  const int single_max = g_decode_single_max.load();
  if (kind == 2 && pl.waves == 0 && g_decode_impl.load() == 0 && p.num_partitions > 1) {
    const int reach = span_bound(p);
    if (Hq / Hkv <= 8 &&
        (reach <= single_max - single_max / 4 || (reach <= single_max && (long)B * Hkv >= 256))) {
      p.partition_size = (reach + 31) & ~31;
      p.num_partitions = 1;
      pl.waves = 8;
    } else {
      const long pairs = (long)B * Hkv * ((Hq / Hkv + 15) / 16);
      const int np_base = num_partitions_for(reach, base_partition(p, kv_dtype));
      const int sized = pairs * np_base > current_num_cus() ? decode_sized_partition(p, kv_dtype, current_num_cus()) : 0;
      p.partition_size = equal_partitions(reach, sized > 0 ? sized : decode_fine_partition(p, kv_dtype));
      p.num_partitions = num_partitions_for(reach, p.partition_size);
    }
  }
  if ((sinks || sliding_window > 0) && kind == 1)
    return fail_arg("%s: sinks and sliding_window need the MFMA kernels (bf16 q, bf16 or fp8 KV, "
                    "head_dim 64 or 128, block_size a power of two >= 16)", who);
  if (take_q_transform(who, q_transform, kind != 1, p.qt)) return -1;
  return 0;
}

// Launches the planned decode.  leave_partials (fixed partitions with more than one partition only): the merge
// launch is left out, the caller's consumer reads p.ws_out / p.ws_ml.  Returns the bytes of workspace used in *used.
static int run_decode(const char* who, DecodePlan& pl, void* workspace, size_t workspace_bytes, bool leave_partials,
                      size_t* used, hipStream_t s) {
  DecodeParams& p = pl.p;
  const int B = p.B, Hq = p.Hq, D = p.D;
  if (used) *used = 0;
  if (!aligned16(workspace)) return fail_arg("%s: workspace must be 16-byte aligned", who);
  if (pl.kind == 3) {
    plan_decode_balanced(p, current_num_cus());
    p.bal_lockstep = lockstep_for(pl.kv_dtype, p.bal_ns);
    const size_t need = decode_balanced_workspace_bytes(B, Hq, D, p.bal_gv);
    if (!workspace || workspace_bytes < need)
      return fail_arg("%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
    if (used) *used = need;
    p.ws_out = (float*)workspace;
    p.ws_ml = p.ws_out + (size_t)Hq * ((size_t)B + p.bal_gv) * D;
    p.ws_start = (int32_t*)(p.ws_ml + (size_t)Hq * ((size_t)B + p.bal_gv) * 2);
    profile_begin(s);
    hipError_t e = launch_decode_balanced(p, pl.kv_dtype, s);
    profile_end(s);
    if (e != hipSuccess) return check_hip(e, "decode launch");
    e = launch_decode_balanced_reduce(p, s);
    return check_hip(e, "decode reduce launch");
  }
  if (p.num_partitions > 1) {
    size_t need = (size_t)B * Hq * p.num_partitions * ((size_t)D + 2) * sizeof(float);
    if ((!workspace || workspace_bytes < need) && p.partition_size != pl.caller_partition) {
      // a workspace sized for the caller's partitions only: those, then
      p.partition_size = pl.caller_partition;
      p.num_partitions = num_partitions_for(span_bound(p), p.partition_size);
      need = (size_t)B * Hq * p.num_partitions * ((size_t)D + 2) * sizeof(float);
    }
    if (p.num_partitions > 1) {
      if (!workspace || workspace_bytes < need)
        return fail_arg("%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
      if (used) *used = need;
      p.ws_out = (float*)workspace;
      p.ws_ml = p.ws_out + (size_t)B * Hq * p.num_partitions * D;
    }
  }
  profile_begin(s);
  hipError_t e = pl.kind == 2 ? launch_decode_mfma(p, pl.kv_dtype, pl.waves, s)
                              : launch_decode_generic(p, pl.q_dtype, pl.kv_dtype, s);
  profile_end(s);
  if (e != hipSuccess) return check_hip(e, "decode launch");
  if (p.num_partitions > 1 && !leave_partials) {
    e = launch_decode_reduce(p, pl.q_dtype, s);
    if (e != hipSuccess) return check_hip(e, "decode reduce launch");
  }
  return 0;
}

int pa_decode(const void* q, const void* k_cache, const void* v_cache,
              const float* k_scale, const float* v_scale,
              const int32_t* block_tables, const int32_t* seq_lens,
              void* out, void* workspace, size_t workspace_bytes,
              int B, int Hq, int Hkv, int D, int block_size,
              int max_blocks_per_seq, int num_blocks, int max_seq_len,
              float scale, int partition_size, int q_dtype, int kv_dtype,
              const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream) {
  tl_error[0] = 0;
  DecodePlan pl;
  if (int rc = plan_decode("pa_decode", pl, q, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, out, true, B, Hq,
                           Hkv, D, block_size, max_blocks_per_seq, num_blocks, max_seq_len, scale, partition_size, q_dtype,
                           kv_dtype, sinks, sliding_window, q_transform))
    return rc;
  if (B == 0) return 0;
  return run_decode("pa_decode", pl, workspace, workspace_bytes, false, nullptr, (hipStream_t)stream);
}

// ---- pa_decode for callers that cannot allocate ------------------------------------------------
// Split-K partials of pa_decode_noalloc live in this array instead of a caller's workspace.  Every
// device the library runs on holds its own copy, at its own address, for the life of the process.
static __device__ __align__(256) unsigned char scratch[PA_DECODE_NOALLOC_SCRATCH_BYTES];

// Device address of `scratch` on the current device, looked up once per device (in host code the
// array's name is not a device address).  Returns nullptr with the error text set on failure.
static void* noalloc_scratch_ptr() {
  static std::mutex mu;
  static void* ptrs[64] = {nullptr};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { check_hip(e, "pa_decode_noalloc: hipGetDevice"); return nullptr; }
  if (dev < 0 || dev >= 64) { set_error("pa_decode_noalloc: device index %d outside [0, 64)", dev); return nullptr; }
  std::lock_guard<std::mutex> lk(mu);
  if (!ptrs[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      check_hip(e == hipSuccess ? hipErrorInvalidSymbol : e, "pa_decode_noalloc: hipGetSymbolAddress(scratch)");
      return nullptr;
    }
    ptrs[dev] = ptr;
  }
  return ptrs[dev];
}

int pa_decode_noalloc(const void* q, const void* k_cache, const void* v_cache,
                      const float* k_scale, const float* v_scale,
                      const int32_t* block_tables, const int32_t* seq_lens, void* out,
                      int B, int Hq, int Hkv, int D, int block_size,
                      int max_blocks_per_seq, int num_blocks, int max_seq_len,
                      float scale, int partition_size, int q_dtype, int kv_dtype,
                      const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream) {
  tl_error[0] = 0;
  if (B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && D > 0 && block_size > 0 && max_blocks_per_seq > 0 && partition_size > 0) {
    const long cap = (long)max_blocks_per_seq * block_size;
    int msl = max_seq_len;
    if (msl <= 0 || msl > cap) msl = (int)(cap > 0x7fffffffL ? 0x7fffffffL : cap);
    const size_t need = pa_decode_workspace_bytes_for(B, Hq, Hkv, D, block_size, msl, partition_size, q_dtype, kv_dtype);
    if (need > (size_t)PA_DECODE_NOALLOC_SCRATCH_BYTES)
      return fail_arg("pa_decode_noalloc: this call needs %zu bytes for its split-K partials, the library's static "
                      "scratch holds %zu (PA_DECODE_NOALLOC_SCRATCH_BYTES); use pa_decode with a workspace of the caller's",
                      need, (size_t)PA_DECODE_NOALLOC_SCRATCH_BYTES);
  }
  void* ws = noalloc_scratch_ptr();
  if (!ws) return 1;
  // same validation, kernels and launches as pa_decode; the partials are rewritten by every call before they are
  // read, so nothing in the scratch has to start at zero
  return pa_decode(q, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, out, ws,
                   (size_t)PA_DECODE_NOALLOC_SCRATCH_BYTES, B, Hq, Hkv, D, block_size, max_blocks_per_seq, num_blocks,
                   max_seq_len, scale, partition_size, q_dtype, kv_dtype, sinks, sliding_window, q_transform, stream);
}

// A caller of verify_launch that can consume the fixed-partition route's split-K partials itself (the projection of
// pa_verify_step) asks for them here: when the call takes that route with more than one partition, the merge launch
// is left out and `f` says where the partials are.
// The same caller hands over the step's cache update: verify_launch either lets it ride on the fixed-partition
// launch (bf16 pools, all rows of a kv head on one wave) or runs the write launch in front of the attention launch.
struct VerifyPartials {
  bool want;
  bool left;
  DecodeParams f;
  const pa_new_kv* new_kv;      // null: the pool already holds the new tokens
  void* k_cache_w;
  void* v_cache_w;
  float* k_scale_w;
  float* v_scale_w;
  bool fuse_rows;               // allowed to take the rows on the attention launch
};

static int verify_write_rows(const VerifyPartials& vp, const pa_q_transform* qt, const int32_t* block_tables,
                             const int32_t* seq_lens, int B, int T, int Hq, int Hkv, int D, int block_size,
                             int max_blocks_per_seq, int num_blocks, int kv_dtype, void* stream) {
  const pa_new_kv* n = vp.new_kv;
  if (qt)
    return pa_qk_norm_rope_kv_write(nullptr, n->xk, n->xv, nullptr, nullptr, n->k_norm_weight, qt->norm_eps, qt->rope_cos,
                                    qt->rope_sin, qt->rope_max_pos, vp.k_cache_w, vp.v_cache_w, vp.k_scale_w, vp.v_scale_w,
                                    block_tables, seq_lens, n->query_lens, B, T, Hq, Hkv, D, block_size, max_blocks_per_seq,
                                    num_blocks, kv_dtype, stream);
  return pa_kv_write(n->xk, n->xv, vp.k_cache_w, vp.v_cache_w, vp.k_scale_w, vp.v_scale_w, block_tables, seq_lens,
                     n->query_lens, B, T, Hkv, D, block_size, max_blocks_per_seq, num_blocks, kv_dtype, stream);
}

// Query tokens [t0, t0 + Tc) of the T tokens per sequence through the decode-shaped kernel (pa_verify: all
// of them in one launch; pa_prefill for shapes the tiled kernel does not take: 64 at a time).
static int verify_launch(const char* who, const void* q, const void* k_cache, const void* v_cache,
                         const float* k_scale, const float* v_scale,
                         const int32_t* block_tables, const int32_t* seq_lens, const int32_t* query_lens,
                         void* out, void* workspace, size_t workspace_bytes,
                         int B, int T, int t0, int Tc, int Hq, int Hkv, int D, int block_size,
                         int max_blocks_per_seq, int num_blocks, int max_seq_len, float scale, int kv_dtype,
                         const float* sinks, int sliding_window, const pa_q_transform* q_transform, hipStream_t s,
                         VerifyPartials* vp = nullptr) {
  const long cap = (long)max_blocks_per_seq * block_size;
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  if (vp) vp->left = false;
  p.q = q; p.k_cache = k_cache; p.v_cache = v_cache; p.k_scale = k_scale; p.v_scale = v_scale;
  p.block_tables = block_tables; p.seq_lens = seq_lens; p.query_lens = query_lens; p.out = out;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.D = D; p.T = Tc; p.T_stride = T; p.t0 = t0;
  {
    // One wave carries 16 query rows of a kv head, or 32 where that measured faster: with more than 16 rows
    // and enough waves either way (a batch of 16 or more, or 128 rows per kv head as in the 64-token launches
    // of a long prefill), for D = 64 and for fp8 pools (which fit the registers), and for bf16 at D = 128
    // (which spills a little) only from four 16-row groups on.
    const int n_rows = (Hq / Hkv) * Tc, forced = g_verify_rows.load();
    // (not under a sliding window: the few tiles a launch then sees are better spread over more waves)
    bool wide = n_rows > 16 && (B >= (D == 64 ? 8 : 16) || (n_rows >= 128 && sliding_window == 0)) &&
                (D == 64 || kv_dtype == PA_FP8_E4M3FN || n_rows > 48);
    // fp8 pools at head dim 128: the two-operand wave is the lean form (Q fragments from LDS, V single-buffered; its
    // some fifty spilled registers lie in the start and end of a sequence, not in the tile loop), which the 16-row
    // wave with K and V streamed two tiles deep has overtaken; it only pays on the largest calls (32 / 8 heads,
    // ragged contexts, us 16 / 32 rows per wave: B = 32 behind 4 K T = 8 63.5 /
    // 86.7, T = 16 98.9 / 103.2, T = 32 178.6 / 159.1; B = 64 behind 1 K T = 8 42.4 / 59.5, T = 32 109.2 / 112.8)
    // ... and at head dim 128 over bf16 pools, the same lean form (32 / 8 heads, T = 16: B = 16 behind 1 K 30.7 / 55.8,
    // B = 32 behind 2 K 80.7 / 90.4; T = 32, B = 16 behind 4 K 122.5 / 114.7).  At head dim 64 it fits, and is ahead once the
    // call is large enough for its half as many waves (64 / 8 heads, on the balanced schedule: T = 4 B = 32 behind 1 K
    // 24.3 / 34.2, B = 64 behind 1 K 39.9 / 36.1, B = 16 behind 4 K 47.5 / 37.4; T = 8 B = 16 behind 1 K 25.2 / 29.5, B = 8
    // behind 4 K 41.2 / 31.3).  The measure is sequences x rows per kv head x length bound.
    if (wide) {
      const long bound = max_seq_len > 0 ? std::min<long>(max_seq_len, cap) : cap;
      const long work = (long)B * n_rows * bound;
      wide = work >= (D == 64 ? 1200000L : kv_dtype == PA_FP8_E4M3FN ? 12L << 20 : 8L << 20);
    }
    p.rows_per_wave = forced == 16 || forced == 32 ? forced : (wide ? 32 : 16);
  }
  p.block_size = block_size; p.max_blocks = max_blocks_per_seq; p.num_blocks = num_blocks;
  p.block_shift = ilog2_exact(block_size);
  p.max_seq_len = (int)(cap > 0x7fffffffL ? 0x7fffffffL : cap);
  p.sinks = sinks; p.window = sliding_window;
  p.partition_size = p.max_seq_len;
  p.num_partitions = 1;
  p.scale_log2e = scale * kLog2e;
  if (!decode_mfma_supported(p, PA_BF16, kv_dtype))
    return fail_arg("%s: unsupported shape (D=%d must be 64 or 128, block_size=%d a power of two >= 16)", who, D, block_size);
  if (take_q_transform(who, q_transform, true, p.qt)) return -1;
  if (max_seq_len > 0 && max_seq_len < p.max_seq_len) p.max_seq_len = max_seq_len;     // the caller's bound on the contexts
  // Small calls (the reference's own use of this path: one sequence, a handful of draft tokens) take fixed partitions,
  // as small pa_decode calls do, by the same rule and for the same reason: the balanced schedule costs what it costs
  // whatever the sizes (256 chunks, each leaving partials of 16 rows).  Inside a verify step of eight attention layers
  // (T = 4, 32 / 8 heads of 128, us per layer replayed from a graph, balanced / fixed partitions): B = 1 behind 4 K
  // 36.0 / 32.9, B = 4 behind 2 K 41.4 / 34.4, B = 4 behind 4 K 47.6 / 38.1, B = 8 behind 2 K 46.8 / 44.0; a single
  // sequence on the finer partitions, B = 1 behind 1 K: 30.5 -> 27.7.  It needs the caller's bound on the lengths (the
  // table capacity says nothing about the sizes), 16 rows per wave, and a workspace that holds the partitions'
  // partials.  Under a sliding window the partitions cover what the window reaches, often a single one, and the
  // window is itself a bound.
  // The fixed partitions take 16 rows per wave, so a call that would take 32 on the balanced schedule is asked first
  // whether it is a small one: it mostly is better off here (64 / 8 heads of 64, T = 4, us fixed partitions / balanced
  // with 32 rows: B = 16 behind 1 K 14.1 / 24.1, B = 32 behind 1 K 23.2 / 33.1; fp8 pool, 32 / 8 heads of 128, T = 8:
  // B = 16 behind 1 K 18.0 / 42.5, behind 4 K 53.6 / 62.3).  Not when every kv head has several 16-row waves, each of
  // which reads its partitions, over long contexts: at head dim 64 (where the two-operand wave fits) from 80 000
  // (sequence x wave x bound) products on the balanced schedule with 32 rows is ahead (B = 8 behind 4 K T = 8 35.6 /
  // 29.4, B = 12 behind 4 K T = 4 45.2 / 35.2; B = 8 behind 4 K T = 4 21.8 / 29.2 is not).
  if ((max_seq_len > 0 || sliding_window > 0) && g_verify_rows.load() != 32 && g_decode_impl.load() == 0) {
    DecodeParams f = p;
    f.rows_per_wave = 16;
    f.partition_size = 512;
    bool small = decode_small_call(f, kv_dtype);
    {
      const int n_rows = (Hq / Hkv) * Tc;
      if (small && D == 64 && n_rows > 16 && p.rows_per_wave == 32 &&
          (long)B * ((n_rows + 15) / 16) * span_bound(f) > 80000) small = false;
    }
    if (small) {
      // a single sequence: finer partitions; many (sequence, kv head) pairs: partitions sized to the device (as pa_decode)
      const long pairs = (long)B * Hkv * (((Hq / Hkv) * Tc + 15) / 16);
      const int sized = pairs * num_partitions_for(span_bound(f), base_partition(f, kv_dtype)) > current_num_cus()
                            ? decode_sized_partition(f, kv_dtype, current_num_cus()) : 0;
      f.partition_size = equal_partitions(span_bound(f), sized > 0 ? sized : decode_fine_partition(f, kv_dtype));
    }
    f.num_partitions = num_partitions_for(span_bound(f), f.partition_size);
    size_t need_f = f.num_partitions <= 1 ? 0 : (size_t)B * Hq * Tc * f.num_partitions * ((size_t)D + 2) * sizeof(float);
    if (small && f.partition_size != 512 && need_f && !(workspace && workspace_bytes >= need_f)) {
      f.partition_size = 512;
      f.num_partitions = num_partitions_for(span_bound(f), f.partition_size);
    }
    need_f = f.num_partitions <= 1 ? 0 : (size_t)B * Hq * Tc * f.num_partitions * ((size_t)D + 2) * sizeof(float);
    if (small && (need_f == 0 || (workspace && workspace_bytes >= need_f))) {
      f.head_major = g_head_major.load();
      f.ws_out = (float*)workspace;
      f.ws_ml = f.ws_out + (size_t)B * Hq * Tc * f.num_partitions * D;
      if (vp && vp->new_kv) {
        // (for one or two sequences: B = 1, T = 4 behind 1 K 27.6 -> 25.9 us per layer of a verify step, behind 4 K
        // 32.5 -> 31.2; with more sequences the start of more workgroups waits for the rows' transform and the write
        // launch is the faster way: B = 8 34.8 -> 35.6.  Debug switch 10 = 2 takes the rows whatever the batch.)
        if (vp->fuse_rows && t0 == 0 && Tc == T && decode_new_row_supported(f, PA_BF16, kv_dtype) &&
            ((long)B * Hkv <= 16 || g_step_fusion.load() == 2)) {
          f.new_k = vp->new_kv->xk; f.new_v = vp->new_kv->xv; f.new_lens = vp->new_kv->query_lens;
          if (q_transform) {
            f.new_kt = f.qt;
            f.new_kt.norm_weight = (const uint16_t*)vp->new_kv->k_norm_weight;
          }
        } else if (int rc = verify_write_rows(*vp, q_transform, block_tables, seq_lens, B, T, Hq, Hkv, D, block_size,
                                              max_blocks_per_seq, num_blocks, kv_dtype, (void*)s)) {
          return rc;
        }
      }
      profile_begin(s);
      hipError_t e = launch_decode_mfma(f, kv_dtype, 0, s);
      profile_end(s);
      if (e != hipSuccess) return check_hip(e, "verify kernel launch");
      if (vp && vp->want && f.num_partitions > 1) {
        vp->left = true;
        vp->f = f;
        return 0;
      }
      if (f.num_partitions > 1) e = launch_decode_reduce(f, PA_BF16, s);
      return check_hip(e, "verify merge launch");
    }
  }
  plan_decode_balanced(p, current_num_cus());
  p.bal_lockstep = lockstep_for(kv_dtype, p.bal_ns);
  const size_t need = decode_balanced_workspace_bytes(B, Hq * Tc, D, p.bal_gv);
  if (!workspace || workspace_bytes < need)
    return fail_arg("%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  if (vp && vp->new_kv) {
    if (int rc = verify_write_rows(*vp, q_transform, block_tables, seq_lens, B, T, Hq, Hkv, D, block_size,
                                   max_blocks_per_seq, num_blocks, kv_dtype, (void*)s))
      return rc;
  }
  p.ws_out = (float*)workspace;
  p.ws_ml = p.ws_out + (size_t)Hq * Tc * ((size_t)B + p.bal_gv) * D;
  p.ws_start = (int32_t*)(p.ws_ml + (size_t)Hq * Tc * ((size_t)B + p.bal_gv) * 2);
  profile_begin(s);
  hipError_t e = launch_decode_balanced(p, kv_dtype, s);
  profile_end(s);
  if (e != hipSuccess) return check_hip(e, "verify kernel launch");
  e = launch_decode_balanced_reduce(p, s);
  return check_hip(e, "verify merge launch");
}

size_t pa_verify_workspace_bytes(int B, int T, int Hq, int D) {
  if (B <= 0 || T <= 0 || Hq <= 0 || D <= 0 || (long)Hq * T > 0x7fffffffL) return 0;
  return decode_balanced_workspace_bytes(B, Hq * T, D, 8 * current_num_cus());
}

int pa_verify(const void* q, const void* k_cache, const void* v_cache,
              const float* k_scale, const float* v_scale,
              const int32_t* block_tables, const int32_t* seq_lens, const int32_t* query_lens,
              void* out, void* workspace, size_t workspace_bytes,
              int B, int T, int Hq, int Hkv, int D, int block_size,
              int max_blocks_per_seq, int num_blocks, int max_seq_len,
              float scale, int kv_dtype, const float* sinks, int sliding_window,
              const pa_q_transform* q_transform, void* stream) {
  tl_error[0] = 0;
  if (sliding_window < 0) return fail_arg("pa_verify: sliding_window=%d must be >= 0 (0 = none)", sliding_window);
  if (B < 0 || T < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return fail_arg("pa_verify: bad sizes B=%d T=%d Hq=%d Hkv=%d D=%d", B, T, Hq, Hkv, D);
  if (Hq % Hkv) return fail_arg("pa_verify: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  if (block_size <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0) return fail_arg("pa_verify: bad paging sizes");
  if (kv_dtype != PA_BF16 && kv_dtype != PA_FP8_E4M3FN)
    return fail_arg("pa_verify: kv_dtype must be bf16 or fp8-e4m3fn (got %d)", kv_dtype);
  if (T > PA_VERIFY_MAX_TOKENS) return fail_arg("pa_verify: T=%d exceeds %d query tokens per sequence; use pa_prefill", T, PA_VERIFY_MAX_TOKENS);
  if (B == 0 || T == 0) return 0;
  if (B > 65535) return fail_arg("pa_verify: B=%d exceeds 65535", B);
  if (!q || !k_cache || !v_cache || !block_tables || !seq_lens || !query_lens || !out)
    return fail_arg("pa_verify: null pointer argument");
  if (kv_dtype == PA_FP8_E4M3FN && (!k_scale || !v_scale)) return fail_arg("pa_verify: fp8 KV needs k_scale and v_scale");
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out) || !aligned16(workspace))
    return fail_arg("pa_verify: q, k_cache, v_cache, out and workspace must be 16-byte aligned");
  return verify_launch("pa_verify", q, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, query_lens, out,
                       workspace, workspace_bytes, B, T, 0, T, Hq, Hkv, D, block_size, max_blocks_per_seq, num_blocks,
                       max_seq_len, scale, kv_dtype, sinks, sliding_window, q_transform, (hipStream_t)stream);
}

static void fill_prefill_shape(PrefillParams& p, int B, int T, int Hq, int Hkv, int D, int block_size,
                               int max_blocks_per_seq, int num_blocks) {
  p.B = B; p.T = T; p.Hq = Hq; p.Hkv = Hkv; p.D = D;
  p.block_size = block_size; p.max_blocks = max_blocks_per_seq; p.num_blocks = num_blocks;
  p.block_shift = ilog2_exact(block_size);
  p.impl = g_prefill_impl.load();
  p.num_cus = current_num_cus();
}

static size_t prefill_split_bytes(const PrefillParams& p, int splits) {
  return splits > 1 ? (size_t)p.B * p.T * p.Hq * splits * ((size_t)p.D + 2) * sizeof(float) : 0;
}

size_t pa_prefill_workspace_bytes(int B, int T, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq) {
  if (B <= 0 || T <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || block_size <= 0 || max_blocks_per_seq <= 0 || Hq % Hkv) return 0;
  PrefillParams p;
  memset(&p, 0, sizeof(p));
  fill_prefill_shape(p, B, T, Hq, Hkv, D, block_size, max_blocks_per_seq, 1);
  p.block_tables = (const int32_t*)16;     // paged form (only tested for null)
  const size_t plain = prefill_split_bytes(p, prefill_async_splits(p, current_num_cus()));
  if (D != 128) {   // what the tiled kernel does not take runs as launches of the decode-shaped kernel, 64 query tokens each
    const size_t chunks = pa_verify_workspace_bytes(B, T < PA_VERIFY_MAX_TOKENS ? T : PA_VERIFY_MAX_TOKENS, Hq, D);
    return plain > chunks ? plain : chunks;
  }
  p.kv_fp8 = 1;                            // fp8 pools use another workgroup shape: cover both
  const size_t fp8 = prefill_split_bytes(p, prefill_async_splits(p, current_num_cus()));
  return plain > fp8 ? plain : fp8;
}

int pa_prefill(const void* q, const void* k_cache, const void* v_cache,
               const float* k_scale, const float* v_scale,
               const int32_t* block_tables, const int32_t* seq_lens,
               const int32_t* query_lens, void* out,
               int B, int T, int Hq, int Hkv, int D, int block_size,
               int max_blocks_per_seq, int num_blocks, int max_seq_len,
               float scale, int dtype, int kv_dtype, const float* sinks, int sliding_window,
               void* workspace, size_t workspace_bytes, const pa_q_transform* q_transform, void* stream) {
  tl_error[0] = 0;
  if (B < 0 || T < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return fail_arg("pa_prefill: bad sizes");
  if (sliding_window < 0) return fail_arg("pa_prefill: sliding_window=%d must be >= 0 (0 = none)", sliding_window);
  if (Hq % Hkv) return fail_arg("pa_prefill: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  if (dtype != PA_BF16) return fail_arg("pa_prefill: only bf16 queries are supported (dtype=%d)", dtype);
  if (kv_dtype != PA_BF16 && kv_dtype != PA_FP8_E4M3FN)
    return fail_arg("pa_prefill: kv_dtype must be bf16 or fp8-e4m3fn (got %d)", kv_dtype);
  const bool fp8 = kv_dtype == PA_FP8_E4M3FN;
  if (block_size <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0) return fail_arg("pa_prefill: bad paging sizes");
  if (max_seq_len < 0 || (long)max_seq_len > (long)max_blocks_per_seq * block_size)
    return fail_arg("pa_prefill: max_seq_len=%d outside [0, max_blocks_per_seq * block_size]", max_seq_len);
  if (B == 0 || T == 0) return 0;
  if ((long)num_blocks * block_size > 0x7fffffffL || (long)block_size * Hkv * D * 2 > 0xffffffffL)
    return fail_arg("pa_prefill: pool of %d blocks x %d rows exceeds 2^31 rows (or a block 4 GiB)", num_blocks, block_size);
  if (!q || !k_cache || !v_cache || !block_tables || !seq_lens || !query_lens || !out)
    return fail_arg("pa_prefill: null pointer argument");
  if (fp8 && (!k_scale || !v_scale)) return fail_arg("pa_prefill: fp8 KV needs k_scale and v_scale");
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
    return fail_arg("pa_prefill: q, k_cache, v_cache and out must be 16-byte aligned");
  PrefillParams p;
  memset(&p, 0, sizeof(p));
  p.q = q; p.k = k_cache; p.v = v_cache; p.block_tables = block_tables; p.seq_lens = seq_lens;
  p.query_lens = query_lens; p.out = out;
  fill_prefill_shape(p, B, T, Hq, Hkv, D, block_size, max_blocks_per_seq, num_blocks);
  p.len_bound = max_seq_len;
  p.scale_log2e = scale * kLog2e;
  p.kv_fp8 = fp8 ? 1 : 0; p.k_scale = k_scale; p.v_scale = v_scale;
  // head_dim 64: the tiled kernel takes two or more kv heads (two heads share its 256-byte rows); short
  // query runs and a single kv head go to the decode-shaped kernel, 64 query tokens per launch, each
  // launch reading the context up to its last token once per kv head
  // (measured crossover for runs of up to 64 tokens: 384 query rows per kv head in a batch of 8 or more)
  const int from64 = g_d64_tiled_from.load();
  const bool many_rows = from64 == PA_VERIFY_MAX_TOKENS + 1 && B >= 8 && (long)T * (Hq / Hkv) >= 384;
  const bool tiled64 = D == 64 && (T >= from64 || many_rows) && p.impl != 1 && prefill_async_supported(p);
  if (!prefill_supported(p) && !tiled64) {
    if (D != 64) return fail_arg("pa_prefill: unsupported shape (D=%d block_size=%d)", D, block_size);
    if (!aligned16(workspace)) return fail_arg("pa_prefill: workspace must be 16-byte aligned");
    if (B > 65535) return fail_arg("pa_prefill: B=%d exceeds 65535", B);
    for (int t0 = 0; t0 < T; t0 += PA_VERIFY_MAX_TOKENS) {
      const int tc = T - t0 < PA_VERIFY_MAX_TOKENS ? T - t0 : PA_VERIFY_MAX_TOKENS;
      const int rc = verify_launch("pa_prefill", q, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, query_lens,
                                   out, workspace, workspace_bytes, B, T, t0, tc, Hq, Hkv, D, block_size,
                                   max_blocks_per_seq, num_blocks, max_seq_len, scale, kv_dtype, sinks, sliding_window, q_transform,
                                   (hipStream_t)stream);
      if (rc) return rc;
    }
    return 0;
  }
  if (sliding_window > 0 && (p.impl == 1 || !prefill_async_supported(p)))
    return fail_arg("pa_prefill: sliding_window needs the asynchronous-copy kernel (block_size a power of two >= 16)");
  p.sinks = sinks; p.window = sliding_window;
  if (take_q_transform("pa_prefill", q_transform, p.impl != 1 && prefill_async_supported(p), p.qt)) return -1;
  // few workgroups and a long table: split the key tiles of a query tile over several workgroups when the
  // caller brought the workspace for it (without one the call runs unsplit)
  p.splits = 1;
  if (workspace) {
    if (!aligned16(workspace)) return fail_arg("pa_prefill: workspace must be 16-byte aligned");
    const int forced = g_prefill_split.load();       // 1: the rule; 0: never; 2-16: that many shares
    const int want = forced == 1 ? prefill_async_splits(p, current_num_cus(), max_seq_len) : forced <= 0 ? 1 : std::min(forced, 16);
    if (want > 1 && workspace_bytes >= prefill_split_bytes(p, want)) {
      p.splits = want;
      p.ws_o = (float*)workspace;
      p.ws_ml = p.ws_o + (size_t)B * T * Hq * want * D;
    }
  }
  hipStream_t s = (hipStream_t)stream;
  profile_begin(s);
  hipError_t e = launch_prefill(p, s);
  profile_end(s);
  return check_hip(e, "pa_prefill launch");
}

int pa_blocksparse_prefill(const void* q, const void* k, const void* v, void* out,
                           int B, int S, int Hq, int Hkv, int D,
                           int block, int local_blocks, int vert_stride,
                           float scale, int dtype, void* stream) {
  tl_error[0] = 0;
  if (B < 0 || S < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return fail_arg("pa_blocksparse_prefill: bad sizes");
  if (Hq % Hkv) return fail_arg("pa_blocksparse_prefill: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  if (dtype != PA_BF16) return fail_arg("pa_blocksparse_prefill: only bf16 is supported (dtype=%d)", dtype);
  if (block != 64) return fail_arg("pa_blocksparse_prefill: sparsity block must be 64 (got %d)", block);
  if (local_blocks < 1 || vert_stride < 1) return fail_arg("pa_blocksparse_prefill: local_blocks and vert_stride must be >= 1");
  if (B == 0 || S == 0) return 0;
  if ((long)B * S > 0x7fffffffL || (long)Hkv * D * 2 > 0x7fffffffL)
    return fail_arg("pa_blocksparse_prefill: B*S=%ld rows exceed 2^31", (long)B * S);
  if (!q || !k || !v || !out) return fail_arg("pa_blocksparse_prefill: null pointer argument");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out))
    return fail_arg("pa_blocksparse_prefill: q, k, v and out must be 16-byte aligned");
  PrefillParams p;
  memset(&p, 0, sizeof(p));
  p.q = q; p.k = k; p.v = v; p.out = out;
  p.B = B; p.T = S; p.S = S; p.Hq = Hq; p.Hkv = Hkv; p.D = D;
  p.sparse_local = local_blocks; p.sparse_stride = vert_stride;
  p.block_shift = -1;
  p.impl = g_prefill_impl.load();
  p.scale_log2e = scale * kLog2e;
  if (!prefill_supported(p)) return fail_arg("pa_blocksparse_prefill: unsupported shape (D=%d)", D);
  hipStream_t s = (hipStream_t)stream;
  profile_begin(s);
  hipError_t e = launch_prefill(p, s);
  profile_end(s);
  return check_hip(e, "pa_blocksparse_prefill launch");
}

int pa_kv_write(const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                float* k_scale, float* v_scale,
                const int32_t* block_tables, const int32_t* seq_lens, const int32_t* query_lens,
                int B, int T, int Hkv, int D, int block_size, int max_blocks_per_seq, int num_blocks,
                int kv_dtype, void* stream) {
  tl_error[0] = 0;
  if (B < 0 || T < 0 || Hkv <= 0 || D <= 0) return fail_arg("pa_kv_write: bad sizes");
  if (block_size <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0) return fail_arg("pa_kv_write: bad paging sizes");
  if (kv_dtype != PA_F32 && kv_dtype != PA_BF16 && kv_dtype != PA_FP8_E4M3FN)
    return fail_arg("pa_kv_write: unknown kv_dtype %d", kv_dtype);
  const int src_esz = kv_dtype == PA_F32 ? 4 : 2;
  if ((D * src_esz) % 16 != 0 || (kv_dtype == PA_FP8_E4M3FN && D % 8 != 0))
    return fail_arg("pa_kv_write: D=%d rows must be a multiple of 16 bytes", D);
  if ((long)max_blocks_per_seq * block_size > 0x7fffffffL) return fail_arg("pa_kv_write: table capacity exceeds 2^31 tokens");
  if (B == 0 || T == 0) return 0;
  if (B > 65535 || Hkv > 65535) return fail_arg("pa_kv_write: B and Hkv are limited to 65535 (grid dimensions)");
  if (!k_new || !v_new || !k_cache || !v_cache || !block_tables || !seq_lens || !query_lens)
    return fail_arg("pa_kv_write: null pointer argument");
  if (kv_dtype == PA_FP8_E4M3FN && (!k_scale || !v_scale)) return fail_arg("pa_kv_write: fp8 pools need k_scale and v_scale");
  if (!aligned16(k_new) || !aligned16(v_new) || !aligned16(k_cache) || !aligned16(v_cache))
    return fail_arg("pa_kv_write: k_new, v_new, k_cache and v_cache must be 16-byte aligned");
  KvWriteParams p;
  memset(&p, 0, sizeof(p));
  p.k_new = k_new; p.v_new = v_new; p.k_cache = k_cache; p.v_cache = v_cache;
  p.k_scale = k_scale; p.v_scale = v_scale;
  p.block_tables = block_tables; p.seq_lens = seq_lens; p.query_lens = query_lens;
  p.B = B; p.T = T; p.Hkv = Hkv; p.D = D; p.block_size = block_size; p.max_blocks = max_blocks_per_seq;
  p.num_blocks = num_blocks; p.kv_dtype = kv_dtype;
  hipStream_t s = (hipStream_t)stream;
  profile_begin(s);
  hipError_t e = launch_kv_write(p, s);
  profile_end(s);
  return check_hip(e, "pa_kv_write launch");
}

int pa_qk_norm_rope_kv_write(const void* xq, const void* xk, const void* xv, void* q_out,
                             const void* q_norm_weight, const void* k_norm_weight, float norm_eps,
                             const void* rope_cos, const void* rope_sin, int rope_max_pos,
                             void* k_cache, void* v_cache, float* k_scale, float* v_scale,
                             const int32_t* block_tables, const int32_t* seq_lens, const int32_t* query_lens,
                             int B, int T, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq,
                             int num_blocks, int kv_dtype, void* stream) {
  tl_error[0] = 0;
  if (B < 0 || T < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return fail_arg("pa_qk_norm_rope_kv_write: bad sizes");
  if (block_size <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0 || rope_max_pos <= 0)
    return fail_arg("pa_qk_norm_rope_kv_write: bad paging or table sizes");
  if (kv_dtype != PA_BF16 && kv_dtype != PA_FP8_E4M3FN)
    return fail_arg("pa_qk_norm_rope_kv_write: kv_dtype must be bf16 or fp8-e4m3fn (got %d)", kv_dtype);
  if (!kv_write_xform_supported(D)) return fail_arg("pa_qk_norm_rope_kv_write: head_dim %d must be 64, 128 or 256", D);
  if ((long)max_blocks_per_seq * block_size > 0x7fffffffL) return fail_arg("pa_qk_norm_rope_kv_write: table capacity exceeds 2^31 tokens");
  if (B == 0 || T == 0) return 0;
  if (B > 65535 || Hkv > 65535) return fail_arg("pa_qk_norm_rope_kv_write: B and Hkv are limited to 65535 (grid dimensions)");
  if (!xk || !xv || !rope_cos || !rope_sin || !k_cache || !v_cache || !block_tables || !seq_lens || !query_lens)
    return fail_arg("pa_qk_norm_rope_kv_write: null pointer argument");
  if ((xq == nullptr) != (q_out == nullptr))
    return fail_arg("pa_qk_norm_rope_kv_write: xq and q_out must both be given, or both be NULL (K and V only)");
  if (kv_dtype == PA_FP8_E4M3FN && (!k_scale || !v_scale)) return fail_arg("pa_qk_norm_rope_kv_write: fp8 pools need k_scale and v_scale");
  if (!aligned16(xq) || !aligned16(xk) || !aligned16(xv) || !aligned16(q_out) || !aligned16(k_cache) || !aligned16(v_cache))
    return fail_arg("pa_qk_norm_rope_kv_write: xq, xk, xv, q_out, k_cache and v_cache must be 16-byte aligned");
  if (!aligned16(rope_cos) || !aligned16(rope_sin) || !aligned16(q_norm_weight) || !aligned16(k_norm_weight))
    return fail_arg("pa_qk_norm_rope_kv_write: rope_cos, rope_sin and the norm weights must be 16-byte aligned");
  KvWriteParams p;
  memset(&p, 0, sizeof(p));
  p.k_new = xk; p.v_new = xv; p.k_cache = k_cache; p.v_cache = v_cache;
  p.k_scale = k_scale; p.v_scale = v_scale;
  p.block_tables = block_tables; p.seq_lens = seq_lens; p.query_lens = query_lens;
  p.B = B; p.T = T; p.Hkv = Hkv; p.D = D; p.block_size = block_size; p.max_blocks = max_blocks_per_seq;
  p.num_blocks = num_blocks; p.kv_dtype = kv_dtype;
  p.q_in = xq; p.q_out = q_out; p.Hq = Hq;
  p.q_norm_weight = (const uint16_t*)q_norm_weight; p.k_norm_weight = (const uint16_t*)k_norm_weight;
  p.rope_cos = (const uint16_t*)rope_cos; p.rope_sin = (const uint16_t*)rope_sin;
  p.norm_eps = norm_eps; p.rope_max_pos = rope_max_pos;
  hipStream_t s = (hipStream_t)stream;
  profile_begin(s);
  hipError_t e = launch_kv_write(p, s);
  profile_end(s);
  return check_hip(e, "pa_qk_norm_rope_kv_write launch");
}

size_t pa_o_proj_workspace_bytes(int M, int K, int N) {
  if (M <= 0 || K <= 0 || N <= 0 || K % 64 || N % 8) return 0;
  const int s = o_proj_splits(M, K, N);
  return s > 1 ? (size_t)s * M * N * sizeof(float) : 0;
}

int pa_o_proj(const void* x, const void* w, const void* bias, void* out, int M, int K, int N, int dtype, void* stream) {
  return pa_o_proj_ws(x, w, bias, out, nullptr, 0, M, K, N, dtype, stream);
}

int pa_o_proj_ws(const void* x, const void* w, const void* bias, void* out, void* workspace, size_t workspace_bytes,
                 int M, int K, int N, int dtype, void* stream) {
  tl_error[0] = 0;
  if (M < 0 || K <= 0 || N <= 0) return fail_arg("pa_o_proj: bad sizes M=%d K=%d N=%d", M, K, N);
  if (dtype != PA_BF16) return fail_arg("pa_o_proj: only bf16 is supported (dtype=%d)", dtype);
  if (K % 64) return fail_arg("pa_o_proj: K=%d (Hq * head_dim) must be a multiple of 64", K);
  if (N % 8) return fail_arg("pa_o_proj: N=%d must be a multiple of 8", N);
  if (M == 0) return 0;
  if ((long)N * 2 * 64 > 0xffffffffL || (long)K * 2 * 256 > 0xffffffffL)
    return fail_arg("pa_o_proj: row of %d (K) or %d (N) elements too long for 32-bit tile offsets", K, N);
  if (!x || !w || !out) return fail_arg("pa_o_proj: null pointer argument");
  if (!aligned16(x) || !aligned16(w) || !aligned16(out) || !aligned16(bias))
    return fail_arg("pa_o_proj: x, w, bias and out must be 16-byte aligned");
  OProjParams p;
  memset(&p, 0, sizeof(p));
  p.x = x; p.w = w; p.bias = bias; p.out = out; p.M = M; p.K = K; p.N = N;
  p.splits = 1;
  if (workspace) {
    if (!aligned16(workspace)) return fail_arg("pa_o_proj: workspace must be 16-byte aligned");
    // as many K ranges as the workspace holds, up to what the shape asks for; too small for two: unsplit
    const size_t per_split = (size_t)M * N * sizeof(float);
    int want = o_proj_splits(M, K, N);
    if ((size_t)want * per_split > workspace_bytes) want = (int)(workspace_bytes / per_split);
    if (want > 1) { p.splits = want; p.ws = (float*)workspace; }
  }
  hipStream_t s = (hipStream_t)stream;
  profile_begin(s);
  hipError_t e = launch_o_proj(p, s);
  profile_end(s);
  return check_hip(e, "pa_o_proj launch");
}

// ---- one decode step of an attention layer in one call -------------------------------------------
static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

size_t pa_decode_step_workspace_bytes(int B, int Hq, int Hkv, int D, int block_size, int max_seq_len, int partition_size,
                                      int N, int q_dtype, int kv_dtype) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || D <= 0 || block_size <= 0 || partition_size <= 0 || N < 0) return 0;
  const size_t dec = pa_decode_workspace_bytes_for(B, Hq, Hkv, D, block_size, max_seq_len, partition_size, q_dtype, kv_dtype);
  const size_t proj = N > 0 ? pa_o_proj_workspace_bytes(B, Hq * D, N) : 0;
  return align256(dec) + align256(proj) + align256((size_t)B * Hq * D * 4) + 256;
}

int pa_decode_step(const void* q, const pa_new_kv* new_kv, void* k_cache, void* v_cache, float* k_scale, float* v_scale,
                   const int32_t* block_tables, const int32_t* seq_lens, void* attn_out, const pa_out_proj* proj,
                   void* workspace, size_t workspace_bytes,
                   int B, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq, int num_blocks, int max_seq_len,
                   float scale, int partition_size, int q_dtype, int kv_dtype,
                   const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream) {
  tl_error[0] = 0;
  const char* who = "pa_decode_step";
  DecodePlan pl;
  if (int rc = plan_decode(who, pl, q, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, attn_out, proj == nullptr,
                           B, Hq, Hkv, D, block_size, max_blocks_per_seq, num_blocks, max_seq_len, scale, partition_size,
                           q_dtype, kv_dtype, sinks, sliding_window, q_transform))
    return rc;
  if (!new_kv) return fail_arg("%s: new_kv is required (pa_decode is the call without a cache update)", who);
  if (B == 0) return 0;
  if (!new_kv->xk || !new_kv->xv || !new_kv->query_lens) return fail_arg("%s: new_kv needs xk, xv and query_lens", who);
  if (!aligned16(new_kv->xk) || !aligned16(new_kv->xv) || !aligned16(new_kv->k_norm_weight))
    return fail_arg("%s: xk, xv and k_norm_weight must be 16-byte aligned", who);
  if (new_kv->k_norm_weight && !q_transform)
    return fail_arg("%s: k_norm_weight comes with q_transform (the norm and rotation are applied to Q and K alike)", who);
  const int K = Hq * D;
  int N = 0;
  if (proj) {
    N = proj->N;
    if (!proj->o_weight || !proj->out) return fail_arg("%s: out_proj needs o_weight and out", who);
    if (q_dtype != PA_BF16) return fail_arg("%s: the output projection is bf16 only", who);
    if (N <= 0 || N % 8) return fail_arg("%s: N=%d must be a positive multiple of 8", who, N);
    if (K % 64) return fail_arg("%s: Hq * head_dim = %d must be a multiple of 64", who, K);
    if ((long)N * 2 * 64 > 0xffffffffL || (long)K * 2 * 256 > 0xffffffffL)
      return fail_arg("%s: row of %d (K) or %d (N) elements too long for 32-bit tile offsets", who, K, N);
    if (!aligned16(proj->o_weight) || !aligned16(proj->o_bias) || !aligned16(proj->out))
      return fail_arg("%s: o_weight, o_bias and out must be 16-byte aligned", who);
  }
  if (!aligned16(workspace)) return fail_arg("%s: workspace must be 16-byte aligned", who);
  hipStream_t s = (hipStream_t)stream;
  DecodeParams& p = pl.p;
  const int fusion = g_step_fusion.load();

  // the cache update: on the decode launch where its kernel takes the row, else a launch of its own in front
  const bool fused_row = pl.kind == 2 && decode_new_row_supported(p, q_dtype, kv_dtype) && fusion != 1 && fusion != 3;
  if (fused_row) {
    p.new_k = new_kv->xk; p.new_v = new_kv->xv; p.new_lens = new_kv->query_lens;
    if (q_transform) {
      p.new_kt = p.qt;
      p.new_kt.norm_weight = (const uint16_t*)new_kv->k_norm_weight;
    }
  }
  if (!fused_row) {
    int rc;
    if (q_transform)
      rc = pa_qk_norm_rope_kv_write(nullptr, new_kv->xk, new_kv->xv, nullptr, nullptr, new_kv->k_norm_weight,
                                    q_transform->norm_eps, q_transform->rope_cos, q_transform->rope_sin,
                                    q_transform->rope_max_pos, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens,
                                    new_kv->query_lens, B, 1, Hq, Hkv, D, block_size, max_blocks_per_seq, num_blocks,
                                    kv_dtype, stream);
    else
      rc = pa_kv_write(new_kv->xk, new_kv->xv, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens,
                       new_kv->query_lens, B, 1, Hkv, D, block_size, max_blocks_per_seq, num_blocks, kv_dtype, stream);
    if (rc) return rc;
  }

  // workspace, from its end: the attention output when the caller wants none, the projection's K-range partials;
  // the decode launch gets what is in front of them
  char* ws = (char*)workspace;
  size_t avail = workspace ? workspace_bytes & ~(size_t)255 : 0;
  const size_t esz = q_dtype == PA_F32 ? 4 : 2;
  void* attn = attn_out;
  if (!attn) {
    const size_t need = align256((size_t)B * Hq * D * esz);
    if (avail < need) return fail_arg("%s: workspace of %zu bytes too small (pa_decode_step_workspace_bytes)", who, workspace_bytes);
    avail -= need;
    attn = ws + avail;
    p.out = attn;
  }
  int splits = 1;
  float* proj_ws = nullptr;
  if (proj) {
    const size_t per_split = (size_t)B * N * sizeof(float);
    int want = o_proj_splits(B, K, N);
    if (align256((size_t)want * per_split) > avail) want = (int)(avail / per_split);
    if (want > 1) {
      splits = want;
      avail -= align256((size_t)splits * per_split);
      proj_ws = (float*)(ws + avail);
    }
  }
  // the merge of the decode partitions on the projection's load of its rows, where both kernels are the small-call ones
  // (up to four partitions: the projection requests that many ahead of its weight tiles; with more, the merge's later
  // loads wait behind the tiles and the separate merge launch is faster: B = 8 at 4 K, eight partitions, 45.5 against 43.2 us)
  // (not under a sliding window: the projection's merge does not know where a window's partitions begin)
  const bool merge_on_load = proj && !attn_out && pl.kind == 2 && p.num_partitions > 1 && (p.num_partitions <= 4 || fusion == 3) && fusion != 1 && fusion != 2 &&
                             sliding_window == 0 &&
                             q_dtype == PA_BF16 && o_proj_takes_partials(B, K, D, splits, proj_ws != nullptr);
  if (int rc = run_decode(who, pl, ws, avail, merge_on_load, nullptr, s)) return rc;
  if (!proj) return 0;

  OProjParams o;
  memset(&o, 0, sizeof(o));
  o.w = proj->o_weight; o.bias = proj->o_bias; o.out = proj->out; o.M = B; o.K = K; o.N = N;
  o.splits = splits; o.ws = proj_ws;
  if (merge_on_load && p.num_partitions > 1) {
    o.part_o = p.ws_out; o.part_ml = p.ws_ml; o.part_seq_lens = seq_lens;
    o.part_np = p.num_partitions; o.part_size = p.partition_size; o.part_max_seq_len = p.max_seq_len; o.part_D = D;
    o.part_T = 1; o.part_n_rep = Hq / Hkv; o.part_sinks = sinks;
  } else {
    o.x = attn;
  }
  profile_begin(s);
  hipError_t e = launch_o_proj(o, s);
  profile_end(s);
  return check_hip(e, "pa_decode_step projection launch");
}

size_t pa_verify_step_workspace_bytes(int B, int T, int Hq, int D, int N) {
  if (B <= 0 || T <= 0 || Hq <= 0 || D <= 0 || N < 0 || (long)B * T > 0x7fffffffL) return 0;
  const size_t proj = N > 0 ? pa_o_proj_workspace_bytes(B * T, Hq * D, N) : 0;
  return align256(pa_verify_workspace_bytes(B, T, Hq, D)) + align256(proj) + align256((size_t)B * T * Hq * D * 2) + 256;
}

int pa_verify_step(const void* q, const pa_new_kv* new_kv, void* k_cache, void* v_cache, float* k_scale, float* v_scale,
                   const int32_t* block_tables, const int32_t* seq_lens, void* attn_out, const pa_out_proj* proj,
                   void* workspace, size_t workspace_bytes,
                   int B, int T, int Hq, int Hkv, int D, int block_size, int max_blocks_per_seq, int num_blocks,
                   int max_seq_len, float scale, int kv_dtype,
                   const float* sinks, int sliding_window, const pa_q_transform* q_transform, void* stream) {
  tl_error[0] = 0;
  const char* who = "pa_verify_step";
  if (!new_kv) return fail_arg("%s: new_kv is required (pa_verify is the call without a cache update)", who);
  if (B < 0 || T < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return fail_arg("%s: bad sizes", who);
  if (T > PA_VERIFY_MAX_TOKENS) return fail_arg("%s: T=%d exceeds %d query tokens per sequence", who, T, PA_VERIFY_MAX_TOKENS);
  if (new_kv->k_norm_weight && !q_transform)
    return fail_arg("%s: k_norm_weight comes with q_transform (the norm and rotation are applied to Q and K alike)", who);
  if (!attn_out && !proj) return fail_arg("%s: neither attn_out nor out_proj given", who);
  const int K = Hq * D;
  int N = 0;
  if (proj) {
    N = proj->N;
    if (!proj->o_weight || !proj->out) return fail_arg("%s: out_proj needs o_weight and out", who);
    if (N <= 0 || N % 8) return fail_arg("%s: N=%d must be a positive multiple of 8", who, N);
    if (K % 64) return fail_arg("%s: Hq * head_dim = %d must be a multiple of 64", who, K);
    if ((long)N * 2 * 64 > 0xffffffffL || (long)K * 2 * 256 > 0xffffffffL)
      return fail_arg("%s: row of %d (K) or %d (N) elements too long for 32-bit tile offsets", who, K, N);
    if (!aligned16(proj->o_weight) || !aligned16(proj->o_bias) || !aligned16(proj->out))
      return fail_arg("%s: o_weight, o_bias and out must be 16-byte aligned", who);
  }
  if (!aligned16(workspace) || !aligned16(attn_out)) return fail_arg("%s: workspace and attn_out must be 16-byte aligned", who);
  int rc;
  if (!new_kv->xk || !new_kv->xv || !new_kv->query_lens) {
    if (B > 0 && T > 0) return fail_arg("%s: new_kv needs xk, xv and query_lens", who);
  }
  if (B == 0 || T == 0) return 0;
  if (Hq % Hkv) return fail_arg("%s: Hq=%d is not a multiple of Hkv=%d", who, Hq, Hkv);
  if (kv_dtype != PA_BF16 && kv_dtype != PA_FP8_E4M3FN) return fail_arg("%s: kv_dtype must be bf16 or fp8-e4m3fn", who);
  if (!q) return fail_arg("%s: null pointer argument", who);
  const long M = (long)B * T;
  hipStream_t s = (hipStream_t)stream;
  char* ws = (char*)workspace;
  size_t avail = workspace ? workspace_bytes & ~(size_t)255 : 0;
  void* attn = attn_out;
  if (!attn) {
    const size_t need = align256((size_t)M * K * 2);
    if (avail < need) return fail_arg("%s: workspace of %zu bytes too small (pa_verify_step_workspace_bytes)", who, workspace_bytes);
    avail -= need;
    attn = ws + avail;
  }
  int splits = 1;
  float* proj_ws = nullptr;
  if (proj) {
    const size_t per_split = (size_t)M * N * sizeof(float);
    int want = o_proj_splits((int)M, K, N);
    if (align256((size_t)want * per_split) > avail) want = (int)(avail / per_split);
    if (want > 1) {
      splits = want;
      avail -= align256((size_t)splits * per_split);
      proj_ws = (float*)(ws + avail);
    }
  }
  // the cache update (on the attention launch, or a launch with argument checks of its own in front of it), the
  // attention, the projection
  const int fusion = g_step_fusion.load();
  VerifyPartials vp;
  memset(&vp, 0, sizeof(vp));
  vp.new_kv = new_kv; vp.k_cache_w = k_cache; vp.v_cache_w = v_cache; vp.k_scale_w = k_scale; vp.v_scale_w = v_scale;
  vp.fuse_rows = fusion != 1 && fusion != 3;
  vp.want = proj && !attn_out && fusion != 1 && fusion != 2 && sliding_window == 0 &&
            o_proj_takes_partials((int)M, K, D, splits, proj_ws != nullptr);
  rc = verify_launch(who, q, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, new_kv->query_lens, attn, ws, avail,
                     B, T, 0, T, Hq, Hkv, D, block_size, max_blocks_per_seq, num_blocks, max_seq_len, scale, kv_dtype, sinks,
                     sliding_window, q_transform, s, &vp);
  if (rc || !proj) return rc;
  if (vp.left && vp.f.num_partitions > 4) {
    // the projection requests up to four partitions ahead of its weight tiles; more are merged by the launch after all
    hipError_t e = launch_decode_reduce(vp.f, PA_BF16, s);
    if (e != hipSuccess) return check_hip(e, "verify merge launch");
    vp.left = false;
  }
  OProjParams o;
  memset(&o, 0, sizeof(o));
  o.w = proj->o_weight; o.bias = proj->o_bias; o.out = proj->out; o.M = (int)M; o.K = K; o.N = N;
  o.splits = splits; o.ws = proj_ws;
  if (vp.left) {
    o.part_o = vp.f.ws_out; o.part_ml = vp.f.ws_ml; o.part_seq_lens = seq_lens; o.part_query_lens = new_kv->query_lens;
    o.part_np = vp.f.num_partitions; o.part_size = vp.f.partition_size; o.part_max_seq_len = vp.f.max_seq_len; o.part_D = D;
    o.part_T = T; o.part_n_rep = Hq / Hkv; o.part_sinks = sinks;
  } else {
    o.x = attn;
  }
  profile_begin(s);
  hipError_t e = launch_o_proj(o, s);
  profile_end(s);
  return check_hip(e, "pa_verify_step projection launch");
}

int pa_gather_kv(const void* cache, const int32_t* block_tables, const int32_t* seq_lens,
                 void* out, int B, int Hkv, int D, int block_size,
                 int max_blocks_per_seq, int num_blocks, int max_seq_len,
                 int elem_bytes, void* stream) {
  tl_error[0] = 0;
  if (B < 0 || Hkv <= 0 || D <= 0 || block_size <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0 ||
      max_seq_len < 0 || elem_bytes <= 0)
    return fail_arg("pa_gather_kv: bad sizes");
  if ((long)max_seq_len > (long)max_blocks_per_seq * block_size)
    return fail_arg("pa_gather_kv: max_seq_len=%d exceeds table capacity %ld", max_seq_len,
                    (long)max_blocks_per_seq * block_size);
  if (B == 0 || max_seq_len == 0) return 0;
  if (!cache || !block_tables || !seq_lens || !out) return fail_arg("pa_gather_kv: null pointer argument");
  if (B > 65535) return fail_arg("pa_gather_kv: B too large");
  hipError_t e = launch_gather(cache, block_tables, seq_lens, out, B, Hkv * D * elem_bytes, block_size,
                               max_blocks_per_seq, num_blocks, max_seq_len, (hipStream_t)stream);
  return check_hip(e, "pa_gather_kv launch");
}

}  // extern "C"
