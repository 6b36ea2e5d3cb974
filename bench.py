#!/usr/bin/env python3
"""Benchmark of the paged attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2|5|3|4|6|...]

A step is one pass of the op over one batch of synthetic input that is already
resident in HBM.  Prints ONE JSON line.  Without --config the line is config 2
(Llama-3-8B-shape paged decode, bf16, batch 64, context U[512, 8192], block 32) and
carries, under "configs", one record each for config 3 (paged chunked prefill),
config 4 (blocksparse prefill) and config 5 (fp8-KV long-context decode), timed in
the same run with the same protocol: both halves of the headline metric and every
benchmark-sized configuration, plus "o_proj", the output projection behind config 3's
attention, and under "layer_steps" the microseconds per layer of the small-batch decode and
verify steps (configs 13, 15, 16).  --config N prints that configuration alone (6-17: the kernels and steps around the
attention call; their docstrings say what each one is).

value      whole-step throughput: algorithmic HBM bytes / step time for the decode
           configs (GB/s), attention FLOPs / step time for the prefill configs
           (TFLOP/s); the step includes every kernel the op launches.
roofline   the dominant kernel alone, timed with HIP events on its launch stream
           inside the library (pa_profile_*), over the K launches right behind the K the step time is
           taken from ("ms_per_step_with_events" is that second block's own step time).
warm-up    --warmup is a minimum; blocks of K launches follow until two consecutive blocks agree within
           2 % (the clock ramps for tens of launches after the allocation phase); the last block is the
           measurement ("warmup_effective_steps", "warmup_converged" say what happened).
cpu_baseline  the NumPy oracle on a bounded sample of the same workload, on this
           box's host cores: 1 warm-up + 3 repetitions, median (reported, not a target).
parity     the device result against the oracle's on that same sample: max abs error,
           the tolerance of the configuration, pass / fail.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

_NO_CPU = False
_CONST_DATA = False         # --const-data: every Q / K / V element the same value (a power probe, see main)
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published


def _collect_kernel_ms(lib, n):
    buf = (ctypes.c_float * max(n, 1))()
    got = lib.pa_profile_collect(buf, n)
    return [buf[i] for i in range(got)]


def _time_steps(step, steps, warmup):
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


WARMUP_AGREE = 0.02      # two consecutive blocks of `steps` launches must agree within this
WARMUP_CAP_S = 1.5       # ... or the warm-up ends after this long (and says so)


def _measure(step, steps, warmup, lib):
    """Step time and the dominant kernel's time from two adjacent blocks of `steps` launches in the steady state.

    `warmup` is a minimum: after it, blocks of `steps` launches are timed until two consecutive blocks agree
    within WARMUP_AGREE (the shader clock keeps ramping for some tens of launches after an allocation phase,
    however few warm-up steps the command line asked for), for at most WARMUP_CAP_S.  The block that agreed
    with its predecessor gives the step time (wall clock between two synchronisations, nothing else on the
    stream).  The block right behind it runs with the library's HIP events around the dominant kernel and gives
    the kernel time; its own wall time is reported too (`ms_per_step_with_events`: two event records per step
    cost a few microseconds, which is why the step time is not taken from that block), so that step >= kernel
    can be read off one and the same block.  Returns (seconds per step, kernel milliseconds per launch, info)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()

    def block():
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    prev, blocks, t_begin, converged = None, 0, time.perf_counter(), False
    while True:
        sec = block()
        blocks += 1
        if prev is not None and abs(sec - prev) <= WARMUP_AGREE * min(sec, prev):
            converged = True
            break
        if time.perf_counter() - t_begin > WARMUP_CAP_S and blocks >= 2:
            break
        prev = sec
    lib.pa_profile_enable(1)
    step()                                   # creates the events the timed block reuses
    torch.cuda.synchronize()
    _collect_kernel_ms(lib, 0)
    sec_ev = block()
    kms = _collect_kernel_ms(lib, 4 * steps)
    # what the same pair of events reads around a kernel that does nothing, interleaved with real steps so that the
    # device is in the state of the timed block: the share of `kms` that is not kernel time (a kernel trace, which
    # stamps first wave to last, reads that much less than the events)
    stream = torch.cuda.current_stream().cuda_stream
    empty = []
    for _ in range(10):
        lib.pa_profile_enable(0)
        step()
        lib.pa_profile_enable(1)
        lib.pa_profile_empty_launch(stream)
        torch.cuda.synchronize()
        empty += _collect_kernel_ms(lib, 4)
    lib.pa_profile_enable(0)
    info = {"warmup_effective_steps": warmup + (blocks - 1) * steps, "warmup_converged": converged,
            "ms_per_step_with_events": round(sec_ev * 1e3, 5),
            "event_pair_around_empty_kernel_ms": round(float(np.median(empty)), 5) if empty else None}
    return sec, kms, info


def _host_info():
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count()
    return cores


def _median3(fn):
    """1 warm-up + 3 timed repetitions of fn(); returns (median seconds, last result)."""
    res = fn()
    times = []
    for _ in range(3):
        t = time.perf_counter()
        res = fn()
        times.append(time.perf_counter() - t)
    return float(np.median(times)), res


def _parity(got, want, tol):
    err = float(np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)).max()) if np.size(want) else 0.0
    ok = bool(np.isfinite(np.asarray(got)).all() and err <= tol)
    # the bar is the plain absolute one: no allowance for large outputs is applied here, so every element counts
    over = int((np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)) > tol).sum()) if np.size(want) else 0
    return {"max_abs_err": round(err, 6), "tol": tol, "pass": ok, "elements_checked": int(np.size(want)),
            "elements_above_tol": over, "widened_bar_used": False}


def _cpu_decode_baseline(w, got, tol, budget_s=16.0):
    """Oracle decode on the first n sequences (n sized so that the 4 runs stay near the budget);
    returns (cpu_baseline, parity of the device rows `got` [B, Hq, D] on those sequences)."""
    from oracle import paged_attention_oracle as O
    from nkipy_amd.workloads import storage_bits
    B = w.q.shape[0]
    kc, vc = storage_bits(w.k_cache), storage_bits(w.v_cache)
    q = storage_bits(w.q)
    tables = w.block_tables.cpu().numpy()
    ks = w.k_scale.cpu().numpy() if w.k_scale is not None else None
    vs = w.v_scale.cpu().numpy() if w.v_scale is not None else None

    def run(n):
        return O.paged_decode(q[:n], kc, vc, tables[:n], w.ctx[:n].astype(np.int32), w.scale,
                              k_scale=ks, v_scale=vs, q_dtype="bf16")

    probe = min(B, 2)
    t0 = time.perf_counter()
    run(probe)
    per_seq = (time.perf_counter() - t0) / probe
    n = int(max(probe, min(B, budget_s / 4.0 / max(per_seq, 1e-6))))
    t, want = _median3(lambda: run(n))
    nb, bs, hkv, d = w.k_cache.shape
    bytes_n = int(w.ctx[:n].sum()) * 2 * hkv * d * w.k_cache.element_size()
    cpu = {"value": round(bytes_n / t / 1e9, 4), "unit": "GB/s", "cores": _host_info(), "kind": "port",
           "tok_per_s": round(n / t, 2),
           "sample": f"NumPy oracle, first {n} of {B} sequences of the same workload, 1 warm-up + 3 runs, median "
                     f"{t:.3f} s, numpy {np.__version__} default BLAS threading"}
    return cpu, _parity(got.float().cpu().numpy()[:n], want, tol)


def _cpu_prefill_baseline(run_fn, flops, desc):
    """run_fn() -> oracle result; flops = attention FLOPs of that sample."""
    t, want = _median3(run_fn)
    return {"value": round(flops / t / 1e12, 5), "unit": "TFLOP/s", "cores": _host_info(), "kind": "port",
            "sample": f"{desc}, 1 warm-up + 3 runs, median {t:.2f} s, numpy {np.__version__} default BLAS threading"}, want


# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this file on the seeded workloads (FETCH_SIZE x 2.00, WRITE_SIZE x 1.00: the factors a plain copy
# of known size shows); the summaries with the commands are under profiles/.  Not re-measured at run time.
MEASURED_TRAFFIC_BYTES = {
    2: {"bytes": 1_099_100_000, "source": "profiles/decode_balanced_kernel_C2.md"},
    3: {"bytes": 380_800_000, "source": "profiles/prefill_async_kernel_C3.md"},
    4: {"bytes": 709_500_000, "source": "profiles/prefill_async_kernel_C4.md"},
    5: {"bytes": 2_404_500_000, "source": "profiles/decode_balanced_kernel_C5.md"},
    8: {"bytes": 1_125_700_000, "source": "profiles/decode_balanced_kernel_verify_T4.md"},
}


def _traffic(cfg):
    t = MEASURED_TRAFFIC_BYTES.get(cfg)
    return (t["bytes"], t["source"]) if t else (None, None)


def bench_decode(cfg, steps, warmup, lib, pa, W):
    w = W.make_decode(cfg)
    out = torch.empty_like(w.q)

    def step():
        pa.decode(w.q, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.scale,
                  k_scale=w.k_scale, v_scale=w.v_scale, partition_size=w.partition_size,
                  max_seq_len=w.max_seq_len, out=out)

    sec, kms, winfo = _measure(step, steps, warmup, lib)
    kavg = float(np.mean(kms)) if kms else float("nan")
    ab = w.algorithmic_bytes()
    B, Hq, D = w.q.shape
    nb, bs, hkv, _ = w.k_cache.shape
    dtype = "fp8-e4m3 KV / bf16 q, fp32 accumulate" if cfg == 5 else "bf16, fp32 accumulate"
    res = {
        "metric": "decode attn HBM GB/s (% peak) + tok/s",
        "value": round(ab / sec / 1e9, 2), "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * ab / sec / 1e9 / HBM_PEAK_GBS, 2),
        "tok_per_s": round(B / sec, 1),
        "ms_per_step": round(sec * 1e3, 5), **winfo,
        "dtype": dtype,
        "config": {"workload": f"C{cfg} paged decode: B={B}, Hq={Hq}, Hkv={hkv}, D={D}, block_size={bs}, "
                               f"ctx sum={int(w.ctx.sum())} (min {int(w.ctx.min())}, max {int(w.ctx.max())}), "
                               f"pool={nb} blocks, split-K by the balanced tile schedule (equal chunks of the "
                               f"flattened 32-token tile stream, one per resident wave group; partition_size="
                               f"{w.partition_size} is passed but sizes only the fixed-partition kernels)",
                   "algorithmic_bytes": ab},
        "roofline": {"bound": "hbm", "achieved": round(ab / (kavg * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(ab / (kavg * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": _traffic(cfg)[0], "traffic_source": _traffic(cfg)[1],
                     "kernel": "decode_balanced_kernel" + (" behind decode_tile_prefix_kernel" if B > 512 else ""),
                     "kernel_avg_ms": round(kavg, 5),
                     "launches_timed": len(kms)},
    }
    if _NO_CPU:
        res["cpu_baseline"] = res["parity"] = None
    else:
        torch.cuda.synchronize()
        res["cpu_baseline"], res["parity"] = _cpu_decode_baseline(w, out, 5e-2 if cfg == 5 else 2e-2)
    return res


def bench_verify(steps, warmup, lib, pa, W, T=4):
    """Speculative verify on the pool and tables of the C2 decode workload: the last T tokens of every
    context are the queries (K = T - 1 drafts plus the last accepted token)."""
    from oracle import paged_attention_oracle as O
    from nkipy_amd.workloads import storage_bits as dev_bits
    w = W.make_decode(2)
    B, Hq, D = w.q.shape
    gen = torch.Generator(device=w.q.device)
    gen.manual_seed(1008)
    q = torch.randn((B, T, Hq, D), generator=gen, device=w.q.device).to(torch.bfloat16)
    qlens = torch.full((B,), T, dtype=torch.int32, device=w.q.device)
    out = torch.empty_like(q)

    def step():
        pa.verify(q, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, qlens, w.scale, out=out)

    sec, kms, winfo = _measure(step, steps, warmup, lib)
    kavg = float(np.mean(kms)) if kms else float("nan")
    ab = w.algorithmic_bytes() + 2 * B * (T - 1) * Hq * D * 2 + 4 * B     # more q / out rows, query_lens
    nb, bs, hkv, _ = w.k_cache.shape
    res = {
        "metric": "verify attn HBM GB/s (% peak) + tok/s",
        "value": round(ab / sec / 1e9, 2), "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * ab / sec / 1e9 / HBM_PEAK_GBS, 2),
        "tok_per_s": round(B * T / sec, 1),
        "ms_per_step": round(sec * 1e3, 5), **winfo,
        "dtype": "bf16, fp32 accumulate",
        "config": {"workload": f"speculative verify on the C2 pool: B={B}, T={T} query tokens per sequence, Hq={Hq}, "
                               f"Hkv={hkv}, D={D}, block_size={bs}, ctx sum={int(w.ctx.sum())}",
                   "algorithmic_bytes": ab},
        "roofline": {"bound": "hbm", "achieved": round(ab / (kavg * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(ab / (kavg * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": _traffic(8)[0], "traffic_source": _traffic(8)[1],
                     "kernel": "decode_balanced_kernel (multi-token rows)",
                     "kernel_avg_ms": round(kavg, 5), "launches_timed": len(kms)},
    }
    res["cpu_baseline"] = res["parity"] = None
    if not _NO_CPU:
        n = 4
        kc, vc = dev_bits(w.k_cache), dev_bits(w.v_cache)
        dt, want = _median3(lambda: O.paged_prefill(
            dev_bits(q)[:n], kc, vc, w.block_tables.cpu().numpy()[:n], w.ctx[:n].astype(np.int32),
            np.full(n, T, np.int32), w.scale, q_dtype="bf16"))
        bytes_n = int(w.ctx[:n].sum()) * 2 * hkv * D * 2
        res["cpu_baseline"] = {"value": round(bytes_n / dt / 1e9, 4), "unit": "GB/s", "cores": _host_info(), "kind": "port",
                               "tok_per_s": round(n * T / dt, 2),
                               "sample": f"NumPy oracle, first {n} of {B} sequences of the same workload, 1 warm-up + 3 runs, "
                                         f"median {dt:.2f} s, numpy {np.__version__} default BLAS threading"}
        res["parity"] = _parity(out.float().cpu().numpy()[:n], want, 2e-2)
    return res


_bench_lib = None


def _load_bench_lib():
    """libpa_bench.so: the matrix-core ceiling probe, a library of its own beside the product library
    (int pa_bench_probe_mfma(const void* operands, void* sink, int blocks, int iters, float* ms, void* stream))."""
    global _bench_lib
    if _bench_lib is None:
        from nkipy_amd.build import BENCH_LIB_PATH
        if not os.path.exists(BENCH_LIB_PATH):
            raise RuntimeError(f"{BENCH_LIB_PATH} not found: build it with `python -m nkipy_amd.build`")
        _bench_lib = ctypes.CDLL(BENCH_LIB_PATH)
        _bench_lib.pa_bench_probe_mfma.restype = ctypes.c_int
        _bench_lib.pa_bench_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                                   ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
        _bench_lib.pa_bench_probe_tile_loop.restype = ctypes.c_int
        _bench_lib.pa_bench_probe_tile_loop.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                                        ctypes.c_int, ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    return _bench_lib


def _mfma_ceiling(lib, sample):
    """Matrix-core rate of a registers-only MFMA loop fed with operands drawn from `sample`
    (a bf16 device tensor of the benchmark's own inputs): what the power-limited chip
    sustains on this data distribution, to read the nominal-peak fraction against."""
    probe = _load_bench_lib()
    blocks, iters = 256, 4000
    need = blocks * 65536 // 2
    flat = sample.reshape(-1)
    ops = flat[:need].contiguous() if flat.numel() >= need else flat.repeat((need + flat.numel() - 1) // flat.numel())[:need].contiguous()
    sink = torch.empty(blocks * 512, dtype=torch.float32, device=ops.device)
    ms = ctypes.c_float(0.0)
    best = 0.0
    for _ in range(3):
        rc = probe.pa_bench_probe_mfma(ops.data_ptr(), sink.data_ptr(), blocks, iters, ctypes.byref(ms),
                                       torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(f"pa_bench_probe_mfma failed ({rc})")
        best = max(best, blocks * 8 * iters * 16 * 32768.0 / (ms.value * 1e-3) / 1e12)
    return round(best, 1)


def bench_tile_loop_probe(steps, warmup):
    """config 14 (a probe, not a benchmark of the product): the key loop of the tiled prefill kernel as a stand-alone
    loop, in the shipped structure (8 waves x 32 query rows, two waves per SIMD) and as 4 waves x 64 rows with one wave
    per SIMD, the whole register file and a software pipeline over 32-key x 32-row units; the same 256 rows x 64 keys
    per workgroup and tile either way.  On N(0,1) and on constant operands: time per tile, shader cycles per tile
    (2048 = matrix pipeline never idle) and the clock the chip ran at."""
    probe = _load_bench_lib()
    blocks, iters = 256, 2000
    nbytes = 2 * 8 * 6144 * 2048 + (1 << 20)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1014)
    src = torch.randn(nbytes // 2, generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    sink = torch.empty(blocks * 512, dtype=torch.float32, device="cuda")
    stamps = torch.zeros(blocks * 2, dtype=torch.int64, device="cuda")
    ms = ctypes.c_float(0.0)
    forms = {0: "8 waves x 32 rows, two waves per SIMD (shipped structure)", 1: "4 waves x 64 rows, one wave per SIMD, pipelined units"}
    out = {}
    for data in ("N(0,1)", "constant"):
        if data == "constant":
            src.fill_(0.011)
        for form, name in forms.items():
            best = None
            for _ in range(max(3, warmup // 10) + max(3, steps // 10)):
                rc = probe.pa_bench_probe_tile_loop(form, src.data_ptr(), sink.data_ptr(), stamps.data_ptr(), blocks, iters,
                                                    ctypes.byref(ms), torch.cuda.current_stream().cuda_stream)
                if rc != 0:
                    raise RuntimeError(f"pa_bench_probe_tile_loop failed ({rc})")
                st = stamps.cpu().numpy().reshape(blocks, 2).astype(np.float64)
                rec = {"ms": round(ms.value, 4), "ns_per_tile": round(ms.value * 1e6 / iters, 1),
                       "tflops": round(blocks * iters * 256 * 32768.0 / (ms.value * 1e-3) / 1e12, 1),
                       "shader_cycles_per_tile": round(float(st[:, 0].mean()) / iters, 1),
                       "clock_mhz": round(float((st[:, 0] / (st[:, 1] * 10.0)).mean()) * 1000.0, 1)}
                rec["matrix_pipe_busy"] = round(2048.0 / rec["shader_cycles_per_tile"], 4)
                if best is None or rec["ms"] < best["ms"]:
                    best = rec
            out[f"{data}: {name}"] = best
    ref = out["N(0,1): " + forms[0]]
    return {
        "metric": "tile-loop probe of the prefill key loop, TFLOP/s (shipped structure, N(0,1) operands)",
        "value": ref["tflops"], "unit": "TFLOP/s", "ms_per_step": ref["ms"], "dtype": "bf16, fp32 accumulate",
        "config": {"workload": f"stand-alone key loop: {blocks} workgroups x {iters} tiles of 256 query rows x 64 keys, head dim 128; "
                               "no masks, tables or lengths"},
        "roofline": {"bound": "mfma", "achieved": ref["tflops"], "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(ref["tflops"] / BF16_PEAK_TFLOPS, 4), "traffic": None, "kernel": "tile_loop_32rows_kernel"},
        "forms": out, "cpu_baseline": None,
    }


def bench_prefill(steps, warmup, lib, pa, W, fp8=False, gpt_oss=False):
    """config 3; with fp8=True the same workload over the pool quantised to e4m3 with per-(block, kv head) scales;
    with gpt_oss=True the same tokens and tables at that model's attention shape (64 q heads and 8 kv heads of 64,
    per-head sinks; examples/models/gpt_oss/kernels/attention.py:117-148)."""
    from oracle import paged_attention_oracle as O
    from nkipy_amd.workloads import storage_bits as dev_bits
    w = W.make_prefill(heads=(64, 8), head_dim=64, name="C3 tokens, gpt-oss heads") if gpt_oss else W.make_prefill()
    sinks = torch.linspace(-1.0, 1.0, w.q.shape[2], device="cuda") if gpt_oss else None
    out = torch.empty_like(w.q)
    if _CONST_DATA:
        for t in (w.q, w.k_cache, w.v_cache):
            t.fill_(0.011)
    kc, vc, ks, vs = w.k_cache, w.v_cache, None, None
    if fp8:
        kc, ks = W.quantize_pool_fp8(w.k_cache)
        vc, vs = W.quantize_pool_fp8(w.v_cache)

    def step():
        pa.prefill(w.q, kc, vc, w.block_tables, w.seq_lens, w.query_lens, w.scale, out=out, k_scale=ks, v_scale=vs,
                   sinks=sinks)

    sec, kms, winfo = _measure(step, steps, warmup, lib)
    kavg = float(np.mean(kms))
    fl = w.flops()
    B, T, Hq, D = w.q.shape

    heads, seq = list(range(0, w.q.shape[2], 2)), 7        # every other q head: two per kv group at 4:1
    host = None

    def cpu():
        nonlocal host
        if host is None:
            host = (dev_bits(w.q), dev_bits(kc), dev_bits(vc), w.block_tables.cpu().numpy(), w.seq_lens.cpu().numpy(),
                    w.query_lens.cpu().numpy(), None if ks is None else ks.cpu().numpy(),
                    None if vs is None else vs.cpu().numpy(), None if sinks is None else sinks.cpu().numpy())
        return O.paged_prefill(host[0], host[1], host[2], host[3], host[4], host[5], w.scale, seqs=[seq], heads=heads,
                               k_scale=host[6], v_scale=host[7], sinks=host[8])

    cpu_flops = 4 * D * len(heads) * (T * int(w.prefix[seq]) + T * (T + 1) // 2)

    res = {
        "metric": "prefill attn TFLOP/s (% MFMA peak)",
        "value": round(fl / sec / 1e12, 2), "unit": "TFLOP/s",
        "pct_of_bf16_peak": round(100.0 * fl / sec / 1e12 / BF16_PEAK_TFLOPS, 2),
        "ms_per_step": round(sec * 1e3, 5), **winfo,
        "dtype": "fp8-e4m3 KV expanded to bf16 in LDS / bf16 q, fp32 accumulate" if fp8 else "bf16, fp32 accumulate",
        "config": {"workload": f"{'gpt-oss-shape' if gpt_oss else 'C3'} paged chunked prefill{' over the fp8-quantised pool' if fp8 else ''}"
                               f"{' with sinks' if gpt_oss else ''}: B={B}, T={T}, "
                               f"Hq={Hq}, Hkv={w.k_cache.shape[2]}, "
                               f"D={D}, block_size={w.k_cache.shape[1]}, prefix={w.prefix.tolist()}",
                   "flops": fl},
        "roofline": {"bound": "mfma", "achieved": round(fl / (kavg * 1e-3) / 1e12, 2), "peak": BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(fl / (kavg * 1e-3) / 1e12 / BF16_PEAK_TFLOPS, 4),
                     "traffic": None if fp8 or gpt_oss else _traffic(3)[0],
                     "traffic_source": None if fp8 or gpt_oss else _traffic(3)[1],
                     "kernel": "prefill_async_kernel", "kernel_avg_ms": round(kavg, 5),
                     "launches_timed": len(kms),
                     "mfma_only_loop_same_data": _mfma_ceiling(lib, w.k_cache)},
    }
    res["cpu_baseline"] = res["parity"] = None
    if not _NO_CPU:
        torch.cuda.synchronize()
        res["cpu_baseline"], want = _cpu_prefill_baseline(cpu, cpu_flops, f"NumPy oracle, sequence {seq}, every other q head ({len(heads)} of {Hq}) of the same workload")
        res["parity"] = _parity(out[seq][:, heads].float().cpu().numpy(), want[seq][:, heads], 5e-2 if fp8 else 2e-2)
    return res


def bench_blocksparse(steps, warmup, lib, pa, W):
    from oracle import paged_attention_oracle as O
    from nkipy_amd.workloads import storage_bits as dev_bits
    w = W.make_blocksparse()
    out = torch.empty_like(w.q)

    def step():
        pa.blocksparse_prefill(w.q, w.k, w.v, w.scale, block=w.block, local_blocks=w.local_blocks,
                               vert_stride=w.vert_stride, out=out)

    sec, kms, winfo = _measure(step, steps, warmup, lib)
    kavg = float(np.mean(kms))
    fl = w.flops()
    B, S, H, D = w.q.shape

    items = [(1, 5), (0, 8), (1, 19), (0, 30), (1, 2), (0, 15)]     # six (batch, head) pairs, six phase offsets
    host = None

    def cpu():
        nonlocal host
        if host is None:     # one head of one batch entry per slice: what the oracle touches
            host = [tuple(dev_bits(x[b_:b_ + 1, :, h_:h_ + 1].contiguous()) for x in (w.q, w.k, w.v)) for b_, h_ in items]
        # a slice holds one head; head_ids keeps its phase offset (head number % vert_stride)
        return np.stack([O.blocksparse_prefill(hq_, hk_, hv_, w.scale, block=w.block, local_blocks=w.local_blocks,
                                               vert_stride=w.vert_stride, head_ids=[h_])[0, :, 0]
                         for (hq_, hk_, hv_), (_, h_) in zip(host, items)])

    def item_flops():
        nb, total = S // w.block, 0
        for _, h_ in items:
            m = O.blocksparse_block_mask(nb, h_, w.local_blocks, w.vert_stride)
            n_diag = int(np.trace(m))
            total += 4 * D * ((int(m.sum()) - n_diag) * w.block * w.block + n_diag * w.block * (w.block + 1) // 2)
        return total

    res = {
        "metric": "prefill attn TFLOP/s (% MFMA peak)",
        "value": round(fl / sec / 1e12, 2), "unit": "TFLOP/s",
        "pct_of_bf16_peak": round(100.0 * fl / sec / 1e12 / BF16_PEAK_TFLOPS, 2),
        "ms_per_step": round(sec * 1e3, 5), **winfo, "dtype": "bf16, fp32 accumulate",
        "config": {"workload": f"C4 blocksparse prefill: B={B}, S={S}, H={H}, D={D}, block={w.block}, "
                               f"local={w.local_blocks}, vert_stride={w.vert_stride}", "flops": fl},
        "roofline": {"bound": "mfma", "achieved": round(fl / (kavg * 1e-3) / 1e12, 2), "peak": BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(fl / (kavg * 1e-3) / 1e12 / BF16_PEAK_TFLOPS, 4),
                     "traffic": _traffic(4)[0], "traffic_source": _traffic(4)[1],
                     "kernel": "prefill_async_kernel", "kernel_avg_ms": round(kavg, 5),
                     "launches_timed": len(kms),
                     "mfma_only_loop_same_data": _mfma_ceiling(lib, w.k)},
    }
    res["cpu_baseline"] = res["parity"] = None
    if not _NO_CPU:
        torch.cuda.synchronize()
        res["cpu_baseline"], want = _cpu_prefill_baseline(
            cpu, item_flops(), f"NumPy oracle (dense masked scores), (batch, head) pairs {items} of the same workload; "
                               "FLOPs counted as the sparse ones")
        res["parity"] = _parity(np.stack([out[b_][:, h_].float().cpu().numpy() for b_, h_ in items]), want, 2e-2)
    return res


def bench_o_proj(steps, warmup, lib, pa, W, M=None):
    """config 12: the output projection behind config 3's attention (examples/models/qwen3/kernels/
    attention.py:143-147): out [B * T, hidden] = attention output [B * T, Hq * D] @ o_weight [Hq * D, hidden],
    Llama-3-8B / Qwen3-8B sizes (32 heads of 128, hidden 4096), N(0,1) activations, N(0, 1/K) weights."""
    from oracle import paged_attention_oracle as O
    from nkipy_amd.workloads import storage_bits as dev_bits
    B, T, Hq, D, N = 8, 2048, 32, 128, 4096
    K = Hq * D
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1012)
    x = torch.randn((B, T, Hq, D), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn((K, N), generator=gen, device="cuda", dtype=torch.float32) / K ** 0.5).to(torch.bfloat16)
    out = torch.empty((B, T, N), dtype=torch.bfloat16, device="cuda")
    if _CONST_DATA:
        x.fill_(0.011)
        w.fill_(0.011)

    def step():
        pa.o_proj(x, w, out=out)

    sec, kms, winfo = _measure(step, steps, warmup, lib)
    kavg = float(np.mean(kms))
    fl = 2 * B * T * K * N
    res = {
        "metric": "post-attention output projection TFLOP/s (% MFMA peak)",
        "value": round(fl / sec / 1e12, 2), "unit": "TFLOP/s",
        "pct_of_bf16_peak": round(100.0 * fl / sec / 1e12 / BF16_PEAK_TFLOPS, 2),
        "ms_per_step": round(sec * 1e3, 5), **winfo, "dtype": "bf16, fp32 accumulate",
        "config": {"workload": f"C12 o_proj behind config 3: tokens M={B * T} (B={B}, T={T}), K=Hq*D={K}, N=hidden={N}", "flops": fl},
        "roofline": {"bound": "mfma", "achieved": round(fl / (kavg * 1e-3) / 1e12, 2), "peak": BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(fl / (kavg * 1e-3) / 1e12 / BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "o_proj_kernel", "kernel_avg_ms": round(kavg, 5), "launches_timed": len(kms),
                     "mfma_only_loop_same_data": _mfma_ceiling(lib, x)},
    }
    res["cpu_baseline"] = res["parity"] = None
    if not _NO_CPU:
        # 512 token rows, 8 from each of the 64 row tiles of 256, at in-tile positions that change from tile to tile
        ridx = np.arange(0, B * T, 32) + (np.arange(B * T // 32) * 7) % 32
        rows = len(ridx)
        torch.cuda.synchronize()
        sel = torch.from_numpy(ridx).to(x.device)
        xh, wh = dev_bits(x.reshape(B * T, K)[sel].contiguous()), dev_bits(w)
        dt, want = _median3(lambda: O.o_proj(xh, wh))
        res["cpu_baseline"] = {"value": round(2 * rows * K * N / dt / 1e12, 5), "unit": "TFLOP/s", "cores": _host_info(), "kind": "port",
                               "sample": f"NumPy oracle (float32 matmul), {rows} of {B * T} token rows of the same workload (8 from every "
                                         f"256-row tile), 1 warm-up + 3 runs, median {dt:.2f} s, numpy {np.__version__} default BLAS threading"}
        got = out.reshape(B * T, N)[sel].float().cpu().numpy()
        err = np.abs(got.astype(np.float64) - want)
        tol = 2.0 ** -7 * np.abs(want) + 1e-5 * float(np.abs(want).max())
        res["parity"] = {"max_abs_err": round(float(err.max()), 6), "tol": "2^-7 |want| + 1e-5 max|want| per element (one bf16 step + float32 summation order)",
                         "pass": bool(np.isfinite(got).all() and np.all(err <= tol))}
    return res


def bench_kv_write(steps, warmup, lib, pa, W):
    """Paged KV write with fp8 quantise-on-write (the step in front of the attention call).
    The kernel mutates the pool; every step rewrites the same rows with the same values, so the
    steady state (scales already at their maximum: no re-encode of earlier rows) is what is timed."""
    from oracle import paged_attention_oracle as O
    from nkipy_amd.workloads import storage_bits as dev_bits
    w = W.make_kv_write()

    def step():
        pa.kv_write(w.k_new, w.v_new, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.query_lens,
                    k_scale=w.k_scale, v_scale=w.v_scale)

    sec, kms, winfo = _measure(step, steps, warmup, lib)
    kavg = float(np.mean(kms))
    ab = w.algorithmic_bytes()
    B, T, Hkv, D = w.k_new.shape
    res = {
        "metric": "paged KV write HBM GB/s (% peak)",
        "value": round(ab / sec / 1e9, 2), "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * ab / sec / 1e9 / HBM_PEAK_GBS, 2),
        "tok_per_s": round(B * T / sec, 1),
        "ms_per_step": round(sec * 1e3, 5), **winfo, "dtype": "bf16 rows -> fp8-e4m3 pool, fp32 scales",
        "config": {"workload": f"C6 paged KV write: B={B}, T={T} new tokens, Hkv={Hkv}, D={D}, block_size={w.k_cache.shape[1]}, "
                               f"prefix={w.prefix.tolist()}, pool={w.k_cache.shape[0]} blocks",
                   "algorithmic_bytes": ab},
        "roofline": {"bound": "hbm", "achieved": round(ab / (kavg * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(ab / (kavg * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": None, "kernel": "kv_write_kernel", "kernel_avg_ms": round(kavg, 5),
                     "launches_timed": len(kms)},
    }

    def cpu():
        n = 2
        kn, vn = dev_bits(w.k_new[:n]), dev_bits(w.v_new[:n])
        kc, vc = dev_bits(w.k_cache), dev_bits(w.v_cache)
        ks, vs = w.k_scale.cpu().numpy(), w.v_scale.cpu().numpy()
        t = time.perf_counter()
        O.kv_write(kn, vn, kc, vc, w.block_tables[:n].cpu().numpy(), w.seq_lens[:n].cpu().numpy(),
                   w.query_lens[:n].cpu().numpy(), k_scale=ks, v_scale=vs)
        dt = time.perf_counter() - t
        return {"value": round(ab * n / B / dt / 1e9, 4), "unit": "GB/s", "cores": _host_info(), "kind": "port",
                "sample": f"NumPy oracle, first {n} of {B} sequences of the same workload, one run of {dt:.2f} s"}

    res["cpu_baseline"] = None if _NO_CPU else cpu()
    return res


def bench_pre_attention(steps, warmup, lib, pa, W):
    """QK RMSNorm + RoPE on q and k fused with the fp8 KV write (config 6's write plus the q tensor)."""
    w = W.make_kv_write()
    B, T, Hkv, D = w.k_new.shape
    Hq = 4 * Hkv
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1007)
    xq = torch.randn((B, T, Hq, D), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    wq = (1.0 + 0.1 * torch.randn(D, generator=gen, device="cuda")).to(torch.bfloat16)
    wk = (1.0 + 0.1 * torch.randn(D, generator=gen, device="cuda")).to(torch.bfloat16)
    max_pos = int(w.seq_lens.max().item())
    cos, sin = pa.rope_tables(D, max_pos, 1000000.0)
    q_out = torch.empty_like(xq)

    def step():
        pa.qk_norm_rope_kv_write(xq, w.k_new, w.v_new, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.query_lens,
                                 cos, sin, q_norm_weight=wq, k_norm_weight=wk, eps=1e-6,
                                 k_scale=w.k_scale, v_scale=w.v_scale, out=q_out)

    sec = _time_steps(step, steps, warmup)
    ab = w.algorithmic_bytes() + 2 * xq.numel() * 2 + 2 * cos.numel() * 2
    res = {
        "metric": "fused QK-norm + RoPE + paged KV write HBM GB/s (% peak)",
        "value": round(ab / sec / 1e9, 2), "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * ab / sec / 1e9 / HBM_PEAK_GBS, 2),
        "tok_per_s": round(B * T / sec, 1),
        "ms_per_step": round(sec * 1e3, 5), "dtype": "bf16 rows, float32 norm, bf16 rotation -> fp8-e4m3 pool",
        "config": {"workload": f"C7 pre-attention: B={B}, T={T} new tokens, Hq={Hq}, Hkv={Hkv}, D={D}, "
                               f"block_size={w.k_cache.shape[1]}, prefix={w.prefix.tolist()}",
                   "algorithmic_bytes": ab},
        "roofline": {"bound": "hbm", "achieved": round(ab / sec / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(ab / sec / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "q_norm_rope_kernel + kv_write_kernel (two launches, step time)",
                     "kernel_avg_ms": round(sec * 1e3, 5), "launches_timed": steps},
        "cpu_baseline": None,
    }
    return res


def bench_prefill_layer_step(steps, warmup, lib, pa, W):
    """config 10: what one attention layer of a prefill step does on config 3's workload: QK RMSNorm +
    RoPE, K/V rows into the pool, attention.  The Q half of the transform rides on the attention
    kernel's Q load; the two-step form (Q transformed by a kernel of its own) is timed beside it."""
    w = W.make_prefill()
    B, T, Hq, D = w.q.shape
    Hkv = w.k_cache.shape[2]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1010)
    xk = torch.randn((B, T, Hkv, D), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    xv = torch.randn((B, T, Hkv, D), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    wq = (1.0 + 0.1 * torch.randn(D, generator=gen, device="cuda")).to(torch.bfloat16)
    wk = (1.0 + 0.1 * torch.randn(D, generator=gen, device="cuda")).to(torch.bfloat16)
    cos, sin = pa.rope_tables(D, int(w.seq_lens.max().item()), 1000000.0)
    out, q2 = torch.empty_like(w.q), torch.empty_like(w.q)
    qt = pa.QTransform(cos, sin, wq, 1e-6)
    common = (w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.query_lens)

    def fused():
        pa.qk_norm_rope_kv_write(None, xk, xv, *common, cos, sin, k_norm_weight=wk, eps=1e-6)
        pa.prefill(w.q, *common, w.scale, out=out, q_transform=qt)

    def two_step():
        pa.qk_norm_rope_kv_write(w.q, xk, xv, *common, cos, sin, q_norm_weight=wq, k_norm_weight=wk, eps=1e-6, out=q2)
        pa.prefill(q2, *common, w.scale, out=out)

    sec2 = _time_steps(two_step, steps, warmup)
    ref = out.clone()
    sec = _time_steps(fused, steps, warmup)
    same = bool(torch.equal(out, ref))
    lib.pa_profile_enable(1)
    _time_steps(fused, steps, 0)
    lib.pa_profile_enable(0)
    kms = [x for x in _collect_kernel_ms(lib, 2 * steps)]
    katt = float(np.mean(sorted(kms)[len(kms) // 2:]))      # the attention launches are the longer half
    fl = w.flops()
    return {
        "metric": "prefill layer step (QK-norm + RoPE + KV write + attention) attn TFLOP/s",
        "value": round(fl / sec / 1e12, 2), "unit": "TFLOP/s",
        "ms_per_step": round(sec * 1e3, 5),
        "two_step_ms_per_step": round(sec2 * 1e3, 5), "fused_equals_two_step_bits": same,
        "dtype": "bf16, float32 norm, bf16 rotation, fp32 accumulate",
        "config": {"workload": f"C3 prefill layer step: B={B}, T={T}, Hq={Hq}, Hkv={Hkv}, D={D}, "
                               f"block_size={w.k_cache.shape[1]}, prefix={w.prefix.tolist()}", "flops": fl},
        "roofline": {"bound": "mfma", "achieved": round(fl / (katt * 1e-3) / 1e12, 2), "peak": BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(fl / (katt * 1e-3) / 1e12 / BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "prefill_async_kernel with the Q transform in its prologue", "kernel_avg_ms": round(katt, 5),
                     "launches_timed": len(kms) // 2},
        "cpu_baseline": None,
    }


def _decode_layer_step_times(steps, warmup, B, ctx, layers, capacity, bound, T=1, gpt_oss=False):
    """Seconds per step of `layers` attention layers, issued call by call and replayed from one HIP graph, on a cache
    whose tables hold `capacity` tokens per sequence; `bound` is the length bound given to `attend` (None: the
    engine's own choice, which under capture is the longest context the cache admits).  T new tokens per sequence
    (1: a decode step; more: a speculative verify step) behind `ctx` cached ones.  gpt_oss: the layer of
    examples/models/gpt_oss/kernels/attention.py:80-163 instead of qwen3's (64 / 8 heads of 64, hidden 2 880 with a
    bias, RoPE without QK norm, a sink logit per head, a 128-token window on every other layer)."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    Hq, Hkv, D, bs, N = (64, 8, 64, 32, 2880) if gpt_oss else (32, 8, 128, 32, 4096)
    nblk = (capacity + bs - 1) // bs
    cache = PagedKVCache(B * nblk + 8, bs, Hkv, D, max_seqs=B, max_blocks_per_seq=nblk, num_layers=layers)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1313)
    one = torch.ones(D, dtype=torch.bfloat16, device="cuda")
    if gpt_oss:
        att = [PagedAttention(cache, Hq, layer=l, rope_base=150000.0, max_positions=nblk * bs,
                              sinks=torch.randn(Hq, generator=gen, device="cuda"), sliding_window=128 if l % 2 == 0 else None,
                              o_weight=(torch.randn(Hq * D, N, generator=gen, device="cuda") / 64).to(torch.bfloat16),
                              o_bias=torch.randn(N, generator=gen, device="cuda").to(torch.bfloat16))
               for l in range(layers)]
    else:
        att = [PagedAttention(cache, Hq, layer=l, rope_base=1e6, max_positions=nblk * bs, q_norm_weight=one, k_norm_weight=one,
                              o_weight=(torch.randn(Hq * D, N, generator=gen, device="cuda") / 64).to(torch.bfloat16))
               for l in range(layers)]
    for pool in cache.k_caches + cache.v_caches:
        pool.copy_(torch.randn(pool.shape, generator=gen, device="cuda", dtype=torch.float32))
    cache.extend(list(range(B)), [ctx] * B)      # contexts of `ctx` tokens (the pool holds whatever it holds)
    q1 = torch.randn(B, T, Hq, D, generator=gen, device="cuda").to(torch.bfloat16)
    k1 = torch.randn(B, T, Hkv, D, generator=gen, device="cuda").to(torch.bfloat16)

    def step():
        for a in att:
            a.attend(q1, k1, k1, max_seq_len=bound)

    cache.begin_step([T] * B, T)
    sec_eager = _time_steps(step, steps, warmup)
    global _LAST_STEP_WITH_BOOKKEEPING
    _LAST_STEP_WITH_BOOKKEEPING = None
    if T == 1:
        # the same with the step's bookkeeping in front (tables, lengths and query lengths published to the device):
        # steps that append nothing, so that the contexts stay what they are; the decode kernels treat every slot as live
        def full_step():
            cache.begin_step([0] * B, 1)
            step()
        _LAST_STEP_WITH_BOOKKEEPING = _time_steps(full_step, steps, 5)
        cache.begin_step([1] * B, 1)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    sec = _time_steps(graph.replay, steps, 5)
    del graph
    return sec, sec_eager, nblk * bs


_LAST_STEP_WITH_BOOKKEEPING = None


def bench_decode_layer_step(steps, warmup, lib, pa, W, B=8, ctx=1024, layers=8):
    """config 13: a decode step of a small batch through the engine glue, per attention layer: QK RMSNorm + RoPE +
    K/V row into the pool + paged decode + output projection (`PagedAttention.attend`), `layers` layers with a pool
    and weights of their own, issued call by call and replayed from one HIP graph.  Launch-bound: the figure is
    microseconds per layer; the bytes a layer has to move (its contexts' K and V, the projection weight) are given
    for scale.  The length bound a captured step carries picks its decode kernel, so the figure depends on what the
    caller can promise: the headline is a cache whose tables end just above the contexts (the bound is then the
    table capacity); `capacity_8k` repeats it on tables of 8 192 tokens per sequence, once with no promise (the
    captured step must serve any length: the balanced kernel) and once with `attend(max_seq_len=1088)`."""
    Hq, Hkv, D, bs, N = 32, 8, 128, 32, 4096
    sec, sec_eager, cap = _decode_layer_step_times(steps, warmup, B, ctx, layers, ctx + 96, None)
    with_books = _LAST_STEP_WITH_BOOKKEEPING
    big_free, _, big_cap = _decode_layer_step_times(steps, warmup, B, ctx, layers, 8192, None)
    big_bound, _, _ = _decode_layer_step_times(steps, warmup, B, ctx, layers, 8192, ctx + 64)
    kv_bytes = 2 * B * (ctx + 1) * Hkv * D * 2
    byts = kv_bytes + Hq * D * N * 2 + B * (2 * Hq * D + 2 * Hkv * D + N) * 2
    us = sec / layers * 1e6
    return {
        "metric": "decode layer step (QK-norm + RoPE + KV write + paged decode + o_proj), layers/s, HIP graph replay",
        "value": round(1e6 / us, 1), "unit": "layer steps/s",
        "ms_per_step": round(sec * 1e3, 5), "us_per_layer": round(us, 2),
        "eager_us_per_layer": round(sec_eager / layers * 1e6, 2),
        "eager_us_per_step_with_begin_step": round(with_books * 1e6, 1), "eager_us_per_step": round(sec_eager * 1e6, 1),
        "capacity_8k": {"table_capacity_tokens": big_cap,
                        "us_per_layer_no_bound": round(big_free / layers * 1e6, 2),
                        f"us_per_layer_max_seq_len_{ctx + 64}": round(big_bound / layers * 1e6, 2)},
        "dtype": "bf16, float32 norm, bf16 rotation, fp32 accumulate",
        "config": {"workload": f"decode layer step: B={B}, context={ctx}, table capacity={cap} tokens per sequence, "
                               f"layers={layers}, Hq={Hq}, Hkv={Hkv}, D={D}, block_size={bs}, hidden={N}; "
                               f"one step = {layers} layers", "algorithmic_bytes_per_layer": byts},
        "roofline": {"bound": "hbm", "achieved": round(byts / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(byts / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "three launches per layer (decode with the new row on it, merge, projection with its merge "
                               "on the load); five without a length bound",
                     "kernel_avg_ms": round(us * 1e-3, 5), "launches_timed": steps * layers},
        "cpu_baseline": None,
    }


def bench_verify_layer_step(steps, warmup, lib, pa, W, B=1, T=4, ctx=1024, layers=8):
    """config 15: a speculative verify step at the reference's operating point (one sequence, K + 1 = 4 tokens), per
    attention layer through `PagedAttention.attend`: the T tokens' K / V rows into the pool, causal attention of the
    T tokens over the cache, output projection; tables that end just above the context.  Launch-bound like config
    13; `batches` repeats it for 4 sequences behind 2 K and 8 behind 1 K."""
    Hq, Hkv, D, bs, N = 32, 8, 128, 32, 4096
    sec, sec_eager, cap = _decode_layer_step_times(steps, warmup, B, ctx, layers, ctx + 96, None, T=T)
    others = {}
    for b2, c2 in ((4, 2048), (8, 1024)):
        s2, e2, _ = _decode_layer_step_times(steps, warmup, b2, c2, layers, c2 + 96, None, T=T)
        others[f"B{b2}_ctx{c2}"] = {"us_per_layer": round(s2 / layers * 1e6, 2),
                                    "eager_us_per_layer": round(e2 / layers * 1e6, 2)}
    byts = 2 * B * (ctx + T) * Hkv * D * 2 + Hq * D * N * 2 + B * T * (2 * Hq * D + 2 * Hkv * D + N) * 2
    us = sec / layers * 1e6
    return {
        "metric": "verify layer step (QK-norm + RoPE + KV write + causal verify + o_proj), layers/s, HIP graph replay",
        "value": round(1e6 / us, 1), "unit": "layer steps/s",
        "ms_per_step": round(sec * 1e3, 5), "us_per_layer": round(us, 2),
        "eager_us_per_layer": round(sec_eager / layers * 1e6, 2), "batches": others,
        "dtype": "bf16, float32 norm, bf16 rotation, fp32 accumulate",
        "config": {"workload": f"verify layer step: B={B}, T={T}, context={ctx}, table capacity={cap} tokens per sequence, "
                               f"layers={layers}, Hq={Hq}, Hkv={Hkv}, D={D}, block_size={bs}, hidden={N}; "
                               f"one step = {layers} layers", "algorithmic_bytes_per_layer": byts},
        "roofline": {"bound": "hbm", "achieved": round(byts / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(byts / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "three launches per layer (verify with the new rows on it, merge, projection)",
                     "kernel_avg_ms": round(us * 1e-3, 5), "launches_timed": steps * layers},
        "cpu_baseline": None,
    }


def bench_gpt_oss_layer_step(steps, warmup, lib, pa, W, B=1, ctx=1024, layers=8):
    """config 16: the decode and verify steps of configs 13 and 15 on the gpt-oss layer, the reference's other model
    family and its published operating point (one sequence, K + 1 = 4 draft tokens: peagle/speculate.py:137-202):
    sinks on every layer, a 128-token sliding window on every other one, 64 / 8 heads of 64, output projection to
    2 880 with a bias.  Launch-bound; microseconds per layer, HIP graph replay and issued call by call."""
    Hq, Hkv, D, bs, N = 64, 8, 64, 32, 2880
    sec, sec_eager, cap = _decode_layer_step_times(steps, warmup, B, ctx, layers, ctx + 96, None, gpt_oss=True)
    with_books = _LAST_STEP_WITH_BOOKKEEPING
    others = {}
    for b2, c2, t2 in ((1, 1024, 4), (8, 1024, 1), (1, 4000, 1), (4, 2048, 4)):
        s2, e2, _ = _decode_layer_step_times(steps, warmup, b2, c2, layers, c2 + 96, None, T=t2, gpt_oss=True)
        others[f"B{b2}_ctx{c2}_T{t2}"] = {"us_per_layer": round(s2 / layers * 1e6, 2),
                                          "eager_us_per_layer": round(e2 / layers * 1e6, 2)}
    # a windowed layer reads its last 128 tokens, a full one the whole context: the mean of the two
    kv_bytes = B * ((ctx + 1) + min(ctx + 1, 128)) * Hkv * D * 2
    byts = kv_bytes + Hq * D * N * 2 + B * (2 * Hq * D + 2 * Hkv * D + N) * 2
    us = sec / layers * 1e6
    return {
        "metric": "gpt-oss decode layer step (RoPE + KV write + paged decode with sinks / window + o_proj), layers/s, HIP graph replay",
        "value": round(1e6 / us, 1), "unit": "layer steps/s",
        "ms_per_step": round(sec * 1e3, 5), "us_per_layer": round(us, 2),
        "eager_us_per_layer": round(sec_eager / layers * 1e6, 2), "other_steps": others,
        "eager_us_per_step_with_begin_step": round(with_books * 1e6, 1), "eager_us_per_step": round(sec_eager * 1e6, 1),
        "dtype": "bf16, bf16 rotation, fp32 accumulate",
        "config": {"workload": f"gpt-oss decode layer step: B={B}, context={ctx}, table capacity={cap} tokens per sequence, "
                               f"layers={layers} (window 128 on the even ones, sinks on all), Hq={Hq}, Hkv={Hkv}, D={D}, "
                               f"block_size={bs}, hidden={N} with bias; one step = {layers} layers",
                   "algorithmic_bytes_per_layer": byts},
        "roofline": {"bound": "hbm", "achieved": round(byts / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(byts / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "per layer: decode with the new row on it (one partition under the window; else + merge), "
                               "projection + its merge",
                     "kernel_avg_ms": round(us * 1e-3, 5), "launches_timed": steps * layers},
        "cpu_baseline": None,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=60)
    ap.add_argument("--config", type=int, default=0, choices=[0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17],
                    help="0 (default): config 2 as the line, configs 3, 4 and 5 under \"configs\"; N: that configuration alone")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and parity legs")
    ap.add_argument("--prefill-impl", type=int, default=0,
                    help="force a form of the tiled prefill kernel through the library's debug switch 3 (4 / 8: waves per "
                         "workgroup; for config 4, 8 is the staggered 256-row form); 0: the library's own choice.  For "
                         "comparisons of kernel forms; recorded in the line as prefill_impl")
    ap.add_argument("--const-data", action="store_true",
                    help="prefill configs 3 / 9 / 11 and the projection 12: every Q, K and V (x and w) element is the same value instead of N(0,1).  Same "
                         "kernel, same instruction stream, far fewer bit flips in the matrix cores' operands: the time "
                         "difference to the normal run is what the chip's power limit costs on random data")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is measured on ONE GPU (the kernel on one GPU's share at its real "
              "shape); --gpus N with N > 1 is not supported.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no ROCm device visible; this benchmark has no CPU path.", file=sys.stderr)
        sys.exit(3)
    import gc

    if args.prefill_impl:
        os.environ["PA_ENABLE_DEBUG"] = "1"      # read by the library at its first use
    import nkipy_amd as pa
    from nkipy_amd import _lib, workloads as W
    lib = _lib.load()
    torch.cuda.set_device(0)
    if args.prefill_impl and lib.pa_debug_set(3, args.prefill_impl) != 0:
        print(f"bench.py: {lib.pa_last_error().decode()}", file=sys.stderr)
        sys.exit(2)
    if args.no_cpu:
        global _NO_CPU
        _NO_CPU = True
    if args.const_data:
        global _CONST_DATA
        _CONST_DATA = True

    def run(cfg):
        if cfg in (2, 5, 17):     # 17: config 2's shape with 8 192 sequences of 10-90 tokens
            res = bench_decode(cfg, args.steps, args.warmup, lib, pa, W)
        elif cfg == 3:
            res = bench_prefill(args.steps, args.warmup, lib, pa, W)
        elif cfg == 4:
            res = bench_blocksparse(args.steps, args.warmup, lib, pa, W)
        elif cfg == 6:
            res = bench_kv_write(args.steps, args.warmup, lib, pa, W)
        elif cfg == 7:
            res = bench_pre_attention(args.steps, args.warmup, lib, pa, W)
        elif cfg == 8:
            res = bench_verify(args.steps, args.warmup, lib, pa, W)
        elif cfg == 9:
            res = bench_prefill(args.steps, args.warmup, lib, pa, W, fp8=True)
        elif cfg == 11:
            res = bench_prefill(args.steps, args.warmup, lib, pa, W, gpt_oss=True)
        elif cfg == 12:
            res = bench_o_proj(args.steps, args.warmup, lib, pa, W)
        elif cfg == 13:
            res = bench_decode_layer_step(args.steps, args.warmup, lib, pa, W)
        elif cfg == 14:
            res = bench_tile_loop_probe(args.steps, args.warmup)
        elif cfg == 15:
            res = bench_verify_layer_step(args.steps, args.warmup, lib, pa, W)
        elif cfg == 16:
            res = bench_gpt_oss_layer_step(args.steps, args.warmup, lib, pa, W)
        else:
            res = bench_prefill_layer_step(args.steps, args.warmup, lib, pa, W)
        gc.collect()
        torch.cuda.empty_cache()
        return res

    t_start = time.perf_counter()
    res = run(args.config or 2)
    line = {"metric": res.pop("metric"), "value": res.pop("value"), "unit": res.pop("unit"),
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": res.pop("dtype"), "data": "synthetic (seeded N(0,1), random block tables)",
            "config": res.pop("config")}
    line.update(res)
    if args.config == 0:
        # the other benchmark-sized configurations, same protocol, same process: the prefill half of the
        # headline metric (config 3), the blocksparse form (config 4) and the fp8-KV decode (config 5)
        line["metric"] = "decode attn HBM GB/s (% peak) + tok/s; prefill attn TFLOP/s (% MFMA peak)"
        subs = {}
        for cfg in (3, 4, 5, 12):
            r = run(cfg)
            r["steps"], r["warmup"] = args.steps, args.warmup
            subs["o_proj" if cfg == 12 else f"C{cfg}"] = r
        line["configs"] = subs
        line["prefill_value"] = subs["C3"]["value"]
        line["prefill_unit"] = subs["C3"]["unit"]
        line["prefill_roofline_frac"] = subs["C3"]["roofline"]["frac"]
        par = [line.get("parity")] + [r.get("parity") for r in subs.values()]
        line["parity_all_pass"] = None if any(x is None for x in par) else all(x["pass"] for x in par)
        # the launch-bound steps of a small batch (a second each): decode and verify steps of a layer on the qwen3
        # and gpt-oss shapes, per layer, replayed from a graph and issued call by call
        steps = {}
        for cfg, name in ((13, "decode_B8_ctx1K"), (15, "verify_B1_T4_ctx1K"), (16, "gpt_oss_decode_B1_ctx1K")):
            r = run(cfg)
            steps[name] = {k: r[k] for k in ("us_per_layer", "eager_us_per_layer", "eager_us_per_step", "eager_us_per_step_with_begin_step",
                                             "capacity_8k", "batches", "other_steps")
                           if k in r}
            steps[name]["workload"] = r["config"]["workload"]
        line["layer_steps"] = steps
    if args.prefill_impl:
        line["prefill_impl"] = args.prefill_impl
    if args.const_data:
        line["data"] = "synthetic CONSTANT operands (power probe: not a benchmark result)"
    line["device"] = torch.cuda.get_device_name(0)
    line["bench_wall_s"] = round(time.perf_counter() - t_start, 1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
