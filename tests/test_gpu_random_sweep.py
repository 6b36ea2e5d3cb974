"""GPU parity over seeded random combinations of every option of the attention ops (shape, GQA ratio,
block size, fp8 pool, ragged query lengths, sliding window, sinks, Q transform on load, kernel route): each
case against the oracle.  The cases are drawn from a fixed seed, so a failure names a reproducible case."""
import os

import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, bf16_to_dev, dev_to_f32, make_paged

pytestmark = pytest.mark.gpu

# elements whose error lay above the plain absolute bar and inside the allowance for large outputs, per case
WIDENED = {}

N_CASES = int(os.environ.get("PA_SWEEP_CASES", "60"))      # more cases for an occasional longer soak of the same generator
FIRST_CASE = int(os.environ.get("PA_SWEEP_FIRST", "0"))


def _i32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.int32)).cuda()


def _draw(case):
    rng = np.random.default_rng(9000 + case)
    D = int(rng.choice([64, 128]))
    Hkv = int(rng.choice([1, 2, 4, 8]))
    n_rep = int(rng.choice([1, 2, 4, 5, 8, 16]))
    bs = int(rng.choice([16, 32, 64, 128]))
    B = int(rng.integers(1, 7))
    kind = rng.choice(["decode", "verify", "tiled"])
    T = 1 if kind == "decode" else int(rng.integers(2, 20)) if kind == "verify" else int(rng.integers(65, 300))
    fp8 = bool(rng.integers(0, 2))
    window = None if rng.integers(0, 2) else int(rng.choice([1, 7, 32, 33, 100, 700]))
    sinks = bool(rng.integers(0, 2))
    long_ctx = rng.integers(0, 4) == 0
    prefixes = [int(rng.integers(0, 3000 if long_ctx else 300)) for _ in range(B)]
    qlens = [int(rng.integers(0 if kind != "decode" and B > 1 else 1, T + 1)) for _ in range(B)]
    if kind != "decode" and max(qlens) == 0:
        qlens[0] = T
    qt = int(rng.integers(0, 3))           # 0: q as given; 1: rotated on load; 2: normed and rotated on load
    return dict(qt=qt, rng=rng, D=D, Hkv=Hkv, Hq=Hkv * n_rep, bs=bs, B=B, kind=kind, T=T, fp8=fp8, window=window,
                sinks=sinks, prefixes=prefixes, qlens=qlens)


@pytest.mark.parametrize("case", range(FIRST_CASE, FIRST_CASE + N_CASES))
def test_random_case(case):
    import nkipy_amd as pa
    c = _draw(case)
    rng, D, Hkv, Hq, bs, B, T = c["rng"], c["D"], c["Hkv"], c["Hq"], c["bs"], c["B"], c["T"]
    print({k: v for k, v in c.items() if k != "rng"}, flush=True)
    qlens = [1] * B if c["kind"] == "decode" else c["qlens"]
    ctxs = [p + t for p, t in zip(c["prefixes"], qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [max(x, 1) for x in ctxs])
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32) * 2) if c["sinks"] else None
    scale = 1.0 / np.sqrt(D)
    kw_o, kw_d = {}, {}
    if c["fp8"]:
        kq, ks = O.quantize_kv_fp8(k)
        vq, vs = O.quantize_kv_fp8(v)
        kc_o, vc_o = kq, vq
        kc_d = torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn)
        vc_d = torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn)
        kw_o = dict(k_scale=ks, v_scale=vs)
        kw_d = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda())
    else:
        kc_o, vc_o = O.round_to_bf16(k), O.round_to_bf16(v)
        kc_d, vc_d = bf16_to_dev(k), bf16_to_dev(v)
    sinks_d = None if sinks is None else bf16_to_dev(sinks)
    tol = 5e-2 if c["fp8"] else 2e-2
    q_dev, qt = q, None
    if c["qt"]:
        w = O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32)) if c["qt"] == 2 else None
        max_pos = max(ctxs) + 1
        cos, sin = O.rope_tables(D, max_pos, 10000.0)
        dcos, dsin = pa.rope_tables(D, max_pos, 10000.0)
        qt = pa.QTransform(dcos, dsin, None if w is None else bf16_to_dev(w), 1e-6)
        q, _ = O.qk_norm_rope(q_dev, q_dev[:, :, :Hkv], np.asarray(ctxs), np.asarray(qlens), cos, sin,
                              q_norm_weight=w, eps=1e-6)          # what the oracle's attention sees
    if c["kind"] == "decode":
        want = O.paged_decode(q[:, 0], kc_o, vc_o, tables, np.asarray(ctxs, np.int32), scale, q_dtype="bf16",
                              sliding_window=c["window"], sinks=sinks, **kw_o)
        got = pa.decode(bf16_to_dev(q_dev[:, 0]), kc_d, vc_d, _i32(tables), _i32(ctxs), scale,
                        sliding_window=c["window"], sinks=sinks_d, q_transform=qt, **kw_d)
    else:
        want = O.paged_prefill(q, kc_o, vc_o, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), scale,
                               q_dtype="bf16", sliding_window=c["window"], sinks=sinks, **kw_o)
        got = pa.prefill(bf16_to_dev(q_dev), kc_d, vc_d, _i32(tables), _i32(ctxs), _i32(qlens), scale,
                         sliding_window=c["window"], sinks=sinks_d, route=c["kind"], q_transform=qt, **kw_d)
    torch.cuda.synchronize()
    got = dev_to_f32(got)
    # The absolute bar holds for outputs of the usual size (a softmax average of N(0,1) rows).  A window of one
    # key hands a single V row through, and a rare row reaches |v| > 4, where one bf16 step is 2^-5: the device
    # rounds the output once and the oracle its probabilities once, so allow 2^-7 of the largest output (case
    # 4765 of this generator: 4.28 -> 0.031, reproduced by the device arithmetic written out in NumPy).
    plain_tol = tol
    tol = max(tol, 2.0 ** -7 * float(np.abs(want).max()))
    over = int((np.abs(got.astype(np.float64) - want) > plain_tol).sum())
    WIDENED[case] = (over, int(want.size))
    print(f"elements above the plain bar {plain_tol} (allowed up to {tol:.4f}): {over} of {want.size}", flush=True)
    assert_close_abs(got, want, tol)
    if c["kind"] != "decode":
        for b, n in enumerate(qlens):
            assert np.all(got[b, n:] == 0)


def test_sweep_summary_of_the_widened_bar(capsys):
    """Says how many elements of the cases above needed the allowance for large outputs (2^-7 of the largest
    expected value) rather than the plain 2e-2 / 5e-2 absolute bar."""
    cases = sum(1 for over, _ in WIDENED.values() if over)
    elems = sum(over for over, _ in WIDENED.values())
    total = sum(n for _, n in WIDENED.values())
    with capsys.disabled():
        print(f"\n[sweep] {len(WIDENED)} cases, {total} elements: {elems} elements in {cases} cases lay above the plain "
              f"absolute bar and inside the 2^-7 max|want| allowance" + (f" (cases {sorted(c for c, (o, _) in WIDENED.items() if o)})" if cases else ""))
