"""GPU parity of `decode_step` (one call per layer and decode step: cache update + attention + output projection)
against the three calls it stands for, bit for bit, on the outputs and on the pools, and against the NumPy oracle
of the reference's decode branch (examples/models/qwen3/kernels/attention.py:78-147)."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import bf16_to_dev, dev_bits, dev_to_f32, make_paged

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


def _i32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.int32)).cuda()


def _fusion(v):
    from nkipy_amd import _lib
    assert _lib.load().pa_debug_set(10, v) == 0


def _setup(rng, B, Hq, Hkv, D, bs, ctxs, qlens, N, bias, xform, fp8=False, poison=True):
    """Pools that hold the contexts without their newest token (its row and everything behind it poisoned with NaN
    patterns: the step must write the row before anything reads it), the step's rows, weights."""
    ctxs = np.asarray(ctxs, np.int64)
    k, v, tables = make_paged(rng, B, Hkv, D, bs, np.maximum(ctxs, 1), extra_blocks=2)
    kd, vd = bf16_to_dev(k), bf16_to_dev(v)
    if poison:
        for b in range(B):
            start = int(ctxs[b]) - int(qlens[b])
            for t in range(max(start, 0), tables.shape[1] * bs):
                blk = tables[b, t // bs]
                if blk < 0:
                    break
                kd[blk, t % bs] = float("nan")
                vd[blk, t % bs] = float("nan")
    d = dict(
        xq=bf16_to_dev(rng.standard_normal((B, Hq, D)).astype(np.float32)),
        xk=bf16_to_dev(rng.standard_normal((B, Hkv, D)).astype(np.float32)),
        xv=bf16_to_dev(rng.standard_normal((B, Hkv, D)).astype(np.float32)),
        k=kd, v=vd, tables=_i32(tables), lens=_i32(ctxs), qlens=_i32(qlens), ks=None, vs=None)
    if fp8:
        from nkipy_amd.workloads import quantize_pool_fp8
        d["k"], d["ks"] = quantize_pool_fp8(torch.nan_to_num(kd, nan=0.0))
        d["v"], d["vs"] = quantize_pool_fp8(torch.nan_to_num(vd, nan=0.0))
    d["ow"] = None if not N else bf16_to_dev((rng.standard_normal((Hq * D, N)) / np.sqrt(Hq * D)).astype(np.float32))
    d["ob"] = bf16_to_dev(rng.standard_normal(N).astype(np.float32)) if N and bias else None
    d["qt"] = d["wk"] = None
    if xform:
        import nkipy_amd
        cos, sin = nkipy_amd.rope_tables(D, tables.shape[1] * bs, 10000.0)
        d["qt"] = nkipy_amd.QTransform(cos, sin, bf16_to_dev(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32)))
        d["wk"] = bf16_to_dev(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32))
    return d


def _three_calls(pa, d, scale, psize, msl, attn_only=False, **variant):
    """The sequence decode_step stands for, on copies of the pools."""
    k, v = d["k"].clone(), d["v"].clone()
    ks = None if d["ks"] is None else d["ks"].clone()
    vs = None if d["vs"] is None else d["vs"].clone()
    if d["qt"] is not None:
        pa.qk_norm_rope_kv_write(None, d["xk"][:, None], d["xv"][:, None], k, v, d["tables"], d["lens"], d["qlens"],
                                 d["qt"].rope_cos, d["qt"].rope_sin, k_norm_weight=d["wk"], eps=d["qt"].eps,
                                 k_scale=ks, v_scale=vs)
    else:
        pa.kv_write(d["xk"][:, None], d["xv"][:, None], k, v, d["tables"], d["lens"], d["qlens"], k_scale=ks, v_scale=vs)
    att = pa.decode(d["xq"], k, v, d["tables"], d["lens"], scale, k_scale=ks, v_scale=vs, partition_size=psize,
                    max_seq_len=msl, q_transform=d["qt"], **variant)
    out = att if attn_only or d["ow"] is None else pa.o_proj(att, d["ow"], d["ob"])
    return out, att, k, v, ks, vs


def _step(pa, d, scale, psize, msl, **kw):
    k, v = d["k"].clone(), d["v"].clone()
    ks = None if d["ks"] is None else d["ks"].clone()
    vs = None if d["vs"] is None else d["vs"].clone()
    out = pa.decode_step(d["xq"], d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], scale, k_scale=ks,
                         v_scale=vs, partition_size=psize, max_seq_len=msl, q_transform=d["qt"], k_norm_weight=d["wk"],
                         o_weight=d["ow"], o_bias=d["ob"], **kw)
    return out, k, v, ks, vs


def _same_bits(a, b, what):
    assert np.array_equal(dev_bits(a), dev_bits(b)), what


CASES = [
    # B, Hq, Hkv, D, bs, contexts (the new token counted), N, bias, transform
    (8, 32, 8, 128, 32, [1025] * 8, 4096, False, True),                 # the layer step this call is for: five fine partitions
    (8, 32, 8, 128, 32, [1024, 1000, 993, 961, 960, 513, 512, 257], 4096, True, True),   # new token first / last of a tile, of a partition
    (1, 32, 8, 128, 16, [1500], 4096, False, True),
    (3, 16, 4, 128, 16, [300, 1, 40], 512, True, True),                 # one partition on eight waves; a sequence of its first token
    (4, 32, 2, 128, 32, [900, 700, 33, 32], 1024, False, True),         # 16 q heads per kv head: no eight-wave form
    (5, 64, 4, 64, 64, [2000, 1999, 1537, 1536, 65], 2880, True, True),   # head dim 64, 16 q heads per kv head, ragged last column slab
    (6, 8, 8, 64, 16, [1200, 31, 32, 33, 257, 256], 512, False, False),   # no GQA, no transform
    (2, 32, 8, 128, 32, [3000, 2500], 4096, False, True),               # six partitions of 512
    (40, 8, 2, 128, 32, [700 + 7 * i for i in range(40)], 4096, False, True),    # more than 32 rows: the projection takes its rows from memory
    (12, 32, 8, 128, 32, [900 + 7 * i for i in range(12)], 1024, False, True),   # more (sequence, kv head) pairs than the small-call kernels take
    (33, 8, 2, 128, 32, [1100 + i for i in range(33)], 256, True, False),
]


@pytest.mark.parametrize("B,Hq,Hkv,D,bs,ctxs,N,bias,xform", CASES)
def test_decode_step_equals_the_three_calls(pa, B, Hq, Hkv, D, bs, ctxs, N, bias, xform):
    rng = np.random.default_rng(B * 1000 + Hq + D + len(ctxs) + N)
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, [1] * B, N, bias, xform)
    scale, msl = 1.0 / np.sqrt(D), int(max(ctxs))
    print(f"decode_step B={B} Hq={Hq} Hkv={Hkv} D={D} bs={bs} ctx={ctxs[:4]}.. N={N} bias={bias} xform={xform}", flush=True)
    want, att, wk, wv, _, _ = _three_calls(pa, d, scale, 512, msl)
    for fusion, kw in ((0, {}), (2, {}), (3, {}), (1, {})):
        _fusion(fusion)
        try:
            got, gk, gv, _, _ = _step(pa, d, scale, 512, msl, **kw)
            torch.cuda.synchronize()
        finally:
            _fusion(0)
        _same_bits(got, want, f"projected rows, fusion switch {fusion}")
        _same_bits(gk, wk, f"K pool, fusion switch {fusion}")
        _same_bits(gv, wv, f"V pool, fusion switch {fusion}")
    # the attention output as well, and alone
    a2 = torch.empty_like(d["xq"])
    got, gk, gv, _, _ = _step(pa, d, scale, 512, msl, attn_out=a2)
    _same_bits(got, want, "projected rows with attn_out")
    _same_bits(a2, att, "attention output beside the projection")
    d2 = dict(d, ow=None, ob=None)
    got, gk, gv, _, _ = _step(pa, d2, scale, 512, msl)
    torch.cuda.synchronize()
    _same_bits(got, att, "attention output alone")
    _same_bits(gk, wk, "K pool, attention alone")
    assert not torch.isnan(got.float()).any()


def test_decode_step_against_the_oracle(pa):
    """The step against the reference's arithmetic: rows normed and rotated (rmsnorm.py:4-21, rope.py:23-48), the
    cache row written, attention over the sequence's history, the projection."""
    rng = np.random.default_rng(77)
    B, Hq, Hkv, D, bs, N = 4, 16, 4, 128, 32, 512
    ctxs = [1030, 517, 64, 1]
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, [1] * B, N, True, True)
    scale = 1.0 / np.sqrt(D)
    got, gk, gv, _, _ = _step(pa, d, scale, 512, max(ctxs))
    torch.cuda.synchronize()
    cos, sin = dev_to_f32(d["qt"].rope_cos), dev_to_f32(d["qt"].rope_sin)
    kpool, vpool, tables = dev_to_f32(gk), dev_to_f32(gv), d["tables"].cpu().numpy()
    xq, xk, xv = dev_to_f32(d["xq"]), dev_to_f32(d["xk"]), dev_to_f32(d["xv"])
    qn, kn = O.qk_norm_rope(xq[:, None], xk[:, None], ctxs, [1] * B, cos, sin, q_norm_weight=dev_to_f32(d["qt"].norm_weight),
                            k_norm_weight=dev_to_f32(d["wk"]), eps=d["qt"].eps)
    for b in range(B):
        pos = ctxs[b] - 1
        blk = tables[b, pos // bs]
        # the new rows, as stored: V bit for bit, K within a bf16 step of the oracle's float32-then-round transform
        assert np.array_equal(xv[b], vpool[blk, pos % bs]), b
        assert np.abs(kn[b, 0] - kpool[blk, pos % bs]).max() <= 2 ** -6 * np.abs(kn[b, 0]).max(), b
    # attention over the pools the step left (the row it wrote included), then the projection
    want_att = O.paged_decode(qn[:, 0], kpool, vpool, tables, np.asarray(ctxs, np.int32), scale, q_dtype="bf16")
    want = O.o_proj(O.round_to_bf16(want_att), dev_to_f32(d["ow"]), dev_to_f32(d["ob"]))
    err = np.abs(dev_to_f32(got) - want)
    assert (err <= 2e-2 + 2 ** -7 * np.abs(want)).all(), err.max()


def test_sequences_that_take_no_token_and_empty_slots(pa):
    """query_lens 0: the sequence is attended to as it is and its pool rows are left alone (whatever its row of xk
    holds); a slot of length 0 comes back as zeros."""
    rng = np.random.default_rng(5)
    B, Hq, Hkv, D, bs, N = 6, 16, 4, 128, 16, 256
    ctxs, qlens = [600, 599, 0, 1, 1030, 48], [1, 0, 0, 1, 0, 1]
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, qlens, N, False, True)
    d["xk"][1] = float("nan")
    d["xv"][4] = float("nan")
    scale = 1.0 / np.sqrt(D)
    want, att, wk, wv, _, _ = _three_calls(pa, d, scale, 512, 1030)
    got, gk, gv, _, _ = _step(pa, d, scale, 512, 1030)
    torch.cuda.synchronize()
    _same_bits(got, want, "projected rows")
    _same_bits(gk, wk, "K pool")
    _same_bits(gv, wv, "V pool")
    g = dev_to_f32(got)
    assert not np.isnan(g).any()
    assert np.array_equal(g[2], np.zeros_like(g[2]))


@pytest.mark.parametrize("B", [3, 24], ids=["fixed_partitions", "balanced_schedule"])
def test_length_bound_below_the_new_token(pa, B):
    """A bound that clamps a context below its newest token (pa_decode's rule): the token is stored all the same
    and the attention is over the clamped context."""
    rng = np.random.default_rng(6)
    Hq, Hkv, D, bs, N = 16, 4, 128, 32, 256
    ctxs = ([1000, 1200, 1100] * 8)[:B]
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, [1] * B, N, False, True, poison=False)
    scale = 1.0 / np.sqrt(D)
    want, att, wk, wv, _, _ = _three_calls(pa, d, scale, 512, 1100)
    got, gk, gv, _, _ = _step(pa, d, scale, 512, 1100)
    torch.cuda.synchronize()
    _same_bits(got, want, "projected rows")
    _same_bits(gk, wk, "K pool")
    _same_bits(gv, wv, "V pool")


@pytest.mark.parametrize("B,Hq,Hkv,D,bs,lo,hi,window", [
    (24, 32, 8, 128, 32, 900, 1400, None),     # more (sequence, kv head) pairs than the small-call kernels take
    (3, 32, 8, 128, 32, 9000, 20000, None),    # few long sequences: every sequence cut into many chunks
    (70, 8, 2, 64, 16, 1, 300, None),          # many short ones, some of a single token, some idle
    (6, 40, 2, 128, 64, 3000, 5000, 1000),     # 20 q heads per kv head (two waves per kv head), a window, sinks
    (600, 8, 2, 128, 32, 1, 90, None),         # more sequences than are scanned in registers
])
def test_steps_that_take_the_balanced_schedule(pa, B, Hq, Hkv, D, bs, lo, hi, window):
    """Steps of more sequences or longer contexts than the small-call kernels take: the write launch, the balanced
    kernel, its merge and the projection inside the one call; pools poisoned from the new token on (the row must be
    in the pool before any wave reads it).  Bit for bit the three calls."""
    rng = np.random.default_rng(B + Hq + hi)
    ctxs = rng.integers(lo, hi + 1, size=B)
    ctxs[::5] = (ctxs[::5] // 32) * 32 + 1        # new token first of a tile
    ctxs[1::5] = np.maximum((ctxs[1::5] // 32) * 32, 1)   # ... last of a tile
    qlens = np.ones(B, np.int64)
    if B > 8:
        qlens[3::7] = 0                           # idle sequences: nothing written, attended to as they are
    N = 256
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, qlens, N, True, True)
    scale, msl = 1.0 / np.sqrt(D), int(ctxs.max())
    kw = {}
    if window:
        kw = dict(sinks=torch.from_numpy(rng.standard_normal(Hq).astype(np.float32)).cuda(), sliding_window=window)
    print(f"balanced decode_step B={B} Hq={Hq} Hkv={Hkv} D={D} bs={bs} ctx={ctxs[:6].tolist()}.. window={window}", flush=True)
    want, att, wk, wv, _, _ = _three_calls(pa, d, scale, 512, msl, **kw)
    for fusion in (0, 1):
        _fusion(fusion)
        try:
            got, gk, gv, _, _ = _step(pa, d, scale, 512, msl, **kw)
            torch.cuda.synchronize()
        finally:
            _fusion(0)
        _same_bits(got, want, f"projected rows, fusion switch {fusion}")
        _same_bits(gk, wk, f"K pool, fusion switch {fusion}")
        _same_bits(gv, wv, f"V pool, fusion switch {fusion}")
    assert not torch.isnan(got.float()).any()


SINK_CASES = [
    # B, Hq, Hkv, D, bs, contexts, N, window, transform
    (1, 64, 8, 64, 32, [1025], 2880, None, True),            # the gpt-oss layer: sinks on every layer ...
    (1, 64, 8, 64, 32, [1025], 2880, 128, True),             # ... a 128-token window on every other one: one partition
    (4, 64, 8, 64, 16, [1500, 129, 128, 1], 2880, 128, True),
    (3, 32, 8, 128, 32, [2000, 700, 513], 1024, 600, True),  # a window of several partitions
    (2, 16, 4, 128, 32, [300, 257], 512, 40, False),         # the new token first of a tile, window inside one tile pair
    (5, 32, 8, 128, 32, [1024, 993, 961, 512, 33], 4096, None, True),
]


@pytest.mark.parametrize("B,Hq,Hkv,D,bs,ctxs,N,window,xform", SINK_CASES)
def test_decode_step_with_sinks_and_window(pa, B, Hq, Hkv, D, bs, ctxs, N, window, xform):
    """The gpt-oss variant of the layer (examples/models/gpt_oss/kernels/attention.py:117-148) through the one call:
    sinks and window ride on the small-call kernels, the new row on the decode launch; bit for bit the three calls,
    and the oracle's values."""
    rng = np.random.default_rng(B * 100 + Hq + (window or 0))
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, [1] * B, N, True, xform)
    scale, msl = 1.0 / np.sqrt(D), int(max(ctxs))
    kw = dict(sinks=torch.from_numpy(rng.standard_normal(Hq).astype(np.float32)).cuda(), sliding_window=window)
    print(f"decode_step with sinks B={B} Hq={Hq} Hkv={Hkv} D={D} ctx={ctxs} window={window}", flush=True)
    want, att, wk, wv, _, _ = _three_calls(pa, d, scale, 512, msl, **kw)
    for fusion in (0, 2, 3, 1):
        _fusion(fusion)
        try:
            got, gk, gv, _, _ = _step(pa, d, scale, 512, msl, **kw)
            torch.cuda.synchronize()
        finally:
            _fusion(0)
        _same_bits(got, want, f"projected rows, fusion switch {fusion}")
        _same_bits(gk, wk, f"K pool, fusion switch {fusion}")
        _same_bits(gv, wv, f"V pool, fusion switch {fusion}")
    # the attention output against the oracle on the pools the step left
    a2 = torch.empty_like(d["xq"])
    _step(pa, d, scale, 512, msl, attn_out=a2, **kw)
    torch.cuda.synchronize()
    q = dev_to_f32(d["xq"])
    if xform:
        cos, sin = dev_to_f32(d["qt"].rope_cos), dev_to_f32(d["qt"].rope_sin)
        q = O.qk_norm_rope(q[:, None], dev_to_f32(d["xk"])[:, None], ctxs, [1] * B, cos, sin,
                           q_norm_weight=dev_to_f32(d["qt"].norm_weight), eps=d["qt"].eps)[0][:, 0]
    ref = O.paged_decode(O.round_to_bf16(q), dev_to_f32(wk), dev_to_f32(wv), d["tables"].cpu().numpy(), np.asarray(ctxs, np.int32),
                         scale, q_dtype="bf16", sliding_window=window, sinks=kw["sinks"].cpu().numpy())
    assert np.abs(dev_to_f32(a2) - ref).max() <= 2e-2


@pytest.mark.parametrize("what", ["fp8", "large", "sinks"])
def test_calls_the_small_step_kernels_do_not_take(pa, what):
    """fp8 pools (the scale of a block can grow with the new row) and calls beyond the small-call bounds, with sinks
    and a window too, run the separate launches inside the one call: same results."""
    rng = np.random.default_rng(8)
    if what == "large":
        B, Hq, Hkv, D, bs, N = 48, 32, 8, 128, 32, 1024
        ctxs = [3000 + 13 * i for i in range(B)]
    elif what == "sinks":
        B, Hq, Hkv, D, bs, N = 24, 32, 8, 128, 32, 1024
        ctxs = [1000 + 17 * i for i in range(B)]
    else:
        B, Hq, Hkv, D, bs, N = 4, 32, 8, 128, 32, 1024
        ctxs = [1000, 513, 100, 31]
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, [1] * B, N, True, True, fp8=what == "fp8", poison=what != "fp8")
    scale = 1.0 / np.sqrt(D)
    kw = {}
    if what == "sinks":
        kw = dict(sinks=torch.from_numpy(rng.standard_normal(Hq).astype(np.float32)).cuda(), sliding_window=300)
    k, v = d["k"].clone(), d["v"].clone()
    ks = None if d["ks"] is None else d["ks"].clone()
    vs = None if d["vs"] is None else d["vs"].clone()
    pa.qk_norm_rope_kv_write(None, d["xk"][:, None], d["xv"][:, None], k, v, d["tables"], d["lens"], d["qlens"],
                             d["qt"].rope_cos, d["qt"].rope_sin, k_norm_weight=d["wk"], eps=d["qt"].eps, k_scale=ks, v_scale=vs)
    att = pa.decode(d["xq"], k, v, d["tables"], d["lens"], scale, k_scale=ks, v_scale=vs, max_seq_len=max(ctxs),
                    q_transform=d["qt"], **kw)
    want = pa.o_proj(att, d["ow"], d["ob"])
    got, gk, gv, gks, gvs = _step(pa, d, scale, 512, max(ctxs), **kw)
    torch.cuda.synchronize()
    _same_bits(got, want, "projected rows")
    _same_bits(gk, k, "K pool")
    _same_bits(gv, v, "V pool")
    if ks is not None:
        _same_bits(gks, ks, "K scales")
        _same_bits(gvs, vs, "V scales")


def test_prepared_step_is_the_call_it_was_prepared_from(pa):
    """prepare_decode_step / prepare_verify_step check and marshal once; launch() on the same buffers with new contents
    (rows copied in, lengths advanced in place) gives what a fresh call on those contents gives, bit for bit."""
    rng = np.random.default_rng(31)
    B, Hq, Hkv, D, bs, N = 3, 32, 8, 128, 32, 1024
    ctxs = np.array([700, 513, 31])
    for T in (1, 3):
        d = (_setup(rng, B, Hq, Hkv, D, bs, ctxs + 8 * T, [T] * B, N, True, True, poison=False) if T == 1 else
             _setup_multi(rng, B, T, Hq, Hkv, D, bs, ctxs + 8 * T, [T] * B, N, True, True))
        scale, msl = 1.0 / np.sqrt(D), 800
        k, v = d["k"].clone(), d["v"].clone()
        k2, v2 = k.clone(), v.clone()
        d["lens"].copy_(_i32(ctxs))
        kw = dict(max_seq_len=msl, q_transform=d["qt"], k_norm_weight=d["wk"], o_weight=d["ow"], o_bias=d["ob"])
        prep = (pa.prepare_decode_step if T == 1 else pa.prepare_verify_step)(
            d["xq"], d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], scale, **kw)
        fresh = pa.decode_step if T == 1 else pa.verify_step
        for step in range(4):
            d["lens"].add_(T)
            for name in ("xq", "xk", "xv"):
                d[name].copy_(bf16_to_dev(rng.standard_normal(tuple(d[name].shape)).astype(np.float32)))
            got = prep.launch().clone()
            want = fresh(d["xq"].clone(), d["xk"].clone(), d["xv"].clone(), k2, v2, d["tables"], d["lens"], d["qlens"], scale, **kw)
            torch.cuda.synchronize()
            _same_bits(got, want, f"T={T} step {step}")
            _same_bits(k, k2, "K pool")
            _same_bits(v, v2, "V pool")


def test_decode_step_in_a_graph(pa):
    """Captured once with a caller-owned workspace, replayed on growing contexts; every replay equals the three calls."""
    rng = np.random.default_rng(9)
    B, Hq, Hkv, D, bs, N = 4, 32, 8, 128, 32, 1024
    ctxs = np.array([1000, 513, 255, 31])
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs + 40, [1] * B, N, False, True, poison=False)
    scale, msl = 1.0 / np.sqrt(D), 1100
    from nkipy_amd import _lib
    need = _lib.load().pa_decode_step_workspace_bytes(B, Hq, Hkv, D, bs, msl, 512, N, 1, 1)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.empty((B, N), dtype=torch.bfloat16, device="cuda")
    k, v = d["k"].clone(), d["v"].clone()
    d["lens"].copy_(_i32(ctxs))

    def step():
        pa.decode_step(d["xq"], d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], scale, max_seq_len=msl,
                       q_transform=d["qt"], k_norm_weight=d["wk"], o_weight=d["ow"], out=out, workspace=ws)

    step()
    torch.cuda.synchronize()
    k2, v2 = k.clone(), v.clone()         # the twin the three calls work on, level with the pools after the first step
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for i in range(1, 36):
        d["lens"].copy_(_i32(ctxs + i))
        for t in ("xq", "xk", "xv"):
            d[t].copy_(bf16_to_dev(rng.standard_normal(tuple(d[t].shape)).astype(np.float32)))
        print(f"replay {i}", flush=True)
        g.replay()
        pa.qk_norm_rope_kv_write(None, d["xk"][:, None], d["xv"][:, None], k2, v2, d["tables"], d["lens"], d["qlens"],
                                 d["qt"].rope_cos, d["qt"].rope_sin, k_norm_weight=d["wk"], eps=d["qt"].eps)
        want = pa.o_proj(pa.decode(d["xq"], k2, v2, d["tables"], d["lens"], scale, max_seq_len=msl, q_transform=d["qt"]), d["ow"])
        torch.cuda.synchronize()
        _same_bits(out, want, f"replay {i}")
        _same_bits(k, k2, f"K pool after replay {i}")
        _same_bits(v, v2, f"V pool after replay {i}")


def test_through_the_dispatcher(pa):
    """torch.ops.nkipy_amd.decode_step / decode_step_fp8: the same bits as the Python op."""
    import nkipy_amd.torch_ops  # noqa: F401
    rng = np.random.default_rng(11)
    for fp8 in (False, True):
        B, Hq, Hkv, D, bs, N = 3, 16, 4, 128, 32, 512
        ctxs = [700, 64, 1031]
        d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, [1] * B, N, True, True, fp8=fp8, poison=not fp8)
        scale = 1.0 / np.sqrt(D)
        want, wk, wv, wks, wvs = _step(pa, d, scale, 512, max(ctxs))
        k, v = d["k"].clone(), d["v"].clone()
        out = torch.empty((B, N), dtype=torch.bfloat16, device="cuda")
        common = dict(max_seq_len=max(ctxs), rope_cos=d["qt"].rope_cos, rope_sin=d["qt"].rope_sin,
                      q_norm_weight=d["qt"].norm_weight, k_norm_weight=d["wk"], norm_eps=d["qt"].eps, o_weight=d["ow"],
                      o_bias=d["ob"])
        if fp8:
            ks, vs = d["ks"].clone(), d["vs"].clone()
            torch.ops.nkipy_amd.decode_step_fp8(d["xq"], d["xk"], d["xv"], k, v, ks, vs, d["tables"], d["lens"], d["qlens"],
                                                scale, out, **common)
            _same_bits(ks, wks, "K scales")
        else:
            torch.ops.nkipy_amd.decode_step(d["xq"], d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], scale, out,
                                            **common)
        torch.cuda.synchronize()
        _same_bits(out, want, f"projected rows, fp8={fp8}")
        _same_bits(k, wk, "K pool")
        _same_bits(v, wv, "V pool")


def test_random_steps_equal_the_three_calls(pa):
    """Seeded random decode and verify steps (head shapes, batch, contexts around tile / partition / block borders,
    idle sequences, sinks, windows, bounds, bias, transform): the one call against the three calls, bit for bit,
    outputs and pools."""
    rng = np.random.default_rng(2024)
    shapes = [(32, 8, 128), (64, 8, 64), (16, 16, 64), (8, 1, 128), (32, 2, 128), (12, 4, 64)]
    borders = np.array([1, 2, 31, 32, 33, 63, 64, 65, 255, 256, 257, 511, 512, 513, 767, 768, 769, 1023, 1024, 1025, 1500])
    cases = 0
    for case in range(40):
        Hq, Hkv, D = shapes[rng.integers(len(shapes))]
        bs = int(rng.choice([16, 32, 64]))
        B = int(rng.choice([1, 2, 3, 5, 9]))
        T = int(rng.choice([1, 1, 2, 4, 8]))
        if (Hq // Hkv) * T > 64:
            T = 1
        qlens = rng.integers(0 if B > 1 else 1, T + 1, size=B)
        qlens[rng.integers(B)] = T
        ctxs = np.maximum(rng.choice(borders, size=B) + rng.integers(0, 3, size=B), qlens)
        ctxs = np.where(qlens == 0, np.maximum(ctxs, 1), ctxs)
        N = int(rng.choice([0, 256, 520, 1024]))
        xform = bool(rng.integers(2))
        window = [None, None, 1, 40, 128, 600][rng.integers(6)]
        sinks = torch.from_numpy(rng.standard_normal(Hq).astype(np.float32)).cuda() if rng.integers(2) else None
        bounded = bool(rng.integers(4))
        msl = int(ctxs.max()) + int(rng.integers(0, 40)) if bounded else None
        kw = dict(sinks=sinks, sliding_window=window)
        tag = f"case {case}: B={B} T={T} Hq={Hq} Hkv={Hkv} D={D} bs={bs} ctx={ctxs.tolist()} q={qlens.tolist()} N={N} xform={xform} window={window} sinks={sinks is not None} msl={msl}"
        print(tag, flush=True)
        if T == 1:
            d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, qlens, N, bool(N) and bool(rng.integers(2)), xform)
            want, att, wk, wv, _, _ = _three_calls(pa, d, 0.11, 512, msl, **kw)
            got, gk, gv, _, _ = _step(pa, d, 0.11, 512, msl, **kw)
        else:
            d = _setup_multi(rng, B, T, Hq, Hkv, D, bs, ctxs, qlens, N, bool(N) and bool(rng.integers(2)), xform)
            want, att, wk, wv, _, _ = _verify_three_calls(pa, d, 0.11, msl, **kw)
            got, gk, gv, _, _ = _verify_step(pa, d, 0.11, msl, **kw)
        torch.cuda.synchronize()
        _same_bits(got, want, tag)
        _same_bits(gk, wk, "K pool, " + tag)
        _same_bits(gv, wv, "V pool, " + tag)
        if N == 0:
            # attention only: the oracle's values too, on the pools the step left
            q = dev_to_f32(d["xq"]).reshape(B, T, Hq, D)
            if xform:
                cos, sin = dev_to_f32(d["qt"].rope_cos), dev_to_f32(d["qt"].rope_sin)
                q = O.qk_norm_rope(q, dev_to_f32(d["xk"]).reshape(B, T, Hkv, D), ctxs, qlens, cos, sin,
                                   q_norm_weight=dev_to_f32(d["qt"].norm_weight), eps=d["qt"].eps)[0]
            lens = np.minimum(ctxs, msl) if msl else ctxs
            ref = O.paged_prefill(O.round_to_bf16(q), dev_to_f32(wk), dev_to_f32(wv), d["tables"].cpu().numpy(),
                                  np.asarray(lens, np.int32), np.asarray(qlens, np.int32), 0.11, q_dtype="bf16",
                                  sliding_window=window, sinks=None if sinks is None else sinks.cpu().numpy())
            g = dev_to_f32(got).reshape(B, T, Hq, D)
            if T == 1:                      # decode treats every slot as live: an idle one attends from its last token
                live = qlens > 0
                g, ref = g[live], ref[live]
            assert np.abs(g - ref).max() <= 2e-2, tag
        cases += 1
    assert cases == 40


def test_verify_step_through_the_dispatcher(pa):
    """torch.ops.nkipy_amd.verify_step / verify_step_fp8: the same bits as the Python op."""
    import nkipy_amd.torch_ops  # noqa: F401
    rng = np.random.default_rng(12)
    for fp8 in (False, True):
        B, T, Hq, Hkv, D, bs, N = 2, 4, 16, 4, 128, 32, 512
        ctxs, qlens = [700, 1031], [4, 3]
        d = _setup_multi(rng, B, T, Hq, Hkv, D, bs, ctxs, qlens, N, True, True, fp8=fp8)
        scale = 1.0 / np.sqrt(D)
        want, wk, wv, wks, wvs = _verify_step(pa, d, scale, max(ctxs))
        k, v = d["k"].clone(), d["v"].clone()
        out = torch.empty((B, T, N), dtype=torch.bfloat16, device="cuda")
        common = dict(max_seq_len=max(ctxs), rope_cos=d["qt"].rope_cos, rope_sin=d["qt"].rope_sin,
                      q_norm_weight=d["qt"].norm_weight, k_norm_weight=d["wk"], norm_eps=d["qt"].eps, o_weight=d["ow"],
                      o_bias=d["ob"])
        if fp8:
            ks, vs = d["ks"].clone(), d["vs"].clone()
            torch.ops.nkipy_amd.verify_step_fp8(d["xq"], d["xk"], d["xv"], k, v, ks, vs, d["tables"], d["lens"], d["qlens"],
                                                scale, out, **common)
            _same_bits(ks, wks, "K scales")
        else:
            torch.ops.nkipy_amd.verify_step(d["xq"], d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], scale, out,
                                            **common)
        torch.cuda.synchronize()
        _same_bits(out, want, f"projected rows, fp8={fp8}")
        _same_bits(k, wk, "K pool")
        _same_bits(v, wv, "V pool")


def test_argument_errors(pa):
    rng = np.random.default_rng(10)
    d = _setup(rng, 2, 8, 2, 128, 16, [40, 50], [1, 1], 256, False, True, poison=False)
    scale = 1.0 / np.sqrt(128)
    with pytest.raises(ValueError):
        pa.decode_step(d["xq"], d["xk"][:, :1], d["xv"], d["k"], d["v"], d["tables"], d["lens"], d["qlens"], scale)
    with pytest.raises(ValueError):
        pa.decode_step(d["xq"], d["xk"], d["xv"], d["k"], d["v"], d["tables"], d["lens"], d["qlens"], scale, k_norm_weight=d["wk"])
    with pytest.raises(ValueError):
        pa.decode_step(d["xq"], d["xk"], d["xv"], d["k"], d["v"], d["tables"], d["lens"], d["qlens"].long(), scale)
    with pytest.raises(ValueError):
        pa.decode_step(d["xq"], d["xk"], d["xv"], d["k"], d["v"], d["tables"], d["lens"], d["qlens"], scale,
                       o_weight=d["ow"][:-64])
    with pytest.raises(ValueError):
        pa.decode_step(d["xq"], d["xk"], d["xv"], d["k"], d["v"], d["tables"], d["lens"], d["qlens"], scale,
                       o_weight=d["ow"], workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    with pytest.raises(NotImplementedError):
        pa.decode_step(d["xq"].cpu(), d["xk"], d["xv"], d["k"], d["v"], d["tables"], d["lens"], d["qlens"], scale)


# ---- the same for a few tokens per sequence: verify_step -----------------------------------------------------------

def _setup_multi(rng, B, T, Hq, Hkv, D, bs, ctxs, qlens, N, bias, xform, fp8=False):
    d = _setup(rng, B, Hq, Hkv, D, bs, ctxs, qlens, N, bias, xform, fp8=fp8, poison=not fp8)
    d["xq"] = bf16_to_dev(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    d["xk"] = bf16_to_dev(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    d["xv"] = bf16_to_dev(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    return d


def _verify_three_calls(pa, d, scale, msl, **kw):
    k, v = d["k"].clone(), d["v"].clone()
    ks = None if d["ks"] is None else d["ks"].clone()
    vs = None if d["vs"] is None else d["vs"].clone()
    if d["qt"] is not None:
        pa.qk_norm_rope_kv_write(None, d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], d["qt"].rope_cos,
                                 d["qt"].rope_sin, k_norm_weight=d["wk"], eps=d["qt"].eps, k_scale=ks, v_scale=vs)
    else:
        pa.kv_write(d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], k_scale=ks, v_scale=vs)
    att = pa.verify(d["xq"], k, v, d["tables"], d["lens"], d["qlens"], scale, k_scale=ks, v_scale=vs, max_seq_len=msl,
                    q_transform=d["qt"], **kw)
    out = att if d["ow"] is None else pa.o_proj(att, d["ow"], d["ob"])
    return out, att, k, v, ks, vs


def _verify_step(pa, d, scale, msl, **kw):
    k, v = d["k"].clone(), d["v"].clone()
    ks = None if d["ks"] is None else d["ks"].clone()
    vs = None if d["vs"] is None else d["vs"].clone()
    out = pa.verify_step(d["xq"], d["xk"], d["xv"], k, v, d["tables"], d["lens"], d["qlens"], scale, k_scale=ks, v_scale=vs,
                         max_seq_len=msl, q_transform=d["qt"], k_norm_weight=d["wk"], o_weight=d["ow"], o_bias=d["ob"], **kw)
    return out, k, v, ks, vs


VERIFY_CASES = [
    # B, T, Hq, Hkv, D, bs, contexts (new tokens counted), query lens, N, bias, transform, bound given, fp8
    (1, 4, 32, 8, 128, 32, [1030], [4], 4096, False, True, True, False),           # the reference's own use: one sequence, K + 1 = 4
    (8, 4, 32, 8, 128, 32, [1027, 1000, 513, 515, 516, 64, 3, 300], [4, 3, 4, 4, 4, 2, 3, 0], 4096, True, True, True, False),
    (2, 8, 16, 8, 64, 16, [2050, 700], [8, 5], 512, False, True, True, False),     # head dim 64, five partitions
    (3, 16, 8, 8, 128, 32, [900, 40, 16], [16, 7, 16], 256, True, False, True, False),   # no GQA: 16 rows per kv head
    (4, 4, 32, 8, 128, 32, [1500, 600, 90, 5], [4, 4, 1, 4], 1024, False, True, False, False),   # no bound: the balanced schedule
    (4, 4, 32, 8, 128, 32, [1500, 600, 90, 5], [4, 4, 1, 4], 1024, True, True, True, True),     # fp8 pool
    (16, 4, 32, 8, 128, 32, [700 + 31 * i for i in range(16)], [4] * 16, 1024, False, True, True, False),   # 64 rows: the projection reads them from memory
    (2, 8, 32, 8, 128, 32, [1200, 800], [8, 8], 1024, False, True, True, False),   # 32 rows per kv head: not a small call
    (6, 4, 32, 8, 128, 16, [514, 513, 515, 34, 4, 1026], [4, 4, 4, 4, 4, 4], 512, False, True, True, False),   # new tokens across a partition, tile, block border; a sequence of only new tokens
    (3, 16, 8, 8, 64, 32, [530, 16, 1040], [16, 16, 9], 256, True, True, True, False),     # 16 new tokens, head dim 64, across borders
    (2, 4, 32, 8, 128, 32, [600, 900], [4, 4], 512, False, False, True, False),    # no transform: rows stored as given
]


@pytest.mark.parametrize("B,T,Hq,Hkv,D,bs,ctxs,qlens,N,window", [
    (1, 4, 64, 8, 64, 32, [1030], [4], 2880, None),           # the gpt-oss layer at the reference's operating point
    (1, 4, 64, 8, 64, 32, [1030], [4], 2880, 128),            # ... its windowed layers: one partition
    (3, 4, 32, 8, 128, 32, [1500, 515, 4], [4, 3, 4], 1024, 600),
    (2, 4, 32, 8, 128, 16, [700, 258], [4, 4], 512, None),    # two partitions of 512: merged on the projection's load
])
def test_verify_step_with_sinks_and_window(pa, B, T, Hq, Hkv, D, bs, ctxs, qlens, N, window):
    rng = np.random.default_rng(B * 10 + T + Hq + (window or 0))
    d = _setup_multi(rng, B, T, Hq, Hkv, D, bs, ctxs, qlens, N, True, True)
    scale, msl = 1.0 / np.sqrt(D), int(max(ctxs))
    kw = dict(sinks=torch.from_numpy(rng.standard_normal(Hq).astype(np.float32)).cuda(), sliding_window=window)
    print(f"verify_step with sinks B={B} T={T} Hq={Hq} D={D} ctx={ctxs} window={window}", flush=True)
    want, att, wk, wv, _, _ = _verify_three_calls(pa, d, scale, msl, **kw)
    for fusion in (0, 2, 3, 1):
        _fusion(fusion)
        try:
            got, gk, gv, _, _ = _verify_step(pa, d, scale, msl, **kw)
            torch.cuda.synchronize()
        finally:
            _fusion(0)
        _same_bits(got, want, f"projected rows, fusion switch {fusion}")
        _same_bits(gk, wk, "K pool")
        _same_bits(gv, wv, "V pool")


@pytest.mark.parametrize("B,T,Hq,Hkv,D,bs,ctxs,qlens,N,bias,xform,bounded,fp8", VERIFY_CASES)
def test_verify_step_equals_the_three_calls(pa, B, T, Hq, Hkv, D, bs, ctxs, qlens, N, bias, xform, bounded, fp8):
    rng = np.random.default_rng(B * 100 + T * 7 + Hq + D + N)
    d = _setup_multi(rng, B, T, Hq, Hkv, D, bs, ctxs, qlens, N, bias, xform, fp8=fp8)
    scale, msl = 1.0 / np.sqrt(D), (int(max(ctxs)) if bounded else None)
    print(f"verify_step B={B} T={T} Hq={Hq} Hkv={Hkv} D={D} bs={bs} ctx={ctxs[:4]}.. q={qlens[:4]}.. N={N} fp8={fp8}", flush=True)
    want, att, wk, wv, wks, wvs = _verify_three_calls(pa, d, scale, msl)
    for fusion in (0, 2, 3, 1):
        _fusion(fusion)
        try:
            got, gk, gv, gks, gvs = _verify_step(pa, d, scale, msl)
            torch.cuda.synchronize()
        finally:
            _fusion(0)
        _same_bits(got, want, f"projected rows, fusion switch {fusion}")
        _same_bits(gk, wk, "K pool")
        _same_bits(gv, wv, "V pool")
        if fp8:
            _same_bits(gks, wks, "K scales")
    a2 = torch.empty_like(d["xq"])
    got, _, _, _, _ = _verify_step(pa, d, scale, msl, attn_out=a2)
    _same_bits(got, want, "projected rows with attn_out")
    _same_bits(a2, att, "attention output beside the projection")
    got, _, _, _, _ = _verify_step(pa, dict(d, ow=None, ob=None), scale, msl)
    torch.cuda.synchronize()
    _same_bits(got, att, "attention output alone")
    g = dev_to_f32(got)
    assert not np.isnan(g).any()
    for b in range(B):
        assert np.array_equal(g[b, qlens[b]:], np.zeros_like(g[b, qlens[b]:]))     # padding rows


def test_verify_step_argument_errors(pa):
    rng = np.random.default_rng(12)
    d = _setup_multi(rng, 2, 4, 8, 2, 128, 16, [40, 50], [4, 4], 256, False, True)
    scale = 1.0 / np.sqrt(128)
    args = (d["k"], d["v"], d["tables"], d["lens"], d["qlens"], scale)
    with pytest.raises(ValueError):
        pa.verify_step(d["xq"], d["xk"][:, :2], d["xv"], *args)
    with pytest.raises(ValueError):
        pa.verify_step(d["xq"], d["xk"], d["xv"], *args, k_norm_weight=d["wk"])
    with pytest.raises(ValueError):
        pa.verify_step(d["xq"].float(), d["xk"], d["xv"], *args)
    with pytest.raises(ValueError):
        big = torch.zeros((2, 65, 8, 128), dtype=torch.bfloat16, device="cuda")
        pa.verify_step(big, big[:, :, :2], big[:, :, :2], *args)
    with pytest.raises(NotImplementedError):
        pa.verify_step(d["xq"].cpu(), d["xk"], d["xv"], *args)
