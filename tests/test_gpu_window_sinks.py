"""GPU parity: sliding window and attention sinks (the gpt-oss attention variant,
examples/models/gpt_oss/kernels/attention.py:117-148) in decode and speculative verify vs the oracle."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, bf16_to_dev, dev_bits, dev_to_f32, make_paged

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2
FP8_TOL = 5e-2


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


def _i32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.int32)).cuda()


def _f32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).cuda()


CTXS = [1, 31, 32, 33, 64, 65, 200, 1500, 4097]


@pytest.mark.parametrize("window", [None, 1, 2, 31, 32, 33, 128, 5000])
@pytest.mark.parametrize("with_sinks", [False, True])
@pytest.mark.parametrize("D,Hq,Hkv,bs", [(64, 8, 1, 16), (128, 32, 8, 32)])
def test_decode_window_and_sinks(pa, window, with_sinks, D, Hq, Hkv, bs):
    if window is None and not with_sinks:
        pytest.skip("plain decode is covered elsewhere")
    rng = np.random.default_rng(7 + (window or 0) + D)
    B = len(CTXS)
    k, v, tables = make_paged(rng, B, Hkv, D, bs, CTXS)
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    q = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32) * 2) if with_sinks else None
    scale = 1.0 / np.sqrt(D)
    want = O.paged_decode(q, k, v, tables, np.asarray(CTXS, np.int32), scale, q_dtype="bf16",
                          sliding_window=window, sinks=sinks)
    got = pa.decode(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(CTXS), scale,
                    sliding_window=window, sinks=None if sinks is None else bf16_to_dev(sinks))
    torch.cuda.synchronize()
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_decode_window_fp8_long_single_sequence(pa):
    """One 20 000-token sequence cut into every chunk of the schedule; with a 128-token window only the
    last five tiles are streamed."""
    rng = np.random.default_rng(21)
    D, Hq, Hkv, bs, ctx = 128, 16, 2, 64, 20000
    k, v, tables = make_paged(rng, 1, Hkv, D, bs, [ctx])
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    q = O.round_to_bf16(rng.standard_normal((1, Hq, D)).astype(np.float32))
    sinks = rng.standard_normal(Hq).astype(np.float32)
    for window in (128, 3000, None):
        want = O.paged_decode(q, kq, vq, tables, np.asarray([ctx], np.int32), 0.09, k_scale=ks, v_scale=vs,
                              q_dtype="bf16", sliding_window=window, sinks=sinks)
        got = pa.decode(bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
                        torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(tables), _i32([ctx]), 0.09,
                        k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda(),
                        sliding_window=window, sinks=_f32(sinks))
        torch.cuda.synchronize()
        assert_close_abs(dev_to_f32(got), want, FP8_TOL)


def test_neutral_options_change_nothing(pa):
    """A window at least as long as every context and sinks of -inf give the plain result bit for bit, in the
    balanced kernel and in the fixed-partition kernel (which serves a call this small by default, and whose sums are
    taken in another order than the balanced kernel's: equal to the tolerance between the two)."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(22)
    D, Hq, Hkv, bs = 128, 8, 2, 32
    ctxs = [5, 700, 2049]
    k, v, tables = make_paged(rng, len(ctxs), Hkv, D, bs, ctxs)
    q = rng.standard_normal((len(ctxs), Hq, D)).astype(np.float32)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), 0.09)
    lib.pa_debug_set(0, 3)
    try:
        plain = pa.decode(*args)
        assert np.array_equal(dev_bits(pa.decode(*args, sliding_window=2049)), dev_bits(plain))
        assert np.array_equal(dev_bits(pa.decode(*args, sinks=_f32(np.full(Hq, -np.inf)))), dev_bits(plain))
        assert not np.array_equal(dev_bits(pa.decode(*args, sliding_window=2048)), dev_bits(plain))
    finally:
        lib.pa_debug_set(0, 0)
    small = pa.decode(*args)
    assert_close_abs(dev_to_f32(small), dev_to_f32(plain), BF16_TOL)
    assert np.array_equal(dev_bits(pa.decode(*args, sliding_window=2049)), dev_bits(small))
    assert np.array_equal(dev_bits(pa.decode(*args, sinks=_f32(np.full(Hq, -np.inf)))), dev_bits(small))
    assert not np.array_equal(dev_bits(pa.decode(*args, sliding_window=2048)), dev_bits(small))


@pytest.mark.parametrize("window,part", [(None, 1024), (1, 512), (33, 32), (100, 64), (128, 512), (129, 64), (600, 256),
                                         (1000, 128), (5000, 1024)])
@pytest.mark.parametrize("with_sinks", [False, True])
@pytest.mark.parametrize("D,Hq,Hkv,bs", [(64, 64, 8, 16), (128, 32, 8, 32), (128, 16, 1, 32)])
def test_decode_window_and_sinks_on_fixed_partitions(pa, window, part, with_sinks, D, Hq, Hkv, bs):
    """Small calls with a length bound: the fixed-partition kernel, whose partitions count from the first tile the
    window reaches (one partition on eight waves, one on four, several with the merge launch), forced and by the
    library's own choice; contexts shorter than the window, ending on tile and partition boundaries."""
    from nkipy_amd import _lib
    lib = _lib.load()
    if window is None and not with_sinks:
        pytest.skip("plain decode is covered elsewhere")
    rng = np.random.default_rng(11 + (window or 0) + D + part)
    ctxs = [1, 31, 32, 33, 64, 65, 200, 1500, 4097][: 5 if Hkv == 8 else 9] + [part, part + 1, 2 * part + 32]
    B = len(ctxs)
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    q = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32) * 2) if with_sinks else None
    scale = 1.0 / np.sqrt(D)
    want = O.paged_decode(q, k, v, tables, np.asarray(ctxs, np.int32), scale, q_dtype="bf16",
                          sliding_window=window, sinks=sinks)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), scale)
    kw = dict(sliding_window=window, sinks=None if sinks is None else bf16_to_dev(sinks), partition_size=part,
              max_seq_len=max(ctxs))
    for impl in (2, 0):
        lib.pa_debug_set(0, impl)
        try:
            got = pa.decode(*args, **kw)
            torch.cuda.synchronize()
        finally:
            lib.pa_debug_set(0, 0)
        assert_close_abs(dev_to_f32(got), want, BF16_TOL)


@pytest.fixture(params=[16, 32], ids=["rows16", "rows32"])
def rows(request):
    from nkipy_amd import _lib
    lib = _lib.load()
    lib.pa_debug_set(5, request.param)
    yield request.param
    lib.pa_debug_set(5, 0)


@pytest.mark.parametrize("window", [1, 3, 30, 33, 64, 128, 4000])
@pytest.mark.parametrize("T,Hq,Hkv,D,bs", [(4, 16, 2, 64, 16), (4, 32, 8, 128, 32), (40, 2, 1, 128, 32)])
def test_verify_window_and_sinks(pa, rows, window, T, Hq, Hkv, D, bs):
    """Query tokens of one sequence have different window starts, up to T - 1 tokens apart: rows that see
    nothing in the first tiles of the span, and (T = 40) windows shorter than the query run."""
    rng = np.random.default_rng(100 * T + window)
    qlens = [T, max(T - 1, 1), 1, T, 0, T]
    prefixes = [0, 300, 65, 1533, 40, 31]
    B = len(qlens)
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [max(c, 1) for c in ctxs])
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32))
    scale = 1.0 / np.sqrt(D)
    want = O.paged_prefill(q, k, v, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), scale,
                           q_dtype="bf16", sliding_window=window, sinks=sinks)
    got = pa.prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(qlens), scale,
                     sliding_window=window, sinks=bf16_to_dev(sinks))
    torch.cuda.synchronize()
    got = dev_to_f32(got)
    assert_close_abs(got, want, BF16_TOL)
    for b, n in enumerate(qlens):
        assert np.all(got[b, n:] == 0)


@pytest.mark.parametrize("window", [None, 1, 30, 64, 128, 700])
@pytest.mark.parametrize("T,Hq,Hkv,D,bs", [(4, 64, 8, 64, 16), (4, 32, 8, 128, 32), (3, 8, 2, 128, 32)])
def test_verify_window_and_sinks_small_calls(pa, window, T, Hq, Hkv, D, bs):
    """With the caller's length bound a small verify call takes the fixed partitions, sinks and window included:
    rows of one sequence whose windows begin in different tiles, 16 and 32 rows per kv head."""
    rng = np.random.default_rng(100 * T + (window or 7) + D)
    qlens = [T, max(T - 1, 1), 1, T, 0]
    prefixes = [0, 300, 65, 1533, 40]
    B = len(qlens)
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [max(c, 1) for c in ctxs])
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32))
    scale = 1.0 / np.sqrt(D)
    want = O.paged_prefill(q, k, v, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), scale,
                           q_dtype="bf16", sliding_window=window, sinks=sinks)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(qlens), scale)
    got = pa.verify(*args, sliding_window=window, sinks=bf16_to_dev(sinks), max_seq_len=max(ctxs))
    free = pa.verify(*args, sliding_window=window, sinks=bf16_to_dev(sinks))
    torch.cuda.synchronize()
    got = dev_to_f32(got)
    assert_close_abs(got, want, BF16_TOL)
    assert_close_abs(dev_to_f32(free), want, BF16_TOL)
    for b, n in enumerate(qlens):
        assert np.all(got[b, n:] == 0)


def test_variant_argument_errors(pa):
    rng = np.random.default_rng(23)
    k, v, tables = make_paged(rng, 1, 2, 128, 32, [40])
    q = bf16_to_dev(rng.standard_normal((1, 4, 128)).astype(np.float32))
    args = (q, bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32([40]), 0.09)
    with pytest.raises(ValueError):
        pa.decode(*args, sliding_window=0)
    with pytest.raises(ValueError):
        pa.decode(*args, sinks=_f32(np.zeros(3)))
    with pytest.raises(RuntimeError):      # fp32 decode runs the scalar kernel, which has no window
        pa.decode(q.float(), args[1].float(), args[2].float(), *args[3:], sliding_window=8)
    k8, v8, t8 = make_paged(rng, 1, 2, 128, 24, [140])
    q4 = bf16_to_dev(rng.standard_normal((1, 100, 4, 128)).astype(np.float32))
    with pytest.raises(RuntimeError):      # a block size of 24 takes the register-staged prefill kernel, which has no window
        pa.prefill(q4, bf16_to_dev(k8), bf16_to_dev(v8), _i32(t8), _i32([140]), _i32([100]), 0.09, sliding_window=8)


@pytest.mark.parametrize("window", [1, 50, 64, 65, 128, 300, 5000])
@pytest.mark.parametrize("waves", [4, 8])
def test_tiled_prefill_window_and_sinks(pa, window, waves):
    """Long query runs through the tiled kernel: windows shorter and longer than a 64-key tile, than a
    wave's 32 rows and than the whole chunk; first tiles in which a wave's later rows see nothing."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(300 + window)
    T, Hq, Hkv, D, bs = 200, 4, 2, 128, 32
    qlens, prefixes = [200, 77, 1, 130], [0, 300, 65, 1000]
    B = len(qlens)
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32))
    scale = 1.0 / np.sqrt(D)
    want = O.paged_prefill(q, k, v, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), scale,
                           q_dtype="bf16", sliding_window=window, sinks=sinks)
    lib.pa_debug_set(3, waves)
    try:
        got = pa.prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(qlens), scale,
                         sliding_window=window, sinks=bf16_to_dev(sinks), route="tiled")
        torch.cuda.synchronize()
    finally:
        lib.pa_debug_set(3, 0)
    got = dev_to_f32(got)
    assert_close_abs(got, want, BF16_TOL)
    assert np.all(got[1, 77:] == 0) and np.all(got[2, 1:] == 0)


def test_tiled_prefill_neutral_options_change_nothing(pa):
    rng = np.random.default_rng(31)
    T, Hq, Hkv, D, bs = 300, 4, 2, 128, 32
    ctxs = [300 + 700, 150 + 0]
    k, v, tables = make_paged(rng, 2, Hkv, D, bs, ctxs)
    q = rng.standard_normal((2, T, Hq, D)).astype(np.float32)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32([300, 150]), 0.09)
    plain = dev_bits(pa.prefill(*args))
    assert np.array_equal(dev_bits(pa.prefill(*args, sliding_window=1000)), plain)
    assert np.array_equal(dev_bits(pa.prefill(*args, sinks=_f32(np.full(Hq, -np.inf)))), plain)
    assert not np.array_equal(dev_bits(pa.prefill(*args, sliding_window=999)), plain)
