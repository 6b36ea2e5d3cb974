"""GPU parity: the Q half of the pre-attention step (QK RMSNorm + RoPE) done by the attention kernels
as they load Q (`q_transform`) gives the bits of the two-step form (qk_norm_rope_kv_write, then the
attention call), and matches the oracle's norm + rotation + attention."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, bf16_to_dev, dev_bits, dev_to_f32, make_paged

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


def _i32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.int32)).cuda()


def _pool(rng, B, Hkv, D, bs, ctxs, fp8):
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [max(int(c), 1) for c in ctxs])
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    if not fp8:
        return dict(k=k, v=v, tables=tables, dev=(bf16_to_dev(k), bf16_to_dev(v)), kw={}, okw={})
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    dev = (torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn), torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn))
    return dict(k=kq, v=vq, tables=tables, dev=dev, okw=dict(k_scale=ks, v_scale=vs),
                kw=dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda()))


def _two_step_q(pa, xq, ctxs, qlens, dcos, dsin, w):
    """Q as the stand-alone transform kernel writes it (its K/V scatter goes to a throw-away pool)."""
    B, T, _, D = xq.shape
    nblk = (int(max(ctxs)) + 15) // 16 + 1
    tables = _i32(np.arange(B * nblk).reshape(B, nblk))
    pool = torch.zeros((B * nblk, 16, 1, D), dtype=torch.bfloat16, device="cuda")
    kv = torch.zeros((B, T, 1, D), dtype=torch.bfloat16, device="cuda")
    return pa.qk_norm_rope_kv_write(xq, kv, kv, pool, pool.clone(), tables, _i32(ctxs), _i32(qlens), dcos, dsin,
                                    q_norm_weight=w)


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("norm", [False, True], ids=["rope", "norm_rope"])
@pytest.mark.parametrize("D,bs,Hq,Hkv", [(128, 32, 32, 8), (64, 16, 8, 2), (128, 16, 5, 1)])
def test_decode_matches_two_step_bits(pa, fp8, norm, D, bs, Hq, Hkv):
    rng = np.random.default_rng(D + Hq + 2 * fp8 + norm)
    ctxs = [1, 77, 1300, 4097, 33]
    B = len(ctxs)
    pool = _pool(rng, B, Hkv, D, bs, ctxs, fp8)
    xq = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32) * 2)
    w = O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32)) if norm else None
    cos, sin = O.rope_tables(D, 4200, 10000.0)
    dcos, dsin = pa.rope_tables(D, 4200, 10000.0)
    dw = bf16_to_dev(w) if norm else None
    scale = 1.0 / np.sqrt(D)
    dq = bf16_to_dev(xq)
    q2 = _two_step_q(pa, dq[:, None].contiguous(), ctxs, [1] * B, dcos, dsin, dw)[:, 0].contiguous()
    args = (*pool["dev"], _i32(pool["tables"]), _i32(ctxs), scale)
    want_bits = dev_bits(pa.decode(q2, *args, **pool["kw"]))
    got = pa.decode(dq, *args, **pool["kw"], q_transform=pa.QTransform(dcos, dsin, dw, 1e-6))
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(got), want_bits)
    # and the oracle's own transform followed by its attention
    oq, _ = O.qk_norm_rope(xq[:, None], xq[:, None, :Hkv], np.asarray(ctxs), np.ones(B, np.int32), cos, sin,
                           q_norm_weight=w, k_norm_weight=None, eps=1e-6)
    want = O.paged_decode(oq[:, 0], pool["k"], pool["v"], pool["tables"], np.asarray(ctxs, np.int32), scale,
                          q_dtype="bf16", **pool["okw"])
    assert_close_abs(dev_to_f32(got), want, BF16_TOL if not fp8 else 5e-2)


@pytest.mark.parametrize("rows", [16, 32])
@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("D,bs,T,Hq,Hkv", [(128, 32, 4, 32, 8), (64, 16, 6, 8, 1), (128, 64, 8, 16, 4)])
def test_verify_matches_two_step_bits(pa, rows, fp8, D, bs, T, Hq, Hkv):
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(D + T + fp8)
    qlens, prefixes = [T, 1, T - 1, 0, T], [0, 300, 1500, 40, 31]
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    B = len(ctxs)
    pool = _pool(rng, B, Hkv, D, bs, ctxs, fp8)
    xq = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32) * 2)
    w = O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32))
    dcos, dsin = pa.rope_tables(D, 2048, 1000000.0)
    dq, dw = bf16_to_dev(xq), bf16_to_dev(w)
    q2 = _two_step_q(pa, dq, ctxs, qlens, dcos, dsin, dw)
    args = (*pool["dev"], _i32(pool["tables"]), _i32(ctxs), _i32(qlens), 0.09)
    lib.pa_debug_set(5, rows)
    try:
        want_bits = dev_bits(pa.verify(q2, *args, **pool["kw"]))
        got = pa.verify(dq, *args, **pool["kw"], q_transform=pa.QTransform(dcos, dsin, dw))
        torch.cuda.synchronize()
    finally:
        lib.pa_debug_set(5, 0)
    assert np.array_equal(dev_bits(got), want_bits)


@pytest.mark.parametrize("kind", ["plain", "packed", "split", "window", "fp8", "fp8_split"])
def test_tiled_prefill_matches_two_step_bits(pa, kind):
    rng = np.random.default_rng(len(kind))
    D, bs = 128, 32
    fp8 = kind.startswith("fp8")
    if kind == "packed":
        T, Hq, Hkv, qlens, prefixes = 32, 8, 2, [32, 7, 32], [100, 0, 515]
    elif kind in ("split", "fp8_split"):
        T, Hq, Hkv, qlens, prefixes = 256, 2, 1, [256], [6000]
    else:
        T, Hq, Hkv, qlens, prefixes = 200, 4, 2, [200, 131, 1, 0], [0, 300, 64, 9]
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    B = len(ctxs)
    pool = _pool(rng, B, Hkv, D, bs, ctxs, fp8)
    xq = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32) * 2)
    w = O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32))
    cos, sin = O.rope_tables(D, 6400, 10000.0)
    dcos, dsin = pa.rope_tables(D, 6400, 10000.0)
    dq, dw = bf16_to_dev(xq), bf16_to_dev(w)
    q2 = _two_step_q(pa, dq, ctxs, qlens, dcos, dsin, dw)
    kw = dict(pool["kw"], route="tiled")
    if kind == "window":
        kw["sliding_window"] = 100
    args = (*pool["dev"], _i32(pool["tables"]), _i32(ctxs), _i32(qlens), 0.09)
    want_bits = dev_bits(pa.prefill(q2, *args, **kw))
    got = pa.prefill(dq, *args, **kw, q_transform=pa.QTransform(dcos, dsin, dw))
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(got), want_bits)
    if kind == "plain":
        oq, _ = O.qk_norm_rope(xq, xq[:, :, :Hkv], np.asarray(ctxs), np.asarray(qlens), cos, sin,
                               q_norm_weight=w, k_norm_weight=None, eps=1e-6)
        want = O.paged_prefill(oq, pool["k"], pool["v"], pool["tables"], np.asarray(ctxs, np.int32),
                               np.asarray(qlens, np.int32), 0.09, q_dtype="bf16")
        assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_k_only_write_equals_the_full_call(pa):
    """qk_norm_rope_kv_write without xq leaves the pool as the full call does."""
    rng = np.random.default_rng(5)
    B, T, Hq, Hkv, D, bs = 2, 20, 8, 2, 128, 16
    seqs, qlens = [50, 20], [20, 13]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, seqs)
    xq = bf16_to_dev(O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32)))
    xk = bf16_to_dev(O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32)))
    xv = bf16_to_dev(O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32)))
    w = bf16_to_dev(O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32)))
    dcos, dsin = pa.rope_tables(D, 64, 10000.0)
    pools = []
    for q in (xq, None):
        dk, dv = bf16_to_dev(O.round_to_bf16(k)), bf16_to_dev(O.round_to_bf16(v))
        r = pa.qk_norm_rope_kv_write(q, xk, xv, dk, dv, _i32(tables), _i32(seqs), _i32(qlens), dcos, dsin, k_norm_weight=w)
        assert (r is None) == (q is None)
        pools.append((dev_bits(dk), dev_bits(dv)))
    assert np.array_equal(pools[0][0], pools[1][0]) and np.array_equal(pools[0][1], pools[1][1])


def test_argument_errors(pa):
    rng = np.random.default_rng(6)
    pool = _pool(rng, 1, 1, 128, 32, [40], False)
    dcos, dsin = pa.rope_tables(128, 64, 10000.0)
    q = bf16_to_dev(np.zeros((1, 4, 2, 128), np.float32))
    args = (*pool["dev"], _i32(pool["tables"]), _i32([40]), _i32([4]), 0.09)
    with pytest.raises(ValueError):
        pa.prefill(q, *args, q_transform=(dcos, dsin))                       # not a QTransform
    with pytest.raises(ValueError):
        pa.prefill(q, *args, q_transform=pa.QTransform(dcos[:, :32].contiguous(), dsin))
    from nkipy_amd import _lib
    lib = _lib.load()
    lib.pa_debug_set(3, 1)                 # the register-staged prefill kernel has no transform
    try:
        with pytest.raises(RuntimeError, match="q_transform"):
            pa.prefill(q, *args, route="tiled", q_transform=pa.QTransform(dcos, dsin))
    finally:
        lib.pa_debug_set(3, 0)
    f32 = torch.zeros((1, 2, 128), dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError):
        pa.decode(f32, f32.new_zeros((2, 32, 1, 128)), f32.new_zeros((2, 32, 1, 128)), _i32(pool["tables"]), _i32([40]),
                  0.09, q_transform=pa.QTransform(dcos, dsin))
