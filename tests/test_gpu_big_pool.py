"""GPU: pools larger than 4 GiB.  A serving pool on a 288 GB device is tens of GiB, so every byte offset
into it must be computed in 64 bits.  Each case runs an op twice on the same data: once on a small pool,
once with the same blocks placed at block ids spread over a 6.5 - 9.2 GB pool (byte and element offsets
on both sides of 2^31 and 2^32) and the tables renumbered.  Same kernel, same values, only the addresses
differ: the outputs must agree bit for bit.  The rest of the big pool is uninitialised memory."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import bf16_to_dev, dev_bits, make_paged

pytestmark = pytest.mark.gpu

HKV, D, BS = 8, 128, 32
BIG_BF16 = 140_000          # blocks of 64 KiB: 9.2 GB, more than 2^32 elements
BIG_FP8 = 200_000           # blocks of 32 KiB: 6.5 GB, more than 2^32 elements


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


@pytest.fixture(scope="module")
def big_bf16():
    k = torch.empty((BIG_BF16, BS, HKV, D), dtype=torch.bfloat16, device="cuda")
    v = torch.empty_like(k)
    yield k, v
    del k, v
    torch.cuda.empty_cache()


@pytest.fixture(scope="module")
def big_fp8():
    k = torch.empty((BIG_FP8, BS, HKV, D), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    v = torch.empty_like(k)
    ks = torch.empty((BIG_FP8, HKV), dtype=torch.float32, device="cuda")
    vs = torch.empty_like(ks)
    yield k, v, ks, vs
    del k, v, ks, vs
    torch.cuda.empty_cache()


def _i32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.int32)).cuda()


def _spread(n_small, n_big):
    """Distinct big block ids for small ids 0 .. n_small-1, from the top of the pool downwards."""
    stride = (n_big * 3 // 4) // max(n_small, 1)
    ids = n_big - 1 - stride * np.arange(n_small, dtype=np.int64)
    assert ids.min() >= 0 and len(np.unique(ids)) == n_small
    return ids


def _place(small, big, ids):
    big.view(torch.uint8)[torch.from_numpy(ids).cuda()] = small.view(torch.uint8)


def _take(big, dev_ids):
    return big.view(torch.uint8)[dev_ids]


def _remap(tables, ids):
    out = tables.copy()
    live = tables >= 0
    out[live] = ids[tables[live]]
    return out.astype(np.int32)


def _case(rng, ctxs, fp8):
    B = len(ctxs)
    k, v, tables = make_paged(rng, B, HKV, D, BS, [max(c, 1) for c in ctxs])
    if fp8:
        kq, ks = O.quantize_kv_fp8(O.round_to_bf16(k))
        vq, vs = O.quantize_kv_fp8(O.round_to_bf16(v))
        small = (torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn), torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn))
        scales = (torch.from_numpy(ks).cuda(), torch.from_numpy(vs).cuda())
    else:
        small, scales = (bf16_to_dev(k), bf16_to_dev(v)), None
    return small, scales, tables


def _both(pa, run, rng, ctxs, fp8, big):
    """run(k, v, tables, kw) on the small pool and on the big one; returns the two results' bits."""
    small, scales, tables = _case(rng, ctxs, fp8)
    ids = _spread(small[0].shape[0], big[0].shape[0])
    assert int(ids.max()) * BS * HKV * D * small[0].element_size() > 2 ** 32 > int(ids.min()) * BS * HKV * D * small[0].element_size()
    _place(small[0], big[0], ids)
    _place(small[1], big[1], ids)
    kw_s, kw_b = {}, {}
    if fp8:
        _place(scales[0], big[2], ids)
        _place(scales[1], big[3], ids)
        kw_s = dict(k_scale=scales[0], v_scale=scales[1])
        kw_b = dict(k_scale=big[2], v_scale=big[3])
    a = run(small[0], small[1], _i32(tables), kw_s)
    b = run(big[0], big[1], _i32(_remap(tables, ids)), kw_b)
    torch.cuda.synchronize()
    return dev_bits(a), dev_bits(b)


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("impl", [0, 1, 2], ids=["balanced", "scalar", "fixed"])
def test_decode(pa, big_bf16, big_fp8, fp8, impl):
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(31 + impl)
    ctxs = [5000, 77, 1300, 2049]
    q = bf16_to_dev(rng.standard_normal((len(ctxs), 32, D)).astype(np.float32))
    lib.pa_debug_set(0, impl)
    try:
        a, b = _both(pa, lambda k, v, t, kw: pa.decode(q, k, v, t, _i32(ctxs), 0.09, **kw), rng, ctxs, fp8,
                     big_fp8 if fp8 else big_bf16)
    finally:
        lib.pa_debug_set(0, 0)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("route,T,prefixes", [("verify", 4, [3000, 0, 611]), ("tiled", 300, [2500, 0, 77]),
                                               ("tiled", 256, [6000])])
def test_prefill_routes(pa, big_bf16, big_fp8, fp8, route, T, prefixes):
    rng = np.random.default_rng(41 + T)
    qlens = [T] * len(prefixes)
    ctxs = [p + T for p in prefixes]
    q = bf16_to_dev(rng.standard_normal((len(ctxs), T, 16, D)).astype(np.float32))
    run = lambda k, v, t, kw: pa.prefill(q, k, v, t, _i32(ctxs), _i32(qlens), 0.09, route=route, **kw)   # noqa: E731
    a, b = _both(pa, run, rng, ctxs, fp8, big_fp8 if fp8 else big_bf16)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
def test_register_staged_prefill(pa, big_bf16, big_fp8, fp8):
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(51)
    T, prefixes = 200, [2500, 40]
    ctxs = [p + T for p in prefixes]
    q = bf16_to_dev(rng.standard_normal((2, T, 8, D)).astype(np.float32))
    lib.pa_debug_set(3, 1)
    try:
        run = lambda k, v, t, kw: pa.prefill(q, k, v, t, _i32(ctxs), _i32([T, T]), 0.09, route="tiled", **kw)   # noqa: E731
        a, b = _both(pa, run, rng, ctxs, fp8, big_fp8 if fp8 else big_bf16)
    finally:
        lib.pa_debug_set(3, 0)
    assert np.array_equal(a, b)


def test_gather(pa, big_bf16):
    rng = np.random.default_rng(61)
    ctxs = [700, 33]
    a, b = _both(pa, lambda k, v, t, kw: pa.gather_kv(k, t, _i32(ctxs)), rng, ctxs, False, big_bf16)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("mode", ["bf16", "fp8", "bf16_rope", "fp8_rope"])
def test_kv_write(pa, big_bf16, big_fp8, mode):
    """New rows written into the big pool land where the small pool's land (blocks compared after the write)."""
    rng = np.random.default_rng(71)
    fp8, rope = mode.startswith("fp8"), mode.endswith("rope")
    big = big_fp8 if fp8 else big_bf16
    B, T = 3, 70
    seqs, qlens = [700, 70, 133], [70, 70, 40]
    small, scales, tables = _case(rng, seqs, fp8)
    ids = _spread(small[0].shape[0], big[0].shape[0])
    dev_ids = torch.from_numpy(ids).cuda()
    _place(small[0], big[0], ids)
    _place(small[1], big[1], ids)
    if fp8:
        _place(scales[0], big[2], ids)
        _place(scales[1], big[3], ids)
    xk = bf16_to_dev(rng.standard_normal((B, T, HKV, D)).astype(np.float32) * 3)
    xv = bf16_to_dev(rng.standard_normal((B, T, HKV, D)).astype(np.float32))
    cos, sin = pa.rope_tables(D, 1024)

    def write(k, v, t, kw):
        if rope:
            pa.qk_norm_rope_kv_write(None, xk, xv, k, v, t, _i32(seqs), _i32(qlens), cos, sin, **kw)
        else:
            pa.kv_write(xk, xv, k, v, t, _i32(seqs), _i32(qlens), **kw)

    write(small[0], small[1], _i32(tables), dict(k_scale=scales[0], v_scale=scales[1]) if fp8 else {})
    write(big[0], big[1], _i32(_remap(tables, ids)), dict(k_scale=big[2], v_scale=big[3]) if fp8 else {})
    torch.cuda.synchronize()
    u8 = lambda t: dev_bits(t.view(torch.uint8))      # noqa: E731
    assert np.array_equal(u8(small[0]), dev_bits(_take(big[0], dev_ids)))
    assert np.array_equal(u8(small[1]), dev_bits(_take(big[1], dev_ids)))
    if fp8:
        assert np.array_equal(u8(scales[0]), dev_bits(_take(big[2], dev_ids)))
        assert np.array_equal(u8(scales[1]), dev_bits(_take(big[3], dev_ids)))


@pytest.mark.parametrize("T", [4, 300], ids=["verify", "tiled"])
def test_head_dim_64(pa, big_fp8, T):
    """The same memory seen as a bf16 pool of head dim 64 (a row of 8 heads x 64 x 2 B is as long as one of
    8 x 128 fp8 codes): the decode kernels and the tiled prefill kernel's two-heads-per-row form."""
    rng = np.random.default_rng(81 + T)
    D64 = 64
    big = tuple(t.view(torch.uint8).view(torch.bfloat16) for t in big_fp8[:2])        # [BIG_FP8, BS, HKV, 64]
    assert big[0].shape == (BIG_FP8, BS, HKV, D64)
    prefixes = [2500, 0, 77]
    ctxs = [p + T for p in prefixes]
    k, v, tables = make_paged(rng, len(ctxs), HKV, D64, BS, ctxs)
    small = (bf16_to_dev(k), bf16_to_dev(v))
    ids = _spread(small[0].shape[0], BIG_FP8)
    _place(small[0], big[0], ids)
    _place(small[1], big[1], ids)
    q = bf16_to_dev(rng.standard_normal((len(ctxs), T, 16, D64)).astype(np.float32))
    run = lambda kk, vv, t: pa.prefill(q, kk, vv, t, _i32(ctxs), _i32([T] * len(ctxs)), 0.125)   # noqa: E731
    a = run(small[0], small[1], _i32(tables))
    b = run(big[0], big[1], _i32(_remap(tables, ids)))
    qd = q[:, 0].contiguous()
    c = pa.decode(qd, small[0], small[1], _i32(tables), _i32(ctxs), 0.125)
    d = pa.decode(qd, big[0], big[1], _i32(_remap(tables, ids)), _i32(ctxs), 0.125)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(a), dev_bits(b))
    assert np.array_equal(dev_bits(c), dev_bits(d))
