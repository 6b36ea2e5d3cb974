"""GPU parity: HIP paged decode (through the C ABI) vs the NumPy oracle."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import (assert_close_abs, assert_close_fp32, bf16_to_dev, dev_bits, dev_to_f32,
                              make_paged)

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2   # absolute, bf16 configs
FP8_TOL = 5e-2    # absolute, fp8 KV after dequantisation
FP32_REL = 1e-5   # relative to the result's scale, fp32 config


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


def _set_impl(v):
    from nkipy_amd import _lib
    _lib.load().pa_debug_set(0, v)


def _set_waves(v):
    from nkipy_amd import _lib
    _lib.load().pa_debug_set(1, v)


def _i32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.int32)).cuda()


def _run_bf16(pa, rng, B, Hq, Hkv, D, bs, ctxs, part, scale=None, impl=0):
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    scale = scale if scale is not None else 1.0 / np.sqrt(D)
    want = O.paged_decode(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                          np.asarray(ctxs, np.int32), scale, q_dtype="bf16")
    _set_impl(impl)
    try:
        got = pa.decode(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs),
                        scale, partition_size=part, max_seq_len=max(int(max(ctxs)), 1))
        torch.cuda.synchronize()
    finally:
        _set_impl(0)
    return dev_to_f32(got), want


# ----------------------------------------------------------------------------- config 1 (fp32)
def test_config1_fp32_exact_config(pa):
    """BASELINE config 1: B=4, 8/8 heads, D=64, bs=16, ctx U[16,256], pool 128, fp32."""
    rng = np.random.default_rng(1001)
    B, H, D, bs = 4, 8, 64, 16
    ctx = rng.integers(16, 257, size=B)
    perm = rng.permutation(128).astype(np.int32)
    nblk = (ctx + bs - 1) // bs
    tables = np.full((B, 16), -1, np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    q = rng.standard_normal((B, H, D)).astype(np.float32)
    k = rng.standard_normal((128, bs, H, D)).astype(np.float32)
    v = rng.standard_normal((128, bs, H, D)).astype(np.float32)
    want = O.paged_decode(q, k, v, tables, ctx.astype(np.int32), 0.125)
    truth = O.paged_decode(q, k, v, tables, ctx.astype(np.int32), 0.125, acc=np.float64)
    for part in (512, 64, 16):
        got = pa.decode(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                        _i32(tables), _i32(ctx), 0.125, partition_size=part)
        torch.cuda.synchronize()
        assert_close_fp32(dev_to_f32(got), want, FP32_REL)
        assert_close_fp32(dev_to_f32(got), truth, FP32_REL)
        # element-wise as well (the form of the reference's own comparisons, tests/utils.py:17-26):
        # |got - truth| <= atol + rtol |truth| for every element, against the float64 result
        g = dev_to_f32(got).astype(np.float64)
        excess = np.abs(g - truth) - (1e-6 + 1e-5 * np.abs(truth))
        worst = float((np.abs(g - truth) / np.maximum(np.abs(truth), 1e-30)).max())
        print(f"config 1, partition {part}: max abs err {np.abs(g - truth).max():.3e}, max element-wise rel err {worst:.3e}")
        assert excess.max() <= 0, f"element-wise rtol=1e-5, atol=1e-6 exceeded by {excess.max():.3e}"


@pytest.mark.parametrize("D", [32, 64, 128, 256])
@pytest.mark.parametrize("n_rep", [1, 4])
def test_fp32_shapes(pa, D, n_rep):
    rng = np.random.default_rng(7 + D + n_rep)
    B, Hkv, bs = 3, 2, 8
    ctxs = [1, 37, 100]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, Hkv * n_rep, D)).astype(np.float32)
    want = O.paged_decode(q, k, v, tables, np.asarray(ctxs, np.int32), 0.2)
    got = pa.decode(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                    _i32(tables), _i32(ctxs), 0.2, partition_size=24)
    torch.cuda.synchronize()
    assert_close_fp32(dev_to_f32(got), want, FP32_REL)


# ----------------------------------------------------------------------------- bf16
@pytest.mark.parametrize("impl", [3, 2, 1], ids=["balanced", "mfma", "scalar"])
@pytest.mark.parametrize("D,Hq,Hkv,bs", [(128, 32, 8, 32), (128, 8, 8, 16), (64, 16, 2, 16),
                                         (128, 64, 8, 64), (64, 4, 4, 128), (128, 40, 2, 32)])
def test_bf16_shapes(pa, impl, D, Hq, Hkv, bs):
    rng = np.random.default_rng(D * 1000 + Hq * 10 + bs)
    ctxs = [1, 31, 32, 33, 500, 1025, 64, 77]
    got, want = _run_bf16(pa, rng, len(ctxs), Hq, Hkv, D, bs, ctxs, part=256, impl=impl)
    assert_close_abs(got, want, BF16_TOL)


@pytest.mark.parametrize("waves", [1, 2, 4])
def test_bf16_waves_per_workgroup(pa, waves):
    rng = np.random.default_rng(waves)
    ctxs = [5, 300, 777, 2048]
    _set_waves(waves)
    try:
        got, want = _run_bf16(pa, rng, 4, 32, 8, 128, 32, ctxs, part=512, impl=2)
    finally:
        _set_waves(0)
    assert_close_abs(got, want, BF16_TOL)


@pytest.mark.parametrize("B,Hq,Hkv,lo,hi", [
    (150, 8, 2, 0, 200),      # more sequences than lanes: multi-pass scan, many empty ones
    (3, 32, 8, 3000, 9000),   # few long sequences: every sequence split over many chunks
    (1, 8, 1, 20000, 20001),  # one kv head: eight chunks per workgroup
    (40, 48, 3, 1, 700),      # head slots do not divide the workgroup evenly
    (9, 32, 16, 100, 1200),   # more head slots than a workgroup holds: two head groups
    (5, 40, 2, 50, 900),      # 20 q heads per kv head: two 16-column chunks per kv head
    (513, 8, 2, 0, 100),      # more sequences than are scanned in registers: tile sums by a launch of their own
    (4500, 8, 2, 0, 70),      # ... of more than one pass, searched in three rounds; runs of empty sequences
])
def test_balanced_schedule_shapes(pa, B, Hq, Hkv, lo, hi):
    rng = np.random.default_rng(B * 7 + Hq)
    ctxs = rng.integers(lo, hi, size=B).tolist()
    if B > 10:
        ctxs[3] = 0
        ctxs[-1] = 0
    if B > 512:
        ctxs[:70] = [0] * 70
        ctxs[300:420] = [0] * 120
        ctxs[-3:] = [0] * 3
    got, want = _run_bf16(pa, rng, B, Hq, Hkv, 128, 32, ctxs, part=512, impl=3)
    assert_close_abs(got, want, BF16_TOL)


def test_zero_length_and_ragged(pa):
    rng = np.random.default_rng(3)
    for part in (4096, 64):
        got, want = _run_bf16(pa, rng, 4, 8, 2, 128, 16, [0, 1, 16, 700], part=part)
        assert np.all(got[0] == 0)
        assert_close_abs(got, want, BF16_TOL)


def test_partition_size_invariance(pa):
    rng = np.random.default_rng(11)
    B, Hq, Hkv, D, bs = 3, 16, 4, 128, 32
    ctxs = [900, 2000, 64]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    dq, dk, dv = bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v)
    outs = []
    for part in (2048, 512, 256, 32):
        o = pa.decode(dq, dk, dv, _i32(tables), _i32(ctxs), 0.09, partition_size=part, max_seq_len=2000)
        torch.cuda.synchronize()
        outs.append(dev_to_f32(o))
    for o in outs[1:]:
        assert np.max(np.abs(o - outs[0])) <= 2 ** -7 * max(1.0, np.abs(outs[0]).max())  # a bf16 ulp or so


def test_small_calls_take_the_fixed_partition_kernel(pa):
    """pa_decode's own choice: a call that can touch little of the pool by its max_seq_len (at most eight
    partitions per sequence) gives the fixed-partition kernel's bits (on partitions of 256 tokens when the call is
    small enough for those), with sinks as well, the same call with a bound of many partitions the balanced kernel's;
    all of them the oracle's values."""
    rng = np.random.default_rng(77)
    B, Hq, Hkv, D, bs = 5, 16, 4, 128, 32
    ctxs = [1, 700, 1500, 33, 1024]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    wide = np.full((B, 8192 // bs), -1, np.int32)            # the same blocks under a capacity of 16 partitions
    wide[:, :tables.shape[1]] = tables
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    dq, dk, dv = bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v)
    sinks = torch.full((Hq,), -float("inf"), device="cuda")
    want = O.paged_decode(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables, np.asarray(ctxs, np.int32),
                          0.09, q_dtype="bf16")

    def run(impl, tab, **kw):
        _set_impl(impl)
        try:
            o = pa.decode(dq, dk, dv, _i32(tab), _i32(ctxs), 0.09, **kw)
            torch.cuda.synchronize()
        finally:
            _set_impl(0)
        return o

    fixed, balanced = run(2, tables, max_seq_len=1500), run(3, tables, max_seq_len=1500)
    for o in (fixed, balanced):
        assert_close_abs(dev_to_f32(o), want, BF16_TOL)
    assert not np.array_equal(dev_bits(fixed), dev_bits(balanced))        # (else the test below shows nothing)
    assert np.array_equal(dev_bits(run(0, tables, max_seq_len=1500)), dev_bits(run(2, tables, max_seq_len=1500, partition_size=256)))
    assert np.array_equal(dev_bits(run(0, wide)), dev_bits(run(3, wide)))                 # bound = 8 192 tokens
    # sinks of -inf add nothing to the denominator: the same kernel, the same bits
    assert np.array_equal(dev_bits(run(0, tables, max_seq_len=1500, sinks=sinks)), dev_bits(run(0, tables, max_seq_len=1500)))
    assert np.array_equal(dev_bits(run(0, wide, sinks=sinks)), dev_bits(run(3, wide)))


def test_head_dim_64_partitions_are_counted_in_bytes(pa):
    """Head dim 64: a call whose bound gives more than eight partitions of partition_size still takes the
    fixed-partition kernel when twice as long partitions give at most eight (the bits of that kernel forced onto
    partitions of 1 024 tokens), a single sequence behind 4 K runs on 512-token partitions instead of sixteen of 256,
    and the results are the oracle's; with debug switch 13 off the first call is the balanced kernel's."""
    from nkipy_amd import _lib
    rng = np.random.default_rng(64)
    Hq, Hkv, D, bs = 16, 4, 64, 32

    def make(ctxs, cap):
        B = len(ctxs)
        k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
        wide = np.full((B, cap // bs), -1, np.int32)
        wide[:, :tables.shape[1]] = tables
        q = rng.standard_normal((B, Hq, D)).astype(np.float32)
        want = O.paged_decode(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables, np.asarray(ctxs, np.int32),
                              0.125, q_dtype="bf16")
        return bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(wide), _i32(ctxs), want

    def run(args, impl=0, **kw):
        _set_impl(impl)
        try:
            o = pa.decode(*args[:5], 0.125, **kw)
            torch.cuda.synchronize()
        finally:
            _set_impl(0)
        return o

    two = make([7000, 300, 5000, 8100], 8192)           # bound 8 192: sixteen partitions of 512, eight of 1 024
    got = run(two, partition_size=512)
    assert_close_abs(dev_to_f32(got), two[5], BF16_TOL)
    assert np.array_equal(dev_bits(got), dev_bits(run(two, impl=2, partition_size=1024)))
    assert not np.array_equal(dev_bits(got), dev_bits(run(two, impl=3, partition_size=512)))
    lib = _lib.load()
    lib.pa_debug_set(13, 0)
    try:
        assert np.array_equal(dev_bits(run(two, partition_size=512)), dev_bits(run(two, impl=3, partition_size=512)))
    finally:
        lib.pa_debug_set(13, 1)
    one = make([3900], 4096)                            # a single sequence: the finer partitions, 512 tokens here
    got = run(one, partition_size=512)
    assert_close_abs(dev_to_f32(got), one[5], BF16_TOL)
    assert np.array_equal(dev_bits(got), dev_bits(run(one, impl=2, partition_size=512)))
    assert not np.array_equal(dev_bits(got), dev_bits(run(one, impl=2, partition_size=256)))
    many = make([2100] * 3 + [1, 900] + [1800] * 59, 2176)      # 256 (sequence, kv head) pairs: one partition of 2 176
    got = run(many, partition_size=512)
    assert_close_abs(dev_to_f32(got), many[5], BF16_TOL)
    assert np.array_equal(dev_bits(got), dev_bits(run(many, impl=2, partition_size=2176)))


def test_fp8_pool_partitions_are_counted_in_bytes(pa):
    """An fp8 pool of head dim 128 (tokens of 128 bytes, like bf16 ones of head dim 64): a bound of sixteen partitions
    of 512 tokens is taken as eight of 1 024 on the fixed-partition kernel; an fp8 pool of head dim 64 stays with the
    balanced kernel there.  Both the oracle's values."""
    rng = np.random.default_rng(8)
    for D, want_fixed in ((128, True), (64, False)):
        Hq, Hkv, bs = 8, 4, 32
        ctxs = [7000, 300, 5000, 8100]
        B = len(ctxs)
        k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
        wide = np.full((B, 8192 // bs), -1, np.int32)
        wide[:, :tables.shape[1]] = tables
        kq, ks = O.quantize_kv_fp8(k)
        vq, vs = O.quantize_kv_fp8(v)
        q = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
        scale = 1.0 / np.sqrt(D)
        want = O.paged_decode(q, kq, vq, tables, np.asarray(ctxs, np.int32), scale, k_scale=ks, v_scale=vs, q_dtype="bf16")
        args = (bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
                torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(wide), _i32(ctxs), scale)
        kw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda())

        def run(impl, part):
            _set_impl(impl)
            try:
                o = pa.decode(*args, partition_size=part, **kw)
                torch.cuda.synchronize()
            finally:
                _set_impl(0)
            return o

        got = run(0, 512)
        assert_close_abs(dev_to_f32(got), want, BF16_TOL)
        fixed, balanced = run(2, 1024), run(3, 512)
        assert not np.array_equal(dev_bits(fixed), dev_bits(balanced))
        assert np.array_equal(dev_bits(got), dev_bits(fixed if want_fixed else balanced))


def test_identity_table_equals_dense_cache(pa):
    """A dense (B, S, Hkv, D) cache viewed as a pool with an identity table."""
    rng = np.random.default_rng(5)
    B, S, Hq, Hkv, D, bs = 4, 256, 8, 2, 128, 32
    ck = O.round_to_bf16(rng.standard_normal((B, S, Hkv, D)).astype(np.float32))
    cv = O.round_to_bf16(rng.standard_normal((B, S, Hkv, D)).astype(np.float32))
    q = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
    ctx = np.array([256, 1, 130, 77], np.int32)
    tables = np.arange(B * S // bs, dtype=np.int32).reshape(B, S // bs)
    got = pa.decode(bf16_to_dev(q), bf16_to_dev(ck.reshape(-1, bs, Hkv, D)), bf16_to_dev(cv.reshape(-1, bs, Hkv, D)),
                    _i32(tables), _i32(ctx), 0.1, partition_size=128)
    torch.cuda.synchronize()
    want = np.stack([O.dense_attention(q[b][None], ck[b, :ctx[b]], cv[b, :ctx[b]], 0.1, prefix=ctx[b] - 1)[0]
                     for b in range(B)])
    assert_close_abs(dev_to_f32(got), O.round_to_bf16(want), BF16_TOL)


def test_pool_permutation_gives_identical_bits(pa):
    """Moving blocks around the pool (and the table with them) must not change one output bit."""
    rng = np.random.default_rng(9)
    B, Hq, Hkv, D, bs = 3, 8, 2, 128, 32
    ctxs = [100, 700, 33]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs, pad_value=0)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    nb = k.shape[0]
    perm = rng.permutation(nb)
    k2, v2 = np.empty_like(k), np.empty_like(v)
    k2[perm], v2[perm] = k, v
    t2 = perm[tables].astype(np.int32)
    a = pa.decode(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), 0.09, partition_size=256)
    b = pa.decode(bf16_to_dev(q), bf16_to_dev(k2), bf16_to_dev(v2), _i32(t2), _i32(ctxs), 0.09, partition_size=256)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(a), dev_bits(b))


def test_stale_pool_bytes_do_not_leak(pa):
    """Rows past seq_len in the last block, unused blocks and padding table entries may hold
    anything (NaN patterns included) without affecting the result."""
    rng = np.random.default_rng(13)
    B, Hq, Hkv, D, bs = 2, 8, 2, 128, 32
    ctxs = [45, 200]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs, pad_value=-7)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    want = O.paged_decode(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                          np.asarray(ctxs, np.int32), 0.09, q_dtype="bf16")
    kd, vd = bf16_to_dev(k), bf16_to_dev(v)
    used = np.zeros(k.shape[:2], bool)
    for b in range(B):
        for t in range(ctxs[b]):
            used[tables[b, t // bs], t % bs] = True
    mask = torch.from_numpy(~used).cuda()
    kd[mask] = float("nan")
    vd[mask] = float("nan")
    for impl in (3, 2, 1):
        _set_impl(impl)
        try:
            got = pa.decode(bf16_to_dev(q), kd, vd, _i32(tables), _i32(ctxs), 0.09, partition_size=64)
            torch.cuda.synchronize()
        finally:
            _set_impl(0)
        assert_close_abs(dev_to_f32(got), want, BF16_TOL)


# ----------------------------------------------------------------------------- fp8 KV
@pytest.mark.parametrize("impl", [3, 2, 1], ids=["balanced", "mfma", "scalar"])
@pytest.mark.parametrize("D,Hq,Hkv,bs", [(128, 64, 8, 64), (128, 8, 2, 16), (64, 8, 1, 32)])
def test_fp8_kv(pa, impl, D, Hq, Hkv, bs):
    rng = np.random.default_rng(D + Hq + bs)
    ctxs = [1, 63, 64, 65, 1500, 300]
    B = len(ctxs)
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    q = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
    scale = 1.0 / np.sqrt(D)
    want = O.paged_decode(q, kq, vq, tables, np.asarray(ctxs, np.int32), scale, k_scale=ks, v_scale=vs, q_dtype="bf16")
    _set_impl(impl)
    try:
        got = pa.decode(bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
                        torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(tables), _i32(ctxs), scale,
                        k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda(),
                        partition_size=512)
        torch.cuda.synchronize()
    finally:
        _set_impl(0)
    assert_close_abs(dev_to_f32(got), want, FP8_TOL)
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)  # in fact as tight as bf16: dequantisation is exact


def test_fp8_every_code_decodes_exactly(pa):
    """All 254 finite e4m3fn codes pass through the device's expansion unchanged:
    one key, V rows holding each code -> out == decode(code) * scale (ctx = 1)."""
    D, bs = 128, 16
    codes = np.array([c for c in range(256) if c not in (0x7F, 0xFF)], np.uint8)
    nb = (len(codes) + D - 1) // D   # one token per sequence, D codes per row
    pad = np.zeros(nb * D, np.uint8)
    pad[:len(codes)] = codes
    v = np.zeros((nb, bs, 1, D), np.uint8)
    v[:, 0, 0, :] = pad.reshape(nb, D)
    k = np.zeros_like(v)
    sc = np.full((nb, 1), 0.5, np.float32)
    tables = np.arange(nb, dtype=np.int32)[:, None]
    q = np.zeros((nb, 1, D), np.float32)
    for impl in (3, 2, 1):
        _set_impl(impl)
        try:
            got = pa.decode(bf16_to_dev(q), torch.from_numpy(k).cuda().view(torch.float8_e4m3fn),
                            torch.from_numpy(v).cuda().view(torch.float8_e4m3fn), _i32(tables),
                            _i32(np.ones(nb)), 1.0, k_scale=torch.from_numpy(sc).cuda(),
                            v_scale=torch.from_numpy(sc).cuda())
            torch.cuda.synchronize()
        finally:
            _set_impl(0)
        want = O.round_to_bf16(O.fp8_e4m3fn_decode(pad).reshape(nb, 1, D) * np.float32(0.5))
        assert np.array_equal(dev_to_f32(got), want)


# ----------------------------------------------------------------------------- gather (bit exact)
@pytest.mark.parametrize("dtype", ["bf16", "fp8", "fp32"])
def test_gather_bit_exact(pa, dtype):
    rng = np.random.default_rng(21)
    B, Hkv, D, bs = 4, 2, 64, 16
    ctxs = [0, 1, 47, 160]
    nblk = [(c + bs - 1) // bs for c in ctxs]
    nb = sum(nblk) + 4
    perm = rng.permutation(nb).astype(np.int32)
    tables = np.zeros((B, max(nblk) + 1), np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    if dtype == "bf16":
        bits = rng.integers(0, 65536, size=(nb, bs, Hkv, D)).astype(np.uint16)
        dev = torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
    elif dtype == "fp8":
        bits = rng.integers(0, 256, size=(nb, bs, Hkv, D)).astype(np.uint8)
        dev = torch.from_numpy(bits).cuda().view(torch.float8_e4m3fn)
    else:
        bits = rng.integers(0, 2 ** 32, size=(nb, bs, Hkv, D), dtype=np.uint64).astype(np.uint32)
        dev = torch.from_numpy(bits.view(np.int32)).cuda().view(torch.float32)
    msl = max(ctxs)
    got = dev_bits(pa.gather_kv(dev, _i32(tables), _i32(ctxs), max_seq_len=msl))
    for b in range(B):
        want = O.gather_kv(bits, tables[b], ctxs[b])
        assert np.array_equal(got[b, :ctxs[b]], want)
        assert np.all(got[b, ctxs[b]:] == 0)


# ----------------------------------------------------------------------------- host-side errors
def test_argument_errors(pa):
    q = torch.zeros(2, 8, 128, dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros(4, 16, 2, 128, dtype=torch.bfloat16, device="cuda")
    bt = torch.zeros(2, 2, dtype=torch.int32, device="cuda")
    sl = torch.ones(2, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        pa.decode(q, kc, kc[:, :, :, :64].contiguous(), bt, sl, 1.0)
    with pytest.raises(ValueError):
        pa.decode(q, kc, kc, bt.long(), sl, 1.0)
    with pytest.raises(ValueError):
        pa.decode(q[:, :7].contiguous(), kc, kc, bt, sl, 1.0)          # 7 q heads over 2 kv heads
    with pytest.raises(ValueError):
        pa.decode(q.transpose(0, 1), kc, kc, bt, sl, 1.0)              # not contiguous
    with pytest.raises(ValueError):
        pa.decode(q, kc, kc, bt, sl, 1.0, max_seq_len=1000)            # beyond table capacity
    with pytest.raises(ValueError):
        pa.decode(q, kc, kc, torch.full_like(bt, 99), sl, 1.0, validate_tables=True)
    with pytest.raises(NotImplementedError):
        pa.decode(q.cpu(), kc, kc, bt, sl, 1.0)
    with pytest.raises(ValueError):
        pa.decode(q.float(), kc, kc, bt, sl, 1.0)                      # fp32 q with bf16 KV


def test_device_kernel_convention(pa):
    """compile_and_load + name-keyed call with caller-allocated output, as the reference's
    DeviceKernel (device_kernel.py:52-193): same result as the direct op."""
    from nkipy_amd.runtime import DeviceKernel, DeviceTensor
    rng = np.random.default_rng(4)
    B, Hq, Hkv, D, bs = 3, 8, 2, 128, 32
    ctxs = [70, 300, 1]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    ins = dict(q=DeviceTensor.from_numpy(O.f32_to_bf16_bits(q), "bf16"),
               k_cache=DeviceTensor.from_numpy(O.f32_to_bf16_bits(k), "bf16"),
               v_cache=DeviceTensor.from_numpy(O.f32_to_bf16_bits(v), "bf16"),
               block_tables=DeviceTensor.from_numpy(tables), seq_lens=DeviceTensor.from_numpy(np.asarray(ctxs, np.int32)))
    kern = DeviceKernel.compile_and_load(pa.decode, name="paged_decode", scale=0.09, **ins)
    out = DeviceTensor(torch.empty_like(ins["q"].torch()))
    assert kern(inputs=ins, outputs={"output0": out}) is None
    torch.cuda.synchronize()
    want = O.paged_decode(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                          np.asarray(ctxs, np.int32), 0.09, q_dtype="bf16")
    assert_close_abs(O.bf16_bits_to_f32(out.numpy()), want, BF16_TOL)
    ret = kern(inputs=ins)                      # outputs=None: result returned by value
    torch.cuda.synchronize()
    assert np.array_equal(ret.numpy(), out.numpy())


@pytest.mark.parametrize("B,ctx_hi,fp8", [(3, 700, False), (70, 1000, False), (5, 768, True), (2, 520, False)])
def test_small_calls_as_one_partition_on_eight_waves(B, ctx_hi, fp8):
    """Small calls whose length bound is short take one partition per sequence on eight waves (no merge launch):
    against the oracle, and against the same call with that route switched off (two partitions and the merge)."""
    import nkipy_amd as pa
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(B + ctx_hi)
    Hq, Hkv, D, bs = 32, 8, 128, 32
    ctxs = [int(x) for x in rng.integers(1, ctx_hi + 1, B)]
    ctxs[0] = ctx_hi
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
    scale = pa.default_scale(D)
    i32 = lambda x: torch.from_numpy(np.asarray(x, np.int32)).cuda()  # noqa: E731
    if fp8:
        kq, ks = O.quantize_kv_fp8(k)
        vq, vs = O.quantize_kv_fp8(v)
        want = O.paged_decode(q, kq, vq, tables, np.asarray(ctxs, np.int32), scale, k_scale=ks, v_scale=vs, q_dtype="bf16")
        kd, vd = (torch.from_numpy(x).cuda().view(torch.float8_e4m3fn) for x in (kq, vq))
        kw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda())
    else:
        want = O.paged_decode(q, O.round_to_bf16(k), O.round_to_bf16(v), tables, np.asarray(ctxs, np.int32), scale, q_dtype="bf16")
        kd, vd, kw = bf16_to_dev(k), bf16_to_dev(v), {}
    print(f"decode one partition B={B} ctx<={ctx_hi} fp8={fp8}", flush=True)
    got = pa.decode(bf16_to_dev(q), kd, vd, i32(tables), i32(ctxs), scale, max_seq_len=ctx_hi, **kw)
    lib.pa_debug_set(9, 0)
    try:
        two = pa.decode(bf16_to_dev(q), kd, vd, i32(tables), i32(ctxs), scale, max_seq_len=ctx_hi, **kw)
        torch.cuda.synchronize()
    finally:
        lib.pa_debug_set(9, 1024)
    assert np.abs(dev_to_f32(got) - want).max() <= (5e-2 if fp8 else 2e-2)
    assert np.abs(dev_to_f32(got) - dev_to_f32(two)).max() <= 2.0 ** -7 * max(np.abs(want).max(), 1.0)
