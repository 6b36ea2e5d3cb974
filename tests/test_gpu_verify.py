"""GPU parity: speculative verify (a few query tokens per sequence, through pa_verify) vs the oracle
and vs the tiled prefill kernel on the same arguments."""
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


@pytest.fixture(params=[16, 32], ids=["rows16", "rows32"])
def rows(request):
    """Force 16 or 32 query rows per wavefront (the library picks by shape otherwise)."""
    from nkipy_amd import _lib
    lib = _lib.load()
    lib.pa_debug_set(5, request.param)
    yield request.param
    lib.pa_debug_set(5, 0)


def _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D):
    B = len(qlens)
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [max(c, 1) for c in ctxs])
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    return q, O.round_to_bf16(k), O.round_to_bf16(v), tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32)


@pytest.mark.parametrize("T,Hq,Hkv", [(4, 32, 8), (2, 8, 2), (5, 6, 2), (8, 32, 8), (16, 16, 4), (3, 40, 2),
                                      (64, 4, 4), (7, 1, 1)])
@pytest.mark.parametrize("D,bs", [(128, 32), (64, 16)])
def test_verify_matches_oracle(pa, rows, T, Hq, Hkv, D, bs):
    """Rows per kv head from 7 to 64: less than, exactly, and several times the 16-row operand."""
    rng = np.random.default_rng(1000 * T + Hq + D)
    qlens = [T, max(T - 1, 1), 1, T, 0, T]
    prefixes = [0, 300, 65, 1533, 40, 31]
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    scale = 1.0 / np.sqrt(D)
    want = O.paged_prefill(q, k, v, tables, ctxs, ql, scale, q_dtype="bf16")
    got = pa.verify(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), scale)
    torch.cuda.synchronize()
    got = dev_to_f32(got)
    assert_close_abs(got, want, BF16_TOL)
    for b, n in enumerate(qlens):
        assert np.all(got[b, n:] == 0)          # padding rows


def test_verify_of_more_sequences_than_are_scanned_in_registers(pa):
    """600 sequences: the tiles before each sequence come from the prefix launch and every wave finds its first
    sequence by search; idle sequences (no query token) at both ends and in a run in the middle."""
    rng = np.random.default_rng(600)
    T, Hq, Hkv, D, bs, B = 3, 8, 2, 128, 16, 600
    qlens = rng.integers(1, T + 1, size=B).tolist()
    prefixes = rng.integers(0, 60, size=B).tolist()
    for i in list(range(5)) + list(range(200, 290)) + [B - 1]:
        qlens[i] = 0
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.09, q_dtype="bf16")
    got = pa.verify(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.09)
    torch.cuda.synchronize()
    got = dev_to_f32(got)
    assert_close_abs(got, want, BF16_TOL)
    for b, n in enumerate(qlens):
        assert np.all(got[b, n:] == 0)


def test_verify_rows_without_keys_in_the_last_chunk(pa, rows):
    """One long sequence spans every chunk of the schedule; its last 32-token tile holds 3 tokens,
    which the first 5 of 8 query tokens do not see, so their partial of that chunk is empty."""
    rng = np.random.default_rng(11)
    T, Hq, Hkv, D, bs = 8, 8, 2, 128, 32
    for ctx in (32 * 40 + 3, 32 * 700 + 1, 9):
        q, k, v, tables, ctxs, ql = _case(rng, T, [T], [ctx - T], Hq, Hkv, bs, D)
        want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.09, q_dtype="bf16")
        got = pa.verify(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.09)
        torch.cuda.synchronize()
        assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_prefill_picks_the_route_by_rows_batch_and_bound(pa):
    """32 rows per kv head: a batch of 16 sequences under a bound of 2 K takes the tiled kernel, the same batch under a
    bound of 1 K and a single sequence the verify kernel; 64 rows of one sequence under a bound of 2 K the verify
    kernel, without a bound the tiled one.  Whatever the route, the oracle's values."""
    rng = np.random.default_rng(21)
    Hq, Hkv, D, bs = 16, 4, 128, 32

    def check(B, T, hi, bound, expect):
        qlens = [T] * B
        qlens[-1] = max(T - 3, 1)
        prefixes = [int(x) for x in rng.integers(hi // 4, hi - T, size=B)]
        q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
        wide = np.full((B, max(tables.shape[1], (bound or 0) // bs)), -1, np.int32)     # table capacity >= the bound
        wide[:, :tables.shape[1]] = tables
        args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(wide), _i32(ctxs), _i32(ql), 0.09)
        kw = {} if bound is None else {"max_seq_len": bound}
        got = pa.prefill(*args, **kw)
        torch.cuda.synchronize()
        want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.09, q_dtype="bf16")
        assert_close_abs(dev_to_f32(got), want, BF16_TOL)
        forced = {r: pa.prefill(*args, route=r, **kw) for r in ("verify", "tiled")}
        torch.cuda.synchronize()
        assert not np.array_equal(dev_to_f32(forced["verify"]), dev_to_f32(forced["tiled"]))
        assert np.array_equal(dev_to_f32(got), dev_to_f32(forced[expect])), (B, T, hi, bound, expect)

    check(16, 8, 600, 2048, "tiled")
    check(16, 8, 600, 1024, "verify")
    check(1, 8, 1500, 2048, "verify")
    check(1, 16, 1500, 2048, "verify")
    check(1, 16, 1500, None, "tiled")


def test_verify_agrees_with_tiled_prefill_and_decode(pa):
    rng = np.random.default_rng(12)
    T, Hq, Hkv, D, bs = 4, 32, 8, 128, 32
    qlens, prefixes = [4, 4, 2, 4], [700, 0, 129, 4000]
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.09)
    a = dev_to_f32(pa.prefill(*args, route="verify"))
    b = dev_to_f32(pa.prefill(*args, route="tiled"))
    c = dev_to_f32(pa.prefill(*args))                   # 16 rows per kv head: the verify kernel by default
    assert np.max(np.abs(a - b)) <= 2 ** -6
    assert np.array_equal(a, c)
    # the last query token of a full-length sequence is a decode step over the whole context
    full = [i for i, n in enumerate(qlens) if n == T]
    d = pa.decode(args[0][full, T - 1].contiguous(), args[1], args[2], args[3][full].contiguous(),
                  args[4][full].contiguous(), 0.09)
    torch.cuda.synchronize()
    assert np.max(np.abs(dev_to_f32(d) - a[full, T - 1])) <= 2 ** -6


@pytest.mark.parametrize("D,Hq,Hkv,bs,T", [(128, 32, 8, 64, 4), (64, 8, 1, 16, 6), (128, 16, 2, 32, 5)])
def test_verify_fp8_pool(pa, rows, D, Hq, Hkv, bs, T):
    rng = np.random.default_rng(D + T)
    qlens, prefixes = [T, 1, T, T - 1], [0, 63, 1500, 300]
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    scale = 1.0 / np.sqrt(D)
    want = O.paged_prefill(q, kq, vq, tables, ctxs, ql, scale, k_scale=ks, v_scale=vs, q_dtype="bf16")
    got = pa.prefill(bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
                     torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(tables), _i32(ctxs), _i32(ql), scale,
                     k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda())
    torch.cuda.synchronize()
    assert_close_abs(dev_to_f32(got), want, FP8_TOL)
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_verify_stale_pool_bytes_and_padding_rows_do_not_leak(pa, rows):
    rng = np.random.default_rng(13)
    T, Hq, Hkv, D, bs = 6, 8, 2, 128, 32      # 24 rows per kv head
    qlens, prefixes = [6, 3], [45, 3]
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.09)
    kd, vd = bf16_to_dev(k), bf16_to_dev(v)
    used = np.zeros(k.shape[:2], bool)
    for b in range(len(qlens)):
        for t in range(ctxs[b]):
            used[tables[b, t // bs], t % bs] = True
    mask = torch.from_numpy(~used).cuda()
    kd[mask] = float("nan")
    vd[mask] = float("nan")
    qd = bf16_to_dev(q)
    qd[1, 3:] = float("nan")
    got = pa.verify(qd, kd, vd, _i32(tables), _i32(ctxs), _i32(ql), 0.09)
    torch.cuda.synchronize()
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)
    assert np.all(dev_to_f32(got)[1, 3:] == 0)


def test_verify_is_deterministic_and_keeps_out_argument(pa):
    rng = np.random.default_rng(14)
    T, Hq, Hkv, D, bs = 4, 16, 4, 128, 32
    q, k, v, tables, ctxs, ql = _case(rng, T, [4] * 5, [5000, 17, 900, 2222, 64], Hq, Hkv, bs, D)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.09)
    out = torch.full_like(args[0], 7.0)
    r = pa.verify(*args, out=out)
    assert r is out
    again = pa.verify(*args)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(out), dev_bits(again))


def test_verify_argument_errors(pa):
    rng = np.random.default_rng(15)
    q, k, v, tables, ctxs, ql = _case(rng, 4, [4], [10], 4, 2, 32, 128)
    args = [bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.09]
    with pytest.raises(ValueError):
        pa.verify(*args, workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    big = bf16_to_dev(np.zeros((1, 65, 4, 128), np.float32))
    with pytest.raises(ValueError):
        pa.verify(big, *args[1:])
    with pytest.raises(ValueError):     # forced onto the verify kernel, which stops at 64 tokens
        pa.prefill(big, *args[1:], route="verify")


@pytest.fixture(params=["tiled", "chunks"])
def d64_path(request):
    """head_dim 64 beyond 64 query tokens: two or more kv heads take the tiled kernel (two kv heads
    share its 256-byte rows; the last head of an odd count works alone on the 256 bytes that end with
    it); with the tiled kernel switched off, as for a single kv head, pa_prefill covers the query
    tokens with launches of the verify kernel, 64 tokens each."""
    from nkipy_amd import _lib
    lib = _lib.load()
    lib.pa_debug_set(3, 1 if request.param == "chunks" else 0)
    yield request.param
    lib.pa_debug_set(3, 0)


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("T,Hq,Hkv,bs", [(65, 4, 4, 16), (200, 8, 2, 32), (129, 64, 8, 64), (300, 3, 1, 32), (530, 12, 6, 16),
                                         (300, 9, 3, 32), (130, 10, 5, 16), (257, 7, 7, 64)])
def test_head_dim_64_long_prefill(pa, d64_path, fp8, T, Hq, Hkv, bs):
    """Ragged lengths put tile and launch boundaries inside, at the end of and past a sequence's query run;
    the sliding window and the sinks ride along."""
    rng = np.random.default_rng(T + Hq)
    D = 64
    qlens = [T, 64, 65, 0, T - 1, 1]
    prefixes = [0, 300, 65, 40, 1533, 31]
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32))
    okw, dkw = {}, {}
    kd, vd = bf16_to_dev(k), bf16_to_dev(v)
    if fp8:
        k, ks = O.quantize_kv_fp8(k)
        v, vs = O.quantize_kv_fp8(v)
        okw = dict(k_scale=ks, v_scale=vs)
        dkw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda())
        kd = torch.from_numpy(k).cuda().view(torch.float8_e4m3fn)
        vd = torch.from_numpy(v).cuda().view(torch.float8_e4m3fn)
    for win, snk in ((None, None), (100, sinks)):
        want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.125, q_dtype="bf16", sliding_window=win, sinks=snk, **okw)
        got = pa.prefill(bf16_to_dev(q), kd, vd, _i32(tables), _i32(ctxs), _i32(ql), 0.125, sliding_window=win,
                         sinks=None if snk is None else bf16_to_dev(snk), **dkw)
        torch.cuda.synchronize()
        got = dev_to_f32(got)
        assert_close_abs(got, want, FP8_TOL if fp8 else BF16_TOL)
        for b, n in enumerate(qlens):
            assert np.all(got[b, n:] == 0)


def test_head_dim_64_long_prefill_with_q_transform(pa, d64_path):
    rng = np.random.default_rng(77)
    T, Hq, Hkv, bs, D = 150, 8, 2, 32, 64
    qlens, prefixes = [150, 70, 3], [200, 0, 900]
    xq, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    w = O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32))
    cos, sin = O.rope_tables(D, 1200, 10000.0)
    dcos, dsin = pa.rope_tables(D, 1200, 10000.0)
    oq, _ = O.qk_norm_rope(xq, xq[:, :, :Hkv], ctxs, ql, cos, sin, q_norm_weight=w, eps=1e-6)
    want = O.paged_prefill(oq, k, v, tables, ctxs, ql, 0.125, q_dtype="bf16")
    got = pa.prefill(bf16_to_dev(xq), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.125,
                     q_transform=pa.QTransform(dcos, dsin, bf16_to_dev(w)))
    torch.cuda.synchronize()
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_head_dim_64_tiled_split_matches_unsplit(pa):
    """One long-context request at head_dim 64: the key tiles of its query tiles are split over workgroups."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(91)
    T, Hq, Hkv, bs, D = 256, 4, 2, 32, 64
    q, k, v, tables, ctxs, ql = _case(rng, T, [T], [6000], Hq, Hkv, bs, D)
    sinks = bf16_to_dev(O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32)))
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.125)
    want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.125, q_dtype="bf16", sinks=dev_to_f32(sinks))
    got = dev_to_f32(pa.prefill(*args, sinks=sinks))
    lib.pa_debug_set(6, 0)
    try:
        unsplit = dev_to_f32(pa.prefill(*args, sinks=sinks))
    finally:
        lib.pa_debug_set(6, 1)
    torch.cuda.synchronize()
    assert_close_abs(got, want, BF16_TOL)
    assert np.max(np.abs(got - unsplit)) <= 2 ** -6


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
def test_head_dim_64_odd_kv_heads_at_the_end_of_the_pool(pa, fp8):
    """Three kv heads, every sequence's last block the last block of the pool and filled to its last row: the
    unpaired head's 256-byte window ends exactly with the pool.  Checked against the verify-kernel route too."""
    rng = np.random.default_rng(97)
    T, Hq, Hkv, bs, D = 192, 6, 3, 16, 64
    qlens, prefixes = [192, 100, 64], [64, 12 * 16 - 100, 0]
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    last = k.shape[0] - 1
    for b in range(len(qlens)):
        assert ctxs[b] % bs == 0
        tables[b, ctxs[b] // bs - 1] = last
    okw, dkw = {}, {}
    kd, vd = bf16_to_dev(k), bf16_to_dev(v)
    if fp8:
        k, ks = O.quantize_kv_fp8(k)
        v, vs = O.quantize_kv_fp8(v)
        okw = dict(k_scale=ks, v_scale=vs)
        dkw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda())
        kd = torch.from_numpy(k).cuda().view(torch.float8_e4m3fn)
        vd = torch.from_numpy(v).cuda().view(torch.float8_e4m3fn)
    want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.125, q_dtype="bf16", **okw)
    args = (bf16_to_dev(q), kd, vd, _i32(tables), _i32(ctxs), _i32(ql), 0.125)
    got = dev_to_f32(pa.prefill(*args, route="tiled", **dkw))
    torch.cuda.synchronize()
    assert_close_abs(got, want, FP8_TOL if fp8 else BF16_TOL)
    for b, n in enumerate(qlens):
        assert np.all(got[b, n:] == 0)


def test_head_dim_64_many_rows_of_a_short_run_take_the_tiled_kernel(pa):
    """48 tokens x 8 q heads per kv head in a batch of 8: past the measured crossover the default route is the
    tiled kernel; the verify kernel gives the same result."""
    rng = np.random.default_rng(93)
    T, Hq, Hkv, bs, D = 48, 16, 2, 32, 64
    qlens = [48, 48, 7, 48, 0, 48, 33, 48]
    prefixes = [100, 0, 900, 31, 5, 2000, 64, 333]
    q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.125)
    want = O.paged_prefill(q, k, v, tables, ctxs, ql, 0.125, q_dtype="bf16")
    got = dev_to_f32(pa.prefill(*args))
    via_verify = dev_to_f32(pa.prefill(*args, route="verify"))
    torch.cuda.synchronize()
    assert_close_abs(got, want, BF16_TOL)
    assert_close_abs(via_verify, want, BF16_TOL)
    assert not np.array_equal(got, via_verify)          # two kernels: different summation orders
    for b, n in enumerate(qlens):
        assert np.all(got[b, n:] == 0)


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("T,Hq,Hkv,D,bs", [(4, 32, 8, 128, 32), (8, 8, 2, 128, 16), (3, 40, 2, 64, 16), (5, 6, 2, 64, 64),
                                           (16, 16, 4, 128, 32), (7, 1, 1, 128, 32)])
def test_verify_small_calls_with_a_length_bound(pa, T, Hq, Hkv, D, bs, fp8):
    """With the caller's bound on the contexts a small call takes fixed partitions (one to eight of 512 tokens, or finer ones for a single sequence): a
    single sequence behind about 1 K tokens (the reference's own use), a ragged batch with an idle slot and a
    one-token sequence, contexts a few tokens past a partition boundary (the early query rows then see no key in
    the last partition and leave an empty partial), a bound far above the contexts (partitions with no tokens),
    bf16 and fp8 pools.  Against the oracle; rows past the query length are zeros."""
    rng = np.random.default_rng(77 * T + Hq + D)
    for qlens, prefixes, bound in [([T], [1020], 1100), ([T, max(T - 1, 1), 1, T, 0, T], [0, 300, 65, 1533, 40, 512 - 2], 1600),
                                   ([T, T], [512 - 1, 1024 + 1 - T], 2048), ([T, 2], [3, 40], 70), ([T], [100], 2000)]:
        q, k, v, tables, ctxs, ql = _case(rng, T, qlens, prefixes, Hq, Hkv, bs, D)
        bound = min(bound, tables.shape[1] * bs)        # never above the table capacity
        assert ctxs.max() <= bound
        scale = 1.0 / np.sqrt(D)
        if fp8:
            kq, ks = O.quantize_kv_fp8(k)
            vq, vs = O.quantize_kv_fp8(v)
            want = O.paged_prefill(q, kq, vq, tables, ctxs, ql, scale, q_dtype="bf16", k_scale=ks, v_scale=vs)
            kd, vd = (torch.from_numpy(x).cuda().view(torch.float8_e4m3fn) for x in (kq, vq))
            kw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda())
        else:
            want = O.paged_prefill(q, k, v, tables, ctxs, ql, scale, q_dtype="bf16")
            kd, vd, kw = bf16_to_dev(k), bf16_to_dev(v), {}
        print(f"verify small call T={T} Hq={Hq} Hkv={Hkv} D={D} bs={bs} fp8={fp8} qlens={qlens} bound={bound}", flush=True)
        got = pa.verify(bf16_to_dev(q), kd, vd, _i32(tables), _i32(ctxs), _i32(ql), scale, max_seq_len=bound, **kw)
        plain = pa.verify(bf16_to_dev(q), kd, vd, _i32(tables), _i32(ctxs), _i32(ql), scale, **kw)
        torch.cuda.synchronize()
        got = dev_to_f32(got)
        assert_close_abs(got, want, FP8_TOL if fp8 else BF16_TOL)
        assert np.abs(got - dev_to_f32(plain)).max() <= 2.0 ** -7 * max(np.abs(want).max(), 1.0)      # the balanced route, to a bf16 step
        for b, n in enumerate(qlens):
            assert np.all(got[b, n:] == 0)


def test_verify_length_bound_clamps_like_decode(pa):
    """A bound below a context: the kernels read the context up to the bound, as pa_decode does with its max_seq_len."""
    rng = np.random.default_rng(5)
    T, Hq, Hkv, D, bs = 4, 8, 2, 128, 32
    q, k, v, tables, ctxs, ql = _case(rng, T, [T, T], [900, 200], Hq, Hkv, bs, D)
    bound = 600
    want = O.paged_prefill(q, k, v, tables, np.minimum(ctxs, bound).astype(np.int32), ql, 0.09, q_dtype="bf16")
    got = pa.verify(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(ql), 0.09, max_seq_len=bound)
    torch.cuda.synchronize()
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)
