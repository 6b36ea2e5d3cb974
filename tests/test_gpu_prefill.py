"""GPU parity: HIP chunked prefill and blocksparse prefill (through the C ABI) vs the oracle."""
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


def _prefill_case(pa, rng, T, qlens, prefixes, Hq, Hkv, bs, D=128, scale=None):
    B = len(qlens)
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [max(c, 1) for c in ctxs])
    q = rng.standard_normal((B, T, Hq, D)).astype(np.float32)
    scale = scale if scale is not None else 1.0 / np.sqrt(D)
    want = O.paged_prefill(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                           np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), scale, q_dtype="bf16")
    got = pa.prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(qlens), scale)
    torch.cuda.synchronize()
    return dev_to_f32(got), want


@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (4, 4)])
def test_prefill_with_prefix_ragged(pa, bs, Hq, Hkv):
    rng = np.random.default_rng(bs + Hq)
    got, want = _prefill_case(pa, rng, T=200, qlens=[200, 77, 1, 130], prefixes=[0, 300, 65, 1000],
                              Hq=Hq, Hkv=Hkv, bs=bs)
    assert_close_abs(got, want, BF16_TOL)
    assert np.all(got[1, 77:] == 0) and np.all(got[2, 1:] == 0)   # padding rows


def test_prefill_many_tiles_and_exact_multiples(pa):
    rng = np.random.default_rng(5)
    got, want = _prefill_case(pa, rng, T=384, qlens=[384, 256, 128], prefixes=[640, 64, 0], Hq=4, Hkv=1, bs=32)
    assert_close_abs(got, want, BF16_TOL)


def test_prefill_zero_query_sequence(pa):
    rng = np.random.default_rng(6)
    got, want = _prefill_case(pa, rng, T=64, qlens=[0, 64], prefixes=[10, 3], Hq=2, Hkv=2, bs=16)
    assert np.all(got[0] == 0)
    assert_close_abs(got, want, BF16_TOL)


def test_prefill_T1_equals_decode(pa):
    rng = np.random.default_rng(7)
    B, Hq, Hkv, D, bs = 3, 8, 2, 128, 32
    ctxs = [1, 200, 777]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, 1, Hq, D)).astype(np.float32)
    dk, dv = bf16_to_dev(k), bf16_to_dev(v)
    a = pa.prefill(bf16_to_dev(q), dk, dv, _i32(tables), _i32(ctxs), _i32([1, 1, 1]), 0.09)
    b = pa.decode(bf16_to_dev(q[:, 0]), dk, dv, _i32(tables), _i32(ctxs), 0.09)
    torch.cuda.synchronize()
    assert np.max(np.abs(dev_to_f32(a)[:, 0] - dev_to_f32(b))) <= 2 ** -6


def test_prefill_shared_prefix_blocks(pa):
    """Sequences whose tables alias the same physical prefix blocks (and have the same new
    tokens) produce bit-identical outputs."""
    rng = np.random.default_rng(8)
    Hq, Hkv, D, bs, T, P = 4, 2, 128, 32, 96, 128
    nb = 20
    k = rng.standard_normal((nb, bs, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((nb, bs, Hkv, D)).astype(np.float32)
    shared = [3, 9, 1, 14]
    t0 = shared + [5, 6, 7]
    t1 = shared + [10, 11, 12]
    for a_, b_ in zip(t0[4:], t1[4:]):
        k[b_], v[b_] = k[a_], v[a_]
    tables = np.array([t0, t1], np.int32)
    q1 = rng.standard_normal((1, T, Hq, D)).astype(np.float32)
    q = np.concatenate([q1, q1])
    got = pa.prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32([P + T] * 2),
                     _i32([T, T]), 0.09)
    torch.cuda.synchronize()
    bits = dev_bits(got)
    assert np.array_equal(bits[0], bits[1])
    want = O.paged_prefill(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                           np.array([P + T] * 2, np.int32), np.array([T, T], np.int32), 0.09)
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_prefill_stale_pool_bytes_do_not_leak(pa):
    rng = np.random.default_rng(9)
    B, Hq, Hkv, D, bs, T = 2, 4, 2, 128, 32, 70
    prefixes, qlens = [45, 3], [70, 50]
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs, pad_value=-3)
    q = rng.standard_normal((B, T, Hq, D)).astype(np.float32)
    want = O.paged_prefill(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                           np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), 0.09)
    kd, vd = bf16_to_dev(k), bf16_to_dev(v)
    used = np.zeros(k.shape[:2], bool)
    for b in range(B):
        for t in range(ctxs[b]):
            used[tables[b, t // bs], t % bs] = True
    mask = torch.from_numpy(~used).cuda()
    kd[mask] = float("nan")
    vd[mask] = float("nan")
    qd = bf16_to_dev(q)
    qd[1, 50:] = float("nan")      # padding query rows may hold anything as well
    got = pa.prefill(qd, kd, vd, _i32(tables), _i32(ctxs), _i32(qlens), 0.09)
    torch.cuda.synchronize()
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_config3_shape_shrunk(pa):
    """BASELINE config 3 at 1/8 length (T=256, prefix U[0,512]) with aliased prefix blocks."""
    from nkipy_amd import workloads as W
    w = W.make_prefill(shrink=8)
    got = pa.prefill(w.q, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.query_lens, w.scale,
                     validate_tables=True)
    torch.cuda.synchronize()
    want = O.paged_prefill(dev_bits(w.q), dev_bits(w.k_cache), dev_bits(w.v_cache), w.block_tables.cpu().numpy(),
                           w.seq_lens.cpu().numpy(), w.query_lens.cpu().numpy(), w.scale)
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


# ----------------------------------------------------------------------------- blocksparse
@pytest.mark.parametrize("Hq,Hkv,S,local,stride", [(4, 4, 512, 2, 3), (8, 2, 448, 4, 8), (2, 2, 100, 1, 2),
                                                  (9, 9, 704, 3, 4)])
def test_blocksparse_vs_oracle(pa, Hq, Hkv, S, local, stride):
    rng = np.random.default_rng(S + Hq)
    B, D = 2, 128
    q = rng.standard_normal((B, S, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, S, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, S, Hkv, D)).astype(np.float32)
    scale = 1.0 / np.sqrt(D)
    want = O.blocksparse_prefill(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), scale, block=64,
                                 local_blocks=local, vert_stride=stride)
    got = pa.blocksparse_prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), scale, block=64,
                                 local_blocks=local, vert_stride=stride)
    torch.cuda.synchronize()
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


def test_blocksparse_all_active_equals_dense_causal(pa):
    """local_blocks >= number of blocks: the sparse op is plain causal attention, which the
    paged prefill op computes too (identity block table, no prefix)."""
    rng = np.random.default_rng(33)
    B, S, H, D, bs = 2, 320, 4, 128, 32
    q = rng.standard_normal((B, S, H, D)).astype(np.float32)
    k = rng.standard_normal((B, S, H, D)).astype(np.float32)
    v = rng.standard_normal((B, S, H, D)).astype(np.float32)
    dq, dk, dv = bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v)
    a = pa.blocksparse_prefill(dq, dk, dv, 0.09, local_blocks=1000, vert_stride=8)
    tables = np.arange(B * S // bs, dtype=np.int32).reshape(B, S // bs)
    b = pa.prefill(dq, dk.view(-1, bs, H, D), dv.view(-1, bs, H, D), _i32(tables), _i32([S] * B), _i32([S] * B), 0.09)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(a), dev_bits(b))
    want = np.stack([O.dense_attention(O.round_to_bf16(q[i]), O.round_to_bf16(k[i]), O.round_to_bf16(v[i]), 0.09, prefix=0)
                     for i in range(B)])
    assert_close_abs(dev_to_f32(a), O.round_to_bf16(want), BF16_TOL)


def test_config4_shape_shrunk(pa):
    """BASELINE config 4 at 1/8 length (S=1024): 32 heads MHA, local 4 + every 8th, per-head phase."""
    from nkipy_amd import workloads as W
    w = W.make_blocksparse(shrink=8)
    got = pa.blocksparse_prefill(w.q, w.k, w.v, w.scale, block=w.block, local_blocks=w.local_blocks,
                                 vert_stride=w.vert_stride)
    torch.cuda.synchronize()
    want = O.blocksparse_prefill(dev_bits(w.q), dev_bits(w.k), dev_bits(w.v), w.scale, block=w.block,
                                 local_blocks=w.local_blocks, vert_stride=w.vert_stride)
    assert_close_abs(dev_to_f32(got), want, BF16_TOL)


@pytest.mark.parametrize("B,S,Hq,Hkv,local,stride", [(1, 640, 3, 3, 2, 4), (2, 1024, 4, 2, 4, 8), (1, 2048, 8, 8, 4, 8),
                                                    (1, 700, 2, 1, 1, 3), (1, 1500, 2, 2, 6, 2), (1, 900, 2, 2, 1000, 8),
                                                    (1, 512, 9, 9, 3, 1)])
def test_blocksparse_staggered_256_row_form(pa, B, S, Hq, Hkv, local, stride):
    """The 8-wave blocksparse form (debug switch 3 = 8): four q blocks per workgroup walk the vertical-stride tiles
    together and the local band staggered, one key tile apart.  Windows shorter and longer than the four q blocks,
    a window longer than the sequence, every tile vertical (stride 1), sequence lengths that are not multiples of
    256 or 64, GQA: against the oracle, and bit for bit the 4-wave form's result."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(S + local + stride)
    q = O.round_to_bf16(rng.standard_normal((B, S, Hq, 128)).astype(np.float32))
    k = O.round_to_bf16(rng.standard_normal((B, S, Hkv, 128)).astype(np.float32))
    v = O.round_to_bf16(rng.standard_normal((B, S, Hkv, 128)).astype(np.float32))
    want = O.blocksparse_prefill(q, k, v, 0.09, block=64, local_blocks=local, vert_stride=stride)
    got = {}
    try:
        for impl in (4, 8):
            print(f"blocksparse B={B} S={S} Hq={Hq} Hkv={Hkv} local={local} stride={stride} impl={impl}", flush=True)
            lib.pa_debug_set(3, impl)
            out = pa.blocksparse_prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), 0.09, block=64,
                                         local_blocks=local, vert_stride=stride)
            torch.cuda.synchronize()
            got[impl] = out
    finally:
        lib.pa_debug_set(3, 0)
    assert_close_abs(dev_to_f32(got[8]), want, BF16_TOL)
    assert torch.equal(got[4], got[8])


@pytest.mark.parametrize("impl", [1, 4, 8], ids=["staged", "async4", "async8"])
def test_prefill_kernel_variants_agree(pa, impl):
    """Every prefill kernel variant (register-staged, asynchronous ring with 4 or 8 waves, the
    two-group schedule) against the oracle on the dense-causal and the sparse form."""
    from nkipy_amd import _lib
    rng = np.random.default_rng(77)
    lib = _lib.load()
    lib.pa_debug_set(3, impl)
    try:
        got, want = _prefill_case(pa, rng, T=300, qlens=[300, 129, 257], prefixes=[70, 515, 0], Hq=8, Hkv=2, bs=32)
        assert_close_abs(got, want, BF16_TOL)
        B, S, H, D = 1, 640, 3, 128
        q = rng.standard_normal((B, S, H, D)).astype(np.float32)
        k = rng.standard_normal((B, S, H, D)).astype(np.float32)
        v = rng.standard_normal((B, S, H, D)).astype(np.float32)
        want = O.blocksparse_prefill(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), 0.09,
                                     block=64, local_blocks=2, vert_stride=4)
        got = pa.blocksparse_prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), 0.09, block=64,
                                     local_blocks=2, vert_stride=4)
        torch.cuda.synchronize()
        assert_close_abs(dev_to_f32(got), want, BF16_TOL)
    finally:
        lib.pa_debug_set(3, 0)


def test_prefill_generic_block_size(pa):
    """Block sizes that are not a power of two >= 16 take the register-staged kernel."""
    rng = np.random.default_rng(78)
    got, want = _prefill_case(pa, rng, T=100, qlens=[100, 33], prefixes=[50, 7], Hq=4, Hkv=2, bs=8)
    assert_close_abs(got, want, BF16_TOL)
    got, want = _prefill_case(pa, rng, T=100, qlens=[100, 33], prefixes=[50, 7], Hq=4, Hkv=2, bs=24)
    assert_close_abs(got, want, BF16_TOL)


def test_prefill_argument_errors(pa):
    q = torch.zeros(1, 8, 4, 128, dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros(4, 16, 2, 128, dtype=torch.bfloat16, device="cuda")
    bt = torch.zeros(1, 2, dtype=torch.int32, device="cuda")
    one = torch.ones(1, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        pa.prefill(q.float(), kc, kc, bt, one, one, 1.0)
    with pytest.raises(ValueError):
        pa.prefill(q[:, :, :3].contiguous(), kc, kc, bt, one, one, 1.0)
    with pytest.raises(ValueError):
        pa.blocksparse_prefill(q, q, q, 1.0, block=32)
    with pytest.raises(RuntimeError):      # head_dim 128 (tiled kernel) or 64 (verify kernel, 64 tokens per launch) only
        pa.prefill(q[..., :32].contiguous(), kc[..., :32].contiguous(), kc[..., :32].contiguous(), bt, one, one, 1.0,
                   route="tiled")
    with pytest.raises(ValueError):
        pa.prefill(q, kc, kc, bt, one, one, 1.0, route="fast")


@pytest.mark.parametrize("impl", [5, 4], ids=["packed", "one_head_per_workgroup"])
@pytest.mark.parametrize("T,Hq,Hkv", [(20, 8, 2), (32, 16, 4), (64, 32, 8), (100, 10, 2), (127, 4, 2), (33, 16, 1)])
def test_prefill_short_chunks_packed_rows(pa, impl, T, Hq, Hkv):
    """Chunks shorter than a 128-row tile: by default the rows of a workgroup are (token, head) pairs of
    one kv head (ratios 2, 4, 5 and 16: head groups that do and do not divide a wave's 32 rows).  Up to 128 rows
    per kv head (the first two cases, the second exactly 128) one workgroup is the only reader of its keys and values
    and copies them with the streaming policy; beyond, several workgroups share them through the cache."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(T + Hq)
    qlens = [T, max(T - 7, 1), 1, 0, T]
    prefixes = [0, 300, 65, 10, 1500]
    B, D, bs = len(qlens), 128, 32
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [max(c, 1) for c in ctxs])
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32))
    for window in (None, 40):
        want = O.paged_prefill(q, O.round_to_bf16(k), O.round_to_bf16(v), tables, np.asarray(ctxs, np.int32),
                               np.asarray(qlens, np.int32), 0.09, q_dtype="bf16", sliding_window=window, sinks=sinks)
        lib.pa_debug_set(3, impl)
        try:
            got = pa.prefill(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(qlens), 0.09,
                             sliding_window=window, sinks=bf16_to_dev(sinks), route="tiled")
            torch.cuda.synchronize()
        finally:
            lib.pa_debug_set(3, 0)
        got = dev_to_f32(got)
        assert_close_abs(got, want, BF16_TOL)
        for b, n in enumerate(qlens):
            assert np.all(got[b, n:] == 0)


@pytest.mark.parametrize("T,Hq,Hkv,window", [(128, 8, 2, None), (100, 8, 2, None), (300, 4, 4, None), (200, 8, 1, 700),
                                             (90, 4, 1, 64), (256, 2, 2, 1500)])
def test_prefill_split_over_key_tiles(pa, T, Hq, Hkv, window):
    """Few query tiles against long contexts: the key tiles of a query tile are shared by several
    workgroups (4- and 8-wave, packed rows, windowed); shares that are empty for some rows or for a
    whole short sequence; same result as the unsplit kernel."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(T + Hq)
    qlens, prefixes = [T, 5], [5000, 3]
    B, D, bs = 2, 128, 32
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32))
    need = lib.pa_prefill_workspace_bytes(B, T, Hq, Hkv, D, bs, tables.shape[1])
    assert need > 0                                   # this shape is one the launcher wants to split
    want = O.paged_prefill(q, O.round_to_bf16(k), O.round_to_bf16(v), tables, np.asarray(ctxs, np.int32),
                           np.asarray(qlens, np.int32), 0.09, q_dtype="bf16", sliding_window=window, sinks=sinks)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(qlens), 0.09)
    kw = dict(sliding_window=window, sinks=bf16_to_dev(sinks), route="tiled")
    got = dev_to_f32(pa.prefill(*args, **kw))
    lib.pa_debug_set(6, 0)
    try:
        unsplit = dev_to_f32(pa.prefill(*args, **kw))
    finally:
        lib.pa_debug_set(6, 1)
    assert_close_abs(got, want, BF16_TOL)
    assert np.max(np.abs(got - unsplit)) <= 2 ** -6
    assert np.all(got[1, 5:] == 0)
    with pytest.raises(ValueError):
        pa.prefill(*args, workspace=torch.empty(64, dtype=torch.uint8, device="cuda"), **kw)


def test_prompt_with_a_short_prefix_runs_unsplit_under_a_length_bound(pa):
    """One prompt of 600 tokens on tables of 8 192: by the table capacity the launcher splits its key tiles; told
    that no context exceeds 700 tokens (less than three times the chunk) it does not, and gives the unsplit kernel's
    bits; with a bound of 5 000 tokens the split stays.  All of them the oracle's values."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(600)
    B, T, Hq, Hkv, D, bs = 1, 600, 8, 2, 128, 32
    ctxs, qlens = [T + 100], [T]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    wide = np.full((B, 8192 // bs), -1, np.int32)
    wide[:, :tables.shape[1]] = tables
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    want = O.paged_prefill(q, O.round_to_bf16(k), O.round_to_bf16(v), tables, np.asarray(ctxs, np.int32),
                           np.asarray(qlens, np.int32), 0.09, q_dtype="bf16")
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(wide), _i32(ctxs), _i32(qlens), 0.09)
    assert lib.pa_prefill_workspace_bytes(B, T, Hq, Hkv, D, bs, wide.shape[1]) > 0
    by_capacity = pa.prefill(*args, route="tiled")
    bounded = pa.prefill(*args, route="tiled", max_seq_len=700)
    far_bound = pa.prefill(*args, route="tiled", max_seq_len=5000)
    lib.pa_debug_set(6, 0)
    try:
        unsplit = pa.prefill(*args, route="tiled")
    finally:
        lib.pa_debug_set(6, 1)
    torch.cuda.synchronize()
    for o in (by_capacity, bounded, far_bound, unsplit):
        assert_close_abs(dev_to_f32(o), want, BF16_TOL)
    assert torch.equal(bounded, unsplit)
    assert not torch.equal(far_bound, unsplit) and not torch.equal(by_capacity, unsplit)      # both split (the bound sizes the shares)
    assert not torch.equal(by_capacity, unsplit)          # (else the comparisons above show nothing)


@pytest.mark.parametrize("bs", [16, 64, 24])
@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (4, 4)])
def test_prefill_fp8_pool(pa, bs, Hq, Hkv):
    """Long chunks over an fp8 pool: codes times their block's scale become bf16 on the way into LDS
    (block sizes that are and are not a power of two; chunks that start inside a block)."""
    rng = np.random.default_rng(bs + Hq)
    T, D = 200, 128
    qlens, prefixes = [200, 77, 1, 130], [0, 300, 65, 1000]
    B = len(qlens)
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    k *= rng.uniform(0.2, 3.0, size=(k.shape[0], 1, Hkv, 1)).astype(np.float32)     # different scales per block and head
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    q = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    sinks = O.round_to_bf16(rng.standard_normal(Hq).astype(np.float32))
    scale = 1.0 / np.sqrt(D)
    want = O.paged_prefill(q, kq, vq, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), scale,
                           k_scale=ks, v_scale=vs, q_dtype="bf16", sinks=sinks)
    got = pa.prefill(bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
                     torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(tables), _i32(ctxs), _i32(qlens), scale,
                     k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda(), sinks=bf16_to_dev(sinks),
                     route="tiled")
    torch.cuda.synchronize()
    got = dev_to_f32(got)
    assert_close_abs(got, want, 5e-2)
    assert np.all(got[1, 77:] == 0) and np.all(got[2, 1:] == 0)
    # with a sliding window: the asynchronous-copy kernel (power-of-two blocks) takes it, the register-staged one does not
    wargs = (bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
             torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(tables), _i32(ctxs), _i32(qlens), scale)
    wkw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda(), sliding_window=50, route="tiled")
    if bs == 24:
        with pytest.raises(RuntimeError):
            pa.prefill(*wargs, **wkw)
    else:
        want = O.paged_prefill(q, kq, vq, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), scale,
                               k_scale=ks, v_scale=vs, q_dtype="bf16", sliding_window=50)
        assert_close_abs(dev_to_f32(pa.prefill(*wargs, **wkw)), want, 5e-2)


def test_prefill_fp8_pool_kernels_agree(pa):
    """The asynchronous-copy kernel (raw ring + expansion pass) and the register-staged kernel on the same fp8 pool."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(77)
    T, D, Hq, Hkv, bs = 300, 128, 4, 2, 32
    qlens, prefixes = [300, 150, 64], [700, 0, 33]
    ctxs = [p + t for p, t in zip(prefixes, qlens)]
    k, v, tables = make_paged(rng, 3, Hkv, D, bs, ctxs)
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    # unused pool rows and the scales of unused blocks may hold anything
    used = np.zeros(k.shape[0], bool)
    for b in range(3):
        used[tables[b, :(ctxs[b] + bs - 1) // bs]] = True
    ks[~used] = np.nan
    vs[~used] = np.nan
    q = O.round_to_bf16(rng.standard_normal((3, T, Hq, D)).astype(np.float32))
    args = (bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
            torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(tables), _i32(ctxs), _i32(qlens), 0.09)
    kw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda(), route="tiled")
    a = dev_to_f32(pa.prefill(*args, **kw))
    lib.pa_debug_set(3, 1)
    try:
        b_ = dev_to_f32(pa.prefill(*args, **kw))
    finally:
        lib.pa_debug_set(3, 0)
    assert np.isfinite(a).all() and np.isfinite(b_).all()
    assert np.max(np.abs(a - b_)) <= 2 ** -5
    ks0, vs0 = np.nan_to_num(ks, nan=1.0), np.nan_to_num(vs, nan=1.0)
    want = O.paged_prefill(q, kq, vq, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), 0.09,
                           k_scale=ks0, v_scale=vs0, q_dtype="bf16")
    assert_close_abs(a, want, 5e-2)


def test_prefill_fp8_pool_split_over_key_tiles(pa):
    """One long fp8 context, one chunk: the split form of the fp8 kernel, with and without a window."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(91)
    T, D, Hq, Hkv, bs = 200, 128, 4, 1, 32
    ctxs, qlens = [5200], [200]
    k, v, tables = make_paged(rng, 1, Hkv, D, bs, ctxs)
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    q = O.round_to_bf16(rng.standard_normal((1, T, Hq, D)).astype(np.float32))
    assert lib.pa_prefill_workspace_bytes(1, T, Hq, Hkv, D, bs, tables.shape[1]) > 0
    args = (bf16_to_dev(q), torch.from_numpy(kq).cuda().view(torch.float8_e4m3fn),
            torch.from_numpy(vq).cuda().view(torch.float8_e4m3fn), _i32(tables), _i32(ctxs), _i32(qlens), 0.09)
    for window in (None, 900):
        want = O.paged_prefill(q, kq, vq, tables, np.asarray(ctxs, np.int32), np.asarray(qlens, np.int32), 0.09,
                               k_scale=ks, v_scale=vs, q_dtype="bf16", sliding_window=window)
        kw = dict(k_scale=torch.from_numpy(ks).cuda(), v_scale=torch.from_numpy(vs).cuda(), sliding_window=window, route="tiled")
        got = dev_to_f32(pa.prefill(*args, **kw))
        lib.pa_debug_set(6, 0)
        try:
            unsplit = dev_to_f32(pa.prefill(*args, **kw))
        finally:
            lib.pa_debug_set(6, 1)
        assert_close_abs(got, want, 5e-2)
        assert np.max(np.abs(got - unsplit)) <= 2 ** -6


@pytest.mark.parametrize("T,impl", [(40, 0), (200, 0), (200, 1)])
def test_query_lens_beyond_seq_lens_counts_the_first_rows(pa, T, impl):
    """query_lens[b] > seq_lens[b] (a caller's slip): every kernel clamps the query length to the
    context, so the first seq_lens[b] rows of q are the sequence's tokens, without a prefix, and the
    other rows are padding -- the tiled kernels (asynchronous and register-staged) and the verify
    kernel agree with each other and with the oracle on the clamped lengths."""
    from nkipy_amd import _lib
    rng = np.random.default_rng(40 + T)
    B, Hq, Hkv, D, bs = 3, 8, 2, 128, 32
    ctxs = [25, T + 30, 7]
    qlens = [T, T, 9]                 # sequences 0 and 2 claim more query tokens than they have context
    clamped = [min(a, c) for a, c in zip(qlens, ctxs)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, T, Hq, D)).astype(np.float32)
    want = O.paged_prefill(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                           np.asarray(ctxs, np.int32), np.asarray(clamped, np.int32), 0.09)
    args = (bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), _i32(qlens), 0.09)
    _lib.load().pa_debug_set(3, impl)
    try:
        tiled = pa.prefill(*args, route="tiled")
        torch.cuda.synchronize()
    finally:
        _lib.load().pa_debug_set(3, 0)
    assert_close_abs(dev_to_f32(tiled), want, BF16_TOL)
    assert np.all(dev_to_f32(tiled)[0, 25:] == 0) and np.all(dev_to_f32(tiled)[2, 7:] == 0)
    if T <= 64:
        ver = pa.prefill(*args, route="verify")
        torch.cuda.synchronize()
        assert_close_abs(dev_to_f32(ver), want, BF16_TOL)
