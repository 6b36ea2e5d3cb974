"""Pins the oracle's attention math: brute force, torch SDPA, closed forms,
and the invariants that tie the paged forms to the reference's dense form."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


def _make_paged(rng, B, Hkv, D, bs, ctxs, extra_blocks=3, dtype=np.float32):
    nblk = [(c + bs - 1) // bs for c in ctxs]
    total = sum(nblk) + extra_blocks
    perm = rng.permutation(total)
    maxb = max(nblk) + 1
    tables = np.full((B, maxb), -1, dtype=np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    kc = _rand(rng, total, bs, Hkv, D).astype(dtype)
    vc = _rand(rng, total, bs, Hkv, D).astype(dtype)
    return kc, vc, tables


# ------------------------------------------------------------------ dense core
@pytest.mark.parametrize("prefix", [None, 0, 3])
def test_dense_vs_bruteforce_f64(rng, prefix):
    T, S, Hq, Hkv, D = 3, 7, 4, 2, 5
    if prefix is not None:
        S = prefix + T
    q, k, v = _rand(rng, T, Hq, D), _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    got = O.dense_attention(q, k, v, 0.37, prefix=prefix, acc=np.float64)
    want = O.attention_bruteforce_f64(q, k, v, 0.37, prefix=prefix)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-13)
    got32 = O.dense_attention(q, k, v, 0.37, prefix=prefix)
    assert np.allclose(got32, want, rtol=2e-5, atol=2e-6)


def test_dense_vs_bruteforce_with_mask(rng):
    T = S = 6
    Hq, Hkv, D = 2, 1, 4
    q, k, v = _rand(rng, T, Hq, D), _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    mask = rng.random((Hq, T, S)) < 0.6
    mask |= np.eye(T, dtype=bool)[None]
    got = O.dense_attention(q, k, v, 0.5, prefix=0, mask=mask, acc=np.float64)
    want = O.attention_bruteforce_f64(q, k, v, 0.5, prefix=0, mask=mask)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("causal", [False, True])
def test_dense_vs_torch_sdpa(rng, causal):
    T, Hq, Hkv, D = 33, 8, 2, 16
    S = T
    q, k, v = _rand(rng, T, Hq, D), _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    scale = 1.0 / np.sqrt(D)
    got = O.dense_attention(q, k, v, scale, prefix=0 if causal else None)
    tq = torch.from_numpy(q).permute(1, 0, 2)[None]
    tk = torch.from_numpy(k).permute(1, 0, 2)[None]
    tv = torch.from_numpy(v).permute(1, 0, 2)[None]
    ref = torch.nn.functional.scaled_dot_product_attention(
        tq, tk, tv, is_causal=causal, scale=float(scale), enable_gqa=True)
    ref = ref[0].permute(1, 0, 2).numpy()
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_closed_form_special_cases(rng):
    Hq, Hkv, D, S = 4, 2, 8, 9
    k, v = _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    # one key: the output is that value row, whatever q is
    o = O.dense_attention(_rand(rng, 1, Hq, D), k[:1], v[:1], 0.3)
    assert np.allclose(o[0], O.repeat_kv(v[:1], 2)[0], rtol=1e-6)
    # q = 0: uniform weights -> mean of the values
    o = O.dense_attention(np.zeros((1, Hq, D), np.float32), k, v, 0.3)
    assert np.allclose(o[0], O.repeat_kv(v, 2).mean(axis=0), rtol=1e-5, atol=1e-6)
    # one dominant key: output ~ that value row
    kk = k.copy()
    q = _rand(rng, 1, Hq, D)
    kk[5] = 0
    kk[5, :, 0] = 1.0
    q[..., 0] = 200.0
    o = O.dense_attention(q, kk * np.float32(1.0), v, 1.0)
    # make key 5 dominate by construction: score 200 vs O(1)-scale others
    s = np.einsum("hd,shd->hs", q[0], O.repeat_kv(kk, 2))
    assert np.all(s[:, 5] - np.delete(s, 5, axis=1).max(axis=1) > 50)
    assert np.allclose(o[0], O.repeat_kv(v, 2)[5], rtol=1e-5, atol=1e-6)
    # convex hull: every output coordinate lies between min and max of V
    o = O.dense_attention(_rand(rng, 3, Hq, D), k, v, 0.3)
    vr = O.repeat_kv(v, 2)
    assert np.all(o <= vr.max(axis=0)[None] + 1e-6) and np.all(o >= vr.min(axis=0)[None] - 1e-6)
    # first causal query with no prefix sees only key 0
    o = O.dense_attention(_rand(rng, 4, Hq, D), k[:4], v[:4], 0.3, prefix=0)
    assert np.allclose(o[0], vr[0], rtol=1e-6)


def test_gqa_equals_mha_on_repeated_kv(rng):
    T, S, Hq, Hkv, D = 2, 11, 8, 2, 8
    q, k, v = _rand(rng, T, Hq, D), _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    a = O.dense_attention(q, k, v, 0.2, prefix=S - T)
    b = O.dense_attention(q, np.repeat(k, 4, axis=1), np.repeat(v, 4, axis=1), 0.2, prefix=S - T)
    assert np.array_equal(a, b)


# ------------------------------------------------------------------ gather
def test_gather_is_np_take_and_bit_exact(rng):
    bs, Hkv, D = 4, 2, 3
    pool = rng.integers(0, 65536, size=(10, bs, Hkv, D)).astype(np.uint16)
    table = np.array([7, 2, 9, 0, -1], np.int32)
    for ctx in (1, 4, 5, 13, 16):
        g = O.gather_kv(pool, table, ctx)
        want = np.concatenate([pool[t] for t in table[: (ctx + bs - 1) // bs]])[:ctx]
        assert g.dtype == np.uint16 and np.array_equal(g, want)
    with pytest.raises(IndexError):
        O.gather_kv(pool, np.array([10], np.int32), 1)
    with pytest.raises(IndexError):
        O.gather_kv(pool, table, 17)  # would read the -1 padding entry


def test_gather_permutation_invariance(rng):
    pool = _rand(rng, 12, 4, 2, 3)
    table = rng.permutation(12)[:6].astype(np.int32)
    perm = rng.permutation(12)
    pool2 = np.empty_like(pool)
    pool2[perm] = pool  # block i moves to perm[i]
    table2 = perm[table].astype(np.int32)
    assert np.array_equal(O.gather_kv(pool, table, 22), O.gather_kv(pool2, table2, 22))


# ------------------------------------------------------------------ paged == dense
def test_identity_table_equals_dense_cache(rng):
    """A dense cache (B, S, Hkv, D) is a pool with an identity table."""
    B, S, Hq, Hkv, D, bs = 3, 32, 4, 2, 8, 8
    cache_k, cache_v = _rand(rng, B, S, Hkv, D), _rand(rng, B, S, Hkv, D)
    q = _rand(rng, B, Hq, D)
    ctx = np.array([5, 32, 17], np.int32)
    pool_k = cache_k.reshape(B * S // bs, bs, Hkv, D)
    pool_v = cache_v.reshape(B * S // bs, bs, Hkv, D)
    tables = np.arange(B * S // bs, dtype=np.int32).reshape(B, S // bs)
    got = O.paged_decode(q, pool_k, pool_v, tables, ctx, 0.35)
    for b in range(B):
        want = O.dense_attention(q[b][None], cache_k[b, :ctx[b]], cache_v[b, :ctx[b]], 0.35)[0]
        assert np.array_equal(got[b], want)


def test_paged_decode_vs_bruteforce(rng):
    B, Hq, Hkv, D, bs = 3, 4, 2, 4, 4
    ctxs = [1, 6, 9]
    kc, vc, tables = _make_paged(rng, B, Hkv, D, bs, ctxs)
    q = _rand(rng, B, Hq, D)
    got = O.paged_decode(q, kc, vc, tables, np.array(ctxs, np.int32), 0.5, acc=np.float64)
    for b in range(B):
        k = np.concatenate([kc[t] for t in tables[b] if t >= 0])[:ctxs[b]]
        v = np.concatenate([vc[t] for t in tables[b] if t >= 0])[:ctxs[b]]
        want = O.attention_bruteforce_f64(q[b][None], k, v, 0.5)[0]
        assert np.allclose(got[b], want, rtol=1e-6, atol=1e-6)


def test_zero_length_sequence_yields_zeros(rng):
    kc, vc, tables = _make_paged(rng, 2, 1, 4, 4, [0, 5])
    out = O.paged_decode(_rand(rng, 2, 2, 4), kc, vc, tables, np.array([0, 5], np.int32), 1.0)
    assert np.all(out[0] == 0) and np.any(out[1] != 0)


def test_prefill_T1_is_decode_and_P0_is_causal(rng):
    B, Hq, Hkv, D, bs = 2, 4, 2, 8, 4
    ctxs = [7, 12]
    kc, vc, tables = _make_paged(rng, B, Hkv, D, bs, ctxs)
    seq = np.array(ctxs, np.int32)
    q1 = _rand(rng, B, 1, Hq, D)
    a = O.paged_prefill(q1, kc, vc, tables, seq, np.array([1, 1], np.int32), 0.3, q_dtype="fp32")
    b = O.paged_decode(q1[:, 0], kc, vc, tables, seq, 0.3)
    assert np.array_equal(a[:, 0], b)
    # no prefix: plain causal self-attention over the gathered rows
    T = 12
    q = _rand(rng, B, T, Hq, D)
    qlens = np.array([7, 12], np.int32)
    got = O.paged_prefill(q, kc, vc, tables, seq, qlens, 0.3, q_dtype="fp32")
    for bi in range(B):
        k = O.gather_kv(kc, tables[bi], ctxs[bi])
        v = O.gather_kv(vc, tables[bi], ctxs[bi])
        want = O.dense_attention(q[bi, :qlens[bi]], k, v, 0.3, prefix=0)
        assert np.allclose(got[bi, :qlens[bi]], want, rtol=1e-6, atol=1e-6)
        assert np.all(got[bi, qlens[bi]:] == 0)


def test_prefill_with_prefix_vs_bruteforce(rng):
    B, Hq, Hkv, D, bs, T = 2, 2, 1, 4, 4, 3
    ctxs = [3 + 5, 3 + 0]
    kc, vc, tables = _make_paged(rng, B, Hkv, D, bs, ctxs)
    q = _rand(rng, B, T, Hq, D)
    got = O.paged_prefill(q, kc, vc, tables, np.array(ctxs, np.int32),
                          np.array([T, T], np.int32), 0.4, q_dtype="fp32", acc=np.float64)
    for b in range(B):
        k = O.gather_kv(kc, tables[b], ctxs[b])
        v = O.gather_kv(vc, tables[b], ctxs[b])
        want = O.attention_bruteforce_f64(q[b], k, v, 0.4, prefix=ctxs[b] - T)
        assert np.allclose(got[b], want, rtol=1e-6, atol=1e-6)


def test_aliased_prefix_blocks_read_identical_rows(rng):
    """Two sequences whose tables share physical prefix blocks see the same keys."""
    bs, Hkv, D = 4, 1, 4
    pool = _rand(rng, 10, bs, Hkv, D)
    t = np.array([[3, 8, 1], [3, 8, 6]], np.int32)
    a = O.gather_kv(pool, t[0], 8)
    b = O.gather_kv(pool, t[1], 8)
    assert np.array_equal(a, b)


# ------------------------------------------------------------------ fp8 / bf16 storage
def test_fp8_paged_decode_equals_dense_on_dequantised(rng):
    B, Hq, Hkv, D, bs = 2, 8, 1, 16, 8
    ctxs = [13, 24]
    kc, vc, tables = _make_paged(rng, B, Hkv, D, bs, ctxs)
    kq, ks = O.quantize_kv_fp8(kc)
    vq, vs = O.quantize_kv_fp8(vc)
    q = O.round_to_bf16(_rand(rng, B, Hq, D))
    got = O.paged_decode(q, kq, vq, tables, np.array(ctxs, np.int32), 0.25,
                         k_scale=ks, v_scale=vs, q_dtype="bf16")
    kd, vd = O.dequantize_kv_fp8(kq, ks), O.dequantize_kv_fp8(vq, vs)
    want = O.paged_decode(q, kd, vd, tables, np.array(ctxs, np.int32), 0.25, q_dtype="bf16")
    assert np.array_equal(got, want)
    # and the quantisation error itself is small against the unquantised answer
    full = O.paged_decode(q, kc, vc, tables, np.array(ctxs, np.int32), 0.25, q_dtype="bf16")
    assert np.max(np.abs(got - full)) < 0.1


def test_bf16_bits_input_equals_float_input(rng):
    B, Hq, Hkv, D, bs = 2, 4, 2, 8, 4
    ctxs = [5, 9]
    kc, vc, tables = _make_paged(rng, B, Hkv, D, bs, ctxs)
    q = _rand(rng, B, Hq, D)
    a = O.paged_decode(O.f32_to_bf16_bits(q), O.f32_to_bf16_bits(kc), O.f32_to_bf16_bits(vc),
                       tables, np.array(ctxs, np.int32), 0.3, q_dtype="bf16")
    b = O.paged_decode(O.round_to_bf16(q), O.round_to_bf16(kc), O.round_to_bf16(vc),
                       tables, np.array(ctxs, np.int32), 0.3, q_dtype="bf16")
    assert np.array_equal(a, b)
    assert np.array_equal(a, O.round_to_bf16(a))


# ------------------------------------------------------------------ split-K
@pytest.mark.parametrize("psize", [1, 3, 8, 64])
def test_split_k_merge_equals_single_pass(rng, psize):
    S, Hq, Hkv, D = 29, 4, 2, 8
    q, k, v = _rand(rng, Hq, D) * 3, _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    parts = [O.partition_stats(q, k[s:s + psize], v[s:s + psize], 0.7) for s in range(0, S, psize)]
    m, l, o = O.merge_partitions(*zip(*parts))
    want = O.dense_attention(q[None], k, v, 0.7, acc=np.float64)[0]
    assert np.allclose(o, want, rtol=1e-12, atol=1e-13)
    m1, l1, _ = O.partition_stats(q, k, v, 0.7)
    assert np.allclose(m, m1) and np.allclose(l, l1, rtol=1e-12)


# ------------------------------------------------------------------ blocksparse
def test_block_mask_pattern():
    bm = O.blocksparse_block_mask(16, head=0, local_blocks=4, vert_stride=8)
    assert bm[10, 10] and bm[10, 7] and not bm[10, 6] and bm[10, 0] and bm[10, 8]
    assert not bm[3, 4]  # causal
    bm3 = O.blocksparse_block_mask(16, head=3, local_blocks=4, vert_stride=8)
    # phase: (j + 3) % 8 == 0 -> j = 5, 13
    assert bm3[12, 5] and not bm3[12, 0] and not bm3[12, 8]
    assert bm3[15, 13]
    # C4's count: average active blocks per head over 32 heads of a 128x128 grid
    cnt = np.mean([O.blocksparse_block_mask(128, h, 4, 8).sum() for h in range(32)])
    assert cnt == 1474.75


def test_blocksparse_equals_masked_dense_and_dense_limit(rng):
    B, S, H, D, blk = 1, 24, 3, 4, 4
    q, k, v = _rand(rng, B, S, H, D), _rand(rng, B, S, H, D), _rand(rng, B, S, H, D)
    got = O.blocksparse_prefill(q, k, v, 0.5, block=blk, local_blocks=2, vert_stride=3,
                                q_dtype="fp32", acc=np.float64)
    for h in range(H):
        bm = O.blocksparse_block_mask(S // blk, h, 2, 3)
        tok = np.kron(bm, np.ones((blk, blk), bool))
        want = O.attention_bruteforce_f64(q[0][:, h:h + 1], k[0][:, h:h + 1], v[0][:, h:h + 1],
                                          0.5, prefix=0, mask=tok[None])
        assert np.allclose(got[0][:, h:h + 1], want, rtol=1e-6, atol=1e-6)
    dense = O.blocksparse_prefill(q, k, v, 0.5, block=blk, local_blocks=10 ** 6, vert_stride=3,
                                  q_dtype="fp32")
    want = np.stack([O.dense_attention(q[0], k[0], v[0], 0.5, prefix=0)])
    assert np.allclose(dense, want, rtol=1e-6, atol=1e-6)
