"""Pins for the oracle's paged KV write (CPU only).

bf16 / fp32 pools restate the reference's dense cache update; the fp8 scale maintenance has
no reference counterpart and is pinned by its defining properties."""
import numpy as np
import pytest

from oracle import paged_attention_oracle as O


def _tables(rng, B, nblk_each, num_blocks):
    perm = rng.permutation(num_blocks).astype(np.int32)
    return perm[:B * nblk_each].reshape(B, nblk_each)


def test_identity_table_equals_reference_dense_update():
    """examples/models/gpt_oss/kernels/attention.py:85,98-100: cache[:, query_pos] = x with
    query_pos = start_pos + arange(seq_len); prefill form :94-95 is start_pos = 0."""
    rng = np.random.default_rng(5)
    B, T, Hkv, D, bs, max_seq = 3, 6, 2, 8, 4, 16
    dense_k = rng.standard_normal((B, max_seq, Hkv, D)).astype(np.float32)
    dense_v = rng.standard_normal((B, max_seq, Hkv, D)).astype(np.float32)
    xk = rng.standard_normal((B, T, Hkv, D)).astype(np.float32)
    xv = rng.standard_normal((B, T, Hkv, D)).astype(np.float32)
    for start_pos in (0, 3, 10):
        ref_k, ref_v = dense_k.copy(), dense_v.copy()
        query_pos = start_pos + np.arange(T, dtype=np.int32)
        ref_k[:, query_pos] = xk
        ref_v[:, query_pos] = xv
        # the same cache seen as a pool through the identity table
        pool_k = dense_k.copy().reshape(B * max_seq // bs, bs, Hkv, D)
        pool_v = dense_v.copy().reshape(B * max_seq // bs, bs, Hkv, D)
        tables = np.arange(B * max_seq // bs, dtype=np.int32).reshape(B, max_seq // bs)
        seq = np.full(B, start_pos + T, np.int32)
        O.kv_write(xk, xv, pool_k, pool_v, tables, seq, np.full(B, T, np.int32))
        assert np.array_equal(pool_k.reshape(B, max_seq, Hkv, D), ref_k)
        assert np.array_equal(pool_v.reshape(B, max_seq, Hkv, D), ref_v)


def test_bf16_rows_travel_bit_for_bit_and_nothing_else_changes():
    rng = np.random.default_rng(6)
    B, T, Hkv, D, bs, nb = 2, 5, 2, 16, 4, 12
    pool_k = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    pool_v = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    k0, v0 = pool_k.copy(), pool_v.copy()
    xk = rng.integers(0, 65536, size=(B, T, Hkv, D), dtype=np.uint16)      # any bit pattern, NaNs included
    xv = rng.integers(0, 65536, size=(B, T, Hkv, D), dtype=np.uint16)
    tables = _tables(rng, B, 4, nb)
    seq, ql = np.array([7, 3], np.int32), np.array([5, 2], np.int32)      # sequence 1: 3 padding rows
    O.kv_write(xk, xv, pool_k, pool_v, tables, seq, ql)
    touched = np.zeros((nb, bs), bool)
    for b in range(B):
        for t in range(ql[b]):
            pos = seq[b] - ql[b] + t
            blk, off = tables[b, pos // bs], pos % bs
            assert np.array_equal(pool_k[blk, off], xk[b, t]) and np.array_equal(pool_v[blk, off], xv[b, t])
            touched[blk, off] = True
    assert np.array_equal(pool_k[~touched], k0[~touched]) and np.array_equal(pool_v[~touched], v0[~touched])


def test_fp8_whole_fresh_blocks_equal_block_quantisation():
    rng = np.random.default_rng(7)
    B, Hkv, D, bs, nb = 2, 3, 16, 8, 10
    T = 2 * bs
    x = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32) * 3)
    y = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    tables = _tables(rng, B, 3, nb)
    pool_k = rng.integers(0, 256, size=(nb, bs, Hkv, D), dtype=np.uint8)   # stale codes and scales must not matter
    pool_v = rng.integers(0, 256, size=(nb, bs, Hkv, D), dtype=np.uint8)
    ks = rng.random((nb, Hkv)).astype(np.float32) * 100
    vs = rng.random((nb, Hkv)).astype(np.float32) * 100
    O.kv_write(O.f32_to_bf16_bits(x), O.f32_to_bf16_bits(y), pool_k, pool_v, tables,
               np.full(B, T, np.int32), np.full(B, T, np.int32), k_scale=ks, v_scale=vs)
    for b in range(B):
        for j in range(2):
            want_codes, want_scale = O.quantize_kv_fp8(x[b, j * bs:(j + 1) * bs][None])
            assert np.array_equal(pool_k[tables[b, j]], want_codes[0])
            assert np.array_equal(ks[tables[b, j]], want_scale[0])


def test_fp8_append_keeps_codes_when_scale_stays_and_recodes_when_it_grows():
    rng = np.random.default_rng(8)
    Hkv, D, bs, nb = 2, 16, 8, 4
    tables = np.array([[2, 0, 1, 3]], np.int32)
    pool_k = np.zeros((nb, bs, Hkv, D), np.uint8); pool_v = np.zeros_like(pool_k)
    ks = np.zeros((nb, Hkv), np.float32); vs = np.zeros_like(ks)
    toks = rng.standard_normal((bs, Hkv, D)).astype(np.float32)
    toks[0] *= 4.0            # the first token sets a scale the next ones stay under ...
    toks[5, 1] *= 40.0        # ... until token 5 raises it for head 1 only
    toks = O.round_to_bf16(toks)
    hist = []
    for t in range(bs):
        x = O.f32_to_bf16_bits(toks[t][None, None])
        before, s_before = pool_k[2].copy(), ks[2].copy()
        O.kv_write(x, x, pool_k, pool_v, tables, np.array([t + 1], np.int32), np.array([1], np.int32),
                   k_scale=ks, v_scale=vs)
        assert np.all(ks[2] >= s_before) or t == 0                     # scales never shrink
        for h in range(Hkv):
            if t > 0 and ks[2, h] == s_before[h]:
                assert np.array_equal(pool_k[2, :t, h], before[:t, h])  # untouched bits when the scale stays
        hist.append(ks[2].copy())
    assert hist[5][1] > hist[4][1] and hist[5][0] == hist[4][0]
    assert np.array_equal(pool_k, pool_v) and np.array_equal(ks, vs)
    # the final scale is absmax / 448 over everything the block holds, and every row dequantises
    # within the e4m3 rounding bound of the scale in force when it was (re)encoded: one rounding
    # of at most 2^-4 relative (3 mantissa bits) or half a subnormal step, twice for recoded rows
    want_scale = np.max(np.abs(toks), axis=(0, 2)) / np.float32(448.0)
    assert np.allclose(ks[2], want_scale, rtol=1e-6)
    deq = O.fp8_e4m3fn_decode(pool_k[2]) * ks[2][None, :, None]
    bound = 2 * (np.abs(toks) * 2.0 ** -4 + ks[2][None, :, None] * 2.0 ** -10)
    assert np.all(np.abs(deq - toks) <= bound)


def test_zero_rows_and_errors():
    Hkv, D, bs = 1, 8, 4
    pool = np.full((2, bs, Hkv, D), 0x55, np.uint8); pool2 = pool.copy()
    ks = np.full((2, Hkv), 7.0, np.float32); vs = ks.copy()
    z = np.zeros((1, 4, Hkv, D), np.uint16)
    O.kv_write(z, z, pool, pool2, np.array([[1, 0]], np.int32), np.array([4], np.int32), np.array([4], np.int32),
               k_scale=ks, v_scale=vs)
    assert ks[1, 0] == 1.0 and np.all(pool[1] == 0)          # all-zero slab: scale 1 so the division is defined
    assert ks[0, 0] == 7.0 and np.all(pool[0] == 0x55)
    with pytest.raises(ValueError):
        O.kv_write(z, z, pool, pool2, np.array([[1, 0]], np.int32), np.array([2], np.int32), np.array([4], np.int32),
                   k_scale=ks, v_scale=vs)
    with pytest.raises(IndexError):
        O.kv_write(z, z, pool, pool2, np.array([[5, 0]], np.int32), np.array([4], np.int32), np.array([4], np.int32),
                   k_scale=ks, v_scale=vs)
    O.kv_write(z, z, pool, pool2, np.array([[1, 0]], np.int32), np.array([4], np.int32), np.array([0], np.int32),
               k_scale=ks, v_scale=vs)                      # nothing to write
