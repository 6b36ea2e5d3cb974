"""GPU parity: fused QK RMSNorm + RoPE + paged KV write (through the C ABI) vs the oracle."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, bf16_to_dev, dev_bits, dev_to_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


def _i32(a):
    return torch.from_numpy(np.asarray(a, np.int32)).cuda()


def _setup(rng, B, T, Hq, Hkv, D, bs, seqs, qlens):
    seqs, qlens = np.asarray(seqs, np.int32), np.asarray(qlens, np.int32)
    nblk = (np.maximum(seqs, 1) + bs - 1) // bs
    nb = int(nblk.sum()) + 2
    perm = rng.permutation(nb).astype(np.int32)
    tables = np.full((B, int(nblk.max()) + 1), -1, np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    xq = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32) * 2)
    xk = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32) * 2)
    xv = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    wq = O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32))
    wk = O.round_to_bf16(1.0 + 0.2 * rng.standard_normal(D).astype(np.float32))
    return nb, tables, seqs, qlens, xq, xk, xv, wq, wk


def _ulp_close(got, want, ulps):
    """|got - want| within `ulps` bf16 steps of the larger magnitude."""
    tol = ulps * 2.0 ** -8 * np.maximum(np.abs(got), np.abs(want)) + 1e-30
    bad = np.abs(got - want) > tol
    assert not bad.any(), f"{bad.sum()} of {bad.size} beyond {ulps} bf16 ulp, worst {np.abs(got - want).max()}"


@pytest.mark.parametrize("D,bs,base", [(128, 16, 1000000.0), (64, 32, 10000.0), (256, 64, 10000.0)])
def test_rope_only_is_bit_exact(pa, rng, D, bs, base):
    """Without the norm every operation is an exactly specified bf16 rounding: same bits."""
    B, T, Hq, Hkv = 3, 37, 4, 2
    nb, tables, seqs, qlens, xq, xk, xv, _, _ = _setup(rng, B, T, Hq, Hkv, D, bs, seqs=[37, 90, 4], qlens=[37, 20, 0])
    cos, sin = O.rope_tables(D, 128, base)
    dcos, dsin = pa.rope_tables(D, 128, base)
    assert np.array_equal(dev_to_f32(dcos), cos) and np.array_equal(dev_to_f32(dsin), sin)
    pk = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    pv = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    dk = torch.from_numpy(pk.view(np.int16).copy()).cuda().view(torch.bfloat16)
    dv = torch.from_numpy(pv.view(np.int16).copy()).cuda().view(torch.bfloat16)
    q_out = pa.qk_norm_rope_kv_write(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, _i32(tables),
                                     _i32(seqs), _i32(qlens), dcos, dsin)
    want_q, want_k = O.qk_norm_rope(xq, xk, seqs, qlens, cos, sin)
    O.kv_write(O.f32_to_bf16_bits(want_k), O.f32_to_bf16_bits(xv), pk, pv, tables, seqs, qlens)
    assert np.array_equal(dev_bits(q_out), O.f32_to_bf16_bits(want_q))
    assert np.array_equal(dev_bits(dk), pk) and np.array_equal(dev_bits(dv), pv)


def test_norm_and_rope_into_bf16_pool(pa, rng):
    """With the norm the mean of squares is summed in a different order than NumPy's: results
    agree to one bf16 step (two after the rotation's own roundings)."""
    B, T, Hq, Hkv, D, bs = 2, 50, 8, 2, 128, 32
    nb, tables, seqs, qlens, xq, xk, xv, wq, wk = _setup(rng, B, T, Hq, Hkv, D, bs, seqs=[75, 50], qlens=[50, 50])
    cos, sin = O.rope_tables(D, 256, 1000000.0)
    dcos, dsin = pa.rope_tables(D, 256, 1000000.0)
    pk = np.zeros((nb, bs, Hkv, D), np.uint16); pv = np.zeros_like(pk)
    dk = torch.zeros((nb, bs, Hkv, D), dtype=torch.bfloat16, device="cuda"); dv = torch.zeros_like(dk)
    dq = bf16_to_dev(xq)
    out = pa.qk_norm_rope_kv_write(dq, bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, _i32(tables), _i32(seqs), _i32(qlens),
                                   dcos, dsin, q_norm_weight=bf16_to_dev(wq), k_norm_weight=bf16_to_dev(wk), eps=1e-6, out=dq)
    assert out.data_ptr() == dq.data_ptr()                                   # in place on q
    want_q, want_k = O.qk_norm_rope(xq, xk, seqs, qlens, cos, sin, q_norm_weight=wq, k_norm_weight=wk, eps=1e-6)
    O.kv_write(O.f32_to_bf16_bits(want_k), O.f32_to_bf16_bits(xv), pk, pv, tables, seqs, qlens)
    _ulp_close(dev_to_f32(out), want_q, 3)
    _ulp_close(dev_to_f32(dk), O.bf16_bits_to_f32(pk), 3)
    assert np.array_equal(dev_bits(dv), pv)                                  # V is a plain scatter
    exact = (dev_to_f32(out) == want_q).mean()
    assert exact > 0.98, f"only {exact:.3f} of the elements are bit-identical"


def test_norm_rope_fp8_pool_then_prefill_attention(pa, rng):
    """Pre-attention into an fp8 pool followed by the chunked prefill: the attention output matches
    the oracle run on the oracle's own pool."""
    B, T, Hq, Hkv, D, bs = 2, 48, 8, 2, 128, 16
    nb, tables, seqs, qlens, xq, xk, xv, wq, wk = _setup(rng, B, T, Hq, Hkv, D, bs, seqs=[48, 48], qlens=[48, 48])
    cos, sin = O.rope_tables(D, 64, 10000.0)
    dcos, dsin = pa.rope_tables(D, 64, 10000.0)
    pk = np.zeros((nb, bs, Hkv, D), np.uint8); pv = np.zeros_like(pk)
    ks = np.zeros((nb, Hkv), np.float32); vs = np.zeros_like(ks)
    dk = torch.zeros((nb, bs, Hkv, D), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn); dv = torch.zeros_like(dk)
    dks = torch.zeros((nb, Hkv), dtype=torch.float32, device="cuda"); dvs = torch.zeros_like(dks)
    q_out = pa.qk_norm_rope_kv_write(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, _i32(tables), _i32(seqs),
                                     _i32(qlens), dcos, dsin, q_norm_weight=bf16_to_dev(wq), k_norm_weight=bf16_to_dev(wk),
                                     eps=1e-6, k_scale=dks, v_scale=dvs)
    want_q, want_k = O.qk_norm_rope(xq, xk, seqs, qlens, cos, sin, q_norm_weight=wq, k_norm_weight=wk, eps=1e-6)
    O.kv_write(O.f32_to_bf16_bits(want_k), O.f32_to_bf16_bits(xv), pk, pv, tables, seqs, qlens, k_scale=ks, v_scale=vs)
    assert np.array_equal(dev_bits(dv), pv) and np.array_equal(dvs.cpu().numpy(), vs)       # V: no norm in its way
    assert np.allclose(dks.cpu().numpy(), ks, rtol=2.0 ** -7)                               # K scales follow the K values
    deq_got = O.fp8_e4m3fn_decode(dev_bits(dk)) * dks.cpu().numpy()[:, None, :, None]
    deq_want = O.fp8_e4m3fn_decode(pk) * ks[:, None, :, None]
    assert_close_abs(deq_got, deq_want, 0.25 * float(ks.max()) * 448 / 8)                   # at most one e4m3 step of the largest values
    # decode attention over the device's own fp8 pool vs the oracle over the same pool
    scale = float(np.float32(1.0) / np.float32(np.sqrt(D)))
    q1 = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
    got = pa.decode(bf16_to_dev(q1), dk, dv, _i32(tables), _i32(seqs), scale, k_scale=dks, v_scale=dvs)
    want = O.paged_decode(q1, dev_bits(dk), dev_bits(dv), tables, seqs, scale, k_scale=dks.cpu().numpy(),
                          v_scale=dvs.cpu().numpy(), q_dtype="bf16")
    assert_close_abs(dev_to_f32(got), want, 5e-2)
    _ulp_close(dev_to_f32(q_out), want_q, 3)


def test_argument_validation(pa):
    z = torch.zeros((1, 2, 2, 128), dtype=torch.bfloat16, device="cuda")
    kv = torch.zeros((1, 2, 1, 128), dtype=torch.bfloat16, device="cuda")
    pool = torch.zeros((2, 16, 1, 128), dtype=torch.bfloat16, device="cuda")
    t, one = _i32([[0, 1]]), _i32([2])
    cos, sin = pa.rope_tables(128, 8)
    with pytest.raises(ValueError):
        pa.qk_norm_rope_kv_write(z, kv, kv, pool, pool, t, one, one, cos[:, :32].contiguous(), sin)
    with pytest.raises(ValueError):
        pa.qk_norm_rope_kv_write(z, kv, kv, pool, pool, t, one, one, cos, sin, q_norm_weight=torch.ones(64, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        pa.qk_norm_rope_kv_write(z, kv, kv, pool.float(), pool.float(), t, one, one, cos, sin)
    z96 = torch.zeros((1, 2, 2, 96), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        pa.qk_norm_rope_kv_write(z96, z96[:, :, :1].contiguous(), z96[:, :, :1].contiguous(),
                                 torch.zeros((2, 16, 1, 96), dtype=torch.bfloat16, device="cuda"),
                                 torch.zeros((2, 16, 1, 96), dtype=torch.bfloat16, device="cuda"), t, one, one, cos, sin)
