"""Pins for the oracle's QK RMSNorm / RoPE restatement (CPU only): closed forms, a float64
restatement and an independent library routine."""
import numpy as np
import torch

from oracle import paged_attention_oracle as O


def test_rope_tables_follow_the_definition():
    D, n, base = 16, 40, 1000000.0
    cos, sin = O.rope_tables(D, n, base)
    assert cos.shape == (n, D // 2) and sin.shape == (n, D // 2)
    assert np.all(cos[0] == 1.0) and np.all(sin[0] == 0.0)                  # position 0: no rotation
    ang = np.arange(n)[:, None] * (1.0 / base ** (np.arange(0, D, 2) / D))[None, :]
    assert np.allclose(cos, np.cos(ang), atol=2 ** -8) and np.allclose(sin, np.sin(ang), atol=2 ** -8)
    assert np.array_equal(cos, O.round_to_bf16(cos)) and np.array_equal(sin, O.round_to_bf16(sin))   # bf16 values
    assert np.allclose(cos[:, 0], np.cos(np.arange(n)), atol=2 ** -8)       # first pair turns by one radian per token


def test_rmsnorm_against_float64_and_torch():
    rng = np.random.default_rng(11)
    x = O.round_to_bf16(rng.standard_normal((3, 5, 4, 128)).astype(np.float32) * 3)
    w = O.round_to_bf16(rng.standard_normal(128).astype(np.float32))
    got = O.rmsnorm(x, w, 1e-6)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * w64
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-30)   # one bf16 rounding of the exact value
    lib = torch.nn.functional.rms_norm(torch.from_numpy(x), (128,), torch.from_numpy(w), 1e-6).numpy()
    assert np.allclose(got, lib, rtol=2.0 ** -7, atol=1e-6)
    ones = np.ones(128, np.float32)
    unit = O.rmsnorm(x, ones, 0.0)
    assert np.allclose((unit.astype(np.float64) ** 2).mean(-1), 1.0, atol=2e-2)   # unit mean square
    assert np.array_equal(O.rmsnorm(4 * x, ones, 0.0), unit)                      # scale invariance (power of two: exact)


def test_rope_closed_forms():
    rng = np.random.default_rng(12)
    T, H, D = 9, 3, 32
    cos, sin = O.rope_tables(D, 64, 10000.0)
    x = O.round_to_bf16(rng.standard_normal((2, T, H, D)).astype(np.float32))
    pos = np.arange(5, 5 + T)
    y = O.apply_rope(x, cos[pos], sin[pos])
    assert y.shape == x.shape and np.array_equal(y, O.round_to_bf16(y))
    # exact rotation in float64 within a few bf16 roundings (two products, one sum per element)
    c, s = cos[pos][None, :, None, :].astype(np.float64), sin[pos][None, :, None, :].astype(np.float64)
    x0, x1 = x[..., :D // 2].astype(np.float64), x[..., D // 2:].astype(np.float64)
    want = np.concatenate([x0 * c - x1 * s, x0 * s + x1 * c], -1)
    assert np.allclose(y, want, atol=3e-2, rtol=2e-2)
    # position 0 is the identity, bit for bit
    assert np.array_equal(O.apply_rope(x, np.repeat(cos[:1], T, 0), np.repeat(sin[:1], T, 0)), x)
    # a rotation keeps the norm of each (x0, x1) pair
    n_in = np.sqrt(x0 ** 2 + x1 ** 2)
    n_out = np.sqrt(y[..., :D // 2].astype(np.float64) ** 2 + y[..., D // 2:].astype(np.float64) ** 2)
    assert np.allclose(n_in, n_out, rtol=2e-2, atol=1e-2)
    # what attention sees depends on relative position only: <rope(q, m), rope(k, n)> == <rope(q, m+d), rope(k, n+d)>
    q = O.round_to_bf16(rng.standard_normal((1, 1, 1, D)).astype(np.float32))
    k = O.round_to_bf16(rng.standard_normal((1, 1, 1, D)).astype(np.float32))
    def dot(m, n):
        return float((O.apply_rope(q, cos[m:m + 1], sin[m:m + 1]) * O.apply_rope(k, cos[n:n + 1], sin[n:n + 1])).sum())
    assert abs(dot(3, 1) - dot(13, 11)) < 0.15 and abs(dot(7, 7) - float((q * k).sum())) < 0.15


def test_qk_norm_rope_positions_and_padding():
    rng = np.random.default_rng(13)
    B, T, Hq, Hkv, D = 2, 4, 4, 2, 16
    cos, sin = O.rope_tables(D, 32)
    xq = O.round_to_bf16(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    xk = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    w = O.round_to_bf16(rng.standard_normal(D).astype(np.float32))
    seq, ql = np.array([10, 3], np.int32), np.array([4, 2], np.int32)
    qo, ko = O.qk_norm_rope(xq, xk, seq, ql, cos, sin, q_norm_weight=w, k_norm_weight=None, eps=1e-6)
    assert np.all(qo[1, 2:] == 0) and np.all(ko[1, 2:] == 0)              # padding rows
    # sequence 0, token 2 sits at position 10 - 4 + 2 = 8 (gpt_oss/kernels/attention.py:85)
    want_q = O.apply_rope(O.rmsnorm(xq[0, 2], w, 1e-6)[None], cos[8:9], sin[8:9])[0]
    want_k = O.apply_rope(xk[0, 2][None], cos[8:9], sin[8:9])[0]           # no k norm requested
    assert np.array_equal(qo[0, 2], want_q) and np.array_equal(ko[0, 2], want_k)
    # uint16 bf16 bit patterns are accepted like values
    qo2, ko2 = O.qk_norm_rope(O.f32_to_bf16_bits(xq), O.f32_to_bf16_bits(xk), seq, ql, cos, sin,
                              q_norm_weight=O.f32_to_bf16_bits(w), eps=1e-6)
    assert np.array_equal(qo, qo2) and np.array_equal(ko, ko2)
