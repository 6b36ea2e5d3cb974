"""Pins for the oracle's output projection (the reference's `np.matmul(output, o_weight)` (+ o_bias),
examples/models/qwen3/kernels/attention.py:143-147, gpt_oss/kernels/attention.py:155-163):
an independent library, a float64 element-by-element restatement, and closed forms that a
transposed operand, a dropped bias or a wrong reshape would fail."""
import numpy as np
import torch

from oracle import paged_attention_oracle as O


def _bf(rng, *shape):
    return O.round_to_bf16(rng.standard_normal(shape).astype(np.float32))


def test_against_torch_matmul_bf16_inputs(rng):
    x, w, b = _bf(rng, 3, 5, 4, 32), _bf(rng, 128, 48), _bf(rng, 48)
    want = torch.matmul(torch.from_numpy(x).reshape(3, 5, 128).double(), torch.from_numpy(w).double()) + torch.from_numpy(b).double()
    got = O.o_proj(x, w, b)
    assert got.shape == (3, 5, 48)
    # float32 accumulation of 128 products, then one bf16 rounding: within one bf16 step of the exact result
    assert np.all(np.abs(got - want.numpy()) <= 2.0 ** -8 * np.abs(want.numpy()) + 1e-5)
    assert np.array_equal(got, O.round_to_bf16(got))                     # values are bf16-representable
    # bf16 bit patterns in = float values in
    assert np.array_equal(O.o_proj(O.f32_to_bf16_bits(x), O.f32_to_bf16_bits(w), O.f32_to_bf16_bits(b)), got)


def test_float64_element_by_element(rng):
    x, w = _bf(rng, 4, 64), _bf(rng, 64, 8)
    want = np.zeros((4, 8))
    for m in range(4):
        for n in range(8):
            want[m, n] = sum(float(x[m, k]) * float(w[k, n]) for k in range(64))     # x row . w COLUMN
    assert np.array_equal(O.o_proj(x, w, acc=np.float64), O.round_to_bf16(want.astype(np.float32)))


def test_closed_forms(rng):
    x = _bf(rng, 2, 3, 2, 32)
    eye = np.eye(64, dtype=np.float32)
    assert np.array_equal(O.o_proj(x, eye), x.reshape(2, 3, 64))         # identity weight: the reshape (head-major, then d)
    perm = eye[:, ::-1]                                                  # w[k, n] = 1 iff n = 63 - k: out[n] = x[63 - n]
    assert np.array_equal(O.o_proj(x, perm), x.reshape(2, 3, 64)[..., ::-1])
    w = _bf(rng, 64, 16)
    b = _bf(rng, 16)
    zero = np.zeros_like(x)
    assert np.array_equal(O.o_proj(zero, w, b), np.broadcast_to(b, (2, 3, 16)))      # bias alone, same for every row
    assert np.array_equal(O.o_proj(zero, w), np.zeros((2, 3, 16), np.float32))
    # linearity in x (exact in float64 before the rounding): two one-hot rows select and add rows of w
    e = np.zeros((1, 64), np.float32)
    e[0, 5], e[0, 40] = 1.0, 2.0
    assert np.array_equal(O.o_proj(e, w, acc=np.float64)[0], O.round_to_bf16((w[5].astype(np.float64) + 2.0 * w[40]).astype(np.float32)))
