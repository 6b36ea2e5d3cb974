"""GPU parity at the ends of the shape range: one context of a million tokens (32 768 table entries,
2 048 chunks of the balanced schedule for a single sequence) and a batch of 30 000 short sequences."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, bf16_to_dev, dev_to_f32, make_paged

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2


def _i32(x):
    return torch.from_numpy(np.asarray(x, np.int32)).cuda()


def test_million_token_context():
    import nkipy_amd as pa
    rng = np.random.default_rng(0)
    ctxs, Hq, Hkv, D, bs = [1_048_576 + 5, 9], 8, 2, 128, 32
    k, v, tables = make_paged(rng, len(ctxs), Hkv, D, bs, ctxs)
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    kd, vd, td, sd = bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs)
    lens = np.asarray(ctxs, np.int32)
    q = O.round_to_bf16(rng.standard_normal((2, Hq, D)).astype(np.float32))
    want = O.paged_decode(q, k, v, tables, lens, 0.09, q_dtype="bf16")
    assert_close_abs(dev_to_f32(pa.decode(bf16_to_dev(q), kd, vd, td, sd, 0.09)), want, BF16_TOL)
    for T, route, heads in ((4, "verify", None), (130, "tiled", [0, 5])):
        qv = O.round_to_bf16(rng.standard_normal((2, T, Hq, D)).astype(np.float32))
        ql = np.asarray([min(T, c) for c in ctxs], np.int32)
        want = O.paged_prefill(qv, k, v, tables, lens, ql, 0.09, q_dtype="bf16", heads=heads)
        got = dev_to_f32(pa.prefill(bf16_to_dev(qv), kd, vd, td, sd, _i32(ql), 0.09, route=route))
        sel = slice(None) if heads is None else heads
        assert_close_abs(got[:, :, sel], want[:, :, sel], BF16_TOL)


def test_thirty_thousand_sequences():
    import nkipy_amd as pa
    rng = np.random.default_rng(1)
    B = 30000
    ctxs = rng.integers(0, 90, size=B)
    k, v, tables = make_paged(rng, B, 2, 128, 16, np.maximum(ctxs, 1))
    k, v = O.round_to_bf16(k), O.round_to_bf16(v)
    q = O.round_to_bf16(rng.standard_normal((B, 8, 128)).astype(np.float32))
    want = O.paged_decode(q, k, v, tables, ctxs.astype(np.int32), 0.09, q_dtype="bf16")
    got = dev_to_f32(pa.decode(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs), 0.09))
    assert_close_abs(got, want, BF16_TOL)
    assert np.all(got[ctxs == 0] == 0)
