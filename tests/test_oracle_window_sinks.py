"""Pins the oracle's sliding-window and attention-sink options (the reference's
examples/models/gpt_oss/kernels/attention.py:117-148): brute force, the reference's own
mask construction restated with np.triu / np.tril, and closed forms a wrong sign or an
off-by-one in the window would break."""
import numpy as np
import pytest

from oracle import paged_attention_oracle as O


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("window", [None, 1, 2, 5, 100])
@pytest.mark.parametrize("with_sinks", [False, True])
def test_window_and_sinks_vs_bruteforce_f64(rng, window, with_sinks):
    T, P, Hq, Hkv, D = 4, 6, 4, 2, 5
    S = P + T
    q, k, v = _rand(rng, T, Hq, D), _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    sinks = _rand(rng, Hq) * 2 if with_sinks else None
    got = O.dense_attention(q, k, v, 0.37, prefix=P, window=window, sinks=sinks, acc=np.float64)
    want = O.attention_bruteforce_f64(q, k, v, 0.37, prefix=P, window=window, sinks=sinks)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("W", [1, 3, 8])
def test_window_equals_the_reference_mask_construction(rng, W):
    """attention.py:118-135: full_mask = triu(NEG, k=1) + tril(NEG, k=-W), one row per query
    position gathered by start_pos + arange(seq_len), added to the scores."""
    T, P, H, D = 3, 7, 2, 4
    S = P + T
    q, k, v = _rand(rng, T, H, D), _rand(rng, S, H, D), _rand(rng, S, H, D)
    NEG = -100000.0
    full = np.triu(np.ones((S, S)) * NEG, k=1) + np.tril(np.ones((S, S)) * NEG, k=-W)
    rows = full[P + np.arange(T)]                                  # [T, S]
    scores = np.einsum("thd,shd->hts", q.astype(np.float64), k.astype(np.float64)) * 0.5 + rows[None]
    e = np.exp(scores - scores.max(-1, keepdims=True))
    want = np.einsum("hts,shd->thd", e / e.sum(-1, keepdims=True), v.astype(np.float64))
    got = O.dense_attention(q, k, v, 0.5, prefix=P, window=W, acc=np.float64)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-13)
    visible = (rows == 0).sum(axis=1)
    assert list(visible) == [min(W, P + t + 1) for t in range(T)]   # exactly W keys once the context is long enough


def test_window_closed_forms(rng):
    T, P, Hq, Hkv, D = 5, 9, 4, 2, 8
    S = P + T
    q, k, v = _rand(rng, T, Hq, D), _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    plain = O.dense_attention(q, k, v, 0.3, prefix=P, acc=np.float64)
    # a window at least as long as the context changes nothing
    assert np.array_equal(O.dense_attention(q, k, v, 0.3, prefix=P, window=S, acc=np.float64), plain)
    assert not np.allclose(O.dense_attention(q, k, v, 0.3, prefix=P, window=S - 1, acc=np.float64)[-1], plain[-1])
    # W = 1: every query sees only its own key, so the output is its own V row
    own = O.dense_attention(q, k, v, 0.3, prefix=P, window=1, acc=np.float64)
    want = np.repeat(v[P:P + T].astype(np.float64), Hq // Hkv, axis=1)
    assert np.allclose(own, want, rtol=0, atol=1e-12)
    # a window equals dense attention over the last W keys only (decode form)
    W = 4
    dec = O.dense_attention(q[-1:], k, v, 0.3, prefix=S - 1, window=W, acc=np.float64)
    cut = O.dense_attention(q[-1:], k[S - W:], v[S - W:], 0.3, prefix=W - 1, acc=np.float64)
    assert np.allclose(dec, cut, rtol=1e-12, atol=1e-13)


def test_sink_closed_forms(rng):
    T, P, Hq, Hkv, D = 3, 5, 4, 2, 8
    S = P + T
    q, k, v = _rand(rng, T, Hq, D), _rand(rng, S, Hkv, D), _rand(rng, S, Hkv, D)
    plain = O.dense_attention(q, k, v, 0.3, prefix=P, acc=np.float64)
    # a sink of -inf takes no mass
    none = O.dense_attention(q, k, v, 0.3, prefix=P, sinks=np.full(Hq, -np.inf), acc=np.float64)
    assert np.allclose(none, plain, rtol=1e-13, atol=0)
    # a sink only shrinks the output: out = plain * Z / (Z + exp(sink)), Z = sum exp(score)
    sinks = np.array([0.5, -1.0, 2.0, 0.0])
    got = O.dense_attention(q, k, v, 0.3, prefix=P, sinks=sinks, acc=np.float64)
    for t in range(T):
        for h in range(Hq):
            s = 0.3 * (k[:P + t + 1, h // 2].astype(np.float64) @ q[t, h].astype(np.float64))
            z = np.exp(s).sum()
            assert np.allclose(got[t, h], plain[t, h] * z / (z + np.exp(sinks[h])), rtol=1e-12)
    # a huge sink takes everything
    big = O.dense_attention(q, k, v, 0.3, prefix=P, sinks=np.full(Hq, 80.0), acc=np.float64)
    assert np.abs(big).max() < 1e-25
    # a sink is a key that every query of the head sees, with score = sink and a zero value row:
    # for one head, append such a key at the front (visible to all causal rows) with q-independent score
    h = 1
    qh, kh, vh = q[:, h:h + 1], k[:, 0:1], v[:, 0:1]
    got1 = O.dense_attention(qh, kh, vh, 0.3, prefix=P, sinks=sinks[h:h + 1], acc=np.float64)
    # emulate with an extra feature dimension: q gets a constant 1, the sink key is e_extra * sink / scale
    q2 = np.concatenate([qh, np.ones((T, 1, 1), np.float32)], axis=2).astype(np.float64)
    k2 = np.concatenate([kh.astype(np.float64), np.zeros((S, 1, 1))], axis=2)
    sink_key = np.zeros((1, 1, D + 1)); sink_key[0, 0, D] = sinks[h] / 0.3
    k2 = np.concatenate([sink_key, k2], axis=0)
    v2 = np.concatenate([np.zeros((1, 1, D)), vh.astype(np.float64)], axis=0)
    want1 = O.dense_attention(q2, k2, v2, 0.3, prefix=P + 1, acc=np.float64)
    assert np.allclose(got1, want1, rtol=1e-12, atol=1e-14)


def test_paged_forms_pass_the_options_through(rng):
    B, Hq, Hkv, D, bs = 2, 4, 2, 8, 4
    ctxs = np.array([11, 6], np.int32)
    nb = 8
    kc, vc = _rand(rng, nb, bs, Hkv, D), _rand(rng, nb, bs, Hkv, D)
    tables = np.array([[5, 2, 7], [1, 4, -1]], np.int32)
    sinks = _rand(rng, Hq)
    q = _rand(rng, B, 3, Hq, D)
    ql = np.array([3, 2], np.int32)
    got = O.paged_prefill(q, kc, vc, tables, ctxs, ql, 0.4, q_dtype="fp32", sliding_window=5, sinks=sinks)
    for b in range(B):
        k = O.gather_kv(kc, tables[b], ctxs[b])
        v = O.gather_kv(vc, tables[b], ctxs[b])
        want = O.attention_bruteforce_f64(q[b, :ql[b]], k, v, 0.4, prefix=ctxs[b] - ql[b], window=5, sinks=sinks)
        assert np.allclose(got[b, :ql[b]], want, rtol=2e-5, atol=2e-6)
    # decode == the last row of a prefill whose last token is that query
    dec = O.paged_decode(q[:, -1][[0]], kc, vc, tables[[0]], ctxs[[0]], 0.4, sliding_window=5, sinks=sinks)
    assert np.allclose(dec[0], got[0, 2], rtol=1e-6, atol=1e-7)
