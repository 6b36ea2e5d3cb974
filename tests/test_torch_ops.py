"""The dispatcher-level operators: registration, schemas and the CPU refusal without a GPU; on the
GPU the same results as the Python ops, through torch.ops and inside a captured HIP graph."""
import numpy as np
import pytest
import torch

from tests.pa_testlib import bf16_to_dev, dev_bits, make_paged


def test_ops_are_registered_with_mutation_schemas():
    import nkipy_amd.torch_ops as T
    for name in T.OPS:
        assert hasattr(torch.ops.nkipy_amd, name)
    s = str(torch.ops.nkipy_amd.paged_decode.default._schema)
    assert "Tensor(a6!) out" in s and "-> ()" in s
    assert str(torch.ops.nkipy_amd.paged_kv_write.default._schema).count("!") == 2        # both caches
    assert str(torch.ops.nkipy_amd.paged_kv_write_fp8.default._schema).count("!") == 4    # ... and both scale tables
    assert str(torch.ops.nkipy_amd.decode_step.default._schema).count("!") == 3           # both caches and out
    assert str(torch.ops.nkipy_amd.decode_step_fp8.default._schema).count("!") == 5
    assert str(torch.ops.nkipy_amd.verify_step.default._schema).count("!") == 3
    assert str(torch.ops.nkipy_amd.verify_step_fp8.default._schema).count("!") == 5


def test_ops_refuse_cpu_tensors_and_trace_with_fake_tensors():
    import nkipy_amd.torch_ops  # noqa: F401
    q = torch.zeros(2, 4, 64, dtype=torch.bfloat16)
    kc = torch.zeros(4, 16, 2, 64, dtype=torch.bfloat16)
    bt = torch.zeros(2, 2, dtype=torch.int32)
    sl = torch.ones(2, dtype=torch.int32)
    with pytest.raises(NotImplementedError):
        torch.ops.nkipy_amd.paged_decode(q, kc, kc, bt, sl, 0.1, torch.empty_like(q))
    with pytest.raises(NotImplementedError):
        torch.ops.nkipy_amd.decode_step(q, kc[:2, 0], kc[:2, 0], kc, kc, bt, sl, sl, 0.1, torch.empty_like(q))
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        fq = torch.zeros(2, 4, 64, dtype=torch.bfloat16, device="cuda")
        fk = torch.zeros(4, 16, 2, 64, dtype=torch.bfloat16, device="cuda")
        fb = torch.zeros(2, 2, dtype=torch.int32, device="cuda")
        fs = torch.ones(2, dtype=torch.int32, device="cuda")
        assert torch.ops.nkipy_amd.paged_decode(fq, fk, fk, fb, fs, 0.1, torch.empty_like(fq)) is None


def _i32(x):
    return torch.from_numpy(np.asarray(x, dtype=np.int32)).cuda()


@pytest.mark.gpu
def test_ops_match_the_python_ops_and_replay_in_a_graph():
    import nkipy_amd as pa
    import nkipy_amd.torch_ops  # noqa: F401
    rng = np.random.default_rng(5)
    B, Hq, Hkv, D, bs = 3, 8, 2, 128, 32
    ctxs = [40, 700, 2100]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    kd, vd, td, sd = bf16_to_dev(k), bf16_to_dev(v), _i32(tables), _i32(ctxs)
    q = bf16_to_dev(rng.standard_normal((B, Hq, D)).astype(np.float32))
    sinks = torch.randn(Hq, device="cuda")
    want = pa.decode(q, kd, vd, td, sd, 0.09, sinks=sinks, sliding_window=600)
    out = torch.empty_like(q)
    torch.ops.nkipy_amd.paged_decode(q, kd, vd, td, sd, 0.09, out, sinks=sinks, sliding_window=600)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(out), dev_bits(want))

    # verify-sized prefill + the KV write in front of it, as one captured graph replayed on new inputs
    T = 4
    qlens = _i32([4, 4, 4])
    xq = bf16_to_dev(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    xk = bf16_to_dev(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    xv = bf16_to_dev(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    o = torch.empty_like(xq)

    def step():
        torch.ops.nkipy_amd.paged_kv_write(xk, xv, kd, vd, td, sd, qlens)
        torch.ops.nkipy_amd.paged_prefill(xq, kd, vd, td, sd, qlens, 0.09, o)

    step()                                   # eager once: loads the library, sizes the cached workspace
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for _ in range(3):
        for t in (xq, xk, xv):
            t.copy_(bf16_to_dev(rng.standard_normal(tuple(t.shape)).astype(np.float32)))
        g.replay()
        torch.cuda.synchronize()
        got = dev_bits(o).copy()
        step()                               # the program's own eager work between replays
        torch.cuda.synchronize()
        assert np.array_equal(got, dev_bits(o))

    # the Q half of the pre-attention transform on the attention operator, K and V through the write operator
    cos, sin = pa.rope_tables(D, 4096)
    wn = bf16_to_dev(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32))
    torch.ops.nkipy_amd.k_norm_rope_kv_write(xk, xv, kd, vd, td, sd, qlens, cos, sin, wn)
    want = pa.prefill(xq, kd, vd, td, sd, qlens, 0.09, q_transform=pa.QTransform(cos, sin, wn))
    torch.ops.nkipy_amd.paged_prefill(xq, kd, vd, td, sd, qlens, 0.09, o, rope_cos=cos, rope_sin=sin, q_norm_weight=wn)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(o), dev_bits(want))
    two = pa.prefill(pa.qk_norm_rope_kv_write(xq, xk, xv, kd, vd, td, sd, qlens, cos, sin, q_norm_weight=wn,
                                              k_norm_weight=wn), kd, vd, td, sd, qlens, 0.09)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(o), dev_bits(two))


@pytest.mark.gpu
def test_graph_keeps_its_scratch_when_the_batch_grows_and_a_larger_eager_call_follows():
    """A decode + projection step captured through the dispatcher, once with the ops' cached scratch and once
    with the caller's `workspace`, is replayed after (i) more slots have gone live and contexts have grown (the
    lengths and tables are device tensors the replay reads) and (ii) an eager call on the capture stream's
    neighbour, the current stream, that needs a far larger scratch and a cache flush of every eager entry.
    Each replay must equal the eager result on the same state."""
    import nkipy_amd as pa
    import nkipy_amd.torch_ops  # noqa: F401
    from nkipy_amd import paged_attn
    rng = np.random.default_rng(11)
    B, Hq, Hkv, D, bs, N = 16, 8, 2, 128, 32, 512
    cap_tokens = 4096
    ctxs_small = [0] * B
    ctxs_small[0], ctxs_small[1] = 37, 300
    ctxs_big = [int(x) for x in rng.integers(500, cap_tokens, B)]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, [cap_tokens] * B)
    kd, vd, td = bf16_to_dev(k), bf16_to_dev(v), _i32(tables)
    sd = _i32(ctxs_small)
    q = bf16_to_dev(rng.standard_normal((B, Hq, D)).astype(np.float32))
    w = bf16_to_dev((rng.standard_normal((Hq * D, N)) / 32).astype(np.float32))
    att, proj = torch.empty_like(q), torch.empty((B, N), dtype=torch.bfloat16, device="cuda")
    need = max(paged_attn.decode_workspace_bytes(B, Hq, D, cap_tokens, 512), paged_attn.o_proj_workspace_bytes(B, Hq * D, N))
    own = torch.empty(need, dtype=torch.uint8, device="cuda")

    def step(ws):
        torch.ops.nkipy_amd.paged_decode(q, kd, vd, td, sd, 0.09, att, max_seq_len=cap_tokens, workspace=ws, partition_size=512)
        torch.ops.nkipy_amd.o_proj(att, w, proj, workspace=ws)

    step(None)
    torch.cuda.synchronize()
    graphs = []
    for ws in (None, own):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            step(ws)
        graphs.append(g)
    # between capture and replay: the batch grows, and an eager call that outgrows every cached scratch runs
    sd.copy_(_i32(ctxs_big))
    q.copy_(bf16_to_dev(rng.standard_normal((B, Hq, D)).astype(np.float32)))
    big_B = 512
    kb, vb, tb = make_paged(rng, big_B, Hkv, D, bs, [64] * big_B)
    bigq = bf16_to_dev(rng.standard_normal((big_B, 4 * Hkv, D)).astype(np.float32))
    pa.decode(bigq, bf16_to_dev(kb), bf16_to_dev(vb), _i32(tb), _i32([64] * big_B), 0.09)
    paged_attn._workspaces.clear()                      # every eager entry gone: a graph's scratch must not have been one
    torch.cuda.synchronize()
    step(own)
    torch.cuda.synchronize()
    want_att, want_proj = dev_bits(att).copy(), dev_bits(proj).copy()
    for g in graphs:
        for _ in range(2):
            att.zero_()
            proj.zero_()
            g.replay()
            torch.cuda.synchronize()
            assert np.array_equal(dev_bits(att), want_att)
            assert np.array_equal(dev_bits(proj), want_proj)
            pa.decode(bigq, bf16_to_dev(kb), bf16_to_dev(vb), _i32(tb), _i32([64] * big_B), 0.09)   # eager work between replays
            torch.cuda.synchronize()
