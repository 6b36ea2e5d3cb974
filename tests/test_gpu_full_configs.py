"""The five BASELINE configurations at full size on the GPU: the oracle checks every
sequence where it finishes in seconds (configs 1, 2) and a seeded sample of
sequences / heads where it would take minutes (configs 3, 4, 5); size-independent
properties cover the rest of the output."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, dev_bits, dev_to_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    return nkipy_amd


def _decode(pa, w):
    out = pa.decode(w.q, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.scale, k_scale=w.k_scale,
                    v_scale=w.v_scale, partition_size=w.partition_size, max_seq_len=w.max_seq_len,
                    validate_tables=True)
    torch.cuda.synchronize()
    return out


def test_config2_full_size_every_sequence(pa):
    from nkipy_amd import workloads as W
    w = W.make_decode(2)
    got = dev_to_f32(_decode(pa, w))
    want = O.paged_decode(dev_bits(w.q), dev_bits(w.k_cache), dev_bits(w.v_cache), w.block_tables.cpu().numpy(),
                          w.ctx.astype(np.int32), w.scale, q_dtype="bf16")
    assert_close_abs(got, want, 2e-2)
    # convex-hull property on the whole output: |out| <= max |V|
    assert np.abs(got).max() <= float(w.v_cache.float().abs().max()) + 1e-3


def test_config5_full_size_sampled_sequences(pa):
    from nkipy_amd import workloads as W
    w = W.make_decode(5)
    got = dev_to_f32(_decode(pa, w))
    assert np.isfinite(got).all()
    order = np.argsort(w.ctx)
    # shortest, median and longest context, plus every 9th sequence: 18 of 128
    sample = sorted({int(order[0]), int(order[-1]), int(order[len(order) // 2])} | set(range(3, 128, 9)))
    assert len(sample) >= 16
    kc, vc = dev_bits(w.k_cache), dev_bits(w.v_cache)
    ks, vs = w.k_scale.cpu().numpy(), w.v_scale.cpu().numpy()
    tables = w.block_tables.cpu().numpy()
    want = O.paged_decode(dev_bits(w.q)[sample], kc, vc, tables[sample], w.ctx[sample].astype(np.int32), w.scale,
                          k_scale=ks, v_scale=vs, q_dtype="bf16")
    assert_close_abs(got[sample], want, 5e-2)
    # invariance to the physical placement of blocks, over the whole batch: swap two
    # halves of the pool and remap the tables -> identical output bits
    nb = w.k_cache.shape[0]
    perm = torch.roll(torch.arange(nb, device="cuda"), nb // 2)          # block i moves to perm[i]
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nb, device="cuda")
    k2, v2 = w.k_cache[inv].contiguous(), w.v_cache[inv].contiguous()
    ks2, vs2 = w.k_scale[inv].contiguous(), w.v_scale[inv].contiguous()
    t2 = torch.where(w.block_tables >= 0, perm[w.block_tables.clamp(min=0).long()].int(), w.block_tables)
    out2 = pa.decode(w.q, k2, v2, t2.contiguous(), w.seq_lens, w.scale, k_scale=ks2, v_scale=vs2,
                     partition_size=w.partition_size, max_seq_len=w.max_seq_len)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(out2), dev_bits(_decode(pa, w)))


def test_config3_full_size_sampled(pa):
    """Every sequence, one q head of every kv group (the head's place in its group varies with the
    sequence), against the oracle; the rest of the output through the hull property."""
    from nkipy_amd import workloads as W
    w = W.make_prefill()
    got = pa.prefill(w.q, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.query_lens, w.scale,
                     validate_tables=True)
    torch.cuda.synchronize()
    g = dev_to_f32(got)
    assert np.isfinite(g).all()
    qb, kb, vb = dev_bits(w.q), dev_bits(w.k_cache), dev_bits(w.v_cache)
    tables, lens, qlens = w.block_tables.cpu().numpy(), w.seq_lens.cpu().numpy(), w.query_lens.cpu().numpy()
    B, T, Hq, D = w.q.shape
    n_rep = Hq // w.k_cache.shape[2]
    for b in range(B):
        heads = [hk * n_rep + (b + hk) % n_rep for hk in range(w.k_cache.shape[2])]     # 8 heads, one per kv group
        want = O.paged_prefill(qb, kb, vb, tables, lens, qlens, w.scale, seqs=[b], heads=heads)
        assert_close_abs(g[b][:, heads], want[b][:, heads], 2e-2)
    assert np.abs(g).max() <= float(w.v_cache.float().abs().max()) + 1e-3


def test_config3_aliased_prefix_blocks_give_identical_bits(pa):
    """Sequences 0-3 of config 3 read their shared prefix through the same physical blocks.  Give
    sequence 1 the queries and the new tokens' K/V of sequence 0 (copied into its own private
    blocks): everything it attends to is then equal, part of it through aliased blocks and part
    through its own, and its output must equal sequence 0's bit for bit, at full size."""
    from nkipy_amd import workloads as W
    w = W.make_prefill()
    bs = w.k_cache.shape[1]
    shared = int(w.prefix[0]) // bs
    n0 = (int(w.prefix[0]) + w.q.shape[1] + bs - 1) // bs
    assert int(w.prefix[0]) % bs == 0 and int(w.prefix[1]) == int(w.prefix[0]) and shared > 0
    t0, t1 = w.block_tables[0, shared:n0].long(), w.block_tables[1, shared:n0].long()
    assert torch.equal(w.block_tables[0, :shared], w.block_tables[1, :shared])        # aliased prefix
    assert not bool((t0 == t1).any())                                                  # private tails
    w.k_cache[t1] = w.k_cache[t0]
    w.v_cache[t1] = w.v_cache[t0]
    w.q[1] = w.q[0]
    got = pa.prefill(w.q, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.query_lens, w.scale)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(got[0]), dev_bits(got[1]))
    assert not np.array_equal(dev_bits(got[0]), dev_bits(got[2]))      # sequence 2 kept its own tokens


def test_config4_full_size_sampled(pa):
    """Eight (batch, head) pairs, one for every phase offset h mod 8, both batches, against the oracle."""
    from nkipy_amd import workloads as W
    w = W.make_blocksparse()
    got = pa.blocksparse_prefill(w.q, w.k, w.v, w.scale, block=w.block, local_blocks=w.local_blocks,
                                 vert_stride=w.vert_stride)
    torch.cuda.synchronize()
    g = dev_to_f32(got)
    assert np.isfinite(g).all()
    items = [(0, 0), (1, 9), (0, 18), (1, 27), (0, 4), (1, 13), (0, 22), (1, 31)]
    assert sorted(h % 8 for _, h in items) == list(range(8))
    for b, h in items:
        sl = tuple(dev_bits(x[b:b + 1, :, h:h + 1].contiguous()) for x in (w.q, w.k, w.v))
        want = O.blocksparse_prefill(*sl, w.scale, block=w.block, local_blocks=w.local_blocks,
                                     vert_stride=w.vert_stride, head_ids=[h])[0, :, 0]
        assert_close_abs(g[b][:, h], want, 2e-2)
    # the first 64 rows only see block 0: plain causal attention there, for every head
    first = O.blocksparse_prefill(dev_bits(w.q[:, :64]), dev_bits(w.k[:, :64]), dev_bits(w.v[:, :64]), w.scale,
                                  block=64, local_blocks=1, vert_stride=1)
    assert_close_abs(g[:, :64], first, 2e-2)
