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
    sample = sorted({int(order[0]), int(order[-1]), int(order[len(order) // 2]), 3, 77})
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
    from nkipy_amd import workloads as W
    w = W.make_prefill()
    got = pa.prefill(w.q, w.k_cache, w.v_cache, w.block_tables, w.seq_lens, w.query_lens, w.scale,
                     validate_tables=True)
    torch.cuda.synchronize()
    g = dev_to_f32(got)
    assert np.isfinite(g).all()
    heads = [0, 13, 31]
    want = O.paged_prefill(dev_bits(w.q), dev_bits(w.k_cache), dev_bits(w.v_cache), w.block_tables.cpu().numpy(),
                           w.seq_lens.cpu().numpy(), w.query_lens.cpu().numpy(), w.scale, seqs=[0, 6], heads=heads)
    for b in (0, 6):
        assert_close_abs(g[b][:, heads], want[b][:, heads], 2e-2)
    # sequences 0-3 alias the same prefix blocks: with identical new tokens and queries they
    # must agree bit for bit; with their own (different) tokens they must not
    assert not np.array_equal(dev_bits(got[0]), dev_bits(got[1]))
    # first query row of a no-prefix sequence would equal V[0]; here check the property that
    # holds for every row: output inside the hull of V
    assert np.abs(g).max() <= float(w.v_cache.float().abs().max()) + 1e-3


def test_config4_full_size_sampled(pa):
    from nkipy_amd import workloads as W
    w = W.make_blocksparse()
    got = pa.blocksparse_prefill(w.q, w.k, w.v, w.scale, block=w.block, local_blocks=w.local_blocks,
                                 vert_stride=w.vert_stride)
    torch.cuda.synchronize()
    g = dev_to_f32(got)
    assert np.isfinite(g).all()
    items = [(0, 0), (1, 13)]
    want = O.blocksparse_prefill(dev_bits(w.q), dev_bits(w.k), dev_bits(w.v), w.scale, block=w.block,
                                 local_blocks=w.local_blocks, vert_stride=w.vert_stride, items=items)
    for b, h in items:
        assert_close_abs(g[b][:, h], want[b][:, h], 2e-2)
    # the first 64 rows only see block 0: plain causal attention there, for every head
    first = O.blocksparse_prefill(dev_bits(w.q[:, :64]), dev_bits(w.k[:, :64]), dev_bits(w.v[:, :64]), w.scale,
                                  block=64, local_blocks=1, vert_stride=1)
    assert_close_abs(g[:, :64], first, 2e-2)
