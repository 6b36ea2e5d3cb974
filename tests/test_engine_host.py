"""Host logic of the engine glue (no GPU): block allocator and cache bookkeeping."""
import numpy as np
import pytest
import torch

from nkipy_amd.engine import BlockAllocator, OutOfBlocks, PagedKVCache


def test_allocator_alloc_share_free():
    a = BlockAllocator(6)
    x = a.alloc(4)
    assert x == [0, 1, 2, 3] and a.num_free == 2
    with pytest.raises(OutOfBlocks):
        a.alloc(3)
    assert a.num_free == 2                              # a failed request changes nothing
    a.share(x[:2])
    a.free(x)                                           # first user gone: blocks 2, 3 return, 0 and 1 stay
    assert a.num_free == 4 and a.refcount(0) == 1 and a.refcount(2) == 0
    a.free(x[:2])
    assert a.num_free == 6
    with pytest.raises(ValueError):
        a.free([0])                                     # double free
    with pytest.raises(ValueError):
        a.share([5])                                    # never allocated
    y = a.alloc(6)
    assert sorted(y) == list(range(6)) and a.num_free == 0
    with pytest.raises(ValueError):
        BlockAllocator(0)


def _cache(**kw):
    args = dict(num_blocks=10, block_size=4, n_kv_heads=2, head_dim=8, max_seqs=3, max_blocks_per_seq=5, device="cpu")
    args.update(kw)
    return PagedKVCache(**args)


def test_cache_extend_publishes_tables_and_lengths():
    c = _cache()
    c.extend([0, 2], [6, 1])
    assert c.lens == [6, 0, 1] and len(c.blocks[0]) == 2 and len(c.blocks[2]) == 1
    bt, sl = c.block_tables.numpy(), c.seq_lens.numpy()
    assert sl.tolist() == [6, 0, 1]
    assert bt[0, :2].tolist() == c.blocks[0] and np.all(bt[0, 2:] == -1) and np.all(bt[1] == -1)
    c.extend([0], [2])                                  # 8 tokens: still 2 blocks
    assert len(c.blocks[0]) == 2 and c.seq_lens[0].item() == 8
    c.extend([0], [1])                                  # 9 tokens: third block
    assert len(c.blocks[0]) == 3 and c.block_tables[0, 2].item() == c.blocks[0][2]
    assert len(set(c.blocks[0]) | set(c.blocks[2])) == 4   # disjoint blocks
    with pytest.raises(ValueError):
        c.extend([2], [40])                             # beyond the table's capacity
    assert c.lens[2] == 1


def test_cache_out_of_blocks_is_all_or_nothing():
    c = _cache(num_blocks=3)
    c.extend([0], [8])                                  # 2 blocks
    with pytest.raises(OutOfBlocks):
        c.extend([1, 2], [4, 4])                        # needs 2, one free
    assert c.lens == [8, 0, 0] and c.allocator.num_free == 1 and not c.blocks[1] and not c.blocks[2]


def test_cache_fork_shares_full_blocks_and_copies_the_tail():
    c = _cache(dtype=torch.float8_e4m3fn)
    c.extend([0], [10])                                 # blocks: 2 full + 1 partial
    tail = c.blocks[0][2]
    c.k_cache.view(torch.uint8)[tail] = 7
    c.k_scale[tail] = 0.5
    c.fork(0, 1)
    assert c.blocks[1][:2] == c.blocks[0][:2] and c.blocks[1][2] != tail
    assert c.allocator.refcount(c.blocks[0][0]) == 2 and c.allocator.refcount(tail) == 1
    assert torch.all(c.k_cache.view(torch.uint8)[c.blocks[1][2]] == 7) and torch.all(c.k_scale[c.blocks[1][2]] == 0.5)
    assert c.seq_lens.tolist() == [10, 10, 0]
    c.release(0)
    assert c.allocator.refcount(c.blocks[1][0]) == 1 and c.allocator.num_free == 10 - 3
    assert c.seq_lens.tolist() == [0, 10, 0] and torch.all(c.block_tables[0] == -1)
    with pytest.raises(ValueError):
        c.fork(1, 1)
    c.release(1)
    assert c.allocator.num_free == 10


def test_begin_step_is_all_or_nothing_and_layers_share_tables():
    c = _cache(num_layers=3)
    assert len(c.k_caches) == 3 and c.k_caches[1].data_ptr() != c.k_caches[2].data_ptr()
    c.begin_step([5, 0, 2], 5)
    assert c.lens == [5, 0, 2] and c.step_tokens == 5 and c.query_lens.tolist() == [5, 0, 2]
    assert c.allocator.num_free == 10 - 2 - 1                    # one reservation for all layers
    with pytest.raises(ValueError):
        c.begin_step([1, 1], 1)                                  # one length per slot
    with pytest.raises(ValueError):
        c.begin_step([2, 0, 0], 1)                               # longer than the step's token count
    with pytest.raises(OutOfBlocks):
        c.begin_step([0, 20, 12], 20)                            # 5 + 3 blocks wanted, 7 free
    assert c.lens == [5, 0, 2] and c.query_lens.tolist() == [5, 0, 2]   # nothing changed
    # a fork copies the partial tail block in every layer's pool
    for l in range(3):
        c.k_caches[l][c.blocks[0][1]] = float(l + 1)
    c.fork(0, 1)
    assert c.blocks[1][0] == c.blocks[0][0] and c.blocks[1][1] != c.blocks[0][1]
    for l in range(3):
        assert torch.all(c.k_caches[l][c.blocks[1][1]] == float(l + 1))
    with pytest.raises(ValueError):
        _cache(num_layers=0)


def test_rope_table_must_cover_the_longest_admitted_sequence():
    """Positions past the RoPE table are clamped by the kernels, so the layer refuses a table that is shorter
    than the longest sequence the cache admits: the table capacity, or the cache's max_model_len when the
    model's limit is lower (capacity is rounded up to whole blocks)."""
    import torch
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    cache = PagedKVCache(num_blocks=8, block_size=16, n_kv_heads=2, head_dim=64, max_seqs=2, max_blocks_per_seq=4,
                         device="cpu")
    short = (torch.zeros(63, 32, dtype=torch.bfloat16), torch.zeros(63, 32, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="max_positions >= 64"):
        PagedAttention(cache, 4, rope_tables=short)
    exact = (torch.zeros(64, 32, dtype=torch.bfloat16), torch.zeros(64, 32, dtype=torch.bfloat16))
    PagedAttention(cache, 4, rope_tables=exact)
    # a model of 60 positions over blocks of 16: capacity 64, limit 60; a 60-row table is enough, and the cache
    # refuses to grow a sequence past the limit
    limited = PagedKVCache(num_blocks=8, block_size=16, n_kv_heads=2, head_dim=64, max_seqs=2, max_blocks_per_seq=4,
                           device="cpu", max_model_len=60)
    PagedAttention(limited, 4, rope_tables=(torch.zeros(60, 32, dtype=torch.bfloat16), torch.zeros(60, 32, dtype=torch.bfloat16)))
    limited.extend([0], [60])
    with pytest.raises(ValueError, match="longest sequence"):
        limited.extend([0], [1])
    with pytest.raises(ValueError):
        PagedKVCache(num_blocks=8, block_size=16, n_kv_heads=2, head_dim=64, max_seqs=2, max_blocks_per_seq=4,
                     device="cpu", max_model_len=65)


def test_workspace_cache_is_bounded():
    """The per-(device, stream) scratch cache keeps the most recently used entries only."""
    import ctypes
    import torch
    from nkipy_amd import paged_attn
    paged_attn._workspaces.clear()
    dev = torch.device("cpu")
    bufs = [paged_attn._workspace(dev, 64, ctypes.c_void_p(1000 + i)) for i in range(paged_attn._WORKSPACE_SLOTS + 5)]
    assert len(paged_attn._workspaces) == paged_attn._WORKSPACE_SLOTS
    assert (dev, 1000) not in paged_attn._workspaces and (dev, 1000 + len(bufs) - 1) in paged_attn._workspaces
    again = paged_attn._workspace(dev, 32, ctypes.c_void_p(1000 + len(bufs) - 1))
    assert again is bufs[-1]                                  # reused, not reallocated
    bigger = paged_attn._workspace(dev, 4096, ctypes.c_void_p(1000 + len(bufs) - 1))
    assert bigger.numel() >= 4096 and len(paged_attn._workspaces) == paged_attn._WORKSPACE_SLOTS
    paged_attn._workspaces.clear()
