"""Engine glue around the paged attention ops: who owns the pool and who calls the ops.

The reference's model drivers own a dense per-layer cache, hand it to every layer call as
an aliased input/output and keep all buffers preallocated
(examples/models/qwen3/qwen3.py:54-71, 289-336, 372-396).  With a paged pool the same
role needs three small pieces:

* `BlockAllocator`  -- free list with reference counts (a block shared by a forked prefix
                       is freed when its last user goes);
* `PagedKVCache`    -- the K/V pool of one layer (bf16, or fp8-e4m3 with per-(block, kv
                       head) scales), the per-slot block lists and the device-resident
                       `block_tables` / `seq_lens` the kernels read;
* `PagedAttention`  -- one layer's step: optional QK RMSNorm + RoPE, KV write, then
                       prefill or decode attention, all into preallocated outputs
                       (the order of examples/models/qwen3/kernels/attention.py:78-144).

Host bookkeeping is plain Python lists (it is control plane: a few integers per
sequence and step); the per-step device work is one small host->device copy of the
changed table rows and lengths plus the kernels.  Nothing here imports the oracle and
there is no CPU attention path.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from . import paged_attn


class OutOfBlocks(RuntimeError):
    """The pool has fewer free blocks than a request needs (nothing was allocated)."""


class BlockAllocator:
    """Reference-counted free list over block ids 0 .. num_blocks-1."""

    def __init__(self, num_blocks: int):
        if num_blocks <= 0:
            raise ValueError("num_blocks must be positive")
        self.num_blocks = num_blocks
        self._free: List[int] = list(range(num_blocks - 1, -1, -1))   # pop() hands out 0, 1, 2, ...
        self._ref = [0] * num_blocks

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self, n: int) -> List[int]:
        if n < 0:
            raise ValueError("cannot allocate a negative number of blocks")
        if n > len(self._free):
            raise OutOfBlocks(f"{n} blocks requested, {len(self._free)} free")
        out = [self._free.pop() for _ in range(n)]
        for b in out:
            self._ref[b] = 1
        return out

    def share(self, blocks: Sequence[int]) -> None:
        """One more user for each of `blocks` (they must be live)."""
        for b in blocks:
            if self._ref[b] <= 0:
                raise ValueError(f"block {b} is not allocated")
        for b in blocks:
            self._ref[b] += 1

    def free(self, blocks: Sequence[int]) -> None:
        for b in blocks:
            if not 0 <= b < self.num_blocks or self._ref[b] <= 0:
                raise ValueError(f"block {b} is not allocated")
        for b in blocks:
            self._ref[b] -= 1
            if self._ref[b] == 0:
                self._free.append(b)

    def refcount(self, block: int) -> int:
        return self._ref[block]


class PagedKVCache:
    """K/V pool of one attention layer plus the tables the kernels read.

    Slots 0 .. max_seqs-1 are the rows of `block_tables` / `seq_lens`; a slot with
    seq_len 0 is idle.  `dtype` torch.bfloat16, or torch.float8_e4m3fn (then
    `k_scale` / `v_scale` [num_blocks, Hkv] float32 exist and are maintained by the write
    kernel).
    """

    def __init__(self, num_blocks: int, block_size: int, n_kv_heads: int, head_dim: int, *, max_seqs: int,
                 max_blocks_per_seq: int, dtype=torch.bfloat16, device="cuda"):
        if dtype not in (torch.bfloat16, torch.float8_e4m3fn):
            raise ValueError(f"unsupported pool dtype {dtype}")
        self.block_size, self.n_kv_heads, self.head_dim = block_size, n_kv_heads, head_dim
        self.max_seqs, self.max_blocks_per_seq = max_seqs, max_blocks_per_seq
        self.device = torch.device(device)
        shape = (num_blocks, block_size, n_kv_heads, head_dim)
        if dtype == torch.float8_e4m3fn:
            self.k_cache = torch.zeros(shape, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
            self.v_cache = torch.zeros(shape, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
            self.k_scale = torch.zeros((num_blocks, n_kv_heads), dtype=torch.float32, device=device)
            self.v_scale = torch.zeros((num_blocks, n_kv_heads), dtype=torch.float32, device=device)
        else:
            self.k_cache = torch.zeros(shape, dtype=dtype, device=device)
            self.v_cache = torch.zeros(shape, dtype=dtype, device=device)
            self.k_scale = self.v_scale = None
        self.allocator = BlockAllocator(num_blocks)
        self.blocks: List[List[int]] = [[] for _ in range(max_seqs)]
        self.lens = [0] * max_seqs
        self.block_tables = torch.full((max_seqs, max_blocks_per_seq), -1, dtype=torch.int32, device=device)
        self.seq_lens = torch.zeros(max_seqs, dtype=torch.int32, device=device)
        self._host_tables = np.full((max_seqs, max_blocks_per_seq), -1, dtype=np.int32)

    # ---- host bookkeeping ----------------------------------------------------------
    def blocks_needed(self, slot: int, n_new: int) -> int:
        total = self.lens[slot] + n_new
        return (total + self.block_size - 1) // self.block_size - len(self.blocks[slot])

    def extend(self, slots: Sequence[int], n_new: Sequence[int]) -> None:
        """Reserve room for n_new[i] more tokens in slot slots[i] and publish the new lengths
        and table rows to the device (all or nothing: raises OutOfBlocks before changing state)."""
        need = [self.blocks_needed(s, n) for s, n in zip(slots, n_new)]
        for s, n in zip(slots, n_new):
            if n < 0:
                raise ValueError("n_new must be non-negative")
            if (self.lens[s] + n + self.block_size - 1) // self.block_size > self.max_blocks_per_seq:
                raise ValueError(f"slot {s}: {self.lens[s] + n} tokens exceed the table capacity")
        if sum(max(x, 0) for x in need) > self.allocator.num_free:
            raise OutOfBlocks(f"{sum(need)} blocks requested, {self.allocator.num_free} free")
        for s, n, k in zip(slots, n_new, need):
            if k > 0:
                new = self.allocator.alloc(k)
                at = len(self.blocks[s])
                self.blocks[s].extend(new)
                self._host_tables[s, at:at + k] = new
            self.lens[s] += n
        self._publish(slots)

    def release(self, slot: int) -> None:
        self.allocator.free(self.blocks[slot])
        self.blocks[slot] = []
        self.lens[slot] = 0
        self._host_tables[slot] = -1
        self._publish([slot])

    def fork(self, src: int, dst: int) -> None:
        """Make `dst` a copy of `src` that shares its full blocks.  A partially filled last block is
        private to a sequence (the write kernel owns the blocks it writes), so it is copied."""
        if self.blocks[dst]:
            raise ValueError(f"slot {dst} is in use")
        n_full = self.lens[src] // self.block_size
        shared = self.blocks[src][:n_full]
        tail = self.blocks[src][n_full:]
        if len(tail) > self.allocator.num_free:
            raise OutOfBlocks(f"{len(tail)} blocks requested, {self.allocator.num_free} free")
        self.allocator.share(shared)
        mine = self.allocator.alloc(len(tail))
        for a, b in zip(tail, mine):
            self.k_cache.view(torch.uint8)[b].copy_(self.k_cache.view(torch.uint8)[a])
            self.v_cache.view(torch.uint8)[b].copy_(self.v_cache.view(torch.uint8)[a])
            if self.k_scale is not None:
                self.k_scale[b].copy_(self.k_scale[a])
                self.v_scale[b].copy_(self.v_scale[a])
        self.blocks[dst] = list(shared) + mine
        self.lens[dst] = self.lens[src]
        self._host_tables[dst] = -1
        self._host_tables[dst, :len(self.blocks[dst])] = self.blocks[dst]
        self._publish([dst])

    def _publish(self, slots: Sequence[int]) -> None:
        idx = torch.as_tensor(list(slots), dtype=torch.long, device=self.device)
        rows = torch.from_numpy(self._host_tables[list(slots)]).to(self.device, non_blocking=False)
        self.block_tables.index_copy_(0, idx, rows)
        self.seq_lens.index_copy_(0, idx, torch.tensor([self.lens[s] for s in slots], dtype=torch.int32, device=self.device))

    @property
    def max_seq_len(self) -> int:
        return max(self.lens) if self.lens else 0


class PagedAttention:
    """One attention layer's serving step over a `PagedKVCache`.

    `step(xq, xk, xv, query_lens)` takes the projected q/k/v of every slot, [max_seqs, T, H, D]
    bfloat16 (slot b contributes its first query_lens[b] rows; idle slots 0), reserves the
    blocks, applies the optional QK RMSNorm + RoPE, writes K/V into the pool and runs the
    prefill / verify kernel (T > 1) or the decode kernel (T == 1).  Returns [max_seqs, T, Hq, D]
    (a preallocated buffer, overwritten by the next step of the same T).
    """

    def __init__(self, cache: PagedKVCache, n_heads: int, *, scale: Optional[float] = None, rope_base: Optional[float] = None,
                 max_positions: int = 0, q_norm_weight=None, k_norm_weight=None, norm_eps: float = 1e-6,
                 partition_size: int = 512, sinks=None, sliding_window: Optional[int] = None):
        self.cache, self.n_heads = cache, n_heads
        self.scale = paged_attn.default_scale(cache.head_dim) if scale is None else float(scale)
        self.partition_size = partition_size
        self.q_norm_weight, self.k_norm_weight, self.norm_eps = q_norm_weight, k_norm_weight, norm_eps
        # the gpt-oss layer variant (examples/models/gpt_oss/kernels/attention.py:117-148): per-head sink
        # logits [n_heads] and a sliding window, fixed per layer
        self.sinks = None if sinks is None else sinks.to(torch.float32).contiguous()
        self.sliding_window = sliding_window
        self.rope = None
        if rope_base is not None:
            if max_positions <= 0:
                raise ValueError("RoPE needs max_positions")
            self.rope = paged_attn.rope_tables(cache.head_dim, max_positions, rope_base, device=cache.device)
        elif q_norm_weight is not None or k_norm_weight is not None:
            raise ValueError("the fused pre-attention kernel applies the norm together with RoPE: give rope_base")
        self._out: Dict[int, torch.Tensor] = {}
        self._qlens = torch.zeros(cache.max_seqs, dtype=torch.int32, device=cache.device)

    def step(self, xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, query_lens: Sequence[int]) -> torch.Tensor:
        c = self.cache
        B, T = xq.shape[:2]
        if B != c.max_seqs or len(query_lens) != B:
            raise ValueError(f"expected one row per slot ({c.max_seqs}), got {B} rows and {len(query_lens)} lengths")
        if any(n < 0 or n > T for n in query_lens):
            raise ValueError("query_lens must lie in [0, T]")
        active = [s for s in range(B) if query_lens[s] > 0]
        c.extend(active, [query_lens[s] for s in active])
        self._qlens.copy_(torch.tensor(list(query_lens), dtype=torch.int32))
        out = self._out.get(T)
        if out is None:
            out = self._out[T] = torch.empty((B, T, self.n_heads, c.head_dim), dtype=torch.bfloat16, device=c.device)
        if self.rope is not None:
            q = paged_attn.qk_norm_rope_kv_write(xq, xk, xv, c.k_cache, c.v_cache, c.block_tables, c.seq_lens, self._qlens,
                                                 self.rope[0], self.rope[1], q_norm_weight=self.q_norm_weight,
                                                 k_norm_weight=self.k_norm_weight, eps=self.norm_eps,
                                                 k_scale=c.k_scale, v_scale=c.v_scale, out=xq)
        else:
            paged_attn.kv_write(xk, xv, c.k_cache, c.v_cache, c.block_tables, c.seq_lens, self._qlens,
                                k_scale=c.k_scale, v_scale=c.v_scale)
            q = xq
        if T == 1:
            paged_attn.decode(q[:, 0], c.k_cache, c.v_cache, c.block_tables, c.seq_lens, self.scale,
                              k_scale=c.k_scale, v_scale=c.v_scale, partition_size=self.partition_size,
                              max_seq_len=max(c.max_seq_len, 1), out=out[:, 0],
                              sinks=self.sinks, sliding_window=self.sliding_window)
            # the decode kernel treats every slot as live; idle slots (seq_len 0) come back as zeros
        else:
            paged_attn.prefill(q, c.k_cache, c.v_cache, c.block_tables, c.seq_lens, self._qlens, self.scale,
                               k_scale=c.k_scale, v_scale=c.v_scale, out=out,
                               sinks=self.sinks, sliding_window=self.sliding_window)
        return out
