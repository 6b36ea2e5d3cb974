"""Engine glue around the paged attention ops: who owns the pool and who calls the ops.

The reference's model drivers own a dense per-layer cache, hand it to every layer call as
an aliased input/output and keep all buffers preallocated
(examples/models/qwen3/qwen3.py:54-71, 289-336, 372-396).  With a paged pool the same
role needs three small pieces:

* `BlockAllocator`  -- free list with reference counts (a block shared by a forked prefix
                       is freed when its last user goes);
* `PagedKVCache`    -- the K/V pools of the model's layers (bf16, or fp8-e4m3 with
                       per-(block, kv head) scales), the per-slot block lists and the
                       device-resident `block_tables` / `seq_lens` the kernels read; the
                       layers share the tables, as the reference's layers share start_pos
                       (examples/models/qwen3/qwen3.py:310-336), so a step reserves blocks
                       and publishes lengths once, not once per layer;
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
    """K/V pools of `num_layers` attention layers plus the tables the kernels read.

    Slots 0 .. max_seqs-1 are the rows of `block_tables` / `seq_lens`; a slot with
    seq_len 0 is idle.  Every layer has its own pool `k_caches[l]` / `v_caches[l]`; block ids, tables
    and lengths are common to all layers.  `dtype` torch.bfloat16, or torch.float8_e4m3fn (then
    `k_scales[l]` / `v_scales[l]` [num_blocks, Hkv] float32 exist and are maintained by the write
    kernel).  `k_cache`, `v_cache`, `k_scale`, `v_scale` name layer 0.
    """

    def __init__(self, num_blocks: int, block_size: int, n_kv_heads: int, head_dim: int, *, max_seqs: int,
                 max_blocks_per_seq: int, dtype=torch.bfloat16, device="cuda", num_layers: int = 1,
                 max_model_len: Optional[int] = None):
        if dtype not in (torch.bfloat16, torch.float8_e4m3fn):
            raise ValueError(f"unsupported pool dtype {dtype}")
        if num_layers < 1:
            raise ValueError("num_layers must be at least 1")
        # the longest sequence a slot may grow to: the table capacity (whole blocks) unless the model's own limit is
        # lower (a model of 1000 positions over blocks of 64 has a capacity of 1024 and a limit of 1000)
        cap = max_blocks_per_seq * block_size
        if max_model_len is not None and not 0 < max_model_len <= cap:
            raise ValueError(f"max_model_len {max_model_len} outside (0, {cap}] (the table capacity)")
        self.max_model_len = cap if max_model_len is None else int(max_model_len)
        self.block_size, self.n_kv_heads, self.head_dim = block_size, n_kv_heads, head_dim
        self.max_seqs, self.max_blocks_per_seq, self.num_layers = max_seqs, max_blocks_per_seq, num_layers
        self.device = torch.device(device)
        shape = (num_blocks, block_size, n_kv_heads, head_dim)
        fp8 = dtype == torch.float8_e4m3fn

        def pool():
            if fp8:
                return torch.zeros(shape, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
            return torch.zeros(shape, dtype=dtype, device=device)

        def scales():
            return torch.zeros((num_blocks, n_kv_heads), dtype=torch.float32, device=device) if fp8 else None

        self.k_caches = [pool() for _ in range(num_layers)]
        self.v_caches = [pool() for _ in range(num_layers)]
        self.k_scales = [scales() for _ in range(num_layers)]
        self.v_scales = [scales() for _ in range(num_layers)]
        self.k_cache, self.v_cache = self.k_caches[0], self.v_caches[0]
        self.k_scale, self.v_scale = self.k_scales[0], self.v_scales[0]
        self.step_tokens = 0
        self.allocator = BlockAllocator(num_blocks)
        self.blocks: List[List[int]] = [[] for _ in range(max_seqs)]
        self.lens = [0] * max_seqs
        # What the kernels read of the bookkeeping -- table rows, lengths, the query lengths of the step in flight --
        # lives in ONE device buffer (three views, each starting on a 256-byte boundary) with a host mirror of the same
        # layout, so that publishing a step is one copy.  The copy is asynchronous: the mirror goes into one of a few
        # pinned staging buffers, each reused only when the copy that last read it has completed, and the host
        # never waits for the device's queued work (a decode loop issued call by call stays ahead of the GPU).
        n_tab = max_seqs * max_blocks_per_seq
        self._off_lens = (n_tab + 63) // 64 * 64
        self._off_qlens = self._off_lens + (max_seqs + 63) // 64 * 64
        self._host_meta = np.zeros(self._off_qlens + max_seqs, dtype=np.int32)
        self._host_tables = self._host_meta[:n_tab].reshape(max_seqs, max_blocks_per_seq)
        self._host_tables[:] = -1
        self._host_lens = self._host_meta[self._off_lens:self._off_lens + max_seqs]
        self._host_qlens = self._host_meta[self._off_qlens:]
        self._meta = torch.from_numpy(self._host_meta).to(self.device)
        self.block_tables = self._meta[:n_tab].view(max_seqs, max_blocks_per_seq)
        self.seq_lens = self._meta[self._off_lens:self._off_lens + max_seqs]
        self.query_lens = self._meta[self._off_qlens:]
        self._stage = self._stage_done = None
        self._stage_at = 0
        if self.device.type == "cuda":
            self._stage = [torch.empty(self._host_meta.size, dtype=torch.int32, pin_memory=True) for _ in range(4)]
            self._stage_done = [None] * len(self._stage)

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
            if self.lens[s] + n > self.max_model_len:
                raise ValueError(f"slot {s}: {self.lens[s] + n} tokens exceed the longest sequence the cache admits "
                                 f"({self.max_model_len}: the table capacity, or max_model_len if that is lower)")
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
            for l in range(self.num_layers):
                self.k_caches[l].view(torch.uint8)[b].copy_(self.k_caches[l].view(torch.uint8)[a])
                self.v_caches[l].view(torch.uint8)[b].copy_(self.v_caches[l].view(torch.uint8)[a])
                if self.k_scales[l] is not None:
                    self.k_scales[l][b].copy_(self.k_scales[l][a])
                    self.v_scales[l][b].copy_(self.v_scales[l][a])
        self.blocks[dst] = list(shared) + mine
        self.lens[dst] = self.lens[src]
        self._host_tables[dst] = -1
        self._host_tables[dst, :len(self.blocks[dst])] = self.blocks[dst]
        self._publish([dst])

    def begin_step(self, query_lens: Sequence[int], tokens: int) -> None:
        """Open a step in which slot b appends query_lens[b] <= tokens tokens (0: idle): reserves the
        blocks, publishes tables and lengths, and puts the query lengths on the device for every
        layer's `PagedAttention.attend` of this step.  All or nothing, like `extend`."""
        if len(query_lens) != self.max_seqs:
            raise ValueError(f"expected one length per slot ({self.max_seqs}), got {len(query_lens)}")
        if any(n < 0 or n > tokens for n in query_lens):
            raise ValueError("query_lens must lie in [0, tokens]")
        active = [s for s in range(self.max_seqs) if query_lens[s] > 0]
        before = self._host_qlens.copy()
        self._host_qlens[:] = query_lens
        try:
            self.extend(active, [query_lens[s] for s in active])      # publishes the query lengths with the rest
        except Exception:
            self._host_qlens[:] = before
            raise
        self.step_tokens = tokens

    def _publish(self, slots: Sequence[int]) -> None:
        """Host mirror -> device (tables, lengths, query lengths: one copy, queued on the current stream)."""
        for s in slots:
            self._host_lens[s] = self.lens[s]
        if self._stage is None:
            self._meta.copy_(torch.from_numpy(self._host_meta))
            return
        i = self._stage_at
        self._stage_at = (i + 1) % len(self._stage)
        if self._stage_done[i] is None:
            self._stage_done[i] = torch.cuda.Event()
        else:
            self._stage_done[i].synchronize()         # (long done unless the host is four publications ahead)
        self._stage[i].numpy()[:] = self._host_meta
        self._meta.copy_(self._stage[i], non_blocking=True)
        self._stage_done[i].record()

    @property
    def max_seq_len(self) -> int:
        return max(self.lens) if self.lens else 0


class PagedAttention:
    """One attention layer's serving step over layer `layer` of a `PagedKVCache`.

    A model step is `cache.begin_step(query_lens, T)` once, then `attend(xq, xk, xv)` on every
    layer; `step(xq, xk, xv, query_lens)` does both for a single-layer use.  xq/xk/xv are the
    projected q/k/v of every slot, [max_seqs, T, H, D] bfloat16 (slot b contributes its first
    query_lens[b] rows; idle slots 0).  `attend` applies the optional QK RMSNorm + RoPE, writes K/V
    into the layer's pool and runs the prefill / verify kernel (T > 1) or the decode kernel
    (T == 1).  Returns [max_seqs, T, Hq, D] (a preallocated buffer, overwritten by the next step of
    the same T), or, when the layer was given `o_weight`, the output projection of it, [max_seqs, T, hidden].

    `attend` makes no host synchronisation and, after the first call of a given T, no allocation, so the
    launch-bound decode step of a stack of layers can be captured into one HIP graph (`torch.cuda.graph`) with
    xq / xk / xv as static buffers and replayed every step: `begin_step` stays outside the graph (it publishes
    the step's table rows and lengths, which the replayed kernels read from the same device tensors).  A captured
    decode step is sized by `max_seq_len`, the longest context it will be replayed on (default: the longest
    sequence the cache admits).  The bound also picks the decode kernel: a small batch with up to eight partitions
    of `partition_size` tokens takes the fixed-partition kernel, which is what makes small steps cheap, longer
    bounds and larger batches the balanced one; the two agree to the order of their float32 sums, not bit for bit.
    """

    def __init__(self, cache: PagedKVCache, n_heads: int, *, layer: int = 0, scale: Optional[float] = None,
                 rope_base: Optional[float] = None, max_positions: int = 0, q_norm_weight=None, k_norm_weight=None,
                 norm_eps: float = 1e-6, partition_size: int = 512, sinks=None, sliding_window: Optional[int] = None,
                 rope_tables=None, o_weight=None, o_bias=None):
        if not 0 <= layer < cache.num_layers:
            raise ValueError(f"layer {layer} outside the cache's {cache.num_layers} layers")
        self.cache, self.n_heads, self.layer = cache, n_heads, layer
        self.scale = paged_attn.default_scale(cache.head_dim) if scale is None else float(scale)
        self.partition_size = partition_size
        self.q_norm_weight, self.k_norm_weight, self.norm_eps = q_norm_weight, k_norm_weight, norm_eps
        # the gpt-oss layer variant (examples/models/gpt_oss/kernels/attention.py:117-148): per-head sink
        # logits [n_heads] and a sliding window, fixed per layer
        self.sinks = None if sinks is None else sinks.to(torch.float32).contiguous()
        self.sliding_window = sliding_window
        # RoPE tables: built from `rope_base`, or handed in as (cos, sin) [max_positions, D/2] bfloat16 — the
        # way to share one pair between layers and to bring scaled frequencies (gpt_oss/kernels/rope.py:4-24)
        self.rope = None
        if rope_tables is not None:
            self.rope = (rope_tables[0], rope_tables[1])
        elif rope_base is not None:
            if max_positions <= 0:
                raise ValueError("RoPE needs max_positions")
            self.rope = paged_attn.rope_tables(cache.head_dim, max_positions, rope_base, device=cache.device)
        elif q_norm_weight is not None or k_norm_weight is not None:
            raise ValueError("the fused pre-attention kernel applies the norm together with RoPE: give rope_base")
        if self.rope is not None:
            # the kernels clamp positions past the table to its last row: a table shorter than the longest
            # sequence the cache admits would silently rotate late tokens by the wrong angle
            cap = cache.max_model_len
            if self.rope[0].shape[0] < cap:
                raise ValueError(f"RoPE tables cover {self.rope[0].shape[0]} positions, the cache admits sequences of up "
                                 f"to {cap} tokens ({cache.max_blocks_per_seq} blocks of {cache.block_size}, max_model_len "
                                 f"{cache.max_model_len}): give max_positions >= {cap} or the cache a lower max_model_len")
        # output projection behind the attention call (examples/models/qwen3/kernels/attention.py:143-147;
        # with the bias gpt_oss/kernels/attention.py:155-163): o_weight [n_heads * head_dim, hidden] bfloat16 as the
        # reference stores it, this rank's rows; `attend` then returns [max_seqs, T, hidden] for the caller to all-reduce
        self.o_weight, self.o_bias = o_weight, o_bias
        if o_weight is not None and tuple(o_weight.shape[:1]) != (n_heads * cache.head_dim,):
            raise ValueError(f"o_weight must be [{n_heads * cache.head_dim}, hidden], got {tuple(o_weight.shape)}")
        self._out: Dict[int, torch.Tensor] = {}
        self._proj: Dict[int, torch.Tensor] = {}
        # decode / verify steps prepared once per (T, length bound, storage of xq / xk / xv): a loop that feeds the
        # layer from the same buffers every step pays the argument checks once (see paged_attn.PreparedStep)
        self._steps: Dict[tuple, tuple] = {}

    def step(self, xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, query_lens: Sequence[int]) -> torch.Tensor:
        if xq.shape[0] != self.cache.max_seqs or len(query_lens) != xq.shape[0]:
            raise ValueError(f"expected one row per slot ({self.cache.max_seqs}), got {xq.shape[0]} rows and "
                             f"{len(query_lens)} lengths")
        self.cache.begin_step(query_lens, xq.shape[1])
        return self.attend(xq, xk, xv)

    def reset_steps(self) -> None:
        """Forget the prepared steps (after replacing a tensor the layer was built with: weights, sinks, norm weights)."""
        self._steps.clear()

    def _prepared(self, T, bound, xq, xk, xv, make):
        """The prepared step for these row buffers, built by `make()` on first use.  A step is reused only for the
        very storage, shapes and strides it was prepared with (it keeps them alive, so an address cannot come back as
        another tensor's)."""
        key = (T, bound, xq.data_ptr(), xk.data_ptr(), xv.data_ptr())
        sig = (xq.shape, xq.stride(), xk.shape, xk.stride(), xv.shape, xv.stride(), xq.dtype, xk.dtype, xv.dtype)
        hit = self._steps.get(key)
        if hit is not None and hit[0] == sig:
            return hit[1]
        if len(self._steps) >= 4:          # callers that bring fresh tensors every step: nothing to reuse, nothing to hoard
            self._steps.pop(next(iter(self._steps)))
        st = make()
        self._steps[key] = (sig, st)
        return st

    def _q_transform(self):
        """The layer's Q transform for the attention kernels (one object, validated once), None without RoPE."""
        if self.rope is None:
            return None
        qt = getattr(self, "_qt", None)
        if qt is None:
            qt = self._qt = paged_attn.QTransform(self.rope[0], self.rope[1], self.q_norm_weight, self.norm_eps)
        return qt

    def attend(self, xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, *,
               max_seq_len: Optional[int] = None) -> torch.Tensor:
        c, l = self.cache, self.layer
        if max_seq_len is not None and not 0 < max_seq_len <= c.max_model_len:
            raise ValueError(f"max_seq_len {max_seq_len} outside (0, {c.max_model_len}]")
        B, T = xq.shape[:2]
        if B != c.max_seqs or T != c.step_tokens:
            raise ValueError(f"expected [{c.max_seqs}, {c.step_tokens}, ...] as opened by begin_step, got [{B}, {T}, ...]")
        capturing = c.device.type == "cuda" and torch.cuda.is_current_stream_capturing()
        # (the host-known maximum in steps of 256 tokens, the finest partition the kernels choose by it: the bound is part
        # of what a prepared step is prepared for, and contexts grow by a token a step)
        bound = max_seq_len if max_seq_len is not None else (
            c.max_model_len if capturing else min(c.max_model_len, (max(c.max_seq_len, 1) + 255) // 256 * 256))
        if bound < c.max_seq_len:
            raise ValueError(f"max_seq_len {bound} is below a live context of {c.max_seq_len} tokens")
        kc, vc, ks, vs = c.k_caches[l], c.v_caches[l], c.k_scales[l], c.v_scales[l]
        out = self._out.get(T)
        if out is None:
            out = self._out[T] = torch.empty((B, T, self.n_heads, c.head_dim), dtype=torch.bfloat16, device=c.device)
        if T == 1 and (self.rope is None or paged_attn.q_transform_supported(1, c.head_dim, c.block_size)):
            # a decode step: one call for the cache update, the attention and the projection (a small step then runs
            # as three launches: the new row rides on the decode launch, the split-K merge on the projection's load).
            # The bound on the contexts sizes the launch, clamps the lengths the kernel reads and picks the kernel:
            # the caller's bound if given; else what the host knows of this step's contexts, unless the launch is
            # being captured into a HIP graph, which will be replayed on longer contexts and so gets the longest
            # sequence the cache admits.  The decode kernels treat every slot as live; idle slots (seq_len 0) come
            # back as zeros (projected: the bias).
            proj = None
            if self.o_weight is not None:
                proj = self._proj.get(T)
                if proj is None:
                    proj = self._proj[T] = torch.empty((B, T, self.o_weight.shape[1]), dtype=torch.bfloat16, device=c.device)
            res = out if proj is None else proj

            def make():
                return paged_attn.prepare_decode_step(
                    xq[:, 0], xk[:, 0], xv[:, 0], kc, vc, c.block_tables, c.seq_lens, c.query_lens, self.scale,
                    k_scale=ks, v_scale=vs, partition_size=self.partition_size, max_seq_len=bound,
                    q_transform=self._q_transform(), k_norm_weight=None if self.rope is None else self.k_norm_weight,
                    o_weight=self.o_weight, o_bias=self.o_bias, out=res[:, 0], sinks=self.sinks,
                    sliding_window=self.sliding_window)

            self._prepared(T, bound, xq, xk, xv, make).launch()
            return res
        if T > 1 and (self.rope is None or paged_attn.q_transform_supported(T, c.head_dim, c.block_size)) and \
                paged_attn.prefill_route(B, T, self.n_heads, c.n_kv_heads, c.head_dim, c.block_size, ks is not None,
                                         self.sliding_window or 0, bound) == "verify":
            # a verify step (a few tokens per sequence through the decode-shaped kernel): one call as well
            proj = None
            if self.o_weight is not None:
                proj = self._proj.get(T)
                if proj is None:
                    proj = self._proj[T] = torch.empty((B, T, self.o_weight.shape[1]), dtype=torch.bfloat16, device=c.device)
            res = out if proj is None else proj

            def make():
                return paged_attn.prepare_verify_step(
                    xq, xk, xv, kc, vc, c.block_tables, c.seq_lens, c.query_lens, self.scale, k_scale=ks, v_scale=vs,
                    max_seq_len=bound, q_transform=self._q_transform(),
                    k_norm_weight=None if self.rope is None else self.k_norm_weight, o_weight=self.o_weight,
                    o_bias=self.o_bias, out=res, sinks=self.sinks, sliding_window=self.sliding_window)

            self._prepared(T, bound, xq, xk, xv, make).launch()
            return res
        qt = None
        if self.rope is not None:
            # the Q half of the norm and rotation rides on the attention kernel's Q load where that
            # kernel can do it (no pass over Q of its own); K is transformed on its way into the pool
            fused = paged_attn.q_transform_supported(T, c.head_dim, c.block_size)
            q = paged_attn.qk_norm_rope_kv_write(None if fused else xq, xk, xv, kc, vc, c.block_tables, c.seq_lens,
                                                 c.query_lens, self.rope[0], self.rope[1],
                                                 q_norm_weight=None if fused else self.q_norm_weight,
                                                 k_norm_weight=self.k_norm_weight, eps=self.norm_eps,
                                                 k_scale=ks, v_scale=vs, out=None if fused else xq)
            if fused:
                q, qt = xq, self._q_transform()
        else:
            paged_attn.kv_write(xk, xv, kc, vc, c.block_tables, c.seq_lens, c.query_lens, k_scale=ks, v_scale=vs)
            q = xq
        if T == 1:
            # the bound on the contexts sizes the launch, clamps the lengths the kernel reads and picks the kernel.
            # The caller's bound if given; else what the host knows of this step's contexts, unless the launch is
            # being captured into a HIP graph: that will be replayed on longer contexts, so it gets the longest
            # sequence the cache admits.
            paged_attn.decode(q[:, 0], kc, vc, c.block_tables, c.seq_lens, self.scale,
                              k_scale=ks, v_scale=vs, partition_size=self.partition_size,
                              max_seq_len=bound, out=out[:, 0],
                              sinks=self.sinks, sliding_window=self.sliding_window, q_transform=qt)
            # the decode kernel treats every slot as live; idle slots (seq_len 0) come back as zeros
        else:
            paged_attn.prefill(q, kc, vc, c.block_tables, c.seq_lens, c.query_lens, self.scale,
                               k_scale=ks, v_scale=vs, out=out, max_seq_len=bound,
                               sinks=self.sinks, sliding_window=self.sliding_window, q_transform=qt)
        if self.o_weight is None:
            return out
        proj = self._proj.get(T)
        if proj is None:
            proj = self._proj[T] = torch.empty((B, T, self.o_weight.shape[1]), dtype=torch.bfloat16, device=c.device)
        return paged_attn.o_proj(out, self.o_weight, self.o_bias, out=proj)
