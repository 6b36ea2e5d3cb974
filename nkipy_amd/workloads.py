"""Synthetic inputs for the five benchmark configurations of the paged attention path.

Index structures (context lengths, block tables) come from
`np.random.default_rng(1000 + config_index)` so that they are identical on every
machine; the bulk values (Q, K, V ~ N(0,1), rounded to the storage dtype) are
drawn on the device from a torch generator with the same seed, because drawing
gigabytes of normals on the host would dominate every run.

Every maker takes `shrink` (>= 1): batch and context lengths are divided by it so
that the same generator serves CPU-sized parity cases.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch


@dataclass
class DecodeWorkload:
    name: str
    q: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    block_tables: torch.Tensor
    seq_lens: torch.Tensor
    scale: float
    partition_size: int
    max_seq_len: int
    k_scale: Optional[torch.Tensor] = None
    v_scale: Optional[torch.Tensor] = None
    ctx: np.ndarray = field(default=None, repr=False)

    def algorithmic_bytes(self) -> int:
        """HBM bytes the computation cannot avoid: every visible K/V row once,
        q in, out, the used block-table entries and seq_lens (and, for fp8, one
        K and one V scale per used (block, kv head))."""
        nb, bs, hkv, d = self.k_cache.shape
        esz = self.k_cache.element_size()
        B, hq, _ = self.q.shape
        ctx = self.ctx.astype(np.int64)
        nblk = (ctx + bs - 1) // bs
        total = int(ctx.sum()) * 2 * hkv * d * esz
        total += 2 * B * hq * d * self.q.element_size()
        total += 4 * int(nblk.sum()) + 4 * B
        if self.k_scale is not None:
            total += int(nblk.sum()) * 2 * hkv * 4
        return total


@dataclass
class PrefillWorkload:
    name: str
    q: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    block_tables: torch.Tensor
    seq_lens: torch.Tensor
    query_lens: torch.Tensor
    scale: float
    prefix: np.ndarray = field(default=None, repr=False)

    def flops(self) -> int:
        """4 * Hq * D * sum_b (T*P_b + T(T+1)/2): QK^T and PV over visible pairs only."""
        B, T, hq, d = self.q.shape
        tq = self.query_lens.cpu().numpy().astype(np.int64)
        p = self.prefix.astype(np.int64)
        pairs = int((tq * p + tq * (tq + 1) // 2).sum())
        return 4 * hq * d * pairs


@dataclass
class BlocksparseWorkload:
    name: str
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    scale: float
    block: int
    local_blocks: int
    vert_stride: int

    def flops(self) -> int:
        """Token-causal count: off-diagonal active blocks are block^2 pairs, diagonal
        blocks block*(block+1)/2."""
        B, S, hq, d = self.q.shape
        nb = S // self.block
        i = np.arange(nb)[:, None]
        j = np.arange(nb)[None, :]
        pairs = 0
        for h in range(hq):
            m = (j <= i) & (((i - j) < self.local_blocks) | (((j + h % self.vert_stride) % self.vert_stride) == 0))
            n_diag = int(np.trace(m))
            n_off = int(m.sum()) - n_diag
            pairs += n_off * self.block * self.block + n_diag * self.block * (self.block + 1) // 2
        return 4 * d * B * pairs


@dataclass
class KvWriteWorkload:
    name: str
    k_new: torch.Tensor
    v_new: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    k_scale: Optional[torch.Tensor]
    v_scale: Optional[torch.Tensor]
    block_tables: torch.Tensor
    seq_lens: torch.Tensor
    query_lens: torch.Tensor
    prefix: np.ndarray = field(default=None, repr=False)

    def algorithmic_bytes(self) -> int:
        """Every new K and V row read once and stored once in the pool's element size, one scale per
        touched (block, kv head) and tensor, the used table entries and the two length vectors."""
        B, T, hkv, d = self.k_new.shape
        bs = self.k_cache.shape[1]
        tq = self.query_lens.cpu().numpy().astype(np.int64)
        seq = self.seq_lens.cpu().numpy().astype(np.int64)
        rows = int(tq.sum())
        touched = int(((seq - 1) // bs - (seq - tq) // bs + 1)[tq > 0].sum())
        scales = 2 * touched * hkv * 4 if self.k_scale is not None else 0
        return 2 * rows * hkv * d * (self.k_new.element_size() + self.k_cache.element_size()) + scales + 4 * touched + 8 * B


def storage_bits(t: torch.Tensor) -> np.ndarray:
    """Raw storage bits of a device tensor as a NumPy unsigned array (uint16 for bf16, uint8 for
    fp8 codes, uint32 for float32): the form in which host-side checkers take device data."""
    t = t.detach().contiguous().cpu()
    if t.element_size() == 2:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.element_size() == 1:
        return t.view(torch.uint8).numpy()
    return t.view(torch.int32).numpy().view(np.uint32)


def _randn(shape, dtype, gen, device, chunk=1 << 27):
    """N(0,1) drawn in float32 and rounded to `dtype`, in bounded chunks."""
    out = torch.empty(shape, dtype=dtype, device=device)
    flat = out.view(-1)
    for s in range(0, flat.numel(), chunk):
        n = min(chunk, flat.numel() - s)
        flat[s:s + n] = torch.randn(n, generator=gen, device=device, dtype=torch.float32).to(dtype)
    return out


def _tables(rng, nblk, pool_blocks):
    """Disjoint slices of one permutation of the pool, padded with -1."""
    perm = rng.permutation(pool_blocks).astype(np.int32)
    B = len(nblk)
    width = max(int(max(nblk)), 1)
    tables = np.full((B, width), -1, dtype=np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    return tables


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def quantize_pool_fp8(pool: torch.Tensor):
    """[nb, bs, Hkv, D] float -> (e4m3fn codes, scale[nb, Hkv] = absmax / 448)."""
    x = pool.float()
    absmax = x.abs().amax(dim=(1, 3))
    scale = (absmax / 448.0).to(torch.float32)
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    codes = (x / scale[:, None, :, None]).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    return codes, scale


def make_decode(config: int, device="cuda", shrink: int = 1) -> DecodeWorkload:
    """config 1: fp32 B=4 8/8 heads D=64 bs=16 ctx U[16,256] pool 128;
    config 2: bf16 B=64 32/8 heads D=128 bs=32 ctx U[512,8192] partition 512;
    config 5: fp8 KV B=128 64/8 heads D=128 bs=64 ctx logU[1024,32768] partition 1024;
    config 17: config 2's shape with 8 192 sequences of 10-90 tokens (very many very short contexts)."""
    rng = np.random.default_rng(1000 + config)
    gen = _gen(1000 + config, device)
    if config == 1:
        B, Hq, Hkv, D, bs, dtype, part = 4, 8, 8, 64, 16, torch.float32, 512
        ctx = rng.integers(16, 257, size=B)
        pool_blocks = 128
    elif config == 2:
        B, Hq, Hkv, D, bs, dtype, part = max(64 // shrink, 1), 32, 8, 128, 32, torch.bfloat16, 512
        ctx = rng.integers(512 // shrink, 8192 // shrink + 1, size=B)
        pool_blocks = None
    elif config == 5:
        B, Hq, Hkv, D, bs, dtype, part = max(128 // shrink, 1), 64, 8, 128, 64, torch.bfloat16, 1024
        lo, hi = math.log(1024 / shrink), math.log(32768 / shrink)
        ctx = np.floor(np.exp(rng.uniform(lo, hi, size=B))).astype(np.int64)
        pool_blocks = None
    elif config == 17:
        B, Hq, Hkv, D, bs, dtype, part = max(8192 // shrink, 1), 32, 8, 128, 32, torch.bfloat16, 512
        ctx = rng.integers(10, 91, size=B)
        pool_blocks = None
    else:
        raise ValueError(f"config {config} is not a decode configuration")
    ctx = np.asarray(ctx, dtype=np.int64)
    nblk = (ctx + bs - 1) // bs
    if pool_blocks is None:
        pool_blocks = int(math.ceil(1.1 * int(nblk.sum())))
    tables = _tables(rng, nblk, pool_blocks)
    q = _randn((B, Hq, D), dtype, gen, device)
    k = _randn((pool_blocks, bs, Hkv, D), dtype, gen, device)
    v = _randn((pool_blocks, bs, Hkv, D), dtype, gen, device)
    ks = vs = None
    if config == 5:
        k, ks = quantize_pool_fp8(k)
        v, vs = quantize_pool_fp8(v)
    return DecodeWorkload(
        name=f"C{config}" + (f"/shrink{shrink}" if shrink > 1 else ""),
        q=q, k_cache=k, v_cache=v,
        block_tables=torch.from_numpy(tables).to(device),
        seq_lens=torch.from_numpy(ctx.astype(np.int32)).to(device),
        scale=float(np.float32(1.0) / np.float32(math.sqrt(D))),
        partition_size=part, max_seq_len=int(ctx.max()), k_scale=ks, v_scale=vs, ctx=ctx)


def make_prefill(device="cuda", shrink: int = 1, heads=(32, 8), head_dim: int = 128, name: str = "C3") -> PrefillWorkload:
    """config 3: bf16 causal chunked prefill, B=8, T=2048 new tokens, prefix U[0,4096],
    bs=32, 32/8 heads, D=128; sequences 0-3 share one prefix (same length, a multiple of
    the block size, same physical blocks), 4-7 have private prefixes.  `heads` and `head_dim` give the
    same tokens and tables another attention shape (the gpt-oss layers: 64/8 heads of 64)."""
    rng = np.random.default_rng(1003)
    gen = _gen(1003, device)
    B, (Hq, Hkv), D, bs = 8, heads, head_dim, 32
    T = max(2048 // shrink, 1)
    prefix = rng.integers(0, 4096 // shrink + 1, size=B).astype(np.int64)
    shared = (int(prefix[0]) // bs) * bs
    prefix[:4] = shared
    seq = prefix + T
    nblk = (seq + bs - 1) // bs
    shared_blocks = shared // bs
    private = nblk.copy()
    private[1:4] -= shared_blocks
    pool_blocks = int(math.ceil(1.1 * int(private.sum())))
    perm = rng.permutation(pool_blocks).astype(np.int32)
    tables = np.full((B, int(nblk.max())), -1, dtype=np.int32)
    pos = 0
    for b in range(B):
        if 1 <= b < 4:
            tables[b, :shared_blocks] = tables[0, :shared_blocks]
            n = nblk[b] - shared_blocks
            tables[b, shared_blocks:nblk[b]] = perm[pos:pos + n]
        else:
            n = nblk[b]
            tables[b, :n] = perm[pos:pos + n]
        pos += n
    q = _randn((B, T, Hq, D), torch.bfloat16, gen, device)
    k = _randn((pool_blocks, bs, Hkv, D), torch.bfloat16, gen, device)
    v = _randn((pool_blocks, bs, Hkv, D), torch.bfloat16, gen, device)
    return PrefillWorkload(
        name=name + (f"/shrink{shrink}" if shrink > 1 else ""), q=q, k_cache=k, v_cache=v,
        block_tables=torch.from_numpy(tables).to(device),
        seq_lens=torch.from_numpy(seq.astype(np.int32)).to(device),
        query_lens=torch.full((B,), T, dtype=torch.int32, device=device),
        scale=float(np.float32(1.0) / np.float32(math.sqrt(D))), prefix=prefix)


def make_blocksparse(device="cuda", shrink: int = 1) -> BlocksparseWorkload:
    """config 4: bf16, B=2, S=8192, 32 heads (MHA), D=128, block 64, local 4 + every 8th."""
    gen = _gen(1004, device)
    B, H, D = 2, 32, 128
    S = max(8192 // shrink, 64)
    q = _randn((B, S, H, D), torch.bfloat16, gen, device)
    k = _randn((B, S, H, D), torch.bfloat16, gen, device)
    v = _randn((B, S, H, D), torch.bfloat16, gen, device)
    return BlocksparseWorkload(name="C4" + (f"/shrink{shrink}" if shrink > 1 else ""), q=q, k=k, v=v,
                               scale=float(np.float32(1.0) / np.float32(math.sqrt(D))),
                               block=64, local_blocks=4, vert_stride=8)


def make_kv_write(device="cuda", shrink: int = 1, fp8: bool = True) -> KvWriteWorkload:
    """config 6 (the step in front of config 3's attention): the 2048 new tokens of each of 8
    sequences are written behind prefixes U[0,4096] into a block-64 pool, 8 kv heads, D=128;
    fp8-e4m3 pool with per-(block, kv head) scales by default (bf16 new rows quantised on the
    way in), or a bf16 pool (plain scatter)."""
    rng = np.random.default_rng(1006)
    gen = _gen(1006, device)
    B, Hkv, D, bs = 8, 8, 128, 64
    T = max(2048 // shrink, 1)
    prefix = rng.integers(0, 4096 // shrink + 1, size=B).astype(np.int64)
    seq = prefix + T
    nblk = (seq + bs - 1) // bs
    pool_blocks = int(math.ceil(1.1 * int(nblk.sum())))
    tables = _tables(rng, nblk, pool_blocks)
    k_new = _randn((B, T, Hkv, D), torch.bfloat16, gen, device)
    v_new = _randn((B, T, Hkv, D), torch.bfloat16, gen, device)
    if fp8:
        # earlier context already in the pool (the blocks the chunk starts inside carry a scale)
        k_cache, k_scale = quantize_pool_fp8(_randn((pool_blocks, bs, Hkv, D), torch.bfloat16, gen, device))
        v_cache, v_scale = quantize_pool_fp8(_randn((pool_blocks, bs, Hkv, D), torch.bfloat16, gen, device))
    else:
        k_cache = _randn((pool_blocks, bs, Hkv, D), torch.bfloat16, gen, device)
        v_cache = _randn((pool_blocks, bs, Hkv, D), torch.bfloat16, gen, device)
        k_scale = v_scale = None
    return KvWriteWorkload(
        name="C6" + ("" if fp8 else "/bf16") + (f"/shrink{shrink}" if shrink > 1 else ""),
        k_new=k_new, v_new=v_new, k_cache=k_cache, v_cache=v_cache, k_scale=k_scale, v_scale=v_scale,
        block_tables=torch.from_numpy(tables).to(device),
        seq_lens=torch.from_numpy(seq.astype(np.int32)).to(device),
        query_lens=torch.full((B,), T, dtype=torch.int32, device=device), prefix=prefix)
