"""CPU oracle for paged flash attention.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only the test-suite, the smoke
check and the benchmark's CPU-baseline leg may import it.  The shipped path
(`nkipy_amd`) runs hand-written HIP kernels and never falls back to this file.

What it restates
----------------
The reference has no paged attention.  Its serving attention is a dense-cache
NumPy kernel; this oracle composes that math with a block-table gather written
in the one-dynamic-index `np.take` form the reference's tracer supports:

* GQA head sharing      examples/models/qwen3/kernels/attention.py:15-22,109-110
* scores = q.k^T * scale examples/models/qwen3/kernels/attention.py:112-120
* additive causal mask  examples/models/qwen3/kernels/attention.py:124-134
* multi-token-at-offset examples/models/gpt_oss/kernels/attention.py:85,117-135
  ("query at start_pos+i attends to keys <= start_pos+i")
* sliding window, sinks examples/models/gpt_oss/kernels/attention.py:118-125 (keys
                        further back than W tokens masked), 137-148 (per-head logit
                        as one more softmax column, dropped afterwards)
* softmax               examples/models/qwen3/kernels/softmax.py:4-6
* weights @ values      examples/models/qwen3/kernels/attention.py:139-144
* cache layout/write-before-attend   examples/models/qwen3/qwen3.py:54-71,
                        examples/models/qwen3/kernels/attention.py:100-106
* gather primitive      nkipy/src/nkipy/core/tensor.py:575-640 (np.take, one
                        dynamic index per expression)
* QK RMSNorm + RoPE     examples/models/qwen3/kernels/rmsnorm.py:4-21, rope.py:4-48 and
                        their call sites attention.py:78-97 (bf16 tensors: every
                        RoPE product and sum is rounded to bf16, the norm is float32)
* output projection     examples/models/qwen3/kernels/attention.py:143-147 (`np.matmul(output,
                        o_weight)` on the BSHD output reshaped to (B, S, H*D)) and, with the
                        bias, examples/models/gpt_oss/kernels/attention.py:155-163
* cache update          examples/models/gpt_oss/kernels/attention.py:92-100
                        (`cache_k[:, query_pos] = xk`, query_pos = start_pos +
                        arange(seq_len)), examples/models/qwen3/kernels/attention.py:100-106

Dtype policy: inputs are values already rounded to their storage type (bf16 /
fp8-e4m3fn with a per-(block, kv-head) scale / fp32); every product and sum is
float32 (or float64 when `acc=np.float64`); the result is rounded once to the
query's storage type.  The reference's intermediate bf16 rounding of the score
matrix (attention.py:120) is deliberately not reproduced.

How each function is pinned (see tests/test_oracle_*.py)
--------------------------------------------------------
bf16 / fp8 codecs      exhaustive over every bit pattern vs. torch's dtypes and
                       vs. the format definition
gather_kv              np.take semantics; permutation invariance; identity
                       table == dense slice
dense_attention        float64 triple-loop brute force on tiny inputs; torch
                       scaled_dot_product_attention (CPU); closed-form special
                       cases (ctx=1, q=0, dominant key, rows of P sum to one)
paged_decode/prefill   identity table over a reshaped dense cache == dense
                       attention; GQA == MHA on np.repeat'ed KV; T=1 prefill ==
                       decode; P=0 prefill == plain causal
sliding window, sinks  float64 brute force; W >= context == no window; W = 1 ==
                       the query's own V row; sink = -inf == no sink; a sink is a
                       key with a zero value row; a huge sink drives the output to 0
merge_partitions       split-K merge == single pass in float64 for any split
blocksparse_prefill    == dense attention under the expanded boolean mask;
                       all-active pattern == dense causal
o_proj                 torch.matmul on CPU (an independent library); float64 row-by-row
                       dot products on tiny inputs; identity weight returns the input;
                       linearity in x; the bias shifts every row alike
rope_tables / rmsnorm / apply_rope   closed forms (position 0 is the identity,
                       rotation preserves the pair norm, angle addition), float64
                       restatement, torch.nn.functional.rms_norm on CPU
kv_write               bf16/fp32 pools: identity table == the reference's dense
                       `cache[:, query_pos] = x`; untouched pool bytes keep their
                       bits.  fp8 pools (no reference counterpart): a whole fresh
                       block == quantize_kv_fp8 of that block; scales never
                       shrink; codes of earlier tokens keep their bits when the
                       scale stays; token-by-token append dequantises within the
                       e4m3 rounding bound of the final scale
No reference test or fixture exists for the paged / split-K / blocksparse /
fp8-KV forms, so against the reference itself their parity is unpinned; they
are pinned by the mathematics above.
"""

from __future__ import annotations

import numpy as np

NEG_MASK = np.float32(-100000.0)  # examples/models/qwen3/kernels/attention.py:126
FP8_E4M3_MAX = 448.0

# ---------------------------------------------------------------------------
# storage codecs (integer bit manipulation; no ml_dtypes in this image)
# ---------------------------------------------------------------------------


def f32_to_bf16_bits(x) -> np.ndarray:
    """float32 -> bfloat16 bit pattern (uint16), round-to-nearest-even.

    NaN stays NaN (quiet bit forced), +-inf stay inf, overflow rounds to inf.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    is_nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    nan_bits = (u >> np.uint32(16)) | np.uint32(0x0040)
    return np.where(is_nan, nan_bits, rounded).astype(np.uint16)


def bf16_bits_to_f32(b) -> np.ndarray:
    """bfloat16 bit pattern (uint16) -> float32 (exact)."""
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_to_bf16(x) -> np.ndarray:
    """Round float32 values to the nearest bfloat16, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def _build_fp8_e4m3fn_lut() -> np.ndarray:
    """All 256 OCP e4m3fn values from the format definition.

    1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; the all-ones
    exponent with all-ones mantissa (0x7F / 0xFF) is NaN; largest finite 448.
    """
    lut = np.zeros(256, dtype=np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            val = np.nan
        elif e == 0:
            val = sign * (m / 8.0) * 2.0 ** (1 - 7)
        else:
            val = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        lut[code] = val
    return lut.astype(np.float32)


FP8_E4M3FN_LUT = _build_fp8_e4m3fn_lut()


def fp8_e4m3fn_decode(codes) -> np.ndarray:
    """uint8 e4m3fn codes -> float32 (exact; table lookup)."""
    return FP8_E4M3FN_LUT[np.ascontiguousarray(codes, dtype=np.uint8)]


def fp8_e4m3fn_encode(x) -> np.ndarray:
    """float32 -> e4m3fn code (uint8): nearest, ties-to-even, saturating at 448.

    Works on the non-negative half of the code space (codes 0..0x7E are
    monotone in value): find the two neighbouring codes, pick the nearer, on a
    tie the one with an even code (an even code has an even mantissa).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    mags = FP8_E4M3FN_LUT[:0x7F].astype(np.float64)  # 0 .. 448, ascending
    a = np.minimum(np.abs(x.astype(np.float64)), FP8_E4M3_MAX)
    hi = np.searchsorted(mags, a, side="left")  # first code with value >= a
    hi = np.clip(hi, 0, 0x7E)
    lo = np.clip(hi - 1, 0, 0x7E)
    d_hi = mags[hi] - a
    d_lo = a - mags[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & ((lo & 1) == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    code = np.where(np.isnan(x), np.uint8(0x7F), code)
    sign = (x.view(np.uint32) >> np.uint32(24)).astype(np.uint8) & np.uint8(0x80)
    return (code | sign).astype(np.uint8)


def quantize_kv_fp8(pool_f32):
    """Quantise a pool [num_blocks, block_size, Hkv, D] to e4m3fn codes.

    scale[block, kv_head] = absmax / 448 (1.0 for an all-zero slab so that the
    division is defined); code = encode(x / scale).  Returns (codes, scales).
    """
    pool_f32 = np.asarray(pool_f32, dtype=np.float32)
    absmax = np.max(np.abs(pool_f32), axis=(1, 3))  # [num_blocks, Hkv]
    scale = (absmax / np.float32(FP8_E4M3_MAX)).astype(np.float32)
    scale = np.where(scale == 0, np.float32(1.0), scale).astype(np.float32)
    codes = fp8_e4m3fn_encode(pool_f32 / scale[:, None, :, None])
    return codes, scale


def dequantize_kv_fp8(codes, scale) -> np.ndarray:
    """codes [nb, bs, Hkv, D] uint8, scale [nb, Hkv] f32 -> float32 pool."""
    return fp8_e4m3fn_decode(codes) * np.asarray(scale, np.float32)[:, None, :, None]


def to_f32(x, kind=None) -> np.ndarray:
    """View a stored array as float32 values.

    float32/float64 arrays pass through; uint16 arrays are bf16 bit patterns;
    uint8 arrays are e4m3fn codes (no scale applied here).
    """
    x = np.asarray(x)
    if x.dtype == np.uint16:
        return bf16_bits_to_f32(x)
    if x.dtype == np.uint8:
        return fp8_e4m3fn_decode(x)
    return x.astype(np.float32, copy=False)


def round_output(x, q_dtype: str) -> np.ndarray:
    """Round a float result once to the query's storage type (as float32)."""
    x = np.asarray(x).astype(np.float32)
    if q_dtype == "bf16":
        return round_to_bf16(x)
    if q_dtype == "fp32":
        return x
    raise ValueError(f"unknown q_dtype {q_dtype!r}")


# ---------------------------------------------------------------------------
# block-table gather
# ---------------------------------------------------------------------------


def gather_kv(pool, table_row, seq_len: int, block_scale=None) -> np.ndarray:
    """Rows [0, seq_len) of one sequence out of a paged pool.

    pool       [num_blocks, block_size, Hkv, D]   (any dtype; bits are copied)
    table_row  [max_blocks] int32, logical block i -> physical block id
    Returns    [seq_len, Hkv, D] in the pool's dtype — or float32 dequantised
    values when `block_scale` ([num_blocks, Hkv] f32) is given.

    One dynamic index, along axis 0, exactly the `x[idx]` -> np.take form of
    nkipy/src/nkipy/core/tensor.py:575-640.
    """
    num_blocks, block_size = pool.shape[0], pool.shape[1]
    nblk = (int(seq_len) + block_size - 1) // block_size
    idx = np.asarray(table_row[:nblk], dtype=np.int64)
    if idx.size and (idx.min() < 0 or idx.max() >= num_blocks):
        raise IndexError("block table entry outside the pool")
    blocks = np.take(pool, idx, axis=0)  # [nblk, bs, Hkv, D]
    if block_scale is not None:
        sc = np.take(np.asarray(block_scale, np.float32), idx, axis=0)  # [nblk, Hkv]
        blocks = to_f32(blocks) * sc[:, None, :, None]
    return blocks.reshape((nblk * block_size,) + pool.shape[2:])[: int(seq_len)]


# ---------------------------------------------------------------------------
# dense attention core (the reference's math on one sequence)
# ---------------------------------------------------------------------------


def rope_tables(head_dim: int, max_seq_len: int, base: float = 10000.0):
    """cos / sin tables [max_seq_len, head_dim // 2] as bf16-rounded float32 values.

    examples/models/qwen3/kernels/rope.py:4-20: freqs = 1 / base ** (arange(0, D, 2) / D)
    (float64), t = arange(max_seq_len) float32, outer product, cos / sin evaluated in float32,
    then cast to the tensor dtype (bf16 at the call site, attention.py:84-86).
    """
    freqs = 1.0 / (base ** (np.arange(0, head_dim, 2)[: (head_dim // 2)] / head_dim))
    t = np.arange(max_seq_len, dtype=np.float32)
    ang = np.outer(t, freqs)
    return round_to_bf16(np.cos(ang, dtype=np.float32)), round_to_bf16(np.sin(ang, dtype=np.float32))


def rmsnorm(x, weight, eps: float) -> np.ndarray:
    """examples/models/qwen3/kernels/rmsnorm.py:4-21 on bf16 storage: float32 compute,
    x / sqrt(mean(x^2) + eps) * weight, result rounded to bf16 (returned as float32)."""
    x = to_f32(x)
    w = to_f32(weight)
    z = np.mean(np.square(x), axis=-1, keepdims=True, dtype=np.float32)
    z = (z + np.float32(eps)).astype(np.float32)
    return round_to_bf16((x / np.sqrt(z)) * w)


def apply_rope(x, cos, sin) -> np.ndarray:
    """examples/models/qwen3/kernels/rope.py:23-48 for one tensor x [..., T, H, D] with
    cos / sin [T, D/2]: halves (x0, x1) -> (x0 c - x1 s, x0 s + x1 c).  All operands are bf16
    there, so each product and each sum is rounded to bf16."""
    x = to_f32(x)
    c = np.expand_dims(np.asarray(cos, np.float32), axis=-2)      # [T, 1, D/2]
    s_ = np.expand_dims(np.asarray(sin, np.float32), axis=-2)
    half = x.shape[-1] // 2
    x0, x1 = x[..., :half], x[..., half:]
    r = round_to_bf16
    o0 = r(r(x0 * c) - r(x1 * s_))
    o1 = r(r(x0 * s_) + r(x1 * c))
    return np.concatenate([o0, o1], axis=-1)


def qk_norm_rope(xq, xk, seq_lens, query_lens, cos, sin, *, q_norm_weight=None, k_norm_weight=None, eps=1e-6):
    """The reference's pre-attention step on q and k (qwen3/kernels/attention.py:78-97): optional
    QK RMSNorm, then RoPE at the tokens' absolute positions start_pos + t with start_pos =
    seq_lens[b] - query_lens[b] (gpt_oss/kernels/attention.py:85-90).  xq [B, T, Hq, D],
    xk [B, T, Hkv, D] bf16 bits or values; rows t >= query_lens[b] come back as zeros.
    Returns (q_out, k_out) as bf16-rounded float32."""
    q, k = to_f32(xq), to_f32(xk)
    B, T = q.shape[:2]
    qo, ko = np.zeros_like(q), np.zeros_like(k)
    for b in range(B):
        tq = min(max(int(query_lens[b]), 0), T)
        if tq == 0:
            continue
        start = int(seq_lens[b]) - tq
        pos = start + np.arange(tq)
        qb, kb = q[b, :tq], k[b, :tq]
        if q_norm_weight is not None:
            qb = rmsnorm(qb, q_norm_weight, eps)
        if k_norm_weight is not None:
            kb = rmsnorm(kb, k_norm_weight, eps)
        qo[b, :tq] = apply_rope(qb, cos[pos], sin[pos])
        ko[b, :tq] = apply_rope(kb, cos[pos], sin[pos])
    return qo, ko


def kv_write(k_new, v_new, k_cache, v_cache, block_tables, seq_lens, query_lens, *,
             k_scale=None, v_scale=None) -> None:
    """Write the new tokens' K/V into the paged pool, in place, before attention.

    The reference updates a dense cache with `cache_k[:, query_pos] = xk`,
    query_pos = start_pos + arange(seq_len) (gpt_oss/kernels/attention.py:85,92-100;
    qwen3/kernels/attention.py:100-106).  Paged form: token t < query_lens[b] of
    sequence b sits at position pos = seq_lens[b] - query_lens[b] + t and goes to
    pool row (block_tables[b, pos // bs], pos % bs).

    k_new/v_new [B, T, Hkv, D]: uint16 bf16 bit patterns or float32 values.
    k/v_cache [num_blocks, bs, Hkv, D]: uint16 / float32 pools receive the rows bit
    for bit.  uint8 pools hold e4m3fn codes with k_scale/v_scale [num_blocks, Hkv]
    float32, maintained per (block, kv head) -- this part has no counterpart in the
    reference:
      s_old = scale of the block if it already holds earlier tokens of the sequence
              (pos of the first written token is not the block's first row), else 0
      s_new = max(s_old, absmax(new rows of the block) / 448)   (1.0 if that is 0)
      earlier rows are re-encoded as encode(decode(code) * s_old / s_new) when the
      scale grew; new rows are encode(x / s_new).  All arithmetic float32.
    """
    kn, vn = np.asarray(k_new), np.asarray(v_new)
    B, T = kn.shape[:2]
    bs = k_cache.shape[1]
    fp8 = k_cache.dtype == np.uint8
    if fp8 and (k_scale is None or v_scale is None):
        raise ValueError("fp8 pools need k_scale and v_scale")
    for b in range(B):
        seq, tq = int(seq_lens[b]), int(query_lens[b])
        tq = min(max(tq, 0), T)
        if tq == 0:
            continue
        start = seq - tq
        if start < 0:
            raise ValueError("seq_lens must count the new tokens")
        for jb in range(start // bs, (seq - 1) // bs + 1):
            blk = int(block_tables[b, jb])
            if not 0 <= blk < k_cache.shape[0]:
                raise IndexError(f"block table entry {blk} out of range")
            lo = max(start, jb * bs) - jb * bs
            hi = min(seq, (jb + 1) * bs) - jb * bs
            t0 = jb * bs + lo - start
            for new, cache, scale in ((kn, k_cache, k_scale), (vn, v_cache, v_scale)):
                rows = new[b, t0:t0 + (hi - lo)]                      # [n, Hkv, D]
                if not fp8:
                    cache[blk, lo:hi] = rows if cache.dtype == rows.dtype else to_f32(rows).astype(cache.dtype)
                    continue
                x = to_f32(rows)
                amax = np.max(np.abs(x), axis=(0, 2)).astype(np.float32)          # [Hkv]
                s_old = scale[blk].astype(np.float32) if lo > 0 else np.zeros_like(amax)
                s_new = np.maximum(s_old, (amax / np.float32(FP8_E4M3_MAX)).astype(np.float32))
                s_new = np.where(s_new == 0, np.float32(1.0), s_new).astype(np.float32)
                if lo > 0:
                    grew = s_new != s_old
                    old = (fp8_e4m3fn_decode(cache[blk, :lo]) * s_old[None, :, None]).astype(np.float32)
                    recoded = fp8_e4m3fn_encode((old / s_new[None, :, None]).astype(np.float32))
                    cache[blk, :lo] = np.where(grew[None, :, None], recoded, cache[blk, :lo])
                cache[blk, lo:hi] = fp8_e4m3fn_encode((x / s_new[None, :, None]).astype(np.float32))
                scale[blk] = s_new


def repeat_kv(x, n_rep: int) -> np.ndarray:
    """[S, Hkv, D] -> [S, Hkv*n_rep, D]; q head h uses kv head h // n_rep.

    examples/models/qwen3/kernels/attention.py:15-22 (np.repeat on the head axis).
    """
    if n_rep == 1:
        return x
    return np.repeat(x, n_rep, axis=1)


def softmax_lastaxis(x) -> np.ndarray:
    """examples/models/qwen3/kernels/softmax.py:4-6."""
    e = np.exp(x - np.max(x, axis=-1, keepdims=True))
    return e / np.sum(e, axis=-1, keepdims=True)


def dense_attention(q, k, v, scale, *, prefix=None, mask=None, window=None, sinks=None,
                    acc=np.float32) -> np.ndarray:
    """softmax(q k^T * scale + mask) v for ONE sequence.

    q [T, Hq, D], k/v [S, Hkv, D] (float), Hq % Hkv == 0.
    prefix: if not None, query i sees keys j <= prefix + i (additive -100000
            mask as in attention.py:124-134; decode is T == 1, prefix == S-1).
    mask:   optional boolean [Hq or 1, T, S], True = visible (ANDed with causal).
    window: sliding window W (needs prefix): query at position p = prefix + i does not
            see keys j <= p - W, i.e. it sees the W keys (p - W, p]
            (examples/models/gpt_oss/kernels/attention.py:118-125, np.tril(..., k=-W)).
    sinks:  [Hq] per-head logits appended to every score row as one more column
            before the softmax and dropped after it (gpt_oss attention.py:137-148):
            they take probability mass and contribute no value.
    Returns [T, Hq, D] in `acc` precision (no output rounding here).
    """
    q = np.asarray(q, dtype=acc)
    k = np.asarray(k, dtype=acc)
    v = np.asarray(v, dtype=acc)
    T, Hq, D = q.shape
    S, Hkv, _ = k.shape
    n_rep = Hq // Hkv
    assert Hkv * n_rep == Hq
    keys = repeat_kv(k, n_rep).transpose(1, 0, 2)  # [Hq, S, D]
    vals = repeat_kv(v, n_rep).transpose(1, 0, 2)
    qh = q.transpose(1, 0, 2)  # [Hq, T, D]
    scores = np.matmul(qh, keys.transpose(0, 2, 1)) * acc(scale)  # [Hq, T, S]
    visible = np.ones((1, T, S), dtype=bool)
    if prefix is not None:
        jj = np.arange(S)[None, :]
        ii = np.arange(T)[:, None]
        visible = visible & (jj <= (int(prefix) + ii))[None]
    if window is not None:
        assert prefix is not None and int(window) >= 1
        jj = np.arange(S)[None, :]
        ii = np.arange(T)[:, None]
        visible = visible & ((int(prefix) + ii) - jj < int(window))[None]
    if mask is not None:
        visible = visible & np.asarray(mask, dtype=bool)
    scores = scores + np.where(visible, acc(0), acc(NEG_MASK))
    if sinks is not None:
        sink_col = np.broadcast_to(np.asarray(sinks, dtype=acc).reshape(Hq, 1, 1), (Hq, T, 1))
        weights = softmax_lastaxis(np.concatenate([scores, sink_col], axis=-1))[:, :, :S]
    else:
        weights = softmax_lastaxis(scores)
    out = np.matmul(weights, vals)  # [Hq, T, D]
    return out.transpose(1, 0, 2)


def attention_bruteforce_f64(q, k, v, scale, *, prefix=None, mask=None, window=None, sinks=None) -> np.ndarray:
    """Same contract as dense_attention, written as explicit float64 loops with
    hard masking (masked keys are skipped, not offset; a sink is one more term of
    the denominator).  Tiny inputs only."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    T, Hq, D = q.shape
    S, Hkv, _ = k.shape
    n_rep = Hq // Hkv
    out = np.zeros((T, Hq, D), dtype=np.float64)
    for t in range(T):
        for h in range(Hq):
            hk = h // n_rep
            js = []
            for j in range(S):
                if prefix is not None and j > prefix + t:
                    continue
                if window is not None and j <= prefix + t - window:
                    continue
                if mask is not None:
                    mh = h if np.asarray(mask).shape[0] > 1 else 0
                    if not mask[mh][t][j]:
                        continue
                js.append(j)
            s = [float(scale) * sum(q[t, h, d] * k[j, hk, d] for d in range(D)) for j in js]
            mx = max(s) if sinks is None else max(s + [float(sinks[h])])
            w = [np.exp(x - mx) for x in s]
            z = sum(w) + (0.0 if sinks is None else np.exp(float(sinks[h]) - mx))
            for d in range(D):
                out[t, h, d] = sum(wi * v[j, hk, d] for wi, j in zip(w, js)) / z
    return out


# ---------------------------------------------------------------------------
# paged entry points (same argument meaning as the HIP ops)
# ---------------------------------------------------------------------------


def _pool_f32_rows(cache, scale_tbl, table_row, ctx):
    if scale_tbl is not None:
        return gather_kv(cache, table_row, ctx, block_scale=scale_tbl)
    return to_f32(gather_kv(cache, table_row, ctx))


def paged_decode(q, k_cache, v_cache, block_tables, seq_lens, scale, *,
                 k_scale=None, v_scale=None, q_dtype="fp32", acc=np.float32,
                 sliding_window=None, sinks=None) -> np.ndarray:
    """One new query token per sequence against its paged context.

    q            [B, Hq, D]       float32 values (or uint16 bf16 bits)
    k/v_cache    [num_blocks, block_size, Hkv, D]  float32 / uint16 bf16 bits /
                 uint8 e4m3fn codes (then k_scale/v_scale [num_blocks, Hkv])
    block_tables [B, max_blocks] int32;  seq_lens [B] int32 (keys visible,
                 the current token's K/V already written: attention.py:100-106)
    Returns      [B, Hq, D] float32 holding values rounded to `q_dtype`.
    A sequence with seq_len == 0 yields zeros.
    sliding_window / sinks [Hq]: as in dense_attention (gpt_oss attention.py:117-148).
    """
    qf = to_f32(q)
    B, Hq, D = qf.shape
    out = np.zeros((B, Hq, D), dtype=np.float32)
    for b in range(B):
        ctx = int(seq_lens[b])
        if ctx <= 0:
            continue
        k = _pool_f32_rows(k_cache, k_scale, block_tables[b], ctx)
        v = _pool_f32_rows(v_cache, v_scale, block_tables[b], ctx)
        o = dense_attention(qf[b][None], k, v, scale, prefix=ctx - 1, window=sliding_window, sinks=sinks, acc=acc)
        out[b] = o[0]
    return round_output(out, q_dtype)


def paged_prefill(q, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, *,
                  k_scale=None, v_scale=None, q_dtype="bf16", acc=np.float32,
                  seqs=None, heads=None, sliding_window=None, sinks=None) -> np.ndarray:
    """Chunked prefill: the last query_lens[b] tokens of each sequence attend to
    the whole paged context causally (query i sees keys <= prefix_b + i, with
    prefix_b = seq_lens[b] - query_lens[b]); the new tokens' K/V are already in
    the pool.  gpt_oss/kernels/attention.py:85,127-135 with start_pos = prefix.

    q [B, T, Hq, D]; rows t >= query_lens[b] are padding and yield zeros.
    `seqs` / `heads` restrict the work to a subset (others stay zero) so that a
    full-size check can sample.
    """
    qf = to_f32(q)
    B, T, Hq, D = qf.shape
    Hkv = k_cache.shape[2]
    n_rep = Hq // Hkv
    out = np.zeros((B, T, Hq, D), dtype=np.float32)
    for b in (range(B) if seqs is None else seqs):
        ctx, tq = int(seq_lens[b]), int(query_lens[b])
        if tq <= 0:
            continue
        prefix = ctx - tq
        assert prefix >= 0
        k = _pool_f32_rows(k_cache, k_scale, block_tables[b], ctx)
        v = _pool_f32_rows(v_cache, v_scale, block_tables[b], ctx)
        for hk in range(Hkv):  # one kv group at a time bounds the score matrix
            hs = [h for h in range(hk * n_rep, (hk + 1) * n_rep) if heads is None or h in heads]
            if not hs:
                continue
            o = dense_attention(qf[b, :tq][:, hs], k[:, hk:hk + 1], v[:, hk:hk + 1],
                                scale, prefix=prefix, window=sliding_window,
                                sinks=None if sinks is None else np.asarray(sinks)[hs], acc=acc)
            out[b, :tq][:, hs] = o
    return round_output(out, q_dtype)


def blocksparse_block_mask(n_blocks: int, head: int, local_blocks: int, vert_stride: int) -> np.ndarray:
    """[n_blocks, n_blocks] bool: q-block i may attend k-block j iff j <= i and
    (i - j < local_blocks  or  (j + head % vert_stride) % vert_stride == 0)."""
    i = np.arange(n_blocks)[:, None]
    j = np.arange(n_blocks)[None, :]
    local = (i - j) < local_blocks
    vert = ((j + (head % vert_stride)) % vert_stride) == 0
    return (j <= i) & (local | vert)


def blocksparse_prefill(q, k, v, scale, *, block=64, local_blocks=4, vert_stride=8,
                        q_dtype="bf16", acc=np.float32, items=None, head_ids=None) -> np.ndarray:
    """Block-sparse causal self-attention over dense q/k/v [B, S, H(kv), D].

    Equals dense attention under the block mask expanded to tokens, ANDed with
    token-level causality.  `items` = iterable of (b, h) to compute (default all).
    `head_ids[h]` = the head number that sets head h's phase offset (default h itself):
    lets a caller pass a slice of the heads of a larger tensor.
    """
    qf, kf, vf = to_f32(q), to_f32(k), to_f32(v)
    B, S, Hq, D = qf.shape
    Hkv = kf.shape[2]
    n_rep = Hq // Hkv
    nb = (S + block - 1) // block
    out = np.zeros((B, S, Hq, D), dtype=np.float32)
    todo = [(b, h) for b in range(B) for h in range(Hq)] if items is None else list(items)
    for b, h in todo:
        bm = blocksparse_block_mask(nb, h if head_ids is None else int(head_ids[h]), local_blocks, vert_stride)
        tok = np.repeat(np.repeat(bm, block, axis=0), block, axis=1)[:S, :S]
        hk = h // n_rep
        o = dense_attention(qf[b][:, h:h + 1], kf[b][:, hk:hk + 1], vf[b][:, hk:hk + 1],
                            scale, prefix=0, mask=tok[None], acc=acc)
        out[b][:, h:h + 1] = o
    return round_output(out, q_dtype)


def o_proj(x, o_weight, bias=None, *, acc=np.float32) -> np.ndarray:
    """Output projection behind attention: examples/models/qwen3/kernels/attention.py:143-147
    (`output.reshape(batch, seq, -1)` then `np.matmul(output, o_weight)`), with `+ o_bias` as
    examples/models/gpt_oss/kernels/attention.py:155-163 adds it (on one rank).

    x [..., Hq, D] or [..., K] (float32 values or uint16 bf16 bits), o_weight [K, N], bias [N] or
    None.  Products and sums in `acc`, bias added before the single rounding to bf16.  The
    reference rounds the matmul result to bf16 before it adds the bias; that extra rounding (at most
    one bf16 step of the result) is not reproduced, like its rounding of the score matrix.
    Returns [..., N] float32 holding bf16-representable values.
    """
    xf, wf = to_f32(x), to_f32(o_weight)
    K, N = wf.shape
    if xf.shape[-1] != K:
        assert xf.ndim >= 2 and xf.shape[-1] * xf.shape[-2] == K, (xf.shape, wf.shape)
        xf = xf.reshape(xf.shape[:-2] + (K,))
    y = np.matmul(xf.astype(acc), wf.astype(acc))
    if bias is not None:
        y = y + to_f32(bias).astype(acc)
    return round_to_bf16(y.astype(np.float32))


# ---------------------------------------------------------------------------
# split-K algebra (what the device's partition + reduce kernels implement)
# ---------------------------------------------------------------------------


def partition_stats(q, k, v, scale, acc=np.float64):
    """Per-partition (m, l, o): running max, sum of exp, normalised output for
    one query [Hq, D] against keys [S, Hkv, D] (no mask)."""
    q = np.asarray(q, acc)
    k = np.asarray(k, acc)
    v = np.asarray(v, acc)
    Hq = q.shape[0]
    n_rep = Hq // k.shape[1]
    keys = repeat_kv(k, n_rep)
    vals = repeat_kv(v, n_rep)
    s = np.einsum("hd,shd->hs", q, keys) * acc(scale)
    m = s.max(axis=1)
    e = np.exp(s - m[:, None])
    l = e.sum(axis=1)
    o = np.einsum("hs,shd->hd", e, vals) / l[:, None]
    return m, l, o


def merge_partitions(ms, ls, os_):
    """m = max m_i;  l = sum l_i e^{m_i-m};  o = sum o_i l_i e^{m_i-m} / l."""
    ms = np.stack(ms)
    ls = np.stack(ls)
    os_ = np.stack(os_)
    m = ms.max(axis=0)
    w = ls * np.exp(ms - m[None])
    l = w.sum(axis=0)
    o = (os_ * w[..., None]).sum(axis=0) / l[..., None]
    return m, l, o
