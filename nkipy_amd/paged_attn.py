"""Paged flash attention ops on MI355X: NumPy-style signatures over device tensors.

Each op keeps the calling convention of the reference's kernels — positional
arrays in, array out, static options as keywords (README.md:118-152 of the
reference) — with the argument order `(q, k_cache, v_cache, block_tables,
seq_lens, scale) -> out`.  They are hand-kernel ops in the sense of the
reference's `nki_custom_op` (nkipy/src/nkipy/core/nki_op.py:800-884): there is
no CPU implementation behind them, and like that hook on the CPU backend
(nki_op.py:480,557,719-722) they raise NotImplementedError for host arrays.

Ownership follows nkipy/src/nkipy/runtime/device_tensor.py:51-74 and
spike/src/spike/spike_model.py:248-288: the caller may pass `out=` (written in
place, returned); otherwise a new tensor is allocated.  Validation errors are
ValueError (bad shape / dtype / contiguity / device), launch failures are
RuntimeError, mirroring spike_model.py:198-246.
"""
from __future__ import annotations

import ctypes
import math

import numpy as np
import torch

from . import _lib

F32, BF16, FP8 = 0, 1, 2
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16, torch.float8_e4m3fn: FP8}

_workspaces = {}
_o_proj_need = {}           # (M, K, N) -> scratch bytes of o_proj's few-rows form (a pure function of the shape)


def _need_device(name, t):
    if isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous():
        return                               # the usual case first: these checks run some twenty times per layer call
    if isinstance(t, np.ndarray):
        raise NotImplementedError(
            f"{name} is a NumPy array: the paged attention ops run hand-written HIP kernels and have "
            "no CPU path; pass torch tensors on a ROCm device")
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name} must be a torch.Tensor on a ROCm device, got {type(t).__name__}")
    if not t.is_cuda:
        raise NotImplementedError(f"{name} lives on {t.device}: the paged attention ops have no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _check(cond, msg):
    if not cond:
        raise ValueError(msg)


def _same_device(ref, **others):
    idx = ref.get_device()                  # an int: comparing device objects costs several times as much per tensor
    for n, t in others.items():
        if t is not None and t.get_device() != idx:
            raise ValueError(f"{n} is on {t.device}, expected {ref.device}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device):
    """The current stream of `device` as the C ABI takes it.  torch's raw-stream query when this build has it (a
    fraction of a microsecond; the Stream object of the public call costs several, and a decode step of a small batch
    is bound by the host), the public call otherwise."""
    if _raw_stream is not None and device.index is not None:
        return ctypes.c_void_p(_raw_stream(device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on(device):
    """Context in which `device` is the current one for a launch; nothing to switch when it already is
    (the usual case, and the switch costs a few microseconds of a call that launches ten-microsecond kernels)."""
    return _NO_GUARD if torch.cuda.current_device() == device.index else torch.cuda.device(device)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _raise_on(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed ({rc}): {_lib.last_error()}")


def _kv_code(cache, scale_given):
    if cache.dtype == torch.uint8:
        _check(scale_given, "uint8 KV caches are fp8-e4m3fn codes and need k_scale/v_scale")
        return FP8
    _check(cache.dtype in _DTYPE_CODE, f"unsupported KV cache dtype {cache.dtype}")
    return _DTYPE_CODE[cache.dtype]


def _check_paging(k_cache, v_cache, block_tables, seq_lens, B):
    _check(k_cache.dim() == 4, "k_cache must be [num_blocks, block_size, Hkv, D]")
    _check(v_cache.shape == k_cache.shape and v_cache.dtype == k_cache.dtype,
           "v_cache must match k_cache in shape and dtype")
    _check(block_tables.dim() == 2 and block_tables.shape[0] == B and block_tables.dtype == torch.int32,
           "block_tables must be int32 [B, max_blocks_per_seq]")
    _check(block_tables.shape[1] > 0, "block_tables needs at least one column")
    _check(seq_lens.shape == (B,) and seq_lens.dtype == torch.int32, "seq_lens must be int32 [B]")


def check_block_tables(block_tables, seq_lens, num_blocks, block_size):
    """Debug helper (synchronises): every table entry a sequence uses is a valid block id."""
    bt = block_tables.detach().cpu().numpy()
    sl = seq_lens.detach().cpu().numpy()
    for b in range(bt.shape[0]):
        n = (int(sl[b]) + block_size - 1) // block_size
        _check(n <= bt.shape[1], f"sequence {b}: seq_len {int(sl[b])} needs {n} blocks, table has {bt.shape[1]}")
        used = bt[b, :n]
        _check(used.size == 0 or (used.min() >= 0 and used.max() < num_blocks),
               f"sequence {b}: block table entry outside [0, {num_blocks})")


def _check_variant(sinks, sliding_window, Hq, ref):
    """sinks [Hq] (any float dtype; passed on as float32) and the window size of the gpt-oss attention
    variant (examples/models/gpt_oss/kernels/attention.py:117-148).  Returns (sinks_f32 or None, window int)."""
    win = 0 if sliding_window is None else int(sliding_window)
    _check(win >= 0 and (sliding_window is None or win >= 1), "sliding_window must be None or >= 1")
    if sinks is not None:
        _need_device("sinks", sinks)
        _check(sinks.shape == (Hq,), f"sinks must have one logit per q head ([{Hq}])")
        _check(sinks.is_floating_point(), "sinks must be floating point")
        _check(sinks.device == ref.device, f"sinks is on {sinks.device}, expected {ref.device}")
        sinks = sinks.to(torch.float32).contiguous()
    return sinks, win


def decode_workspace_bytes(B, Hq, D, max_seq_len, partition_size) -> int:
    return int(_lib.load().pa_decode_workspace_bytes(B, Hq, D, max_seq_len, partition_size))


_WORKSPACE_SLOTS = 16     # (device, stream) pairs whose eager workspace is kept; the least recently used goes first
_graph_workspaces = {}    # buffers handed out while a stream was being captured: a graph has their address baked in
_graph_retired = []       # ... and those that a later capture outgrew; both are kept until the process ends


def _workspace(device, nbytes, stream=None):
    """Scratch for split-K partials, cached per (device, stream) so that calls on one stream reuse one
    buffer and calls on different streams never share one.

    Eager calls: the cache holds at most _WORKSPACE_SLOTS entries (a server that cycles streams does not
    accumulate device memory); dropping or outgrowing an entry returns its memory to torch's allocator,
    which reuses it in stream order.

    Calls issued while the stream is being captured into a HIP graph take their buffer from a second cache
    that eager calls never touch and that is never evicted or freed: the graph has the address baked in, and
    neither a larger eager call on the same stream after the capture nor the eviction of a stream's entry may
    take that memory away from it.  A capture that needs more than the cached graph buffer retires it (kept
    alive) and takes a new one.  All graphs captured on one capture stream share that one buffer, as all calls
    on a stream do: replays of two of them that overlap on different streams race on it.  Callers that replay
    graphs concurrently pass a `workspace=` of their own per graph, sized with the *_workspace_bytes functions,
    and keep it alive."""
    key = (device, (stream or _stream_ptr(device)).value)
    if torch.device(device).type == "cuda" and torch.cuda.is_current_stream_capturing():
        buf = _graph_workspaces.get(key)
        if buf is None or buf.numel() < nbytes:
            if buf is not None:
                _graph_retired.append(buf)
            buf = _graph_workspaces[key] = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        return buf
    buf = _workspaces.pop(key, None)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
    _workspaces[key] = buf              # (re)inserted last: dict order is the LRU order
    while len(_workspaces) > _WORKSPACE_SLOTS:
        _workspaces.pop(next(iter(_workspaces)))
    return buf


class QTransform:
    """Norm and rotation of the Q rows done by the attention kernel as it loads them: the Q half of
    the reference's pre-attention step (QK RMSNorm, examples/models/qwen3/kernels/rmsnorm.py:4-21;
    RoPE at the row's absolute position, rope.py:23-48), bit for bit what `qk_norm_rope_kv_write`
    writes for Q, without that kernel's pass over Q.  rope_cos / rope_sin [max_pos, D/2] bfloat16
    (`rope_tables`); norm_weight [D] bfloat16 or None for rotation only."""

    def __init__(self, rope_cos, rope_sin, norm_weight=None, eps=1e-6):
        self.rope_cos, self.rope_sin, self.norm_weight, self.eps = rope_cos, rope_sin, norm_weight, float(eps)
        self._checked = None                 # (key, struct) of the last validated state

    def _struct(self, D, q):
        # validated once per state: the same object is passed on every call of every step
        key = (D, q.get_device(), q.dtype, id(self.rope_cos), id(self.rope_sin), id(self.norm_weight), self.eps)
        if self._checked is not None and self._checked[0] == key:
            return self._checked[1]
        st = self._build(D, q)
        self._checked = (key, st)
        return st

    def _build(self, D, q):
        for n, t in (("rope_cos", self.rope_cos), ("rope_sin", self.rope_sin)):
            _need_device(n, t)
            _check(t.dim() == 2 and t.shape[1] == D // 2 and t.dtype == torch.bfloat16 and t.shape[0] > 0,
                   f"q_transform.{n} must be bfloat16 [max_pos, D/2]")
        _check(self.rope_sin.shape == self.rope_cos.shape, "q_transform.rope_sin must match rope_cos")
        if self.norm_weight is not None:
            _need_device("norm_weight", self.norm_weight)
            _check(tuple(self.norm_weight.shape) == (D,) and self.norm_weight.dtype == torch.bfloat16,
                   "q_transform.norm_weight must be bfloat16 [D]")
        _check(q.dtype == torch.bfloat16, "q_transform needs bfloat16 q")
        _same_device(q, rope_cos=self.rope_cos, rope_sin=self.rope_sin, norm_weight=self.norm_weight)
        return _lib.QTransformStruct(None if self.norm_weight is None else self.norm_weight.data_ptr(),
                                     self.rope_cos.data_ptr(), self.rope_sin.data_ptr(),
                                     self.rope_cos.shape[0], self.eps)


def q_transform_supported(T, D, block_size) -> bool:
    """Whether the kernel that `decode` (T = 1) or `prefill` picks for bfloat16 q of this shape can
    take a `QTransform`: the matrix-core kernels, which need a power-of-two block size >= 16 and
    head_dim 128 or 64."""
    if block_size < 16 or block_size & (block_size - 1):
        return False
    return D in (64, 128)


def _qt_arg(q_transform, D, q):
    """(struct kept alive by the caller, pointer value or None) for a C call."""
    if q_transform is None:
        return None, None
    _check(isinstance(q_transform, QTransform), "q_transform must be a QTransform")
    st = q_transform._struct(D, q)
    return st, ctypes.addressof(st)


def decode(q, k_cache, v_cache, block_tables, seq_lens, scale, *, k_scale=None, v_scale=None,
           partition_size=512, max_seq_len=None, out=None, workspace=None, validate_tables=False,
           sinks=None, sliding_window=None, q_transform=None):
    """out[b, h] = softmax(q[b, h] . K_b^T * scale) V_b over the paged context.

    q [B, Hq, D] (float32 or bfloat16); k_cache/v_cache [num_blocks, block_size, Hkv, D]
    in q's dtype, or float8_e4m3fn / uint8 codes with k_scale/v_scale [num_blocks, Hkv]
    float32; block_tables int32 [B, max_blocks]; seq_lens int32 [B].
    max_seq_len: host-known upper bound of seq_lens (sizes the split-K grid
    without a device sync; default = table capacity).
    sinks [Hq]: per-head logits that join the softmax as one more column and carry no value;
    sliding_window W: only the last W keys are visible (bf16 / fp8 pools, head_dim 64 or 128).
    q_transform: a `QTransform`; q then holds the rows before norm and rotation (same shapes).
    """
    lib = _lib.load()
    for n, t in (("q", q), ("k_cache", k_cache), ("v_cache", v_cache),
                 ("block_tables", block_tables), ("seq_lens", seq_lens)):
        _need_device(n, t)
    _check(q.dim() == 3, "q must be [B, Hq, D]")
    B, Hq, D = q.shape
    _check(q.dtype in (torch.float32, torch.bfloat16), f"unsupported q dtype {q.dtype}")
    _check_paging(k_cache, v_cache, block_tables, seq_lens, B)
    num_blocks, block_size, Hkv, Dk = k_cache.shape
    _check(Dk == D, f"head_dim mismatch: q has {D}, cache has {Dk}")
    _check(Hq % Hkv == 0, f"Hq={Hq} is not a multiple of Hkv={Hkv}")
    _check(D in (32, 64, 128, 256), f"head_dim {D} not in (32, 64, 128, 256)")
    scaled = k_scale is not None or v_scale is not None
    kv_code = _kv_code(k_cache, scaled)
    q_code = _DTYPE_CODE[q.dtype]
    if kv_code == FP8:
        _check(q_code == BF16, "fp8 KV needs bfloat16 q")
        _check(k_scale is not None and v_scale is not None, "fp8 KV needs both k_scale and v_scale")
        for n, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            _need_device(n, t)
            _check(t.dtype == torch.float32 and t.shape == (num_blocks, Hkv),
                   f"{n} must be float32 [num_blocks, Hkv]")
    else:
        _check(kv_code == q_code, f"KV dtype {k_cache.dtype} does not match q dtype {q.dtype}")
        _check(not scaled, "k_scale/v_scale are only valid with an fp8 KV cache")
    sinks, win = _check_variant(sinks, sliding_window, Hq, q)
    _check(isinstance(partition_size, int) and partition_size > 0, "partition_size must be a positive int")
    cap = block_tables.shape[1] * block_size
    msl = cap if max_seq_len is None else int(max_seq_len)
    _check(0 < msl <= cap, f"max_seq_len {msl} outside (0, {cap}]")
    _same_device(q, k_cache=k_cache, v_cache=v_cache, block_tables=block_tables, seq_lens=seq_lens,
                 k_scale=k_scale, v_scale=v_scale, out=out)
    if validate_tables:
        check_block_tables(block_tables, seq_lens, num_blocks, block_size)
    if out is None:
        out = torch.empty_like(q)
    else:
        _need_device("out", out)
        _check(out.shape == q.shape and out.dtype == q.dtype, "out must match q in shape and dtype")
    with _on(q.device):
        need = int(lib.pa_decode_workspace_bytes_for(B, Hq, Hkv, D, block_size, msl, partition_size, q_code, kv_code))
    stream = _stream_ptr(q.device)
    if workspace is None:
        workspace = _workspace(q.device, need, stream) if need else None
    else:
        _need_device("workspace", workspace)
        _check(workspace.numel() * workspace.element_size() >= need, f"workspace needs {need} bytes")
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    qt_keep, qt_ptr = _qt_arg(q_transform, D, q)
    with _on(q.device):
        rc = lib.pa_decode(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale),
                           _ptr(block_tables), _ptr(seq_lens), _ptr(out), _ptr(workspace), ws_bytes,
                           B, Hq, Hkv, D, block_size, block_tables.shape[1], num_blocks, msl,
                           float(scale), partition_size, q_code, kv_code, _ptr(sinks), win, qt_ptr, stream)
    _raise_on(rc, "pa_decode")
    return out


# prefill() takes the verify kernel up to this many (query token, q head) rows per kv head: the measured
# crossover against the tiled kernel (rows packed over the kv group, key tiles split over workgroups when
# the grid is small) lies between 16 and 48 rows for batches of 1 to 64 sequences
VERIFY_MAX_ROWS = 32
VERIFY_MAX_ROWS_FP8 = 256     # fp8 pools: the tiled kernel has no packed-rows form for them (B = 64, 4 K prefix: T = 64 718 vs 810 us)
# bf16 pools of head dim 128, more than 16 rows per kv head.  Up to VERIFY_MAX_ROWS rows the verify kernel gives a kv
# head two 16-row waves, each of which streams every tile, and from this many (sequence x bound) tokens on the tiled
# kernel's packed rows are ahead (32 / 8 heads, T = 8, ragged contexts up to the bound, us verify / tiled: B = 8 behind
# 2 K 22.9 / 23.5, behind 4 K 41.0 / 31.3; B = 16 behind 1 K 20.2 / 22.6, behind 2 K 43.0 / 30.1; B = 32 behind 1 K 35.8 /
# 29.5; B = 64 behind 2 K 90.3 / 72.0).  Beyond VERIFY_MAX_ROWS a small call -- few sequences, a bound of a few thousand
# tokens -- is still faster on the verify kernel's fixed partitions (T = 16, us verify / tiled: B = 1 behind 1 K 14.1 /
# 21.0, behind 4 K 20.9 / 25.1; B = 2 behind 2 K 19.7 / 22.4; B = 4 behind 500 15.9 / 18.9), up to this many
# (sequence x row x bound) products.
TILED_FROM_TOKENS = 20_000
VERIFY_SMALL_CALL = 300_000


def prefill_route(B, T, Hq, Hkv, D, block_size, fp8=False, window=0, bound=None) -> str:
    """Which kernel `prefill` takes for a shape: "verify" (the decode-shaped kernel) or "tiled".  bound: what the
    caller knows of the longest context (None: nothing)."""
    can_verify = verify_supported(T, D, block_size)
    # the tiled kernel is built for bf16 pools and head_dim 128; what it cannot take goes to the verify kernel
    rows = T * (Hq // Hkv)
    if D == 64:
        # the tiled kernel takes head dim 64 two kv heads at a time (not a single kv head); below 384 rows per kv head, and for small
        # batches, the verify kernel is faster (measured crossover, as in pa_prefill itself: 64 / 8 heads, us verify /
        # tiled, T = 40: B = 8 behind 1 K 30.5 / 39.9, behind 4 K 58.0 / 74.6; T = 48: B = 8 behind 2 K 48.2 / 45.1)
        return "tiled" if not can_verify or (Hkv >= 2 and B >= 8 and rows >= 384) else "verify"
    if not can_verify:
        return "tiled"
    if D != 128:
        return "verify"
    if fp8:
        return "verify" if window > 0 or rows <= VERIFY_MAX_ROWS_FP8 else "tiled"
    if rows <= 16 or (window > 0 and rows <= VERIFY_MAX_ROWS):
        return "verify"
    if rows <= VERIFY_MAX_ROWS:
        if bound is None:
            return "tiled" if B >= 16 else "verify"
        return "tiled" if B >= 8 and B * bound >= TILED_FROM_TOKENS else "verify"
    return "verify" if bound is not None and window == 0 and B * rows * bound <= VERIFY_SMALL_CALL else "tiled"


def verify_supported(T, D, block_size) -> bool:
    """Shapes the verify kernel is built for."""
    return T <= 64 and D in (64, 128) and block_size >= 16 and block_size & (block_size - 1) == 0


def prefill(q, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, *, k_scale=None, v_scale=None,
            out=None, workspace=None, route=None, validate_tables=False, sinks=None, sliding_window=None,
            q_transform=None, max_seq_len=None):
    """Chunked prefill against a cached prefix (causal).

    q [B, T, Hq, D] bfloat16 holds the last query_lens[b] tokens of each sequence
    (rows t >= query_lens[b] are padding; their output is zero); token i sees keys
    j <= seq_lens[b] - query_lens[b] + i of the paged context, which already
    contains the new tokens' K/V.

    Two kernels stand behind it.  Short query runs -- speculative verify: up to 16 (token, q head) rows per
    kv head always, up to VERIFY_MAX_ROWS for small batches and short bounds, more for a handful of sequences
    under a bound of a few thousand tokens (`prefill_route`) -- go through the decode kernel with the
    (token, head) pairs as its query rows
    (HBM-bound: the context is read once per kv head); everything else through the tiled
    matrix-core prefill kernel (head_dim 128, and 64 with two or more kv heads; long query runs
    at head_dim 64 over a single kv head go through the verify kernel 64 tokens at a time).
    `route` = "verify" or "tiled" forces one.  fp8 pools
    (float8_e4m3fn / uint8 codes with k_scale, v_scale) work on both.  sinks and sliding_window are
    as in `decode`, the window counted back from each query token; so is q_transform, the position of
    row t being seq_lens[b] - query_lens[b] + t.
    max_seq_len: host-known upper bound of seq_lens, as in `decode`; with it a small verify call (a few
    short sequences, or a short sliding window) takes fixed partitions instead of the balanced schedule, whose
    fixed cost dominates at that size.  For the tiled kernel it is a hint: a chunk with less than twice its own
    length cached in front of it (max_seq_len < 3 T) runs unsplit, which is faster there.
    """
    lib = _lib.load()
    for n, t in (("q", q), ("k_cache", k_cache), ("v_cache", v_cache), ("block_tables", block_tables),
                 ("seq_lens", seq_lens), ("query_lens", query_lens)):
        _need_device(n, t)
    _check(q.dim() == 4, "q must be [B, T, Hq, D]")
    B, T, Hq, D = q.shape
    _check(q.dtype == torch.bfloat16, "prefill supports bfloat16 only")
    _check_paging(k_cache, v_cache, block_tables, seq_lens, B)
    scaled = k_scale is not None or v_scale is not None
    kv_code = _kv_code(k_cache, scaled)
    _check(kv_code in (BF16, FP8), "prefill needs a bfloat16 or fp8 KV cache")
    _check(query_lens.shape == (B,) and query_lens.dtype == torch.int32, "query_lens must be int32 [B]")
    num_blocks, block_size, Hkv, Dk = k_cache.shape
    _check(Dk == D, f"head_dim mismatch: q has {D}, cache has {Dk}")
    _check(Hq % Hkv == 0, f"Hq={Hq} is not a multiple of Hkv={Hkv}")
    if kv_code == FP8:
        _check(k_scale is not None and v_scale is not None, "fp8 KV needs both k_scale and v_scale")
        for n, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            _need_device(n, t)
            _check(t.dtype == torch.float32 and t.shape == (num_blocks, Hkv),
                   f"{n} must be float32 [num_blocks, Hkv]")
    else:
        _check(not scaled, "k_scale/v_scale are only valid with an fp8 KV cache")
    _check(route in (None, "verify", "tiled"), "route must be None, 'verify' or 'tiled'")
    sinks, win = _check_variant(sinks, sliding_window, Hq, q)
    can_verify = verify_supported(T, D, block_size)
    if route is None:
        route = prefill_route(B, T, Hq, Hkv, D, block_size, kv_code == FP8, win,
                              None if max_seq_len is None else int(max_seq_len))
    if route == "verify":
        _check(can_verify, f"the verify kernel needs T <= 64, head_dim 64 or 128 and a power-of-two block size >= 16 "
                           f"(T={T}, D={D}, block_size={block_size})")
    _same_device(q, k_cache=k_cache, v_cache=v_cache, block_tables=block_tables, seq_lens=seq_lens,
                 query_lens=query_lens, k_scale=k_scale, v_scale=v_scale, out=out)
    if validate_tables:
        check_block_tables(block_tables, seq_lens, num_blocks, block_size)
    if out is None:
        out = torch.empty_like(q)
    else:
        _need_device("out", out)
        _check(out.shape == q.shape and out.dtype == q.dtype, "out must match q in shape and dtype")
    qt_keep, qt_ptr = _qt_arg(q_transform, D, q)
    stream = _stream_ptr(q.device)
    cap = block_tables.shape[1] * block_size
    msl = 0 if max_seq_len is None else int(max_seq_len)
    _check(max_seq_len is None or 0 < msl <= cap, f"max_seq_len {msl} outside (0, {cap}]")
    if route == "verify":
        need = int(lib.pa_verify_workspace_bytes(B, T, Hq, D))
        if workspace is None:
            workspace = _workspace(q.device, need, stream)
        else:
            _need_device("workspace", workspace)
            _check(workspace.numel() * workspace.element_size() >= need, f"workspace needs {need} bytes")
        ws_bytes = workspace.numel() * workspace.element_size()
        with _on(q.device):
            rc = lib.pa_verify(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale),
                               _ptr(block_tables), _ptr(seq_lens), _ptr(query_lens), _ptr(out),
                               _ptr(workspace), ws_bytes, B, T, Hq, Hkv, D, block_size,
                               block_tables.shape[1], num_blocks, msl, float(scale), kv_code, _ptr(sinks), win,
                               qt_ptr, stream)
        _raise_on(rc, "pa_verify")
        return out
    with _on(q.device):
        need = int(lib.pa_prefill_workspace_bytes(B, T, Hq, Hkv, D, block_size, block_tables.shape[1]))
        if workspace is None:
            workspace = _workspace(q.device, need, stream) if need else None
        else:
            _need_device("workspace", workspace)
            _check(workspace.numel() * workspace.element_size() >= need, f"workspace needs {need} bytes")
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
        rc = lib.pa_prefill(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale),
                            _ptr(block_tables), _ptr(seq_lens),
                            _ptr(query_lens), _ptr(out), B, T, Hq, Hkv, D, block_size,
                            block_tables.shape[1], num_blocks, msl, float(scale), BF16, kv_code, _ptr(sinks), win,
                            _ptr(workspace), ws_bytes, qt_ptr, stream)
    _raise_on(rc, "pa_prefill")
    return out


def verify(q, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, **kw):
    """Speculative verify (gpt_oss/kernels/attention.py:80-100 with seq_len = K+1): prefill through
    the decode-shaped kernel whatever T * (Hq / Hkv) is."""
    return prefill(q, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, route="verify", **kw)


def blocksparse_prefill(q, k, v, scale, *, block=64, local_blocks=4, vert_stride=8, out=None):
    """Block-sparse causal prefill over dense q [B, S, Hq, D], k/v [B, S, Hkv, D] (bfloat16).

    q block i attends k block j iff j <= i and (i - j < local_blocks or
    (j + h % vert_stride) % vert_stride == 0); token-causal inside a block.
    """
    lib = _lib.load()
    for n, t in (("q", q), ("k", k), ("v", v)):
        _need_device(n, t)
    _check(q.dim() == 4 and k.dim() == 4, "q must be [B, S, Hq, D], k/v [B, S, Hkv, D]")
    B, S, Hq, D = q.shape
    _check(q.dtype == torch.bfloat16 and k.dtype == torch.bfloat16 and v.dtype == torch.bfloat16,
           "blocksparse_prefill supports bfloat16 only")
    _check(v.shape == k.shape and k.shape[0] == B and k.shape[1] == S and k.shape[3] == D,
           "k/v must be [B, S, Hkv, D] matching q")
    Hkv = k.shape[2]
    _check(Hq % Hkv == 0, f"Hq={Hq} is not a multiple of Hkv={Hkv}")
    _check(block == 64, "sparsity block must be 64")
    _check(local_blocks >= 1 and vert_stride >= 1, "local_blocks and vert_stride must be >= 1")
    _same_device(q, k=k, v=v, out=out)
    if out is None:
        out = torch.empty_like(q)
    else:
        _need_device("out", out)
        _check(out.shape == q.shape and out.dtype == q.dtype, "out must match q in shape and dtype")
    with _on(q.device):
        rc = lib.pa_blocksparse_prefill(_ptr(q), _ptr(k), _ptr(v), _ptr(out), B, S, Hq, Hkv, D, block,
                                        int(local_blocks), int(vert_stride), float(scale), BF16,
                                        _stream_ptr(q.device))
    _raise_on(rc, "pa_blocksparse_prefill")
    return out


def gather_kv(cache, block_tables, seq_lens, max_seq_len=None):
    """Materialise the block-table gather: [B, max_seq_len, Hkv, D], zero past seq_lens[b]."""
    lib = _lib.load()
    for n, t in (("cache", cache), ("block_tables", block_tables), ("seq_lens", seq_lens)):
        _need_device(n, t)
    _check(cache.dim() == 4, "cache must be [num_blocks, block_size, Hkv, D]")
    B = block_tables.shape[0]
    _check(block_tables.dim() == 2 and block_tables.dtype == torch.int32, "block_tables must be int32 [B, max_blocks]")
    _check(seq_lens.shape == (B,) and seq_lens.dtype == torch.int32, "seq_lens must be int32 [B]")
    num_blocks, block_size, Hkv, D = cache.shape
    cap = block_tables.shape[1] * block_size
    msl = cap if max_seq_len is None else int(max_seq_len)
    _check(0 <= msl <= cap, f"max_seq_len {msl} outside [0, {cap}]")
    out = torch.empty((B, msl, Hkv, D), dtype=cache.dtype, device=cache.device)
    with _on(cache.device):
        rc = lib.pa_gather_kv(_ptr(cache), _ptr(block_tables), _ptr(seq_lens), _ptr(out), B, Hkv, D,
                              block_size, block_tables.shape[1], num_blocks, msl, cache.element_size(),
                              _stream_ptr(cache.device))
    _raise_on(rc, "pa_gather_kv")
    return out


def kv_write(k_new, v_new, k_cache, v_cache, block_tables, seq_lens, query_lens, *, k_scale=None, v_scale=None):
    """Write the new tokens' K/V into the paged pool, in place, before the attention call.

    The reference's `cache_k[:, query_pos] = xk` with query_pos = start_pos + arange(seq_len)
    (examples/models/gpt_oss/kernels/attention.py:85,92-100): token t < query_lens[b] of sequence
    b lands at position seq_lens[b] - query_lens[b] + t, i.e. in pool row
    (block_tables[b, pos // block_size], pos % block_size).  k_new/v_new [B, T, Hkv, D] are
    bfloat16 (float32 for a float32 pool).  float8_e4m3fn pools are quantised on the way in and
    k_scale/v_scale [num_blocks, Hkv] float32 are maintained (running absmax / 448 per block and
    kv head; earlier rows of a block are re-encoded when its scale grows).  Returns None: the
    pool tensors are the outputs, aliased to the inputs as the reference's cache tensors are
    (examples/models/qwen3/qwen3.py:289-301).
    """
    lib = _lib.load()
    for n, t in (("k_new", k_new), ("v_new", v_new), ("k_cache", k_cache), ("v_cache", v_cache),
                 ("block_tables", block_tables), ("seq_lens", seq_lens), ("query_lens", query_lens)):
        _need_device(n, t)
    _check(k_new.dim() == 4, "k_new must be [B, T, Hkv, D]")
    _check(v_new.shape == k_new.shape and v_new.dtype == k_new.dtype, "v_new must match k_new")
    _check(k_cache.dim() == 4, "k_cache must be [num_blocks, block_size, Hkv, D]")
    _check(v_cache.shape == k_cache.shape and v_cache.dtype == k_cache.dtype, "v_cache must match k_cache")
    _check(k_cache.dtype in _DTYPE_CODE, f"unsupported pool dtype {k_cache.dtype}")
    B, T, Hkv, D = k_new.shape
    num_blocks, block_size = k_cache.shape[:2]
    _check(tuple(k_cache.shape[2:]) == (Hkv, D), f"pool rows are {tuple(k_cache.shape[2:])}, new rows {(Hkv, D)}")
    kv_dtype = _DTYPE_CODE[k_cache.dtype]
    want = torch.float32 if kv_dtype == F32 else torch.bfloat16
    _check(k_new.dtype == want, f"k_new must be {want} for a {k_cache.dtype} pool, got {k_new.dtype}")
    _check(block_tables.dim() == 2 and block_tables.shape[0] == B and block_tables.dtype == torch.int32,
           "block_tables must be int32 [B, max_blocks]")
    _check(seq_lens.shape == (B,) and seq_lens.dtype == torch.int32, "seq_lens must be int32 [B]")
    _check(query_lens.shape == (B,) and query_lens.dtype == torch.int32, "query_lens must be int32 [B]")
    if kv_dtype == FP8:
        _check(k_scale is not None and v_scale is not None, "float8 pools need k_scale and v_scale")
        for n, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            _need_device(n, t)
            _check(t.dtype == torch.float32 and tuple(t.shape) == (num_blocks, Hkv), f"{n} must be float32 [num_blocks, Hkv]")
    else:
        _check(k_scale is None and v_scale is None, "k_scale / v_scale are for float8 pools only")
    _same_device(k_new, v_new=v_new, k_cache=k_cache, v_cache=v_cache, block_tables=block_tables,
                 seq_lens=seq_lens, query_lens=query_lens, k_scale=k_scale, v_scale=v_scale)
    with _on(k_new.device):
        rc = lib.pa_kv_write(_ptr(k_new), _ptr(v_new), _ptr(k_cache), _ptr(v_cache),
                             _ptr(k_scale) if k_scale is not None else None,
                             _ptr(v_scale) if v_scale is not None else None,
                             _ptr(block_tables), _ptr(seq_lens), _ptr(query_lens),
                             B, T, Hkv, D, block_size, block_tables.shape[1], num_blocks, kv_dtype,
                             _stream_ptr(k_new.device))
    _raise_on(rc, "pa_kv_write")


def rope_tables(head_dim: int, max_seq_len: int, base: float = 10000.0, device="cuda"):
    """cos / sin tables [max_seq_len, head_dim // 2] in bfloat16 on `device`, computed as
    examples/models/qwen3/kernels/rope.py:4-20 does (float64 frequencies, float32 angles and
    cos / sin, cast to bf16 at the call site attention.py:84-86)."""
    freqs = 1.0 / (base ** (np.arange(0, head_dim, 2)[: (head_dim // 2)] / head_dim))
    ang = np.outer(np.arange(max_seq_len, dtype=np.float32), freqs)
    cos, sin = np.cos(ang, dtype=np.float32), np.sin(ang, dtype=np.float32)
    return (torch.from_numpy(cos).to(device).to(torch.bfloat16), torch.from_numpy(sin).to(device).to(torch.bfloat16))


def qk_norm_rope_kv_write(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, rope_cos, rope_sin, *,
                          q_norm_weight=None, k_norm_weight=None, eps=1e-6, k_scale=None, v_scale=None, out=None):
    """The reference's pre-attention step fused with the paged KV write.

    QK RMSNorm (examples/models/qwen3/kernels/rmsnorm.py:4-21; skipped for a tensor whose weight
    is None), RoPE at absolute positions seq_lens[b] - query_lens[b] + t (rope.py:23-48;
    qwen3/kernels/attention.py:78-97), then `kv_write` of the rotated K and of V.  xq [B, T, Hq, D],
    xk / xv [B, T, Hkv, D] bfloat16; rope_cos / rope_sin [max_pos, D/2] bfloat16 (`rope_tables`).
    Returns the transformed q (`out`, which may be xq itself; padding rows are zero); the pool
    (and its scales for float8) is updated in place.

    xq None: only K and V are done and None is returned; the Q half then rides on the attention
    call as its `q_transform` (a `QTransform` with the same tables), which saves a pass over Q.
    """
    lib = _lib.load()
    for n, t in (("xk", xk), ("xv", xv), ("k_cache", k_cache), ("v_cache", v_cache),
                 ("block_tables", block_tables), ("seq_lens", seq_lens), ("query_lens", query_lens),
                 ("rope_cos", rope_cos), ("rope_sin", rope_sin)):
        _need_device(n, t)
    _check(xk.dim() == 4 and xk.dtype == torch.bfloat16, "xk must be bfloat16 [B, T, Hkv, D]")
    B, T, Hkv, D = xk.shape
    _check(xv.shape == xk.shape and xv.dtype == torch.bfloat16, "xv must match xk")
    if xq is None:
        _check(out is None and q_norm_weight is None, "without xq there is neither out nor q_norm_weight")
        Hq = Hkv
    else:
        _need_device("xq", xq)
        _check(xq.dim() == 4 and xq.dtype == torch.bfloat16 and xq.shape[:2] == (B, T) and xq.shape[3] == D,
               "xq must be bfloat16 [B, T, Hq, D] with xk's B, T and D")
        Hq = xq.shape[2]
    _check(Hq % Hkv == 0, f"Hq={Hq} is not a multiple of Hkv={Hkv}")
    _check(D in (64, 128, 256), f"head_dim {D} must be 64, 128 or 256")
    _check(k_cache.dim() == 4 and tuple(k_cache.shape[2:]) == (Hkv, D), "k_cache must be [num_blocks, block_size, Hkv, D]")
    _check(v_cache.shape == k_cache.shape and v_cache.dtype == k_cache.dtype, "v_cache must match k_cache")
    _check(k_cache.dtype in (torch.bfloat16, torch.float8_e4m3fn), f"unsupported pool dtype {k_cache.dtype}")
    num_blocks, block_size = k_cache.shape[:2]
    kv_dtype = _DTYPE_CODE[k_cache.dtype]
    for n, t in (("rope_cos", rope_cos), ("rope_sin", rope_sin)):
        _check(t.dim() == 2 and t.shape[1] == D // 2 and t.dtype == torch.bfloat16, f"{n} must be bfloat16 [max_pos, D/2]")
    _check(rope_sin.shape == rope_cos.shape, "rope_sin must match rope_cos")
    for n, t in (("q_norm_weight", q_norm_weight), ("k_norm_weight", k_norm_weight)):
        if t is not None:
            _need_device(n, t)
            _check(tuple(t.shape) == (D,) and t.dtype == torch.bfloat16, f"{n} must be bfloat16 [D]")
    _check(block_tables.dim() == 2 and block_tables.shape[0] == B and block_tables.dtype == torch.int32,
           "block_tables must be int32 [B, max_blocks]")
    _check(seq_lens.shape == (B,) and seq_lens.dtype == torch.int32, "seq_lens must be int32 [B]")
    _check(query_lens.shape == (B,) and query_lens.dtype == torch.int32, "query_lens must be int32 [B]")
    if kv_dtype == FP8:
        _check(k_scale is not None and v_scale is not None, "float8 pools need k_scale and v_scale")
        for n, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            _need_device(n, t)
            _check(t.dtype == torch.float32 and tuple(t.shape) == (num_blocks, Hkv), f"{n} must be float32 [num_blocks, Hkv]")
    else:
        _check(k_scale is None and v_scale is None, "k_scale / v_scale are for float8 pools only")
    if xq is not None:
        if out is None:
            out = torch.empty_like(xq)
        else:
            _need_device("out", out)
            _check(out.shape == xq.shape and out.dtype == xq.dtype, "out must match xq")
    _same_device(xk, xq=xq, xv=xv, k_cache=k_cache, v_cache=v_cache, block_tables=block_tables, seq_lens=seq_lens,
                 query_lens=query_lens, rope_cos=rope_cos, rope_sin=rope_sin, q_norm_weight=q_norm_weight,
                 k_norm_weight=k_norm_weight, k_scale=k_scale, v_scale=v_scale, out=out)
    with _on(xk.device):
        rc = lib.pa_qk_norm_rope_kv_write(
            _ptr(xq), _ptr(xk), _ptr(xv), _ptr(out), _ptr(q_norm_weight), _ptr(k_norm_weight), ctypes.c_float(eps),
            _ptr(rope_cos), _ptr(rope_sin), rope_cos.shape[0], _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale),
            _ptr(block_tables), _ptr(seq_lens), _ptr(query_lens), B, T, Hq, Hkv, D, block_size, block_tables.shape[1],
            num_blocks, kv_dtype, _stream_ptr(xk.device))
    _raise_on(rc, "pa_qk_norm_rope_kv_write")
    return out


def o_proj(x, o_weight, bias=None, *, out=None, workspace=None):
    """Output projection behind the attention call: `np.matmul(output, o_weight)` (+ `o_bias`) of
    examples/models/qwen3/kernels/attention.py:143-147 and examples/models/gpt_oss/kernels/attention.py:155-163.

    x: the attention output, bfloat16, [..., Hq, D] (as `decode` / `prefill` return it) or already
    [..., K] (with a single q head the two readings coincide: `out`'s rank decides, and without `out` x is
    read as [..., K]); o_weight [K, N] bfloat16 with K = Hq * D (the reference's transposed o_proj.weight; a
    tensor-parallel rank passes its own K rows and all-reduces the result itself); bias [N]
    bfloat16 or None.  Returns [..., N] bfloat16 (`out`, if given, is written in place).  Products
    and sums are float32; the result is rounded to bfloat16 once.  Calls of up to 128 rows (decode,
    verify steps) spread K over several workgroups per column slab and need scratch memory for the
    partial sums: a uint8 tensor `workspace` of at least `o_proj_workspace_bytes(M, K, N)` bytes, or,
    by default, a buffer cached per (device, stream).
    """
    lib = _lib.load()
    for n, t in (("x", x), ("o_weight", o_weight)):
        _need_device(n, t)
    _check(x.dtype == torch.bfloat16 and o_weight.dtype == torch.bfloat16, "o_proj supports bfloat16 only")
    _check(o_weight.dim() == 2, "o_weight must be [K, N]")
    K, N = o_weight.shape
    heads_form = x.dim() >= 2 and x.shape[-1] * x.shape[-2] == K      # [..., Hq, D] -> [..., Hq * D]
    flat_form = x.dim() >= 1 and x.shape[-1] == K
    if heads_form and flat_form:
        # one q head (Hq = 1, D = K): both readings fit x.  `out`, when given, says which one the caller means (an engine
        # layer with one q head passes x [B, T, 1, D] and out [B, T, N]); without it x is read as [..., K]
        heads_form = isinstance(out, torch.Tensor) and out.dim() == x.dim() - 1
        flat_form = not heads_form
    if heads_form:
        lead = tuple(x.shape[:-2])
    else:
        _check(flat_form, f"x's last dimension(s) {tuple(x.shape[-2:])} do not give K={K}")
        lead = tuple(x.shape[:-1])
    M = 1
    for d in lead:
        M *= d
    _check(K % 64 == 0, f"K={K} must be a multiple of 64")
    _check(N % 8 == 0, f"N={N} must be a multiple of 8")
    if bias is not None:
        _need_device("bias", bias)
        _check(bias.dtype == torch.bfloat16 and tuple(bias.shape) == (N,), "bias must be bfloat16 [N]")
    _same_device(x, o_weight=o_weight, bias=bias, out=out)
    if out is None:
        out = torch.empty(lead + (N,), dtype=torch.bfloat16, device=x.device)
    else:
        _need_device("out", out)
        _check(tuple(out.shape) == lead + (N,) and out.dtype == torch.bfloat16, f"out must be bfloat16 {lead + (N,)}")
    with _on(x.device):
        stream = _stream_ptr(x.device)
        need = _o_proj_need.get((M, K, N))
        if need is None:
            need = _o_proj_need[(M, K, N)] = int(lib.pa_o_proj_workspace_bytes(M, K, N))
        if workspace is not None:
            _need_device("workspace", workspace)
            _check(workspace.dtype == torch.uint8 and workspace.is_contiguous(), "workspace must be a contiguous uint8 tensor")
            _check(workspace.data_ptr() % 16 == 0, "workspace must be 16-byte aligned")
            _same_device(x, workspace=workspace)
        elif need:
            # (the split form is one more launch: where a step of a few rows is launched call by call and bound by the
            # host it costs 5 us per layer, replayed from a HIP graph it saves 6; it is taken either way, so that the
            # result does not depend on how the call was issued)
            workspace = _workspace(x.device, need, stream)
        rc = lib.pa_o_proj_ws(_ptr(x), _ptr(o_weight), _ptr(bias), _ptr(out), _ptr(workspace),
                              workspace.numel() if workspace is not None else 0, M, K, N, BF16, stream)
    _raise_on(rc, "pa_o_proj")
    return out


class PreparedStep:
    """A `decode_step` / `verify_step` call with its arguments checked and marshalled once, for callers that issue
    the same step on the same tensors again and again (a layer of a decode loop run without a HIP graph: the call
    is then bound by the host, and most of the host's time went into re-checking what had not changed).  `launch()`
    issues it on the current stream and returns `out`.  The step is tied to the storage of every tensor it was
    prepared with (they are kept alive): new values are copied into them, not passed."""
    __slots__ = ("fn", "who", "head", "tail", "need", "workspace", "device", "out", "keep")

    def launch(self):
        stream = _stream_ptr(self.device)
        ws = self.workspace if self.workspace is not None else _workspace(self.device, self.need, stream)
        with _on(self.device):
            rc = self.fn(*self.head, ws.data_ptr(), ws.numel(), *self.tail, stream)
        _raise_on(rc, self.who)
        return self.out

    __call__ = launch


def decode_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, **kw):
    """One decode step of an attention layer in one call; arguments and result as `prepare_decode_step`, which this is
    followed by `launch()`."""
    return prepare_decode_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, **kw).launch()


def prepare_decode_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, *, k_scale=None, v_scale=None,
                        partition_size=512, max_seq_len=None, q_transform=None, k_norm_weight=None, o_weight=None, o_bias=None,
                        out=None, attn_out=None, workspace=None, sinks=None, sliding_window=None) -> PreparedStep:
    """One decode step of an attention layer in one call: the cache update, the attention and, with `o_weight`, the
    output projection -- the decode branch of the reference's attention_kernel as a whole
    (examples/models/qwen3/kernels/attention.py:78-147; examples/models/gpt_oss/kernels/attention.py:85-163).

    Bit for bit the result of `qk_norm_rope_kv_write(None, xk, xv, ...)` (`kv_write` without `q_transform`), then
    `decode(xq, ..., q_transform=...)`, then `o_proj(...)`; a small step over a bfloat16 pool runs as three launches
    instead of five (the new row rides on the decode launch, the split-K merge on the projection's load).

    xq [B, Hq, D], xk / xv [B, Hkv, D]: the step's new token per sequence, before norm and rotation when `q_transform`
    (a `QTransform`: Q's norm weight and the RoPE tables) is given; `k_norm_weight` [D] is K's norm weight (None: K is
    rotated only).  seq_lens counts the new token; query_lens [B] int32 is 1 for the sequences that take one and 0 for
    those that do not.  The pools (and the scales of a float8 pool) are updated in place.
    The step's result (`PreparedStep.out`, what `launch()` returns) is the projected rows [B, N] when `o_weight`
    [Hq * D, N] is given (written to `out` if passed; `attn_out` [B, Hq, D], if passed, also receives the attention
    output), else the attention output [B, Hq, D] (`out`).  Nothing is launched here.
    """
    lib = _lib.load()
    for n, t in (("xq", xq), ("xk", xk), ("xv", xv), ("k_cache", k_cache), ("v_cache", v_cache),
                 ("block_tables", block_tables), ("seq_lens", seq_lens), ("query_lens", query_lens)):
        _need_device(n, t)
    _check(xq.dim() == 3, "xq must be [B, Hq, D]")
    B, Hq, D = xq.shape
    _check(xq.dtype in (torch.float32, torch.bfloat16), f"unsupported xq dtype {xq.dtype}")
    _check_paging(k_cache, v_cache, block_tables, seq_lens, B)
    num_blocks, block_size, Hkv, Dk = k_cache.shape
    _check(Dk == D, f"head_dim mismatch: xq has {D}, cache has {Dk}")
    _check(Hq % Hkv == 0, f"Hq={Hq} is not a multiple of Hkv={Hkv}")
    _check(D in (32, 64, 128, 256), f"head_dim {D} not in (32, 64, 128, 256)")
    _check(tuple(xk.shape) == (B, Hkv, D) and xv.shape == xk.shape and xk.dtype == xq.dtype and xv.dtype == xq.dtype,
           f"xk and xv must be {xq.dtype} [B, Hkv, D] = {(B, Hkv, D)}")
    _check(query_lens.shape == (B,) and query_lens.dtype == torch.int32, "query_lens must be int32 [B]")
    scaled = k_scale is not None or v_scale is not None
    kv_code = _kv_code(k_cache, scaled)
    q_code = _DTYPE_CODE[xq.dtype]
    if kv_code == FP8:
        _check(q_code == BF16, "fp8 KV needs bfloat16 rows")
        _check(k_scale is not None and v_scale is not None, "fp8 KV needs both k_scale and v_scale")
        for n, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            _need_device(n, t)
            _check(t.dtype == torch.float32 and t.shape == (num_blocks, Hkv), f"{n} must be float32 [num_blocks, Hkv]")
    else:
        _check(kv_code == q_code, f"KV dtype {k_cache.dtype} does not match the rows' dtype {xq.dtype}")
        _check(not scaled, "k_scale/v_scale are only valid with an fp8 KV cache")
    sinks, win = _check_variant(sinks, sliding_window, Hq, xq)
    _check(isinstance(partition_size, int) and partition_size > 0, "partition_size must be a positive int")
    cap = block_tables.shape[1] * block_size
    msl = cap if max_seq_len is None else int(max_seq_len)
    _check(0 < msl <= cap, f"max_seq_len {msl} outside (0, {cap}]")
    if k_norm_weight is not None:
        _need_device("k_norm_weight", k_norm_weight)
        _check(q_transform is not None, "k_norm_weight comes with q_transform")
        _check(tuple(k_norm_weight.shape) == (D,) and k_norm_weight.dtype == torch.bfloat16, "k_norm_weight must be bfloat16 [D]")
    N = 0
    if o_weight is not None:
        _need_device("o_weight", o_weight)
        _check(xq.dtype == torch.bfloat16 and o_weight.dtype == torch.bfloat16, "the output projection supports bfloat16 only")
        _check(o_weight.dim() == 2 and o_weight.shape[0] == Hq * D, f"o_weight must be [Hq * D = {Hq * D}, N]")
        N = o_weight.shape[1]
        _check((Hq * D) % 64 == 0 and N % 8 == 0, f"Hq * D = {Hq * D} must be a multiple of 64 and N = {N} of 8")
        if o_bias is not None:
            _need_device("o_bias", o_bias)
            _check(o_bias.dtype == torch.bfloat16 and tuple(o_bias.shape) == (N,), "o_bias must be bfloat16 [N]")
        if out is None:
            out = torch.empty((B, N), dtype=torch.bfloat16, device=xq.device)
        else:
            _need_device("out", out)
            _check(tuple(out.shape) == (B, N) and out.dtype == torch.bfloat16, f"out must be bfloat16 {(B, N)}")
        if attn_out is not None:
            _need_device("attn_out", attn_out)
            _check(attn_out.shape == xq.shape and attn_out.dtype == xq.dtype, "attn_out must match xq in shape and dtype")
    else:
        _check(o_bias is None and attn_out is None, "o_bias and attn_out come with o_weight (without it `out` is the attention output)")
        if out is None:
            out = torch.empty_like(xq)
        else:
            _need_device("out", out)
            _check(out.shape == xq.shape and out.dtype == xq.dtype, "out must match xq in shape and dtype")
        attn_out = out
    _same_device(xq, xk=xk, xv=xv, k_cache=k_cache, v_cache=v_cache, block_tables=block_tables, seq_lens=seq_lens,
                 query_lens=query_lens, k_scale=k_scale, v_scale=v_scale, out=out, attn_out=attn_out, o_weight=o_weight,
                 o_bias=o_bias, k_norm_weight=k_norm_weight)
    key = (B, Hq, Hkv, D, block_size, msl, partition_size, N, q_code, kv_code)
    need = _decode_step_need.get(key)
    if need is None:
        with _on(xq.device):
            need = _decode_step_need[key] = int(lib.pa_decode_step_workspace_bytes(*key))
    if workspace is not None:
        _need_device("workspace", workspace)
        _check(workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.data_ptr() % 16 == 0,
               "workspace must be a contiguous, 16-byte aligned uint8 tensor")
        _check(workspace.numel() >= need, f"workspace needs {need} bytes")
    qt_keep, qt_ptr = _qt_arg(q_transform, D, xq)
    addr = lambda t: None if t is None else t.data_ptr()
    nkv = _lib.NewKvStruct(addr(xk), addr(xv), addr(k_norm_weight), addr(query_lens))
    proj = None if o_weight is None else _lib.OutProjStruct(addr(o_weight), addr(o_bias), addr(out), N)
    st = PreparedStep()
    st.fn, st.who, st.need, st.workspace, st.device, st.out = lib.pa_decode_step, "pa_decode_step", need, workspace, xq.device, out
    st.head = (_ptr(xq), ctypes.addressof(nkv), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale),
               _ptr(block_tables), _ptr(seq_lens), _ptr(attn_out), None if proj is None else ctypes.addressof(proj))
    st.tail = (B, Hq, Hkv, D, block_size, block_tables.shape[1], num_blocks, msl,
               float(scale), partition_size, q_code, kv_code, _ptr(sinks), win, qt_ptr)
    # everything an address above points into stays alive with the step
    st.keep = (nkv, proj, qt_keep, xq, xk, xv, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, query_lens,
               attn_out, out, sinks, k_norm_weight, o_weight, o_bias, q_transform)
    return st


_decode_step_need = {}


def verify_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, **kw):
    """A speculative verify step of an attention layer in one call; arguments and result as `prepare_verify_step`,
    which this is followed by `launch()`."""
    return prepare_verify_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, **kw).launch()


def prepare_verify_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, *, k_scale=None, v_scale=None,
                        max_seq_len=None, q_transform=None, k_norm_weight=None, o_weight=None, o_bias=None, out=None,
                        attn_out=None, workspace=None, sinks=None, sliding_window=None) -> PreparedStep:
    """A speculative verify step of an attention layer in one call: `decode_step` for up to 64 new tokens per sequence
    (examples/models/gpt_oss/kernels/attention.py:80-163 with seq_len = K + 1; peagle/speculate.py:137-202).

    Bit for bit `qk_norm_rope_kv_write(None, xk, xv, ...)` (`kv_write` without `q_transform`), `verify(xq, ...)`,
    `o_proj(...)`.  xq [B, T, Hq, D], xk / xv [B, T, Hkv, D] bfloat16; query_lens [B]: new tokens per sequence (rows
    t >= query_lens[b] are padding: zero attention output, bias after the projection).  The step's result is
    [B, T, N] with `o_weight`, else the attention output [B, T, Hq, D].  Nothing is launched here."""
    lib = _lib.load()
    for n, t in (("xq", xq), ("xk", xk), ("xv", xv), ("k_cache", k_cache), ("v_cache", v_cache),
                 ("block_tables", block_tables), ("seq_lens", seq_lens), ("query_lens", query_lens)):
        _need_device(n, t)
    _check(xq.dim() == 4, "xq must be [B, T, Hq, D]")
    B, T, Hq, D = xq.shape
    _check(xq.dtype == torch.bfloat16, "verify_step supports bfloat16 rows only")
    _check_paging(k_cache, v_cache, block_tables, seq_lens, B)
    num_blocks, block_size, Hkv, Dk = k_cache.shape
    _check(Dk == D, f"head_dim mismatch: xq has {D}, cache has {Dk}")
    _check(Hq % Hkv == 0, f"Hq={Hq} is not a multiple of Hkv={Hkv}")
    _check(verify_supported(T, D, block_size),
           f"the verify kernel needs T <= 64, head_dim 64 or 128 and a power-of-two block size >= 16 (T={T}, D={D}, block_size={block_size})")
    _check(tuple(xk.shape) == (B, T, Hkv, D) and xv.shape == xk.shape and xk.dtype == xq.dtype and xv.dtype == xq.dtype,
           f"xk and xv must be bfloat16 [B, T, Hkv, D] = {(B, T, Hkv, D)}")
    _check(query_lens.shape == (B,) and query_lens.dtype == torch.int32, "query_lens must be int32 [B]")
    scaled = k_scale is not None or v_scale is not None
    kv_code = _kv_code(k_cache, scaled)
    _check(kv_code in (BF16, FP8), "verify_step needs a bfloat16 or fp8 KV cache")
    if kv_code == FP8:
        _check(k_scale is not None and v_scale is not None, "fp8 KV needs both k_scale and v_scale")
        for n, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            _need_device(n, t)
            _check(t.dtype == torch.float32 and t.shape == (num_blocks, Hkv), f"{n} must be float32 [num_blocks, Hkv]")
    else:
        _check(not scaled, "k_scale/v_scale are only valid with an fp8 KV cache")
    sinks, win = _check_variant(sinks, sliding_window, Hq, xq)
    cap = block_tables.shape[1] * block_size
    msl = 0 if max_seq_len is None else int(max_seq_len)
    _check(max_seq_len is None or 0 < msl <= cap, f"max_seq_len {msl} outside (0, {cap}]")
    if k_norm_weight is not None:
        _need_device("k_norm_weight", k_norm_weight)
        _check(q_transform is not None, "k_norm_weight comes with q_transform")
        _check(tuple(k_norm_weight.shape) == (D,) and k_norm_weight.dtype == torch.bfloat16, "k_norm_weight must be bfloat16 [D]")
    N = 0
    if o_weight is not None:
        _need_device("o_weight", o_weight)
        _check(o_weight.dtype == torch.bfloat16 and o_weight.dim() == 2 and o_weight.shape[0] == Hq * D,
               f"o_weight must be bfloat16 [Hq * D = {Hq * D}, N]")
        N = o_weight.shape[1]
        _check((Hq * D) % 64 == 0 and N % 8 == 0, f"Hq * D = {Hq * D} must be a multiple of 64 and N = {N} of 8")
        if o_bias is not None:
            _need_device("o_bias", o_bias)
            _check(o_bias.dtype == torch.bfloat16 and tuple(o_bias.shape) == (N,), "o_bias must be bfloat16 [N]")
        if out is None:
            out = torch.empty((B, T, N), dtype=torch.bfloat16, device=xq.device)
        else:
            _need_device("out", out)
            _check(tuple(out.shape) == (B, T, N) and out.dtype == torch.bfloat16, f"out must be bfloat16 {(B, T, N)}")
        if attn_out is not None:
            _need_device("attn_out", attn_out)
            _check(attn_out.shape == xq.shape and attn_out.dtype == xq.dtype, "attn_out must match xq in shape and dtype")
    else:
        _check(o_bias is None and attn_out is None, "o_bias and attn_out come with o_weight (without it `out` is the attention output)")
        if out is None:
            out = torch.empty_like(xq)
        else:
            _need_device("out", out)
            _check(out.shape == xq.shape and out.dtype == xq.dtype, "out must match xq in shape and dtype")
        attn_out = out
    _same_device(xq, xk=xk, xv=xv, k_cache=k_cache, v_cache=v_cache, block_tables=block_tables, seq_lens=seq_lens,
                 query_lens=query_lens, k_scale=k_scale, v_scale=v_scale, out=out, attn_out=attn_out, o_weight=o_weight,
                 o_bias=o_bias, k_norm_weight=k_norm_weight)
    key = ("v", B, T, Hq, D, N)
    need = _decode_step_need.get(key)
    if need is None:
        with _on(xq.device):
            need = _decode_step_need[key] = int(lib.pa_verify_step_workspace_bytes(B, T, Hq, D, N))
    if workspace is not None:
        _need_device("workspace", workspace)
        _check(workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.data_ptr() % 16 == 0,
               "workspace must be a contiguous, 16-byte aligned uint8 tensor")
        _check(workspace.numel() >= need, f"workspace needs {need} bytes")
    qt_keep, qt_ptr = _qt_arg(q_transform, D, xq)
    addr = lambda t: None if t is None else t.data_ptr()
    nkv = _lib.NewKvStruct(addr(xk), addr(xv), addr(k_norm_weight), addr(query_lens))
    proj = None if o_weight is None else _lib.OutProjStruct(addr(o_weight), addr(o_bias), addr(out), N)
    st = PreparedStep()
    st.fn, st.who, st.need, st.workspace, st.device, st.out = lib.pa_verify_step, "pa_verify_step", need, workspace, xq.device, out
    st.head = (_ptr(xq), ctypes.addressof(nkv), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale),
               _ptr(block_tables), _ptr(seq_lens), _ptr(attn_out), None if proj is None else ctypes.addressof(proj))
    st.tail = (B, T, Hq, Hkv, D, block_size, block_tables.shape[1], num_blocks, msl,
               float(scale), kv_code, _ptr(sinks), win, qt_ptr)
    st.keep = (nkv, proj, qt_keep, xq, xk, xv, k_cache, v_cache, k_scale, v_scale, block_tables, seq_lens, query_lens,
               attn_out, out, sinks, k_norm_weight, o_weight, o_bias, q_transform)
    return st
def o_proj_workspace_bytes(M: int, K: int, N: int) -> int:
    """Scratch bytes `o_proj` would use for a call of M rows (0 for shapes that take none)."""
    return int(_lib.load().pa_o_proj_workspace_bytes(int(M), int(K), int(N)))


def default_scale(head_dim: int) -> float:
    """1 / sqrt(head_dim) in float32, as examples/models/qwen3/kernels/attention.py:119."""
    return float(np.float32(1.0) / np.float32(math.sqrt(head_dim)))
