"""The paged attention ops as PyTorch custom operators (`torch.ops.nkipy_amd.*`).

A serving engine built on PyTorch-ROCm calls kernels through the dispatcher so that they can sit
inside traced or compiled graphs; this is the MI355X counterpart of the reference's hook for
hand-written kernels inside a traced function (`nki_custom_op`,
nkipy/src/nkipy/core/nki_op.py:800-884): the operator is opaque to the tracer, declares what it
mutates, and has a shape-only ("fake") implementation for tracing.  There is no CPU kernel behind
any of them: host tensors raise NotImplementedError, as that hook does on the CPU backend
(nki_op.py:480,557,719-722).

Every operator writes into buffers the caller passes (`out`, the caches) and returns nothing, so
the caller-allocates rule of nkipy/src/nkipy/runtime/device_tensor.py:51-74 carries over and a
captured graph replays without allocations.  Optional tensors may be None; `sliding_window` 0 means
none.

`workspace` (paged_decode, paged_prefill, o_proj): optional uint8 scratch for split-K partials, sized with
`paged_attn.decode_workspace_bytes` / `lib.pa_verify_workspace_bytes` / `pa_prefill_workspace_bytes` /
`o_proj_workspace_bytes`.  Without it the ops use a buffer cached per (device, stream), which all graphs
captured on one stream share.  A caller that replays several graphs at once gives each its own.  The
scratch carries nothing from call to call, so it is not declared as a mutated argument.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import paged_attn

_NS = "nkipy_amd"


def _win(w: int):
    return None if w <= 0 else int(w)


def _qt(rope_cos, rope_sin, q_norm_weight, eps):
    return None if rope_cos is None else paged_attn.QTransform(rope_cos, rope_sin, q_norm_weight, eps)


@torch.library.custom_op(f"{_NS}::paged_decode", mutates_args=("out",), device_types="cuda")
def paged_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                 seq_lens: torch.Tensor, scale: float, out: torch.Tensor,
                 k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                 max_seq_len: int = 0, sinks: Optional[torch.Tensor] = None, sliding_window: int = 0,
                 rope_cos: Optional[torch.Tensor] = None, rope_sin: Optional[torch.Tensor] = None,
                 q_norm_weight: Optional[torch.Tensor] = None, norm_eps: float = 1e-6,
                 workspace: Optional[torch.Tensor] = None, partition_size: int = 512) -> None:
    paged_attn.decode(q, k_cache, v_cache, block_tables, seq_lens, scale, k_scale=k_scale, v_scale=v_scale,
                      max_seq_len=max_seq_len or None, out=out, sinks=sinks, sliding_window=_win(sliding_window),
                      q_transform=_qt(rope_cos, rope_sin, q_norm_weight, norm_eps), workspace=workspace,
                      partition_size=partition_size)


@torch.library.custom_op(f"{_NS}::paged_prefill", mutates_args=("out",), device_types="cuda")
def paged_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                  seq_lens: torch.Tensor, query_lens: torch.Tensor, scale: float, out: torch.Tensor,
                  k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                  sinks: Optional[torch.Tensor] = None, sliding_window: int = 0,
                  rope_cos: Optional[torch.Tensor] = None, rope_sin: Optional[torch.Tensor] = None,
                  q_norm_weight: Optional[torch.Tensor] = None, norm_eps: float = 1e-6,
                  workspace: Optional[torch.Tensor] = None, max_seq_len: int = 0) -> None:
    paged_attn.prefill(q, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, k_scale=k_scale,
                       v_scale=v_scale, out=out, sinks=sinks, sliding_window=_win(sliding_window),
                       q_transform=_qt(rope_cos, rope_sin, q_norm_weight, norm_eps), workspace=workspace,
                       max_seq_len=max_seq_len or None)


@torch.library.custom_op(f"{_NS}::blocksparse_prefill", mutates_args=("out",), device_types="cuda")
def blocksparse_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, out: torch.Tensor,
                        block: int = 64, local_blocks: int = 4, vert_stride: int = 8) -> None:
    paged_attn.blocksparse_prefill(q, k, v, scale, block=block, local_blocks=local_blocks, vert_stride=vert_stride,
                                   out=out)


# Operators that write scale tables exist in a second form (`*_fp8`): a mutated argument of a custom
# operator cannot be optional.
@torch.library.custom_op(f"{_NS}::paged_kv_write", mutates_args=("k_cache", "v_cache"), device_types="cuda")
def paged_kv_write(k_new: torch.Tensor, v_new: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   block_tables: torch.Tensor, seq_lens: torch.Tensor, query_lens: torch.Tensor) -> None:
    paged_attn.kv_write(k_new, v_new, k_cache, v_cache, block_tables, seq_lens, query_lens)


@torch.library.custom_op(f"{_NS}::paged_kv_write_fp8", mutates_args=("k_cache", "v_cache", "k_scale", "v_scale"),
                         device_types="cuda")
def paged_kv_write_fp8(k_new: torch.Tensor, v_new: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                       k_scale: torch.Tensor, v_scale: torch.Tensor, block_tables: torch.Tensor,
                       seq_lens: torch.Tensor, query_lens: torch.Tensor) -> None:
    paged_attn.kv_write(k_new, v_new, k_cache, v_cache, block_tables, seq_lens, query_lens,
                        k_scale=k_scale, v_scale=v_scale)


@torch.library.custom_op(f"{_NS}::qk_norm_rope_kv_write", mutates_args=("q_out", "k_cache", "v_cache"),
                         device_types="cuda")
def qk_norm_rope_kv_write(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, q_out: torch.Tensor,
                          k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                          seq_lens: torch.Tensor, query_lens: torch.Tensor, rope_cos: torch.Tensor,
                          rope_sin: torch.Tensor, q_norm_weight: Optional[torch.Tensor] = None,
                          k_norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6) -> None:
    paged_attn.qk_norm_rope_kv_write(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, rope_cos,
                                     rope_sin, q_norm_weight=q_norm_weight, k_norm_weight=k_norm_weight, eps=eps,
                                     out=q_out)


@torch.library.custom_op(f"{_NS}::qk_norm_rope_kv_write_fp8",
                         mutates_args=("q_out", "k_cache", "v_cache", "k_scale", "v_scale"), device_types="cuda")
def qk_norm_rope_kv_write_fp8(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, q_out: torch.Tensor,
                              k_cache: torch.Tensor, v_cache: torch.Tensor, k_scale: torch.Tensor,
                              v_scale: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                              query_lens: torch.Tensor, rope_cos: torch.Tensor, rope_sin: torch.Tensor,
                              q_norm_weight: Optional[torch.Tensor] = None,
                              k_norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6) -> None:
    paged_attn.qk_norm_rope_kv_write(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, rope_cos,
                                     rope_sin, q_norm_weight=q_norm_weight, k_norm_weight=k_norm_weight, eps=eps,
                                     k_scale=k_scale, v_scale=v_scale, out=q_out)


# K and V only: the Q half of the transform then rides on paged_decode / paged_prefill (rope_cos, rope_sin,
# q_norm_weight arguments), which saves the pass over Q
@torch.library.custom_op(f"{_NS}::k_norm_rope_kv_write", mutates_args=("k_cache", "v_cache"), device_types="cuda")
def k_norm_rope_kv_write(xk: torch.Tensor, xv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                         block_tables: torch.Tensor, seq_lens: torch.Tensor, query_lens: torch.Tensor,
                         rope_cos: torch.Tensor, rope_sin: torch.Tensor,
                         k_norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6) -> None:
    paged_attn.qk_norm_rope_kv_write(None, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, rope_cos,
                                     rope_sin, k_norm_weight=k_norm_weight, eps=eps)


@torch.library.custom_op(f"{_NS}::k_norm_rope_kv_write_fp8", mutates_args=("k_cache", "v_cache", "k_scale", "v_scale"),
                         device_types="cuda")
def k_norm_rope_kv_write_fp8(xk: torch.Tensor, xv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                             k_scale: torch.Tensor, v_scale: torch.Tensor, block_tables: torch.Tensor,
                             seq_lens: torch.Tensor, query_lens: torch.Tensor, rope_cos: torch.Tensor,
                             rope_sin: torch.Tensor, k_norm_weight: Optional[torch.Tensor] = None,
                             eps: float = 1e-6) -> None:
    paged_attn.qk_norm_rope_kv_write(None, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, rope_cos,
                                     rope_sin, k_norm_weight=k_norm_weight, eps=eps, k_scale=k_scale, v_scale=v_scale)


# the projection behind the attention call (examples/models/qwen3/kernels/attention.py:143-147; with the bias
# examples/models/gpt_oss/kernels/attention.py:155-163); the tensor-parallel all-reduce stays with the caller
@torch.library.custom_op(f"{_NS}::o_proj", mutates_args=("out",), device_types="cuda")
def o_proj(x: torch.Tensor, o_weight: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
           workspace: Optional[torch.Tensor] = None) -> None:
    paged_attn.o_proj(x, o_weight, bias, out=out, workspace=workspace)


# One decode step of a layer in one call (cache update + attention + optional projection): the decode branch of the
# reference's attention_kernel as a whole (examples/models/qwen3/kernels/attention.py:78-147).  `out` is [B, N] with
# o_weight, else [B, Hq, D].
@torch.library.custom_op(f"{_NS}::decode_step", mutates_args=("k_cache", "v_cache", "out"), device_types="cuda")
def decode_step(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                block_tables: torch.Tensor, seq_lens: torch.Tensor, query_lens: torch.Tensor, scale: float,
                out: torch.Tensor, max_seq_len: int = 0, rope_cos: Optional[torch.Tensor] = None,
                rope_sin: Optional[torch.Tensor] = None, q_norm_weight: Optional[torch.Tensor] = None,
                k_norm_weight: Optional[torch.Tensor] = None, norm_eps: float = 1e-6,
                o_weight: Optional[torch.Tensor] = None, o_bias: Optional[torch.Tensor] = None,
                sinks: Optional[torch.Tensor] = None, sliding_window: int = 0,
                workspace: Optional[torch.Tensor] = None, partition_size: int = 512) -> None:
    paged_attn.decode_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale,
                           partition_size=partition_size, max_seq_len=max_seq_len or None,
                           q_transform=_qt(rope_cos, rope_sin, q_norm_weight, norm_eps), k_norm_weight=k_norm_weight,
                           o_weight=o_weight, o_bias=o_bias, out=out, workspace=workspace, sinks=sinks,
                           sliding_window=_win(sliding_window))


@torch.library.custom_op(f"{_NS}::decode_step_fp8", mutates_args=("k_cache", "v_cache", "k_scale", "v_scale", "out"),
                         device_types="cuda")
def decode_step_fp8(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    k_scale: torch.Tensor, v_scale: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                    query_lens: torch.Tensor, scale: float, out: torch.Tensor, max_seq_len: int = 0,
                    rope_cos: Optional[torch.Tensor] = None, rope_sin: Optional[torch.Tensor] = None,
                    q_norm_weight: Optional[torch.Tensor] = None, k_norm_weight: Optional[torch.Tensor] = None,
                    norm_eps: float = 1e-6, o_weight: Optional[torch.Tensor] = None,
                    o_bias: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None,
                    sliding_window: int = 0, workspace: Optional[torch.Tensor] = None, partition_size: int = 512) -> None:
    paged_attn.decode_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, k_scale=k_scale,
                           v_scale=v_scale, partition_size=partition_size, max_seq_len=max_seq_len or None,
                           q_transform=_qt(rope_cos, rope_sin, q_norm_weight, norm_eps), k_norm_weight=k_norm_weight,
                           o_weight=o_weight, o_bias=o_bias, out=out, workspace=workspace, sinks=sinks,
                           sliding_window=_win(sliding_window))


# A speculative verify step of a layer in one call (the K + 1 tokens of examples/models/gpt_oss/peagle/speculate.py:137-202
# through examples/models/gpt_oss/kernels/attention.py:80-163): xq [B, T, Hq, D], xk / xv [B, T, Hkv, D]; `out` is
# [B, T, N] with o_weight, else [B, T, Hq, D].
@torch.library.custom_op(f"{_NS}::verify_step", mutates_args=("k_cache", "v_cache", "out"), device_types="cuda")
def verify_step(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                block_tables: torch.Tensor, seq_lens: torch.Tensor, query_lens: torch.Tensor, scale: float,
                out: torch.Tensor, max_seq_len: int = 0, rope_cos: Optional[torch.Tensor] = None,
                rope_sin: Optional[torch.Tensor] = None, q_norm_weight: Optional[torch.Tensor] = None,
                k_norm_weight: Optional[torch.Tensor] = None, norm_eps: float = 1e-6,
                o_weight: Optional[torch.Tensor] = None, o_bias: Optional[torch.Tensor] = None,
                sinks: Optional[torch.Tensor] = None, sliding_window: int = 0,
                workspace: Optional[torch.Tensor] = None) -> None:
    paged_attn.verify_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale,
                           max_seq_len=max_seq_len or None,
                           q_transform=_qt(rope_cos, rope_sin, q_norm_weight, norm_eps), k_norm_weight=k_norm_weight,
                           o_weight=o_weight, o_bias=o_bias, out=out, workspace=workspace, sinks=sinks,
                           sliding_window=_win(sliding_window))


@torch.library.custom_op(f"{_NS}::verify_step_fp8", mutates_args=("k_cache", "v_cache", "k_scale", "v_scale", "out"),
                         device_types="cuda")
def verify_step_fp8(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    k_scale: torch.Tensor, v_scale: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                    query_lens: torch.Tensor, scale: float, out: torch.Tensor, max_seq_len: int = 0,
                    rope_cos: Optional[torch.Tensor] = None, rope_sin: Optional[torch.Tensor] = None,
                    q_norm_weight: Optional[torch.Tensor] = None, k_norm_weight: Optional[torch.Tensor] = None,
                    norm_eps: float = 1e-6, o_weight: Optional[torch.Tensor] = None,
                    o_bias: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None,
                    sliding_window: int = 0, workspace: Optional[torch.Tensor] = None) -> None:
    paged_attn.verify_step(xq, xk, xv, k_cache, v_cache, block_tables, seq_lens, query_lens, scale, k_scale=k_scale,
                           v_scale=v_scale, max_seq_len=max_seq_len or None,
                           q_transform=_qt(rope_cos, rope_sin, q_norm_weight, norm_eps), k_norm_weight=k_norm_weight,
                           o_weight=o_weight, o_bias=o_bias, out=out, workspace=workspace, sinks=sinks,
                           sliding_window=_win(sliding_window))


def _no_cpu(name):
    def impl(*args, **kwargs):
        raise NotImplementedError(f"{_NS}::{name} runs hand-written HIP kernels and has no CPU path; "
                                  "pass tensors on a ROCm device")
    return impl


for _op, _name in ((paged_decode, "paged_decode"), (paged_prefill, "paged_prefill"),
                   (blocksparse_prefill, "blocksparse_prefill"), (paged_kv_write, "paged_kv_write"),
                   (paged_kv_write_fp8, "paged_kv_write_fp8"), (qk_norm_rope_kv_write, "qk_norm_rope_kv_write"),
                   (qk_norm_rope_kv_write_fp8, "qk_norm_rope_kv_write_fp8"),
                   (k_norm_rope_kv_write, "k_norm_rope_kv_write"), (k_norm_rope_kv_write_fp8, "k_norm_rope_kv_write_fp8"),
                   (o_proj, "o_proj"), (decode_step, "decode_step"), (decode_step_fp8, "decode_step_fp8"),
                   (verify_step, "verify_step"), (verify_step_fp8, "verify_step_fp8")):
    _op.register_kernel("cpu")(_no_cpu(_name))
    _op.register_fake(lambda *args, **kwargs: None)      # outputs are caller-allocated: nothing to infer

OPS = ("paged_decode", "paged_prefill", "blocksparse_prefill", "paged_kv_write", "paged_kv_write_fp8",
       "qk_norm_rope_kv_write", "qk_norm_rope_kv_write_fp8", "k_norm_rope_kv_write", "k_norm_rope_kv_write_fp8", "o_proj",
       "decode_step", "decode_step_fp8", "verify_step", "verify_step_fp8")
