"""Name-keyed call convention of the reference's runtime, over the HIP ops.

The reference runs a kernel as
    k = DeviceKernel.compile_and_load(fn, name=..., **example_args)
    k(inputs={param_name: DeviceTensor}, outputs={"output0": DeviceTensor})
(nkipy/src/nkipy/runtime/device_kernel.py:52-193, spike/src/spike/spike_model.py:248-288):
the caller allocates inputs and outputs, tensors are addressed by parameter name,
unknown names raise ValueError and shape / dtype mismatches AssertionError
(spike_model.py:198-246).  This module keeps that convention for the paged attention
ops; there is nothing to trace or compile, so "compile_and_load" only loads the native
library and records the I/O signature from the example arguments.

State that a kernel updates in place follows the reference's aliasing names
(nkipy/src/nkipy/core/trace.py:218-256, pinned by tests/unit/test_alias.py:236-349, used at
examples/models/qwen3/qwen3.py:289-301): the mutated parameter `k_cache` is passed as input
"k_cache.must_alias_input" and comes back as output "k_cache", bound to the same buffer;
outputs that are not aliases are "output0", "output1", ... by position.
"""
from __future__ import annotations

import inspect

import numpy as np
import torch

from . import _lib, paged_attn

_TENSOR_PARAMS = {"x", "o_weight", "bias", "q", "k_cache", "v_cache", "block_tables", "seq_lens", "query_lens", "k", "v",
                  "k_scale", "v_scale", "k_new", "v_new", "xq", "xk", "xv", "rope_cos", "rope_sin",
                  "q_norm_weight", "k_norm_weight", "sinks"}
ALIAS_SUFFIX = ".must_alias_input"      # nkipy/src/nkipy/core/trace.py:222
# parameters an op writes in place (when given): they travel under the aliasing names
_MUTATED = {"kv_write": ("k_cache", "v_cache", "k_scale", "v_scale"),
            "qk_norm_rope_kv_write": ("k_cache", "v_cache", "k_scale", "v_scale")}


class DeviceTensor:
    """A named-dtype view of device memory (nkipy/src/nkipy/runtime/device_tensor.py:51-74)."""

    def __init__(self, tensor: torch.Tensor):
        self.tensor = tensor

    @classmethod
    def from_torch(cls, t: torch.Tensor, device="cuda") -> "DeviceTensor":
        return cls(t.to(device).contiguous())

    @classmethod
    def from_numpy(cls, a: np.ndarray, dtype: str | None = None, device="cuda") -> "DeviceTensor":
        """uint16 arrays tagged "bf16" are bf16 bit patterns, uint8 arrays tagged "fp8" e4m3fn codes."""
        t = torch.from_numpy(np.ascontiguousarray(a))
        if dtype == "bf16":
            assert a.dtype == np.uint16, "bf16 host data is passed as uint16 bit patterns"
            t = torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)
        elif dtype == "fp8":
            assert a.dtype == np.uint8, "fp8 host data is passed as uint8 codes"
            t = t.view(torch.float8_e4m3fn)
        return cls(t.to(device))

    @property
    def shape(self):
        return tuple(self.tensor.shape)

    @property
    def dtype(self):
        return self.tensor.dtype

    def torch(self) -> torch.Tensor:
        return self.tensor

    def numpy(self) -> np.ndarray:
        t = self.tensor.detach().cpu()
        if t.dtype == torch.bfloat16:
            return t.view(torch.int16).numpy().view(np.uint16)
        if t.dtype == torch.float8_e4m3fn:
            return t.view(torch.uint8).numpy()
        return t.numpy()


class DeviceKernel:
    """A loaded paged attention op with a fixed I/O signature."""

    _OPS = {"decode": paged_attn.decode, "prefill": paged_attn.prefill,
            "blocksparse_prefill": paged_attn.blocksparse_prefill,
            "kv_write": paged_attn.kv_write, "qk_norm_rope_kv_write": paged_attn.qk_norm_rope_kv_write,
            "o_proj": paged_attn.o_proj}

    def __init__(self, fn, name, signature, static_kwargs):
        self.fn, self.name = fn, name
        self.signature = signature          # param name -> (shape, dtype)
        self.static_kwargs = static_kwargs
        # in-place state: parameter names this op mutates and that the caller passed
        self.aliased = [k for k in _MUTATED.get(fn.__name__, ()) if k in signature]
        # what the op returns by position ("output0"): the attention result, the transformed q, or nothing
        if fn is paged_attn.kv_write or (fn is paged_attn.qk_norm_rope_kv_write and "xq" not in signature):
            self._result_like = None
        else:
            self._result_like = "xq" if fn is paged_attn.qk_norm_rope_kv_write else "q"
        # shape and dtype of "output0"
        self._result_sig = self.signature.get(self._result_like) if self._result_like else None
        if fn is paged_attn.o_proj and "x" in signature and "o_weight" in signature:
            (xs, xd), (ws, _) = signature["x"], signature["o_weight"]
            lead = xs[:-1] if xs[-1] == ws[0] else xs[:-2]          # x is [..., K] or [..., Hq, D]
            self._result_like, self._result_sig = "x", (tuple(lead) + (ws[1],), xd)
        self.output_names = (["output0"] if self._result_like else []) + list(self.aliased)
        # names the caller uses for inputs: mutated parameters carry the alias suffix
        self.input_names = {(k + ALIAS_SUFFIX if k in self.aliased else k): k for k in signature}

    @classmethod
    def compile_and_load(cls, fn, name: str | None = None, **example_args) -> "DeviceKernel":
        """fn: one of nkipy_amd.decode / prefill / blocksparse_prefill / kv_write /
        qk_norm_rope_kv_write (or its name).  Tensor arguments (DeviceTensor or torch tensor), given
        under the op's parameter names, fix the expected shapes and dtypes; every other keyword
        (scale, partition_size, ...) becomes a static argument of the kernel."""
        if isinstance(fn, str):
            if fn not in cls._OPS:
                raise ValueError(f"{fn!r} is not a paged attention op; known: {sorted(cls._OPS)}")
            fn = cls._OPS[fn]
        if fn not in cls._OPS.values():
            raise ValueError(f"{getattr(fn, '__name__', fn)!r} is not a paged attention op")
        _lib.load()
        params = inspect.signature(fn).parameters
        signature, static = {}, {}
        for k, v in example_args.items():
            if k not in params:
                raise ValueError(f"{fn.__name__} has no parameter {k!r}")
            if k in _TENSOR_PARAMS and v is not None:
                t = v.tensor if isinstance(v, DeviceTensor) else v
                signature[k] = (tuple(t.shape), t.dtype)
            else:
                static[k] = v
        return cls(fn, name or fn.__name__, signature, static)

    def __call__(self, inputs: dict, outputs: dict | None = None):
        unknown = [k for k in inputs if k not in self.input_names]
        if unknown:
            raise ValueError(f"kernel {self.name!r}: unknown input name(s) {unknown}; expected {sorted(self.input_names)}")
        missing = [k for k in self.input_names if k not in inputs]
        if missing:
            raise ValueError(f"kernel {self.name!r}: missing input(s) {missing}")
        if outputs is not None:
            bad = [k for k in outputs if k not in self.output_names]
            if bad:
                raise ValueError(f"kernel {self.name!r}: unknown output name(s) {bad}; expected {self.output_names}")
        args = {}
        for name, v in inputs.items():
            k = self.input_names[name]
            t = v.tensor if isinstance(v, DeviceTensor) else v
            shape, dtype = self.signature[k]
            assert tuple(t.shape) == shape, f"input {name!r}: shape {tuple(t.shape)} != {shape}"
            assert t.dtype == dtype, f"input {name!r}: dtype {t.dtype} != {dtype}"
            args[k] = t
        out = None
        if outputs is not None:
            for k in self.aliased:          # an alias output is the buffer that came in under the alias name
                if k in outputs:
                    o = outputs[k]
                    o = o.tensor if isinstance(o, DeviceTensor) else o
                    assert o.data_ptr() == args[k].data_ptr() and tuple(o.shape) == tuple(args[k].shape), \
                        f"output {k!r} must be the buffer passed as input {k + ALIAS_SUFFIX!r}"
            if "output0" in outputs:
                o = outputs["output0"]
                out = o.tensor if isinstance(o, DeviceTensor) else o
                qshape, qdtype = self._result_sig
                assert tuple(out.shape) == qshape and out.dtype == qdtype, \
                    f"output0 must be {qdtype} {qshape}"
        if self._result_like is None:
            self.fn(**args, **self.static_kwargs)
            res = None
        else:
            res = self.fn(**args, **self.static_kwargs, out=out)
        if outputs is None:
            ret = ([DeviceTensor(res)] if self._result_like else []) + [DeviceTensor(args[k]) for k in self.aliased]
            return ret[0] if len(ret) == 1 else (tuple(ret) if ret else None)
        return None
