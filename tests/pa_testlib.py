"""Helpers shared by the GPU parity tests: build seeded paged inputs in NumPy,
move them to the device in their storage dtype, bring results back as float32."""
import numpy as np
import torch

from oracle import paged_attention_oracle as O


def has_gpu():
    return torch.cuda.is_available()


def bf16_to_dev(x_f32, device="cuda"):
    """float32 values -> bf16 device tensor (rounded by the oracle's codec, so the
    device sees exactly the bits the oracle reasons about)."""
    bits = O.f32_to_bf16_bits(x_f32)
    return torch.from_numpy(bits.view(np.int16).copy()).to(device).view(torch.bfloat16)


def dev_to_f32(t):
    return t.detach().float().cpu().numpy()


def dev_bits(t):
    """Raw storage bits of a device tensor as a NumPy unsigned array."""
    t = t.detach().contiguous().cpu()
    if t.element_size() == 2:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.element_size() == 1:
        return t.view(torch.uint8).numpy()
    return t.view(torch.int32).numpy().view(np.uint32)


def make_paged(rng, B, Hkv, D, bs, ctxs, extra_blocks=3, table_pad=2, pad_value=-1):
    """Random pool + disjoint block tables for the given context lengths (NumPy, float32)."""
    ctxs = np.asarray(ctxs, dtype=np.int64)
    nblk = (ctxs + bs - 1) // bs
    total = int(nblk.sum()) + extra_blocks
    perm = rng.permutation(total).astype(np.int32)
    width = max(int(nblk.max()), 1) + table_pad
    tables = np.full((B, width), pad_value, dtype=np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    k = rng.standard_normal((total, bs, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((total, bs, Hkv, D)).astype(np.float32)
    return k, v, tables


def err_stats(got, want):
    d = np.abs(got.astype(np.float64) - want.astype(np.float64))
    return float(d.max()) if d.size else 0.0


def assert_close_fp32(got, want, rel=1e-5):
    """fp32 bar: error relative to the largest magnitude of the reference result
    (a softmax-weighted average of O(1) values; elementwise relative error is
    meaningless where an output crosses zero)."""
    ref = max(float(np.abs(want).max()), 1e-30)
    e = err_stats(got, want)
    assert e <= rel * ref, f"max abs err {e:.3e} > {rel} * {ref:.3e}"


def assert_close_abs(got, want, tol):
    e = err_stats(got, want)
    assert np.isfinite(got).all(), "non-finite values in the device result"
    assert e <= tol, f"max abs err {e:.3e} > {tol}"
