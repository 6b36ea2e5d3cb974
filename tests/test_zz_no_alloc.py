"""pa_decode_noalloc (the entry point for callers that cannot allocate: split-K partials in the
library's static device array) against pa_decode with a caller's workspace, through the C ABI:
identical output bits, on two calls in a row of which the second is smaller (the array keeps the
first call's partials), then a larger one again, bf16 and fp8 pools."""
import ctypes

import numpy as np
import pytest
import torch

from tests.pa_testlib import dev_bits

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _case(seed, B, Hq, Hkv, D, bs, lo, hi, fp8):
    from nkipy_amd import workloads as W
    rng = np.random.default_rng(seed)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    ctx = rng.integers(lo, hi + 1, size=B).astype(np.int64)
    nblk = (ctx + bs - 1) // bs
    pool = int(nblk.sum()) + 5
    perm = rng.permutation(pool).astype(np.int32)
    tables = np.full((B, int(nblk.max()) + 1), -1, np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    mk = lambda *s: torch.randn(s, generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)  # noqa: E731
    q, k, v = mk(B, Hq, D), mk(pool, bs, Hkv, D), mk(pool, bs, Hkv, D)
    ks = vs = None
    if fp8:
        k, ks = W.quantize_pool_fp8(k)
        v, vs = W.quantize_pool_fp8(v)
    return dict(q=q, k=k, v=v, ks=ks, vs=vs, tables=torch.from_numpy(tables).cuda(),
                lens=torch.from_numpy(ctx.astype(np.int32)).cuda(), B=B, Hq=Hq, Hkv=Hkv, D=D, bs=bs,
                mb=tables.shape[1], nb=pool, msl=int(ctx.max()), kd=2 if fp8 else 1)


def _run_both(lib, c):
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = float(np.float32(1.0) / np.float32(np.sqrt(c["D"])))
    need = lib.pa_decode_workspace_bytes_for(c["B"], c["Hq"], c["Hkv"], c["D"], c["bs"], c["msl"], 512, 1, c["kd"])
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    out_ref = torch.full_like(c["q"], 7.0)
    out_new = torch.full_like(c["q"], -7.0)
    common = (c["B"], c["Hq"], c["Hkv"], c["D"], c["bs"], c["mb"], c["nb"], c["msl"], scale, 512, 1, c["kd"],
              ctypes.c_void_p(0), 0, ctypes.c_void_p(0), stream)
    rc = lib.pa_decode(_ptr(c["q"]), _ptr(c["k"]), _ptr(c["v"]), _ptr(c["ks"]), _ptr(c["vs"]), _ptr(c["tables"]),
                       _ptr(c["lens"]), _ptr(out_ref), _ptr(ws), ws.numel(), *common)
    assert rc == 0, lib.pa_last_error()
    rc = lib.pa_decode_noalloc(_ptr(c["q"]), _ptr(c["k"]), _ptr(c["v"]), _ptr(c["ks"]), _ptr(c["vs"]), _ptr(c["tables"]),
                               _ptr(c["lens"]), _ptr(out_new), *common)
    assert rc == 0, lib.pa_last_error()
    torch.cuda.synchronize()
    assert np.isfinite(out_new.float().cpu().numpy()).all()
    assert np.array_equal(dev_bits(out_new), dev_bits(out_ref))


@pytest.mark.parametrize("fp8", [False, True])
def test_noalloc_matches_decode_two_calls_second_smaller(fp8):
    from nkipy_amd import _lib
    lib = _lib.load()
    print(f"pa_decode_noalloc fp8={fp8}: large, small, large", flush=True)
    big = _case(11, 48, 32, 8, 128, 32, 200, 6000, fp8)        # sequences span several chunks: partials + merge
    small = _case(12, 3, 32, 8, 128, 32, 1, 900, fp8)          # fewer sequences, shorter: other slots of the array
    _run_both(lib, big)
    _run_both(lib, small)
    _run_both(lib, big)


def test_noalloc_rejects_what_the_scratch_cannot_hold():
    from nkipy_amd import _lib
    lib = _lib.load()
    z = ctypes.c_void_p(0)
    # 64 q heads x (8192 sequences + 256 chunks) x 130 floats = 281 MB of partials
    rc = lib.pa_decode_noalloc(z, z, z, z, z, z, z, z, 8192, 64, 8, 128, 32, 4, 64, 0, 1.0, 512, 1, 1, z, 0, z, z)
    assert rc == -1 and b"static" in lib.pa_last_error()
