"""CPU-side checks: the C-ABI library loads and exports every declared symbol, host
validation works without a GPU, and the ops refuse host arrays instead of falling back."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from nkipy_amd import _lib, build
    if not os.path.exists(build.LIB_PATH):
        build.build()
    return _lib.load()


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(ROOT, "include", "paged_attn.h")).read()
    names = set(re.findall(r"\b(pa_[a-z0-9_]+)\s*\(", header))
    assert {"pa_decode", "pa_prefill", "pa_blocksparse_prefill", "pa_gather_kv", "pa_version",
            "pa_last_error", "pa_decode_workspace_bytes"} <= names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    from nkipy_amd._lib import SIGNATURES
    assert set(SIGNATURES) == names


def test_version_and_workspace_formula(lib):
    assert lib.pa_version() >= 100
    # enough for the fixed-partition kernels: one partial per (sequence, q head, partition)
    assert lib.pa_decode_workspace_bytes(64, 32, 128, 8192, 512) >= 64 * 32 * 16 * (128 + 2) * 4
    assert lib.pa_decode_workspace_bytes(2, 4, 64, 513, 512) >= 2 * 4 * 2 * 66 * 4
    # and for the balanced schedule: one partial per (q head, sequence + chunk), 8 chunks per CU
    assert lib.pa_decode_workspace_bytes(64, 32, 128, 512, 512) >= 32 * (64 + 8 * 256) * 130 * 4
    assert lib.pa_decode_workspace_bytes(0, 32, 128, 512, 512) == 0


def test_decode_workspace_for_shape_and_noalloc_limit(lib):
    """The exact size query never exceeds the upper bound, and the entry point that uses the
    library's static scratch refuses, on the host, a call whose partials do not fit it."""
    upper = lib.pa_decode_workspace_bytes(64, 32, 128, 1 << 20, 512)
    exact = lib.pa_decode_workspace_bytes_for(64, 32, 8, 128, 32, 1 << 20, 512, 1, 1)     # bf16: balanced schedule
    assert 0 < exact <= upper and exact < 64 << 20          # no term that grows with max_seq_len
    assert lib.pa_decode_workspace_bytes_for(64, 32, 8, 128, 32, 1 << 20, 512, 0, 0) == 64 * 32 * 2048 * 130 * 4   # fp32
    # no bound (max_seq_len 0: pa_decode then uses the table capacity, unknown here): enough for the balanced schedule
    # and for the fixed partitions of a small call (up to eight of the caller's, up to sixteen of the finer ones)
    for B in (4, 128, 600):
        unbounded = lib.pa_decode_workspace_bytes_for(B, 32, 8, 128, 32, 0, 512, 1, 1)
        assert unbounded >= B * 32 * 16 * 130 * 4
        for msl in (100, 512, 2048, 1 << 20):
            assert unbounded >= lib.pa_decode_workspace_bytes_for(B, 32, 8, 128, 32, msl, 512, 1, 1)
    z = ctypes.c_void_p(0)
    rc = lib.pa_decode_noalloc(z, z, z, z, z, z, z, z, 8192, 64, 8, 128, 32, 4, 64, 0, 1.0, 512, 1, 1, z, 0, z, z)
    assert rc == -1 and b"static" in lib.pa_last_error()


def test_c_abi_argument_errors_without_gpu(lib):
    """Argument errors are found on the host before anything touches a device."""
    z = ctypes.c_void_p(0)
    def dec(**kw):
        a = dict(B=2, Hq=8, Hkv=2, D=128, bs=16, mb=4, nb=8, msl=0, scale=1.0, part=512, qd=1, kd=1)
        a.update(kw)
        return lib.pa_decode(z, z, z, z, z, z, z, z, z, 0, a["B"], a["Hq"], a["Hkv"], a["D"], a["bs"],
                             a["mb"], a["nb"], a["msl"], a["scale"], a["part"], a["qd"], a["kd"], z, a.get("win", 0), z, z)
    assert dec(Hq=7) == -1 and b"multiple" in lib.pa_last_error()
    assert dec(D=96) == -1 and b"head_dim" in lib.pa_last_error()
    assert dec(qd=0, kd=1) == -1 and b"dtype" in lib.pa_last_error()
    assert dec(part=0) == -1
    assert dec(bs=0) == -1
    assert dec() == -1 and b"null" in lib.pa_last_error()       # sizes fine, pointers null
    assert dec(B=0) == 0                                        # empty batch is a no-op
    assert lib.pa_blocksparse_prefill(z, z, z, z, 1, 64, 4, 4, 128, 32, 4, 8, 1.0, 1, z) == -1
    assert b"block must be 64" in lib.pa_last_error()
    assert lib.pa_prefill(z, z, z, z, z, z, z, z, z, 1, 4, 4, 4, 128, 16, 4, 8, 0, 1.0, 0, 1, z, 0, z, 0, z, z) == -1
    assert lib.pa_prefill(z, z, z, z, z, z, z, z, z, 1, 4, 4, 4, 128, 16, 4, 8, 0, 1.0, 1, 1, z, -1, z, 0, z, z) == -1 and b"sliding_window" in lib.pa_last_error()
    assert lib.pa_prefill(z, z, z, z, z, z, z, z, z, 1, 4, 4, 4, 128, 16, 4, 8, 0, 1.0, 1, 0, z, 0, z, 0, z, z) == -1 and b"kv_dtype" in lib.pa_last_error()
    assert lib.pa_gather_kv(z, z, z, z, 1, 2, 64, 16, 2, 8, 100, 2, z) == -1  # beyond table capacity
    def kvw(**kw):
        a = dict(B=2, T=4, Hkv=2, D=128, bs=16, mb=4, nb=8, kd=1)
        a.update(kw)
        return lib.pa_kv_write(z, z, z, z, z, z, z, z, z, a["B"], a["T"], a["Hkv"], a["D"], a["bs"], a["mb"], a["nb"], a["kd"], z)
    assert kvw(kd=3) == -1 and b"kv_dtype" in lib.pa_last_error()
    assert kvw(D=100) == -1 and b"16 bytes" in lib.pa_last_error()
    assert kvw(bs=0) == -1
    assert kvw() == -1 and b"null" in lib.pa_last_error()
    assert kvw(T=0) == 0
    def pre(**kw):
        a = dict(B=2, T=4, Hq=4, Hkv=2, D=128, bs=16, mb=4, nb=8, kd=1, mp=64)
        a.update(kw)
        return lib.pa_qk_norm_rope_kv_write(z, z, z, z, z, z, 1e-6, z, z, a["mp"], z, z, z, z, z, z, z, a["B"], a["T"],
                                            a["Hq"], a["Hkv"], a["D"], a["bs"], a["mb"], a["nb"], a["kd"], z)
    assert pre(D=96) == -1 and b"64, 128 or 256" in lib.pa_last_error()
    assert pre(kd=0) == -1 and b"kv_dtype" in lib.pa_last_error()
    assert pre(mp=0) == -1
    assert pre() == -1 and b"null" in lib.pa_last_error()
    assert pre(B=0) == 0
    def ver(**kw):
        a = dict(B=2, T=4, Hq=8, Hkv=2, D=128, bs=16, mb=4, nb=8, kd=1)
        a.update(kw)
        return lib.pa_verify(z, z, z, z, z, z, z, z, z, z, 0, a["B"], a["T"], a["Hq"], a["Hkv"], a["D"], a["bs"],
                             a["mb"], a["nb"], a.get("msl", 0), 1.0, a["kd"], z, a.get("win", 0), z, z)
    assert ver(Hq=7) == -1 and b"multiple" in lib.pa_last_error()
    assert ver(kd=0) == -1 and b"kv_dtype" in lib.pa_last_error()
    assert ver(T=65) == -1 and b"pa_prefill" in lib.pa_last_error()
    assert ver() == -1 and b"null" in lib.pa_last_error()
    assert ver(T=0) == 0
    assert ver(win=-1) == -1 and b"sliding_window" in lib.pa_last_error()
    assert dec(win=-2) == -1 and b"sliding_window" in lib.pa_last_error()
    assert lib.pa_verify_workspace_bytes(0, 4, 8, 128) == 0
    from nkipy_amd._lib import NewKvStruct, OutProjStruct
    nkv, proj = NewKvStruct(None, None, None, None), OutProjStruct(None, None, None, 256)
    def step(new_kv=ctypes.addressof(nkv), out_proj=None, **kw):
        a = dict(B=2, Hq=8, Hkv=2, D=128, bs=16, mb=4, nb=8, msl=0, scale=1.0, part=512, qd=1, kd=1)
        a.update(kw)
        return lib.pa_decode_step(z, new_kv, z, z, z, z, z, z, z, out_proj, z, 0, a["B"], a["Hq"], a["Hkv"], a["D"], a["bs"],
                                  a["mb"], a["nb"], a["msl"], a["scale"], a["part"], a["qd"], a["kd"], z, a.get("win", 0), z, z)
    assert step(Hq=7) == -1 and b"multiple" in lib.pa_last_error()
    assert step(D=96) == -1 and b"head_dim" in lib.pa_last_error()
    assert step(win=-1) == -1 and b"sliding_window" in lib.pa_last_error()
    assert step() == -1 and b"null" in lib.pa_last_error()
    assert step(B=0, new_kv=None) == -1 and b"new_kv" in lib.pa_last_error()      # the call without a cache update is pa_decode
    assert step(B=0) == 0
    # what the one call needs covers what its three parts need
    for B, msl in ((8, 1088), (1, 4096), (64, 8192)):
        need = lib.pa_decode_step_workspace_bytes(B, 32, 8, 128, 32, msl, 512, 4096, 1, 1)
        assert need >= lib.pa_decode_workspace_bytes_for(B, 32, 8, 128, 32, msl, 512, 1, 1) + lib.pa_o_proj_workspace_bytes(B, 4096, 4096) + B * 4096 * 2
    assert lib.pa_decode_step_workspace_bytes(0, 32, 8, 128, 32, 100, 512, 4096, 1, 1) == 0


def test_prefill_route_by_rows_batch_and_bound():
    """Which kernel `prefill` picks for runs of a few tokens (bf16 pools, head dim 128): up to 16 rows per kv head the
    verify kernel; 17-32 rows the tiled kernel from 8 sequences and 20 000 (sequence x bound) tokens on; beyond, the
    tiled kernel but for small calls; windows, fp8 pools and head dim 64 as before."""
    from nkipy_amd.paged_attn import prefill_route as route
    assert route(64, 4, 32, 8, 128, 32, bound=8192) == "verify"                 # 16 rows
    assert route(1, 8, 32, 8, 128, 32, bound=32768) == "verify"                  # 32 rows, one sequence
    assert route(8, 8, 32, 8, 128, 32, bound=2048) == "verify"
    assert route(8, 8, 32, 8, 128, 32, bound=4096) == "tiled"
    assert route(16, 8, 32, 8, 128, 32, bound=1024) == "verify"
    assert route(16, 4, 64, 8, 128, 32, bound=2048) == "tiled"
    assert route(16, 8, 32, 8, 128, 32) == "tiled" and route(8, 8, 32, 8, 128, 32) == "verify"      # no bound
    assert route(32, 8, 32, 8, 128, 32, window=128, bound=4096) == "verify"
    assert route(1, 16, 32, 8, 128, 32, bound=4096) == "verify"                  # 64 rows, a small call
    assert route(1, 16, 32, 8, 128, 32) == "tiled" and route(8, 16, 32, 8, 128, 32, bound=4096) == "tiled"
    assert route(4, 16, 32, 8, 128, 32, bound=1024, window=64) == "tiled"
    assert route(64, 8, 32, 8, 128, 32, fp8=True, bound=4096) == "verify"        # fp8 pools: by rows alone
    assert route(1, 32, 32, 8, 128, 32, fp8=True, bound=1024) == "verify"
    assert route(4, 65, 32, 8, 128, 32, fp8=True, bound=1024) == "tiled"
    assert route(64, 64, 64, 8, 64, 32, bound=4096) == "tiled" and route(4, 64, 64, 8, 64, 32, bound=4096) == "verify"
    assert route(4, 65, 32, 8, 128, 32, bound=512) == "tiled"                    # more tokens than the verify kernel takes


def test_ops_refuse_host_arrays():
    import nkipy_amd
    a = np.zeros((1, 1, 64), np.float32)
    with pytest.raises(NotImplementedError):
        nkipy_amd.decode(a, a, a, a, a, 1.0)
    t = torch.zeros(1, 1, 64)
    with pytest.raises(NotImplementedError):
        nkipy_amd.decode(t, t, t, t, t, 1.0)
    with pytest.raises(NotImplementedError):
        nkipy_amd.prefill(a, a, a, a, a, a, 1.0)
    with pytest.raises(NotImplementedError):
        nkipy_amd.blocksparse_prefill(a, a, a, 1.0)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from nkipy_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.PagedAttnLibraryError):
        _lib.load()


def test_workload_index_structures_are_seeded_and_consistent():
    from nkipy_amd import workloads as W
    a = W.make_decode(2, device="cpu", shrink=16)
    b = W.make_decode(2, device="cpu", shrink=16)
    assert torch.equal(a.block_tables, b.block_tables) and torch.equal(a.seq_lens, b.seq_lens)
    bt = a.block_tables.numpy()
    used = bt[bt >= 0]
    assert len(np.unique(used)) == len(used) and used.max() < a.k_cache.shape[0]
    nblk = (a.ctx + 31) // 32
    assert (bt >= 0).sum() == nblk.sum()
    assert a.k_cache.shape[0] == int(np.ceil(1.1 * nblk.sum()))
    # algorithmic bytes: K+V rows dominate
    assert a.algorithmic_bytes() > int(a.ctx.sum()) * 2 * 8 * 128 * 2
    p = W.make_prefill(device="cpu", shrink=32)
    t = p.block_tables.numpy()
    sb = int(p.prefix[0]) // 32
    assert np.all(p.prefix[:4] == p.prefix[0]) and p.prefix[0] % 32 == 0
    for b_ in (1, 2, 3):
        assert np.array_equal(t[b_, :sb], t[0, :sb])
    priv = np.concatenate([t[0][t[0] >= 0]] + [t[b_, sb:][t[b_, sb:] >= 0] for b_ in (1, 2, 3)] +
                          [t[b_][t[b_] >= 0] for b_ in range(4, 8)])
    assert len(np.unique(priv)) == len(priv)
    s = W.make_blocksparse(device="cpu", shrink=64)
    assert s.flops() > 0


def test_device_kernel_name_validation_without_gpu(lib):
    """The name-keyed call convention rejects unknown tensors before touching a device."""
    import nkipy_amd
    from nkipy_amd.runtime import DeviceKernel
    q = torch.zeros(2, 8, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 16, 2, 128, dtype=torch.bfloat16)
    bt = torch.zeros(2, 2, dtype=torch.int32)
    sl = torch.ones(2, dtype=torch.int32)
    k = DeviceKernel.compile_and_load(nkipy_amd.decode, name="dec", q=q, k_cache=kc, v_cache=kc,
                                      block_tables=bt, seq_lens=sl, scale=0.1, partition_size=256)
    assert k.static_kwargs == {"scale": 0.1, "partition_size": 256}
    good = dict(q=q, k_cache=kc, v_cache=kc, block_tables=bt, seq_lens=sl)
    with pytest.raises(ValueError):
        k(inputs=dict(good, bogus=q))
    with pytest.raises(ValueError):
        k(inputs={n: t for n, t in good.items() if n != "seq_lens"})
    with pytest.raises(ValueError):
        k(inputs=good, outputs={"output1": q})
    with pytest.raises(AssertionError):
        k(inputs=dict(good, q=q[:1]))
    with pytest.raises(AssertionError):
        k(inputs=dict(good, q=q.float()))
    with pytest.raises(ValueError):
        DeviceKernel.compile_and_load(nkipy_amd.decode, q=q, nonsense=1)
    with pytest.raises(ValueError):
        DeviceKernel.compile_and_load(print)
    with pytest.raises(NotImplementedError):      # host tensors: no CPU path behind the op
        k(inputs=good)


def test_device_kernel_alias_names_without_gpu(lib):
    """In-place state travels under the reference's aliasing names (trace.py:218-256,
    tests/unit/test_alias.py:236-349): input "k_cache.must_alias_input", output "k_cache" bound to
    the same buffer; the plain parameter name is not an input name of such a kernel."""
    import nkipy_amd
    from nkipy_amd.runtime import ALIAS_SUFFIX, DeviceKernel
    assert ALIAS_SUFFIX == ".must_alias_input"
    kn = torch.zeros(2, 3, 2, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 16, 2, 128, dtype=torch.bfloat16)
    vc = torch.zeros(4, 16, 2, 128, dtype=torch.bfloat16)
    bt = torch.zeros(2, 2, dtype=torch.int32)
    sl = torch.full((2,), 3, dtype=torch.int32)
    k = DeviceKernel.compile_and_load("kv_write", name="write", k_new=kn, v_new=kn, k_cache=kc, v_cache=vc,
                                      block_tables=bt, seq_lens=sl, query_lens=sl)
    assert k.output_names == ["k_cache", "v_cache"]          # no positional output: the op returns nothing
    assert set(k.input_names) == {"k_new", "v_new", "k_cache.must_alias_input", "v_cache.must_alias_input",
                                  "block_tables", "seq_lens", "query_lens"}
    good = {"k_new": kn, "v_new": kn, "k_cache.must_alias_input": kc, "v_cache.must_alias_input": vc,
            "block_tables": bt, "seq_lens": sl, "query_lens": sl}
    with pytest.raises(ValueError):                           # the un-suffixed name is not an input
        k(inputs={**{n: t for n, t in good.items() if n != "k_cache.must_alias_input"}, "k_cache": kc})
    with pytest.raises(ValueError):
        k(inputs=good, outputs={"output0": kc})
    with pytest.raises(AssertionError):                       # alias output bound to another buffer
        k(inputs=good, outputs={"k_cache": vc, "v_cache": vc})
    with pytest.raises(NotImplementedError):                  # names and aliases fine; host tensors have no path
        k(inputs=good, outputs={"k_cache": kc, "v_cache": vc})
    # the fused pre-attention step returns the transformed q as output0 and aliases the pool
    xq = torch.zeros(2, 3, 4, 128, dtype=torch.bfloat16)
    cs = torch.zeros(8, 64, dtype=torch.bfloat16)
    k2 = DeviceKernel.compile_and_load("qk_norm_rope_kv_write", xq=xq, xk=kn, xv=kn, k_cache=kc, v_cache=vc,
                                       block_tables=bt, seq_lens=sl, query_lens=sl, rope_cos=cs, rope_sin=cs, eps=1e-6)
    assert k2.output_names == ["output0", "k_cache", "v_cache"] and k2.static_kwargs == {"eps": 1e-6}
    k3 = DeviceKernel.compile_and_load("qk_norm_rope_kv_write", xq=None, xk=kn, xv=kn, k_cache=kc, v_cache=vc,
                                       block_tables=bt, seq_lens=sl, query_lens=sl, rope_cos=cs, rope_sin=cs)
    assert k3.output_names == ["k_cache", "v_cache"]
    with pytest.raises(ValueError):
        DeviceKernel.compile_and_load("no_such_op")


def test_device_kernel_o_proj_signature_without_gpu(lib):
    """The projection's positional output has its own shape, [..., N], checked like any other."""
    import nkipy_amd
    from nkipy_amd.runtime import DeviceKernel
    x = torch.zeros(2, 3, 4, 32, dtype=torch.bfloat16)
    w = torch.zeros(128, 48, dtype=torch.bfloat16)
    k = DeviceKernel.compile_and_load(nkipy_amd.o_proj, x=x, o_weight=w)
    assert k.output_names == ["output0"] and k._result_sig == ((2, 3, 48), torch.bfloat16)
    with pytest.raises(AssertionError):
        k(inputs={"x": x, "o_weight": w}, outputs={"output0": torch.zeros(2, 3, 128, dtype=torch.bfloat16)})
    with pytest.raises(NotImplementedError):
        k(inputs={"x": x, "o_weight": w}, outputs={"output0": torch.zeros(2, 3, 48, dtype=torch.bfloat16)})
    z = ctypes.c_void_p(0)
    assert lib.pa_o_proj(z, z, z, z, 4, 96, 64, 1, z) == -1 and b"multiple of 64" in lib.pa_last_error()
    assert lib.pa_o_proj(z, z, z, z, 4, 128, 20, 1, z) == -1 and b"multiple of 8" in lib.pa_last_error()
    assert lib.pa_o_proj(z, z, z, z, 4, 128, 64, 0, z) == -1 and b"bf16" in lib.pa_last_error()
    assert lib.pa_o_proj(z, z, z, z, 0, 128, 64, 1, z) == 0
    assert lib.pa_o_proj(z, z, z, z, 4, 128, 64, 1, z) == -1 and b"null" in lib.pa_last_error()


def test_debug_switches_are_refused_without_the_environment_variable():
    """pa_debug_set reroutes kernels for the whole process, so it only works when PA_ENABLE_DEBUG=1 was set
    before the library's first use (these tests set it); a process without it gets an argument error."""
    import subprocess
    import sys
    from nkipy_amd import build
    code = ("import ctypes, sys\n"
            f"lib = ctypes.CDLL({build.LIB_PATH!r})\n"
            "lib.pa_last_error.restype = ctypes.c_char_p\n"
            "rc = lib.pa_debug_set(0, 1)\n"
            "sys.exit(0 if rc == -1 and b'PA_ENABLE_DEBUG' in lib.pa_last_error() else 1)\n")
    env = {k: v for k, v in os.environ.items() if k != "PA_ENABLE_DEBUG"}
    assert subprocess.run([sys.executable, "-c", code], env=env).returncode == 0
    env["PA_ENABLE_DEBUG"] = "1"
    code_on = code.replace("rc == -1 and b'PA_ENABLE_DEBUG' in lib.pa_last_error()", "rc == 0 and lib.pa_debug_set(0, 0) == 0")
    assert subprocess.run([sys.executable, "-c", code_on], env=env).returncode == 0


def test_bench_probe_library_is_separate():
    """The matrix-core ceiling probe is built into a library of its own; the product library exports no
    pa_probe / pa_bench symbol."""
    from nkipy_amd import _lib, build
    if not os.path.exists(build.BENCH_LIB_PATH):
        build.build()
    probe = ctypes.CDLL(build.BENCH_LIB_PATH)
    assert hasattr(probe, "pa_bench_probe_mfma")
    lib = _lib.load()
    assert not hasattr(lib, "pa_probe_mfma") and not hasattr(lib, "pa_bench_probe_mfma")
