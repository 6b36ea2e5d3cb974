"""Golden fixtures (float64 brute-force expectations, see tests/golden/make_golden.py):
the oracle is checked against them on the CPU, the HIP ops on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "paged_attention_golden.npz"))


def _bf16_close(got, exp64, extra=0.0):
    """got holds bf16-rounded values: within one bf16 rounding step of the exact answer."""
    tol = np.abs(exp64) * 2.0 ** -8 + 1e-6 + extra
    assert np.all(np.abs(got - exp64) <= tol), float(np.max(np.abs(got - exp64) - tol))


# ------------------------------------------------------------------------- oracle (CPU)
def test_oracle_decode_fp32_golden():
    got = O.paged_decode(G["dec32_q"], G["dec32_k"], G["dec32_v"], G["dec32_tables"], G["dec32_ctx"],
                         float(G["dec32_scale"]))
    exp = G["dec32_expected"]
    assert np.max(np.abs(got - exp)) <= 1e-5 * np.max(np.abs(exp))


def test_oracle_decode_bf16_golden():
    got = O.paged_decode(G["dec16_q"], G["dec16_k"], G["dec16_v"], G["dec16_tables"], G["dec16_ctx"],
                         float(G["dec16_scale"]), q_dtype="bf16")
    _bf16_close(got, G["dec16_expected"])


def test_oracle_decode_fp8_golden():
    got = O.paged_decode(G["dec8_q"], G["dec8_k"], G["dec8_v"], G["dec8_tables"], G["dec8_ctx"],
                         float(G["dec8_scale"]), k_scale=G["dec8_kscale"], v_scale=G["dec8_vscale"], q_dtype="bf16")
    _bf16_close(got, G["dec8_expected"])


def test_oracle_prefill_golden():
    got = O.paged_prefill(G["pre_q"], G["pre_k"], G["pre_v"], G["pre_tables"], G["pre_ctx"], G["pre_qlens"],
                          float(G["pre_scale"]))
    _bf16_close(got, G["pre_expected"])


def test_oracle_blocksparse_golden():
    got = O.blocksparse_prefill(G["bsp_q"], G["bsp_k"], G["bsp_v"], float(G["bsp_scale"]), block=64,
                                local_blocks=int(G["bsp_local"]), vert_stride=int(G["bsp_stride"]))
    _bf16_close(got, G["bsp_expected"])


def test_oracle_window_and_sinks_golden():
    got = O.paged_prefill(G["ver_q"], G["ver_k"], G["ver_v"], G["ver_tables"], G["ver_ctx"], G["ver_qlens"],
                          float(G["ver_scale"]), sliding_window=int(G["ver_window"]), sinks=G["ver_sinks"])
    _bf16_close(got, G["ver_expected"])
    got = O.paged_decode(G["win8_q"], G["win8_k"], G["win8_v"], G["win8_tables"], G["win8_ctx"], float(G["win8_scale"]),
                         k_scale=G["win8_kscale"], v_scale=G["win8_vscale"], q_dtype="bf16",
                         sliding_window=int(G["win8_window"]), sinks=G["win8_sinks"])
    _bf16_close(got, G["win8_expected"])


# ------------------------------------------------------------------------- HIP ops (GPU)
def _bf(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16)


def _i32(x):
    return torch.from_numpy(np.asarray(x, np.int32)).cuda()


def test_oracle_long_head_dim_64_chunk_golden():
    got = O.paged_prefill(G["long64_q"], G["long64_k"], G["long64_v"], G["long64_tables"], G["long64_ctx"], G["long64_qlens"],
                          float(G["long64_scale"]), sliding_window=int(G["long64_window"]), sinks=G["long64_sinks"])
    _bf16_close(got, G["long64_expected"])


@pytest.mark.gpu
def test_hip_decode_fp32_golden():
    import nkipy_amd as pa
    got = pa.decode(torch.from_numpy(G["dec32_q"]).cuda(), torch.from_numpy(G["dec32_k"]).cuda(),
                    torch.from_numpy(G["dec32_v"]).cuda(), _i32(G["dec32_tables"]), _i32(G["dec32_ctx"]),
                    float(G["dec32_scale"]), partition_size=16).cpu().numpy()
    exp = G["dec32_expected"]
    assert np.max(np.abs(got - exp)) <= 1e-5 * np.max(np.abs(exp))


@pytest.mark.gpu
@pytest.mark.parametrize("impl", [0, 2, 1])
def test_hip_decode_bf16_and_fp8_golden(impl):
    import nkipy_amd as pa
    from nkipy_amd import _lib
    _lib.load().pa_debug_set(0, impl)
    try:
        got = pa.decode(_bf(G["dec16_q"]), _bf(G["dec16_k"]), _bf(G["dec16_v"]), _i32(G["dec16_tables"]),
                        _i32(G["dec16_ctx"]), float(G["dec16_scale"]), partition_size=32).float().cpu().numpy()
        assert np.max(np.abs(got - G["dec16_expected"])) <= 2e-2
        got8 = pa.decode(_bf(G["dec8_q"]), torch.from_numpy(G["dec8_k"]).cuda().view(torch.float8_e4m3fn),
                         torch.from_numpy(G["dec8_v"]).cuda().view(torch.float8_e4m3fn), _i32(G["dec8_tables"]),
                         _i32(G["dec8_ctx"]), float(G["dec8_scale"]), k_scale=torch.from_numpy(G["dec8_kscale"]).cuda(),
                         v_scale=torch.from_numpy(G["dec8_vscale"]).cuda(), partition_size=64).float().cpu().numpy()
        assert np.max(np.abs(got8 - G["dec8_expected"])) <= 5e-2
    finally:
        _lib.load().pa_debug_set(0, 0)


@pytest.mark.gpu
def test_hip_prefill_and_blocksparse_golden():
    import nkipy_amd as pa
    got = pa.prefill(_bf(G["pre_q"]), _bf(G["pre_k"]), _bf(G["pre_v"]), _i32(G["pre_tables"]), _i32(G["pre_ctx"]),
                     _i32(G["pre_qlens"]), float(G["pre_scale"])).float().cpu().numpy()
    assert np.max(np.abs(got - G["pre_expected"])) <= 2e-2
    got = pa.blocksparse_prefill(_bf(G["bsp_q"]), _bf(G["bsp_k"]), _bf(G["bsp_v"]), float(G["bsp_scale"]),
                                 block=64, local_blocks=int(G["bsp_local"]), vert_stride=int(G["bsp_stride"]))
    assert np.max(np.abs(got.float().cpu().numpy() - G["bsp_expected"])) <= 2e-2


@pytest.mark.gpu
@pytest.mark.parametrize("route", ["verify", None])
def test_hip_window_and_sinks_golden(route):
    import nkipy_amd as pa
    got = pa.prefill(_bf(G["ver_q"]), _bf(G["ver_k"]), _bf(G["ver_v"]), _i32(G["ver_tables"]), _i32(G["ver_ctx"]),
                     _i32(G["ver_qlens"]), float(G["ver_scale"]), sliding_window=int(G["ver_window"]),
                     sinks=torch.from_numpy(G["ver_sinks"]).cuda(), route=route).float().cpu().numpy()
    assert np.max(np.abs(got - G["ver_expected"])) <= 2e-2
    got8 = pa.decode(_bf(G["win8_q"]), torch.from_numpy(G["win8_k"]).cuda().view(torch.float8_e4m3fn),
                     torch.from_numpy(G["win8_v"]).cuda().view(torch.float8_e4m3fn), _i32(G["win8_tables"]),
                     _i32(G["win8_ctx"]), float(G["win8_scale"]), k_scale=torch.from_numpy(G["win8_kscale"]).cuda(),
                     v_scale=torch.from_numpy(G["win8_vscale"]).cuda(), sliding_window=int(G["win8_window"]),
                     sinks=torch.from_numpy(G["win8_sinks"]).cuda()).float().cpu().numpy()
    assert np.max(np.abs(got8 - G["win8_expected"])) <= 5e-2


@pytest.mark.gpu
@pytest.mark.parametrize("path", ["tiled", "chunks"])
def test_hip_long_head_dim_64_chunk_golden(path):
    """100 query tokens at head dim 64: the tiled kernel's two-heads-per-row form, and the verify kernel's
    64-token launches (tiled kernel switched off)."""
    import nkipy_amd as pa
    from nkipy_amd import _lib
    lib = _lib.load()
    lib.pa_debug_set(3, 1 if path == "chunks" else 0)
    try:
        got = pa.prefill(_bf(G["long64_q"]), _bf(G["long64_k"]), _bf(G["long64_v"]), _i32(G["long64_tables"]),
                         _i32(G["long64_ctx"]), _i32(G["long64_qlens"]), float(G["long64_scale"]),
                         sliding_window=int(G["long64_window"]), sinks=torch.from_numpy(G["long64_sinks"]).cuda()).float().cpu().numpy()
    finally:
        lib.pa_debug_set(3, 0)
    assert np.max(np.abs(got - G["long64_expected"])) <= 2e-2
    assert np.all(got[1, 70:] == 0)
