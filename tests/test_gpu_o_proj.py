"""GPU parity: HIP output projection (through the C ABI) vs the NumPy oracle."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import bf16_to_dev, dev_bits, dev_to_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


def _close(got, want):
    """bf16 output of a float32-accumulated dot product: one bf16 step of the result (2^-8 relative)
    plus the float32 summation-order term, which scales with the size of the terms, not of the sum."""
    scale = float(np.abs(want).max()) if want.size else 0.0
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bar = 2.0 ** -7 * np.abs(want) + 1e-5 * scale + 1e-6
    assert np.isfinite(got).all()
    assert np.all(err <= bar), f"max excess {(err - bar).max():.3e} at scale {scale:.3e}"


@pytest.mark.parametrize("M,K,N,bias", [(1, 64, 8, False), (37, 128, 72, True), (256, 4096, 256, False),
                                        (300, 512, 2880, True), (513, 1024, 520, True), (64, 4096, 4096, False),
                                        (100, 2048, 2880, True), (129, 512, 200, False), (200, 4096, 1024, True),
                                        (257, 64, 64, True)])
def test_o_proj_vs_oracle(pa, M, K, N, bias):
    rng = np.random.default_rng(M + K + N)
    x = O.round_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = O.round_to_bf16((rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32))
    b = O.round_to_bf16(rng.standard_normal(N).astype(np.float32)) if bias else None
    want = O.o_proj(x, w, b)
    print(f"o_proj M={M} K={K} N={N} bias={bias}", flush=True)
    got = pa.o_proj(bf16_to_dev(x), bf16_to_dev(w), None if b is None else bf16_to_dev(b))
    torch.cuda.synchronize()
    assert tuple(got.shape) == (M, N)
    _close(dev_to_f32(got), want)


@pytest.mark.parametrize("M,K,N,bias,force_large", [(1100, 256, 4096, True, False),   # 128 x 128 tiles, more tiles than CUs (two-stage ring)
                                                    (900, 320, 2880, False, False),    # 128 x 128 tiles, deep ring, ragged edges
                                                    (700, 320, 1032, True, False),     # the 128-row few-rows form over 6 row blocks
                                                    (700, 320, 1032, True, True),      # the same through the 256 x 256 tiles
                                                    (3900, 128, 4096, False, False)])  # enough 256 x 256 tiles by itself
def test_o_proj_tile_forms(pa, M, K, N, bias, force_large):
    """A few hundred rows take the 128-row few-rows form over several row blocks, the row counts between those and a
    device full of 256 x 256 tiles take 128 x 128 tiles; debug switch 8 sends them through the large tiles instead.
    All against the oracle."""
    from nkipy_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(M + N + int(force_large))
    x = O.round_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = O.round_to_bf16((rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32))
    b = O.round_to_bf16(rng.standard_normal(N).astype(np.float32)) if bias else None
    want = O.o_proj(x, w, b)
    print(f"o_proj tile forms M={M} K={K} N={N} bias={bias} force_large={force_large}", flush=True)
    lib.pa_debug_set(8, 1 if force_large else 0)
    try:
        got = pa.o_proj(bf16_to_dev(x), bf16_to_dev(w), None if b is None else bf16_to_dev(b))
        torch.cuda.synchronize()
    finally:
        lib.pa_debug_set(8, 0)
    _close(dev_to_f32(got), want)


@pytest.mark.parametrize("M,K,N,bias", [(4352, 4096, 4096, True),      # 256 x 256 tiles: 17 row tiles (so row tiles 8.. of an XCD's walk), 64 k-steps
                                        (1024, 4096, 4096, False),     # 128 x 128 tiles, deep ring (one workgroup per CU)
                                        (2048, 4096, 2880, True),      # 128 x 128 tiles, two-stage ring, ragged last column tile
                                        (600, 8192, 5120, True),       # the 128-row few-rows form, two workgroups per CU (K >= 5 120), ragged last row block
                                        (1024, 8192, 5120, False)])    # 128 x 128 tiles at 128 k-steps
def test_o_proj_long_k_every_row_tile(pa, M, K, N, bias):
    """The tiled forms at the projection's real depth (K = 4096: 64 steps through the ring, far more than the
    ring is deep or the loop is rotated by), rows checked in every row tile: 16 per 128 rows, at in-tile
    positions that change from block to block, against the oracle on those rows."""
    rng = np.random.default_rng(M + K + N)
    x = O.round_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = O.round_to_bf16((rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32))
    b = O.round_to_bf16(rng.standard_normal(N).astype(np.float32)) if bias else None
    rows = np.unique(np.minimum(np.arange(0, M, 8) + (np.arange((M + 7) // 8) * 5) % 8, M - 1))
    rows = np.union1d(rows, [0, M - 1])
    want = O.o_proj(x[rows], w, b)
    print(f"o_proj long K M={M} K={K} N={N} bias={bias}, {len(rows)} rows checked", flush=True)
    got = pa.o_proj(bf16_to_dev(x), bf16_to_dev(w), None if b is None else bf16_to_dev(b))
    torch.cuda.synchronize()
    assert tuple(got.shape) == (M, N)
    _close(dev_to_f32(got)[rows], want)


def test_identity_and_permutation_weights_move_bits(pa, rng):
    """Exact cases: an identity weight returns x bit for bit (which also pins the [.., Hq, D] -> [.., Hq*D]
    view), a column permutation permutes it, a zero x returns the bias in every row."""
    B, T, Hq, D = 2, 70, 4, 64
    K = Hq * D
    x = bf16_to_dev(rng.standard_normal((B, T, Hq, D)).astype(np.float32))
    eye = torch.eye(K, dtype=torch.bfloat16, device="cuda")
    got = pa.o_proj(x, eye)
    torch.cuda.synchronize()
    assert tuple(got.shape) == (B, T, K)
    assert np.array_equal(dev_bits(got), dev_bits(x).reshape(B, T, K))
    perm = torch.randperm(K, device="cuda")
    got_p = pa.o_proj(x, eye[:, perm].contiguous())          # out[:, n] = x[:, perm[n]]
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(got_p), dev_bits(x).reshape(B, T, K)[..., perm.cpu().numpy()])
    b = bf16_to_dev(rng.standard_normal(K).astype(np.float32))
    got_b = pa.o_proj(torch.zeros_like(x), eye, b)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(got_b), np.broadcast_to(dev_bits(b), (B, T, K)))


def test_fed_by_the_attention_output_and_preallocated_out(pa, rng):
    """decode -> o_proj on the device equals the oracle's decode -> o_proj; `out=` is written in place."""
    from tests.pa_testlib import make_paged
    B, Hq, Hkv, D, bs, N = 5, 8, 2, 128, 32, 264
    ctxs = [3, 200, 64, 900, 33]
    k, v, tables = make_paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    w = O.round_to_bf16((rng.standard_normal((Hq * D, N)) / np.sqrt(Hq * D)).astype(np.float32))
    i32 = lambda a: torch.from_numpy(np.asarray(a, np.int32)).cuda()  # noqa: E731
    att = pa.decode(bf16_to_dev(q), bf16_to_dev(k), bf16_to_dev(v), i32(tables), i32(ctxs), 0.09)
    out = torch.empty((B, N), dtype=torch.bfloat16, device="cuda")
    ret = pa.o_proj(att, bf16_to_dev(w), out=out)
    torch.cuda.synchronize()
    assert ret is out
    want = O.o_proj(dev_bits(att), w)                      # the projection of the device's own attention bits
    _close(dev_to_f32(out), want)
    want_all = O.o_proj(O.paged_decode(O.round_to_bf16(q), O.round_to_bf16(k), O.round_to_bf16(v), tables,
                                       np.asarray(ctxs, np.int32), 0.09, q_dtype="bf16"), w)
    assert np.abs(dev_to_f32(out) - want_all).max() <= 2e-2


@pytest.mark.parametrize("M,K,N,bias", [(1, 4096, 4096, False), (16, 4096, 4096, True), (64, 4096, 2880, True),
                                        (128, 2048, 4096, False), (33, 1088, 1024, True), (32, 4096, 2880, True),
                                        (8, 1088, 520, False), (5, 2048, 4096, True), (20, 3584, 136, True)])
def test_few_rows_split_over_k(pa, M, K, N, bias):
    """Up to 128 rows with a workspace: several workgroups per column slab take ranges of K (17 steps of 64 at
    K = 1088: ranges of 8 and 9, or of 5, 6 and 6 in the all-resident form that calls of up to 32 rows take, whose
    ranges are at most 8 steps long) and a second kernel sums their float32 partials.  Against the oracle; the same bits
    from the cached and from a caller's workspace and from call to call; without a workspace, or with one too small for
    two ranges, the call runs unsplit, as pa_o_proj does."""
    from nkipy_amd import _lib
    from nkipy_amd.paged_attn import BF16, _ptr, _stream_ptr
    lib = _lib.load()
    rng = np.random.default_rng(M + K + N)
    x = O.round_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = O.round_to_bf16((rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32))
    b = O.round_to_bf16(rng.standard_normal(N).astype(np.float32)) if bias else None
    want = O.o_proj(x, w, b)
    xd, wd, bd = bf16_to_dev(x), bf16_to_dev(w), None if b is None else bf16_to_dev(b)
    need = pa.o_proj_workspace_bytes(M, K, N)
    print(f"o_proj split M={M} K={K} N={N} bias={bias} workspace={need}", flush=True)
    assert need > 0 and need % (M * N * 4) == 0 and 2 <= need // (M * N * 4) <= 8
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")      # stale bytes (NaN patterns) must not matter
    got = pa.o_proj(xd, wd, bd, workspace=ws)
    torch.cuda.synchronize()
    _close(dev_to_f32(got), want)
    again = pa.o_proj(xd, wd, bd, workspace=torch.zeros(need + 64, dtype=torch.uint8, device="cuda"))
    default = pa.o_proj(xd, wd, bd)
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(again), dev_bits(got))
    # unsplit: the entry point without a workspace, and a workspace that holds less than two ranges
    plain = torch.empty_like(got)
    rc = lib.pa_o_proj(_ptr(xd), _ptr(wd), _ptr(bd), _ptr(plain), M, K, N, BF16, _stream_ptr(xd.device))
    assert rc == 0
    small = pa.o_proj(xd, wd, bd, workspace=ws[:2 * M * N * 4 - 16])
    torch.cuda.synchronize()
    _close(dev_to_f32(plain), want)
    assert np.array_equal(dev_bits(small), dev_bits(plain))
    assert np.array_equal(dev_bits(default), dev_bits(got))       # the operator's default: split, with its cached scratch
    # the two orders of summation agree to the last bf16 step
    assert np.abs(dev_to_f32(plain) - dev_to_f32(got)).max() <= 2.0 ** -7 * np.abs(want).max()
    assert pa.o_proj_workspace_bytes(300, K, N) == 0


def test_argument_errors(pa):
    x = torch.zeros(4, 96, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        pa.o_proj(x, torch.zeros(96, 64, dtype=torch.bfloat16, device="cuda"))        # K not a multiple of 64
    x = torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        pa.o_proj(x, torch.zeros(128, 20, dtype=torch.bfloat16, device="cuda"))       # N not a multiple of 8
    with pytest.raises(ValueError):
        pa.o_proj(x, torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda"))        # K mismatch
    with pytest.raises(ValueError):
        pa.o_proj(x.float(), torch.zeros(128, 64, dtype=torch.float32, device="cuda"))
    with pytest.raises(NotImplementedError):
        pa.o_proj(np.zeros((4, 128), np.float32), np.zeros((128, 64), np.float32))
    w = torch.zeros(1024, 256, dtype=torch.bfloat16, device="cuda")
    x = torch.zeros(4, 1024, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(pa.o_proj_workspace_bytes(4, 1024, 256) + 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError):
        pa.o_proj(x, w, workspace=ws[1:])                                             # workspace not 16-byte aligned
    with pytest.raises(ValueError):
        pa.o_proj(x, w, workspace=ws.float())                                         # not a uint8 tensor
    assert pa.o_proj_workspace_bytes(4, 100, 256) == 0 and pa.o_proj_workspace_bytes(0, 1024, 256) == 0


def test_single_q_head_layouts(pa, rng):
    """With one q head [.., 1, D] and [.., K] both fit x (K = D): `out`'s rank says which is meant — an engine
    layer of one q head per rank passes x [B, T, 1, D] and out [B, T, N] — and without `out` x is read as [.., K]."""
    B, T, D, N = 3, 5, 128, 72
    x = O.round_to_bf16(rng.standard_normal((B, T, 1, D)).astype(np.float32))
    w = O.round_to_bf16((rng.standard_normal((D, N)) / np.sqrt(D)).astype(np.float32))
    want = O.o_proj(x.reshape(B * T, D), w).reshape(B, T, N)
    xd, wd = bf16_to_dev(x), bf16_to_dev(w)
    out3 = torch.empty((B, T, N), dtype=torch.bfloat16, device="cuda")
    assert pa.o_proj(xd, wd, out=out3) is out3
    out4 = torch.empty((B, T, 1, N), dtype=torch.bfloat16, device="cuda")
    pa.o_proj(xd, wd, out=out4)
    plain = pa.o_proj(xd, wd)
    torch.cuda.synchronize()
    assert tuple(plain.shape) == (B, T, 1, N)
    _close(dev_to_f32(out3), want)
    assert np.array_equal(dev_bits(out4).reshape(B, T, N), dev_bits(out3))
    assert np.array_equal(dev_bits(plain).reshape(B, T, N), dev_bits(out3))
    with pytest.raises(ValueError):
        pa.o_proj(xd, wd, out=torch.empty((B, N), dtype=torch.bfloat16, device="cuda"))
