"""GPU parity: HIP paged KV write (through the C ABI) vs the NumPy oracle, bit for bit."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, bf16_to_dev, dev_bits, dev_to_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pa():
    import nkipy_amd
    from nkipy_amd import _lib
    _lib.load()
    return nkipy_amd


def _i32(a):
    return torch.from_numpy(np.asarray(a, np.int32)).cuda()


def _case(rng, B, T, Hkv, D, bs, seqs, qlens, extra=2):
    seqs, qlens = np.asarray(seqs, np.int32), np.asarray(qlens, np.int32)
    nblk = (np.maximum(seqs, 1) + bs - 1) // bs
    nb = int(nblk.sum()) + extra
    perm = rng.permutation(nb).astype(np.int32)
    tables = np.full((B, int(nblk.max()) + 1), -1, np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    xk = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32) * rng.uniform(0.1, 8.0, size=(B, T, Hkv, 1)).astype(np.float32))
    xv = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    return nb, tables, seqs, qlens, xk, xv


@pytest.mark.parametrize("bs,D", [(16, 128), (32, 64), (48, 128), (64, 256), (16, 80), (32, 96), (16, 8)])
def test_bf16_pool_rows_bit_exact(pa, rng, bs, D):
    B, T, Hkv = 3, 40, 2
    nb, tables, seqs, qlens, xk, xv = _case(rng, B, T, Hkv, D, bs, seqs=[40, 97, 5], qlens=[40, 33, 0])
    pk = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    pv = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    dk = torch.from_numpy(pk.view(np.int16).copy()).cuda().view(torch.bfloat16)
    dv = torch.from_numpy(pv.view(np.int16).copy()).cuda().view(torch.bfloat16)
    pa.kv_write(bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, _i32(tables), _i32(seqs), _i32(qlens))
    O.kv_write(O.f32_to_bf16_bits(xk), O.f32_to_bf16_bits(xv), pk, pv, tables, seqs, qlens)
    assert np.array_equal(dev_bits(dk), pk) and np.array_equal(dev_bits(dv), pv)


def test_fp32_pool_rows_bit_exact(pa, rng):
    B, T, Hkv, D, bs = 2, 9, 3, 64, 16
    nb, tables, seqs, qlens, xk, xv = _case(rng, B, T, Hkv, D, bs, seqs=[20, 9], qlens=[9, 9])
    pk = rng.standard_normal((nb, bs, Hkv, D)).astype(np.float32)
    pv = rng.standard_normal((nb, bs, Hkv, D)).astype(np.float32)
    dk, dv = torch.from_numpy(pk.copy()).cuda(), torch.from_numpy(pv.copy()).cuda()
    pa.kv_write(torch.from_numpy(xk).cuda(), torch.from_numpy(xv).cuda(), dk, dv, _i32(tables), _i32(seqs), _i32(qlens))
    O.kv_write(xk, xv, pk, pv, tables, seqs, qlens)
    assert np.array_equal(dk.cpu().numpy(), pk) and np.array_equal(dv.cpu().numpy(), pv)


def _fp8_state(rng, nb, bs, Hkv, D):
    pk = rng.integers(0, 256, size=(nb, bs, Hkv, D), dtype=np.uint8)
    pk[(pk & 0x7f) == 0x7f] = 0x3a              # no NaN codes in the stale pool: a recode of NaN is not defined
    pv = pk[::-1].copy()
    ks = rng.uniform(1e-3, 0.05, size=(nb, Hkv)).astype(np.float32)
    vs = rng.uniform(1e-3, 0.05, size=(nb, Hkv)).astype(np.float32)
    return pk, pv, ks, vs


def _to_fp8_dev(codes):
    return torch.from_numpy(codes.copy()).cuda().view(torch.float8_e4m3fn)


@pytest.mark.parametrize("bs,D", [(16, 128), (64, 128), (32, 64), (16, 80), (32, 160), (64, 256)])
def test_fp8_pool_codes_and_scales_bit_exact(pa, rng, bs, D):
    """Chunks that start inside a block (stale scale kept or raised, earlier rows recoded),
    whole fresh blocks, single tokens, an empty and an all-zero chunk."""
    B, T, Hkv = 5, 70, 2
    nb, tables, seqs, qlens, xk, xv = _case(rng, B, T, Hkv, D, bs, seqs=[70, 133, 41, 9, 64], qlens=[70, 50, 1, 0, 64])
    xk[4] = 0.0                                                       # all-zero new rows into fresh blocks
    xk[1, :, 1] *= 1e-3                                               # head 1 of sequence 1 stays under the stale scale
    pk, pv, ks, vs = _fp8_state(rng, nb, bs, Hkv, D)
    dk, dv = _to_fp8_dev(pk), _to_fp8_dev(pv)
    dks, dvs = torch.from_numpy(ks.copy()).cuda(), torch.from_numpy(vs.copy()).cuda()
    pa.kv_write(bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, _i32(tables), _i32(seqs), _i32(qlens), k_scale=dks, v_scale=dvs)
    O.kv_write(O.f32_to_bf16_bits(xk), O.f32_to_bf16_bits(xv), pk, pv, tables, seqs, qlens, k_scale=ks, v_scale=vs)
    assert np.array_equal(dks.cpu().numpy(), ks) and np.array_equal(dvs.cpu().numpy(), vs)
    assert np.array_equal(dev_bits(dk), pk)
    assert np.array_equal(dev_bits(dv), pv)


def test_fp8_extreme_values_saturate_like_the_oracle(pa, rng):
    B, T, Hkv, D, bs = 1, 8, 1, 128, 16
    nb, tables, seqs, qlens, xk, xv = _case(rng, B, T, Hkv, D, bs, seqs=[12], qlens=[8])
    xk[0, 0, 0, :8] = [3.0e38, -3.0e38, 1e-30, -1e-30, 0.0, -0.0, 448.0, -448.0]
    xk = O.round_to_bf16(xk)
    pk, pv, ks, vs = _fp8_state(rng, nb, bs, Hkv, D)
    ks[:] = 1.0                                    # old rows (4 of them) decode to values a huge new scale flushes
    dk, dv = _to_fp8_dev(pk), _to_fp8_dev(pv)
    dks, dvs = torch.from_numpy(ks.copy()).cuda(), torch.from_numpy(vs.copy()).cuda()
    pa.kv_write(bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, _i32(tables), _i32(seqs), _i32(qlens), k_scale=dks, v_scale=dvs)
    O.kv_write(O.f32_to_bf16_bits(xk), O.f32_to_bf16_bits(xv), pk, pv, tables, seqs, qlens, k_scale=ks, v_scale=vs)
    assert np.array_equal(dks.cpu().numpy(), ks)
    assert np.array_equal(dev_bits(dk), pk) and np.array_equal(dev_bits(dv), pv)


@pytest.mark.parametrize("scale_bits,why", [
    (0x3cffffff, "mantissa all ones: the reciprocal form would turn x = 2^-15 into a tie and round it to code 0"),
    (0x3cfffffe, "its neighbour, which the reciprocal form takes"),
    (0x2b000000, "2^-41, below the range the reciprocal form is used in"),
    (0x2b800000, "2^-40, its lower end"),
    (0x53800000, "2^40, its upper end"),
    (0x54000000, "2^41, above it"),
])
def test_fp8_quotient_at_the_edges_of_the_reciprocal_form(pa, rng, scale_bits, why):
    """The encode forms x / scale from a refined reciprocal where that is proven to give the division's bits and
    divides elsewhere.  A block that already holds tokens under a stale scale larger than the new rows need keeps
    that scale, so any float32 can be made the divisor: the edges of the proven range, and the one mantissa it
    excludes together with the value that tells the two forms apart."""
    B, T, Hkv, D, bs = 1, 8, 1, 128, 16
    nb, tables, seqs, qlens, xk, xv = _case(rng, B, T, Hkv, D, bs, seqs=[12], qlens=[8])    # 4 earlier rows in block 0
    s = np.array([scale_bits], np.uint32).view(np.float32)[0]
    mags = np.float32(2.0) ** rng.integers(-14, 9, size=xk.shape).astype(np.float32)           # quotients 2^-14 .. 2^8
    xk = (rng.standard_normal(xk.shape).astype(np.float32) * mags * s).astype(np.float32)
    xk[0, 0, 0, :6] = np.array([2.0 ** -10, -2.0 ** -10, 3 * 2.0 ** -10, 447.0, 2.0 ** -9, 0.0], np.float32) * s
    xk[0, 1, 0, :2] = [-0.0, 0.0]
    xk = O.round_to_bf16(np.clip(xk, -400 * s, 400 * s).astype(np.float32))                    # stay under the stale scale
    xv = xk[:, ::-1].copy()
    pk, pv, ks, vs = _fp8_state(rng, nb, bs, Hkv, D)
    ks[:] = s
    vs[:] = s
    dk, dv = _to_fp8_dev(pk), _to_fp8_dev(pv)
    dks, dvs = torch.from_numpy(ks.copy()).cuda(), torch.from_numpy(vs.copy()).cuda()
    print(f"scale {s!r} ({why})", flush=True)
    pa.kv_write(bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, _i32(tables), _i32(seqs), _i32(qlens), k_scale=dks, v_scale=dvs)
    O.kv_write(O.f32_to_bf16_bits(xk), O.f32_to_bf16_bits(xv), pk, pv, tables, seqs, qlens, k_scale=ks, v_scale=vs)
    assert np.array_equal(dks.cpu().numpy(), ks) and np.all(ks[tables[0, 0]] == s)              # the stale scale stayed
    assert np.array_equal(dev_bits(dk), pk) and np.array_equal(dev_bits(dv), pv)


def test_token_by_token_append_then_decode_attention(pa, rng):
    """A serving loop in miniature: prefill write, then single-token writes, each followed by the
    decode attention over the fp8 pool; pool, scales and attention output follow the oracle."""
    B, Hq, Hkv, D, bs = 2, 8, 2, 128, 16
    prompt, steps = [21, 34], 5
    nblk = [(p + steps + bs - 1) // bs for p in prompt]
    nb = sum(nblk) + 1
    perm = rng.permutation(nb).astype(np.int32)
    tables = np.full((B, max(nblk)), -1, np.int32)
    tables[0, :nblk[0]] = perm[:nblk[0]]
    tables[1, :nblk[1]] = perm[nblk[0]:nblk[0] + nblk[1]]
    pk = np.zeros((nb, bs, Hkv, D), np.uint8); pv = np.zeros_like(pk)
    ks = np.zeros((nb, Hkv), np.float32); vs = np.zeros_like(ks)
    dk, dv = _to_fp8_dev(pk), _to_fp8_dev(pv)
    dks, dvs = torch.from_numpy(ks.copy()).cuda(), torch.from_numpy(vs.copy()).cuda()
    dt = _i32(tables)
    T = max(prompt)
    xk = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    xv = O.round_to_bf16(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    seq = np.asarray(prompt, np.int32)
    pa.kv_write(bf16_to_dev(xk), bf16_to_dev(xv), dk, dv, dt, _i32(seq), _i32(seq), k_scale=dks, v_scale=dvs)
    O.kv_write(O.f32_to_bf16_bits(xk), O.f32_to_bf16_bits(xv), pk, pv, tables, seq, seq, k_scale=ks, v_scale=vs)
    scale = float(np.float32(1.0) / np.float32(np.sqrt(D)))
    one = np.ones(B, np.int32)
    for s in range(steps):
        seq = seq + 1
        nk = O.round_to_bf16(rng.standard_normal((B, 1, Hkv, D)).astype(np.float32) * (1.0 + s))
        nv = O.round_to_bf16(rng.standard_normal((B, 1, Hkv, D)).astype(np.float32))
        q = O.round_to_bf16(rng.standard_normal((B, Hq, D)).astype(np.float32))
        pa.kv_write(bf16_to_dev(nk), bf16_to_dev(nv), dk, dv, dt, _i32(seq), _i32(one), k_scale=dks, v_scale=dvs)
        O.kv_write(O.f32_to_bf16_bits(nk), O.f32_to_bf16_bits(nv), pk, pv, tables, seq, one, k_scale=ks, v_scale=vs)
        assert np.array_equal(dev_bits(dk), pk) and np.array_equal(dks.cpu().numpy(), ks)
        assert np.array_equal(dev_bits(dv), pv) and np.array_equal(dvs.cpu().numpy(), vs)
        got = pa.decode(bf16_to_dev(q), dk, dv, dt, _i32(seq), scale, k_scale=dks, v_scale=dvs)
        want = O.paged_decode(q, pk, pv, tables, seq, scale, k_scale=ks, v_scale=vs, q_dtype="bf16")
        assert_close_abs(dev_to_f32(got), want, 5e-2)


def test_bad_lengths_and_table_entries_write_nothing(pa, rng):
    B, T, Hkv, D, bs = 3, 4, 1, 128, 16
    nb = 4
    pk = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    dk = torch.from_numpy(pk.view(np.int16).copy()).cuda().view(torch.bfloat16)
    dv = dk.clone()
    x = bf16_to_dev(rng.standard_normal((B, T, Hkv, D)).astype(np.float32))
    tables = np.array([[0, 1], [7, -3], [2, 3]], np.int32)         # sequence 1: entries outside the pool
    seqs, qlens = np.array([2, 4, 4], np.int32), np.array([4, 4, 0], np.int32)   # sequence 0: more new tokens than context
    pa.kv_write(x, x, dk, dv, _i32(tables), _i32(seqs), _i32(qlens))
    torch.cuda.synchronize()
    assert np.array_equal(dev_bits(dk), pk) and np.array_equal(dev_bits(dv), pk)


def test_argument_validation(pa):
    z = torch.zeros((1, 2, 1, 128), dtype=torch.bfloat16, device="cuda")
    pool = torch.zeros((2, 16, 1, 128), dtype=torch.bfloat16, device="cuda")
    t, one = _i32([[0, 1]]), _i32([2])
    with pytest.raises(ValueError):
        pa.kv_write(z, z, pool, pool.view(torch.int16), t, one, one)
    with pytest.raises(ValueError):
        pa.kv_write(z.float(), z.float(), pool, pool, t, one, one)
    with pytest.raises(ValueError):
        pa.kv_write(z, z, pool.view(torch.uint8)[..., :128].contiguous().view(torch.float8_e4m3fn),
                    pool.view(torch.uint8)[..., :128].contiguous().view(torch.float8_e4m3fn), t, one, one)   # fp8 without scales
    with pytest.raises(NotImplementedError):
        pa.kv_write(z.cpu().float().numpy(), z, pool, pool, t, one, one)


def test_device_kernel_alias_convention_writes_in_place(pa, rng):
    """The write through the name-keyed call convention with the reference's aliasing names
    (examples/models/qwen3/qwen3.py:289-301: "cache_k.must_alias_input" in, "cache_k" out, same
    buffer) gives the bits of the direct call."""
    from nkipy_amd.runtime import DeviceKernel, DeviceTensor
    B, T, Hkv, D, bs = 3, 40, 2, 128, 32
    nb, tables, seqs, qlens, xk, xv = _case(rng, B, T, Hkv, D, bs, seqs=[40, 97, 5], qlens=[40, 33, 0])
    pk = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    pv = rng.integers(0, 65536, size=(nb, bs, Hkv, D), dtype=np.uint16)
    mk = lambda a: torch.from_numpy(a.view(np.int16).copy()).cuda().view(torch.bfloat16)  # noqa: E731
    dk, dv, dk2, dv2 = mk(pk), mk(pv), mk(pk), mk(pv)
    ins = dict(k_new=bf16_to_dev(xk), v_new=bf16_to_dev(xv), block_tables=_i32(tables), seq_lens=_i32(seqs),
               query_lens=_i32(qlens))
    pa.kv_write(ins["k_new"], ins["v_new"], dk, dv, ins["block_tables"], ins["seq_lens"], ins["query_lens"])
    kern = DeviceKernel.compile_and_load(pa.kv_write, name="kv_write", k_cache=dk2, v_cache=dv2, **ins)
    ret = kern(inputs={**{n: DeviceTensor(t) for n, t in ins.items()},
                       "k_cache.must_alias_input": DeviceTensor(dk2), "v_cache.must_alias_input": DeviceTensor(dv2)},
               outputs={"k_cache": DeviceTensor(dk2), "v_cache": DeviceTensor(dv2)})
    torch.cuda.synchronize()
    assert ret is None
    assert np.array_equal(dev_bits(dk2), dev_bits(dk)) and np.array_equal(dev_bits(dv2), dev_bits(dv))
    assert not np.array_equal(dev_bits(dk2), pk)            # something was written
    with pytest.raises(AssertionError):                     # alias output must be the aliased input's buffer
        kern(inputs={**ins, "k_cache.must_alias_input": dk2, "v_cache.must_alias_input": dv2},
             outputs={"k_cache": dk, "v_cache": dv2})
