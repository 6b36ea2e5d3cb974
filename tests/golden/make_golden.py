#!/usr/bin/env python3
"""Writes tests/golden/paged_attention_golden.npz.

The reference repository holds no vectors for paged attention (its tests recompute
every expectation from the NumPy kernel itself), so these fixtures are derived from
first principles instead: seeded inputs, expected outputs from explicit float64
loops with hard masking (`attention_bruteforce_f64`), which shares no code path
with the vectorised oracle or the device kernels.  Inputs are stored in their
storage encodings (fp32, bf16 bit patterns, e4m3fn codes + scales).

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import paged_attention_oracle as O  # noqa: E402


def paged(rng, B, Hkv, D, bs, ctxs, extra=2):
    nblk = [(c + bs - 1) // bs for c in ctxs]
    total = sum(nblk) + extra
    perm = rng.permutation(total).astype(np.int32)
    tables = np.zeros((B, max(nblk) + 1), np.int32)
    pos = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    k = rng.standard_normal((total, bs, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((total, bs, Hkv, D)).astype(np.float32)
    return k, v, tables


def rows(pool, table, ctx, bs):
    return np.concatenate([pool[t] for t in table[:(ctx + bs - 1) // bs]])[:ctx]


def main():
    rng = np.random.default_rng(20240607)
    out = {}

    # 1. fp32 decode, D=64, block 16 (the shape family of config 1)
    B, Hq, Hkv, D, bs = 3, 4, 4, 64, 16
    ctxs = [1, 23, 40]
    k, v, t = paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    exp = np.stack([O.attention_bruteforce_f64(q[b][None], rows(k, t[b], ctxs[b], bs), rows(v, t[b], ctxs[b], bs), 0.125)[0]
                    for b in range(B)])
    out.update(dec32_q=q, dec32_k=k, dec32_v=v, dec32_tables=t, dec32_ctx=np.array(ctxs, np.int32),
               dec32_scale=np.float32(0.125), dec32_expected=exp)

    # 2. bf16 GQA decode, D=128, block 32
    B, Hq, Hkv, D, bs = 2, 8, 2, 128, 32
    ctxs = [37, 70]
    k, v, t = paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    qb, kb, vb = O.f32_to_bf16_bits(q), O.f32_to_bf16_bits(k), O.f32_to_bf16_bits(v)
    qf, kf, vf = O.bf16_bits_to_f32(qb), O.bf16_bits_to_f32(kb), O.bf16_bits_to_f32(vb)
    sc = float(np.float32(1 / np.sqrt(D)))
    exp = np.stack([O.attention_bruteforce_f64(qf[b][None], rows(kf, t[b], ctxs[b], bs), rows(vf, t[b], ctxs[b], bs), sc)[0]
                    for b in range(B)])
    out.update(dec16_q=qb, dec16_k=kb, dec16_v=vb, dec16_tables=t, dec16_ctx=np.array(ctxs, np.int32),
               dec16_scale=np.float32(sc), dec16_expected=exp)

    # 3. fp8 KV decode, D=128, block 64, GQA 8
    B, Hq, Hkv, D, bs = 2, 8, 1, 128, 64
    ctxs = [50, 100]
    k, v, t = paged(rng, B, Hkv, D, bs, ctxs)
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    qb = O.f32_to_bf16_bits(q)
    qf = O.bf16_bits_to_f32(qb)
    kd = O.FP8_E4M3FN_LUT[kq].astype(np.float64) * ks[:, None, :, None]
    vd = O.FP8_E4M3FN_LUT[vq].astype(np.float64) * vs[:, None, :, None]
    exp = np.stack([O.attention_bruteforce_f64(qf[b][None], rows(kd, t[b], ctxs[b], bs), rows(vd, t[b], ctxs[b], bs), sc)[0]
                    for b in range(B)])
    out.update(dec8_q=qb, dec8_k=kq, dec8_v=vq, dec8_kscale=ks, dec8_vscale=vs, dec8_tables=t,
               dec8_ctx=np.array(ctxs, np.int32), dec8_scale=np.float32(sc), dec8_expected=exp)

    # 4. bf16 chunked prefill with prefix, D=128, block 32, ragged query lengths
    B, T, Hq, Hkv, D, bs = 2, 24, 2, 1, 128, 32
    qlens, prefixes = [24, 9], [41, 0]
    ctxs = [p + n for p, n in zip(prefixes, qlens)]
    k, v, t = paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, T, Hq, D)).astype(np.float32)
    qb, kb, vb = O.f32_to_bf16_bits(q), O.f32_to_bf16_bits(k), O.f32_to_bf16_bits(v)
    qf, kf, vf = O.bf16_bits_to_f32(qb), O.bf16_bits_to_f32(kb), O.bf16_bits_to_f32(vb)
    exp = np.zeros((B, T, Hq, D))
    for b in range(B):
        exp[b, :qlens[b]] = O.attention_bruteforce_f64(qf[b, :qlens[b]], rows(kf, t[b], ctxs[b], bs),
                                                       rows(vf, t[b], ctxs[b], bs), sc, prefix=prefixes[b])
    out.update(pre_q=qb, pre_k=kb, pre_v=vb, pre_tables=t, pre_ctx=np.array(ctxs, np.int32),
               pre_qlens=np.array(qlens, np.int32), pre_scale=np.float32(sc), pre_expected=exp)

    # 5. blocksparse prefill, block 64, local 1 + every 2nd block, 2 heads (phase differs per head)
    B, S, H, D = 1, 192, 2, 128
    q = rng.standard_normal((B, S, H, D)).astype(np.float32)
    k = rng.standard_normal((B, S, H, D)).astype(np.float32)
    v = rng.standard_normal((B, S, H, D)).astype(np.float32)
    qb, kb, vb = O.f32_to_bf16_bits(q), O.f32_to_bf16_bits(k), O.f32_to_bf16_bits(v)
    qf, kf, vf = O.bf16_bits_to_f32(qb), O.bf16_bits_to_f32(kb), O.bf16_bits_to_f32(vb)
    exp = np.zeros((B, S, H, D))
    nb = S // 64
    for h in range(H):
        bm = np.zeros((nb, nb), bool)
        for i in range(nb):
            for j in range(nb):
                bm[i, j] = j <= i and ((i - j) < 1 or ((j + h % 2) % 2) == 0)
        tok = np.kron(bm, np.ones((64, 64), bool))
        exp[0][:, h:h + 1] = O.attention_bruteforce_f64(qf[0][:, h:h + 1], kf[0][:, h:h + 1], vf[0][:, h:h + 1],
                                                        sc, prefix=0, mask=tok[None])
    out.update(bsp_q=qb, bsp_k=kb, bsp_v=vb, bsp_scale=np.float32(sc), bsp_local=np.int32(1),
               bsp_stride=np.int32(2), bsp_expected=exp)

    # 6. the gpt-oss variant on a verify-sized chunk: bf16, D=64, 8 q heads on one kv head, 4 query tokens
    #    (ragged), sliding window 20 and per-head sinks
    B, T, Hq, Hkv, D, bs = 2, 4, 8, 1, 64, 16
    qlens, prefixes, window = [4, 3], [37, 5], 20
    ctxs = [p_ + n for p_, n in zip(prefixes, qlens)]
    k, v, t = paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, T, Hq, D)).astype(np.float32)
    sinks = O.bf16_bits_to_f32(O.f32_to_bf16_bits(rng.standard_normal(Hq).astype(np.float32) * 2))
    qb, kb, vb = O.f32_to_bf16_bits(q), O.f32_to_bf16_bits(k), O.f32_to_bf16_bits(v)
    qf, kf, vf = O.bf16_bits_to_f32(qb), O.bf16_bits_to_f32(kb), O.bf16_bits_to_f32(vb)
    sc6 = float(np.float32(1 / np.sqrt(D)))
    exp = np.zeros((B, T, Hq, D))
    for b in range(B):
        exp[b, :qlens[b]] = O.attention_bruteforce_f64(qf[b, :qlens[b]], rows(kf, t[b], ctxs[b], bs), rows(vf, t[b], ctxs[b], bs),
                                                       sc6, prefix=prefixes[b], window=window, sinks=sinks)
    out.update(ver_q=qb, ver_k=kb, ver_v=vb, ver_tables=t, ver_ctx=np.array(ctxs, np.int32),
               ver_qlens=np.array(qlens, np.int32), ver_scale=np.float32(sc6), ver_window=np.int32(window),
               ver_sinks=sinks.astype(np.float32), ver_expected=exp)

    # 7. fp8 KV decode with a sliding window of 48 and sinks, D=128, block 32
    B, Hq, Hkv, D, bs = 2, 4, 2, 128, 32
    ctxs, window = [50, 130], 48
    k, v, t = paged(rng, B, Hkv, D, bs, ctxs)
    kq, ks = O.quantize_kv_fp8(k)
    vq, vs = O.quantize_kv_fp8(v)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    sinks = rng.standard_normal(Hq).astype(np.float32)
    qb = O.f32_to_bf16_bits(q)
    qf = O.bf16_bits_to_f32(qb)
    kd = O.FP8_E4M3FN_LUT[kq].astype(np.float64) * ks[:, None, :, None]
    vd = O.FP8_E4M3FN_LUT[vq].astype(np.float64) * vs[:, None, :, None]
    exp = np.stack([O.attention_bruteforce_f64(qf[b][None], rows(kd, t[b], ctxs[b], bs), rows(vd, t[b], ctxs[b], bs), sc,
                                               prefix=ctxs[b] - 1, window=window, sinks=sinks)[0] for b in range(B)])
    out.update(win8_q=qb, win8_k=kq, win8_v=vq, win8_kscale=ks, win8_vscale=vs, win8_tables=t,
               win8_ctx=np.array(ctxs, np.int32), win8_scale=np.float32(sc), win8_window=np.int32(window),
               win8_sinks=sinks, win8_expected=exp)

    # 8. a long chunk of the gpt-oss variant: bf16, D=64, 8 q heads on 2 kv heads, 100 query tokens (ragged)
    #    behind cached prefixes, sliding window 50 and per-head sinks
    B, T, Hq, Hkv, D, bs = 2, 100, 8, 2, 64, 16
    qlens, prefixes, window = [100, 70], [30, 200], 50
    ctxs = [p_ + n for p_, n in zip(prefixes, qlens)]
    k, v, t = paged(rng, B, Hkv, D, bs, ctxs)
    q = rng.standard_normal((B, T, Hq, D)).astype(np.float32)
    sinks = O.bf16_bits_to_f32(O.f32_to_bf16_bits(rng.standard_normal(Hq).astype(np.float32) * 2))
    qb, kb, vb = O.f32_to_bf16_bits(q), O.f32_to_bf16_bits(k), O.f32_to_bf16_bits(v)
    qf, kf, vf = O.bf16_bits_to_f32(qb), O.bf16_bits_to_f32(kb), O.bf16_bits_to_f32(vb)
    exp = np.zeros((B, T, Hq, D))
    for b in range(B):
        exp[b, :qlens[b]] = O.attention_bruteforce_f64(qf[b, :qlens[b]], rows(kf, t[b], ctxs[b], bs), rows(vf, t[b], ctxs[b], bs),
                                                       sc6, prefix=prefixes[b], window=window, sinks=sinks)
    out.update(long64_q=qb, long64_k=kb, long64_v=vb, long64_tables=t, long64_ctx=np.array(ctxs, np.int32),
               long64_qlens=np.array(qlens, np.int32), long64_scale=np.float32(sc6), long64_window=np.int32(window),
               long64_sinks=sinks.astype(np.float32), long64_expected=exp.astype(np.float32))   # float32: 2^-24 of the values, far below the bf16 bar

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "paged_attention_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
