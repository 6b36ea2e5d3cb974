"""GPU end-to-end: a serving loop in miniature (ragged prompts, decode steps, a forked prefix,
slot reuse) through the engine glue, every step checked against the oracle's dense attention
over the tokens each sequence has seen."""
import numpy as np
import pytest
import torch

from oracle import paged_attention_oracle as O
from tests.pa_testlib import assert_close_abs, bf16_to_dev, dev_to_f32

pytestmark = pytest.mark.gpu


class _Mirror:
    """Dense per-sequence history kept by the oracle: rotated K, V as the reference's cache holds them."""

    def __init__(self, n_slots, cos, sin, wq, wk, eps, window=None, sinks=None):
        self.k = [None] * n_slots
        self.v = [None] * n_slots
        self.cos, self.sin, self.wq, self.wk, self.eps = cos, sin, wq, wk, eps
        self.window, self.sinks = window, sinks

    def step(self, xq, xk, xv, qlens, scale):
        B, T, Hq, D = xq.shape
        out = np.zeros((B, T, Hq, D), np.float32)
        for b in range(B):
            n = qlens[b]
            if n == 0:
                continue
            start = 0 if self.k[b] is None else self.k[b].shape[0]
            seq = np.array([start + n], np.int32)
            if self.cos is not None:
                q, k = O.qk_norm_rope(xq[b:b + 1, :n], xk[b:b + 1, :n], seq, np.array([n], np.int32), self.cos, self.sin,
                                      q_norm_weight=self.wq, k_norm_weight=self.wk, eps=self.eps)
                q, k = q[0], k[0]
            else:
                q, k = xq[b, :n], xk[b, :n]
            self.k[b] = k if self.k[b] is None else np.concatenate([self.k[b], k])
            self.v[b] = xv[b, :n] if self.v[b] is None else np.concatenate([self.v[b], xv[b, :n]])
            n_rep = Hq // k.shape[1]
            o = O.dense_attention(q, O.repeat_kv(self.k[b], n_rep), O.repeat_kv(self.v[b], n_rep), scale, prefix=start,
                                  window=self.window, sinks=self.sinks)
            out[b, :n] = O.round_output(o, "bf16")
        return out


def _rand(rng, shape, amp=1.0):
    return O.round_to_bf16(rng.standard_normal(shape).astype(np.float32) * amp)


@pytest.mark.parametrize("rope", [False, True])
def test_serving_loop_bf16_pool(rng, rope):
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    S, Hq, Hkv, D, bs = 4, 8, 2, 128, 16
    cache = PagedKVCache(num_blocks=40, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=12)
    wq = wk = cos = sin = None
    kw = {}
    if rope:
        wq, wk = _rand(rng, D) * 0.1 + 1.0, _rand(rng, D) * 0.1 + 1.0
        wq, wk = O.round_to_bf16(wq), O.round_to_bf16(wk)
        cos, sin = O.rope_tables(D, 256, 1000000.0)
        kw = dict(rope_base=1000000.0, max_positions=256, q_norm_weight=bf16_to_dev(wq), k_norm_weight=bf16_to_dev(wk), norm_eps=1e-6)
    layer = PagedAttention(cache, Hq, **kw)
    mirror = _Mirror(S, cos, sin, wq, wk, 1e-6)
    tol = 2e-2 if not rope else 3e-2        # with the norm q/k differ from the oracle's by a bf16 step here and there

    def run(T, qlens):
        xq, xk, xv = _rand(rng, (S, T, Hq, D)), _rand(rng, (S, T, Hkv, D)), _rand(rng, (S, T, Hkv, D))
        got = dev_to_f32(layer.step(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), qlens))
        want = mirror.step(xq, xk, xv, qlens, layer.scale)
        for b in range(S):
            if qlens[b]:
                assert_close_abs(got[b, :qlens[b]], want[b, :qlens[b]], tol)

    run(37, [37, 20, 0, 5])                      # ragged prompts, slot 2 idle
    for _ in range(3):
        run(1, [1, 1, 0, 1])                     # decode
    run(9, [0, 9, 0, 0])                         # a second chunk for slot 1 (chunked prefill against its cached prefix)
    # fork slot 0 into slot 2: shared full blocks, private tail; both continue independently
    cache.fork(0, 2)
    mirror.k[2], mirror.v[2] = mirror.k[0].copy(), mirror.v[0].copy()
    shared = cache.blocks[0][:cache.lens[0] // bs]
    assert shared and all(cache.allocator.refcount(b) == 2 for b in shared)
    for _ in range(bs + 2):                      # long enough to fill the tail and open new blocks on both sides
        run(1, [1, 1, 1, 1])
    assert cache.blocks[0][len(shared):] != cache.blocks[2][len(shared):]
    # release a slot and reuse it for a new prompt: its blocks go back and stale contents do not leak
    free_before = cache.allocator.num_free
    cache.release(1)
    mirror.k[1] = mirror.v[1] = None
    assert cache.allocator.num_free > free_before
    run(21, [0, 21, 0, 0])
    run(1, [1, 1, 1, 1])


def test_serving_loop_gpt_oss_variant(rng):
    """head_dim 64, RoPE, per-head sinks and a 24-token sliding window (shorter than the prompts): prompt
    chunks (one of them longer than a launch of that kernel takes), verify-sized steps and decode steps all go
    through the decode-shaped kernel."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    S, Hq, Hkv, D, bs = 3, 8, 2, 64, 16
    cache = PagedKVCache(num_blocks=40, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=12)
    sinks = _rand(rng, Hq)
    cos, sin = O.rope_tables(D, 192, 150000.0)
    layer = PagedAttention(cache, Hq, rope_base=150000.0, max_positions=192, sinks=bf16_to_dev(sinks), sliding_window=24)
    mirror = _Mirror(S, cos, sin, None, None, 1e-6, window=24, sinks=sinks)

    def run(T, qlens):
        xq, xk, xv = _rand(rng, (S, T, Hq, D)), _rand(rng, (S, T, Hkv, D)), _rand(rng, (S, T, Hkv, D))
        got = dev_to_f32(layer.step(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), qlens))
        want = mirror.step(xq, xk, xv, qlens, layer.scale)
        for b in range(S):
            if qlens[b]:
                assert_close_abs(got[b, :qlens[b]], want[b, :qlens[b]], 2e-2)

    run(40, [40, 13, 0])            # prompts; slot 0's is longer than the window
    for _ in range(3):
        run(1, [1, 1, 0])
    run(4, [4, 4, 0])               # speculative verify: the last accepted token plus three drafts
    run(30, [0, 0, 30])
    for _ in range(20):
        run(1, [1, 1, 1])
    run(100, [0, 100, 70])          # a long chunk at head_dim 64: the verify kernel, 64 tokens per launch
    run(1, [1, 1, 1])


def test_steps_published_while_the_device_is_busy():
    """A loop issued call by call runs ahead of the GPU: the bookkeeping of a dozen later steps is published while the
    first step's kernels have not started (a long matmul holds the stream).  Every step must still read its own
    tables, lengths and query lengths: same results as a twin that waits for the device after every step."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    torch.manual_seed(3)
    S, Hq, Hkv, D, bs = 3, 8, 2, 128, 16

    def make():
        cache = PagedKVCache(num_blocks=60, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=16)
        return cache, PagedAttention(cache, Hq, rope_base=10000.0, max_positions=256)

    rows = [(torch.randn(S, 1, Hq, D, device="cuda").to(torch.bfloat16), torch.randn(S, 1, Hkv, D, device="cuda").to(torch.bfloat16),
             torch.randn(S, 1, Hkv, D, device="cuda").to(torch.bfloat16)) for _ in range(14)]
    qlens = [[1, 1, 1], [1, 0, 1], [1, 1, 0]]
    prompt = (torch.randn(S, 20, Hq, D, device="cuda").to(torch.bfloat16), torch.randn(S, 20, Hkv, D, device="cuda").to(torch.bfloat16),
              torch.randn(S, 20, Hkv, D, device="cuda").to(torch.bfloat16))

    def run(wait):
        cache, layer = make()
        layer.step(*prompt, [20, 7, 15])
        torch.cuda.synchronize()
        if not wait:
            big = torch.randn(8192, 8192, device="cuda")
            for _ in range(6):
                big = big @ big * 1e-4                 # tens of milliseconds of queued work ahead of the steps
        outs = []
        for i, (xq, xk, xv) in enumerate(rows):
            outs.append(layer.step(xq, xk, xv, qlens[i % 3]).clone())
            if wait:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        return outs, cache.k_cache.clone()

    a, ka = run(True)
    b, kb = run(False)
    for i, (x, y) in enumerate(zip(a, b)):
        assert torch.equal(x.view(torch.int16), y.view(torch.int16)), f"step {i}"
    assert torch.equal(ka.view(torch.int16), kb.view(torch.int16))


def test_serving_loop_fp8_pool(rng):
    """fp8 pool: the write kernel maintains the scales; attention follows the oracle run on the
    dequantised pool within the fp8 bar."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    S, Hq, Hkv, D, bs = 2, 8, 2, 128, 16
    cache = PagedKVCache(num_blocks=12, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=5,
                         dtype=torch.float8_e4m3fn)
    layer = PagedAttention(cache, Hq)
    for step in range(40):
        xq, xk, xv = _rand(rng, (S, 1, Hq, D)), _rand(rng, (S, 1, Hkv, D), 1.0 + 0.05 * step), _rand(rng, (S, 1, Hkv, D))
        got = dev_to_f32(layer.step(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), [1, 1]))[:, 0]
        codes_k = cache.k_cache.view(torch.uint8).cpu().numpy()
        codes_v = cache.v_cache.view(torch.uint8).cpu().numpy()
        want = O.paged_decode(xq[:, 0], codes_k, codes_v, cache.block_tables.cpu().numpy(), cache.seq_lens.cpu().numpy(),
                              layer.scale, k_scale=cache.k_scale.cpu().numpy(), v_scale=cache.v_scale.cpu().numpy(), q_dtype="bf16")
        assert_close_abs(got, want, 5e-2)
    assert cache.lens == [40, 40] and len(cache.blocks[0]) == 3
    # a speculative-verify step (3 tokens for slot 0, 2 for slot 1) reads the fp8 pool as well
    xq, xk, xv = _rand(rng, (S, 3, Hq, D)), _rand(rng, (S, 3, Hkv, D)), _rand(rng, (S, 3, Hkv, D))
    got = dev_to_f32(layer.step(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), [3, 2]))
    want = O.paged_prefill(xq, cache.k_cache.view(torch.uint8).cpu().numpy(), cache.v_cache.view(torch.uint8).cpu().numpy(),
                           cache.block_tables.cpu().numpy(), cache.seq_lens.cpu().numpy(), np.array([3, 2], np.int32),
                           layer.scale, k_scale=cache.k_scale.cpu().numpy(), v_scale=cache.v_scale.cpu().numpy(), q_dtype="bf16")
    assert_close_abs(got, want, 5e-2)
    assert cache.lens == [43, 42] and np.all(got[1, 2] == 0)
    # a longer chunk goes through the tiled kernel, which expands the fp8 codes on their way into LDS
    cache.release(1)
    xq, xk, xv = _rand(rng, (S, 70, Hq, D)), _rand(rng, (S, 70, Hkv, D)), _rand(rng, (S, 70, Hkv, D))
    got = dev_to_f32(layer.step(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), [0, 70]))
    want = O.paged_prefill(xq, cache.k_cache.view(torch.uint8).cpu().numpy(), cache.v_cache.view(torch.uint8).cpu().numpy(),
                           cache.block_tables.cpu().numpy(), cache.seq_lens.cpu().numpy(), np.array([0, 70], np.int32),
                           layer.scale, k_scale=cache.k_scale.cpu().numpy(), v_scale=cache.v_scale.cpu().numpy(), q_dtype="bf16")
    assert_close_abs(got, want, 5e-2)
    assert cache.lens == [43, 70] and np.all(got[0] == 0)


def test_two_layers_share_tables(rng):
    """A model step opens once (`begin_step`) and every layer attends into its own pool through the shared
    block tables; a fork copies the partial tail block of every layer."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    S, Hq, Hkv, D, bs, L = 3, 8, 2, 128, 16, 2
    cache = PagedKVCache(num_blocks=30, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=8,
                         num_layers=L)
    cos, sin = O.rope_tables(D, 128, 10000.0)
    tables = (bf16_to_dev(cos), bf16_to_dev(sin))                   # one pair of RoPE tables for both layers
    layers = [PagedAttention(cache, Hq, layer=l, rope_tables=tables) for l in range(L)]
    mirrors = [_Mirror(S, cos, sin, None, None, 1e-6) for _ in range(L)]
    assert cache.k_caches[0].data_ptr() != cache.k_caches[1].data_ptr()

    def run(T, qlens):
        free_before = cache.allocator.num_free
        cache.begin_step(qlens, T)
        for l in range(L):
            xq, xk, xv = _rand(rng, (S, T, Hq, D)), _rand(rng, (S, T, Hkv, D)), _rand(rng, (S, T, Hkv, D))
            got = dev_to_f32(layers[l].attend(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv)))
            want = mirrors[l].step(xq, xk, xv, qlens, layers[l].scale)
            for b in range(S):
                if qlens[b]:
                    assert_close_abs(got[b, :qlens[b]], want[b, :qlens[b]], 3e-2)
        return free_before - cache.allocator.num_free

    used = run(21, [21, 9, 0])
    assert used == 2 + 1                                             # blocks are reserved once per step, not per layer
    run(1, [1, 1, 0])
    cache.fork(0, 2)
    for m in mirrors:
        m.k[2], m.v[2] = m.k[0].copy(), m.v[0].copy()
    for _ in range(3):
        run(1, [1, 1, 1])
    with pytest.raises(ValueError):
        layers[0].attend(bf16_to_dev(_rand(rng, (S, 2, Hq, D))), bf16_to_dev(_rand(rng, (S, 2, Hkv, D))),
                         bf16_to_dev(_rand(rng, (S, 2, Hkv, D))))   # not the step begin_step opened


@pytest.mark.parametrize("seed,variant", [(0, "qwen"), (1, "qwen"), (2, "gpt_oss"), (3, "gpt_oss")])
def test_serving_loop_random_schedule(seed, variant):
    """A random schedule of prompt chunks, verify-sized steps, decode steps, forks and releases over two
    layers' worth of history (one layer computed), every step against the oracle's dense attention; the pool
    is small enough that slots must be released to make room."""
    from nkipy_amd.engine import OutOfBlocks, PagedAttention, PagedKVCache
    rng = np.random.default_rng(500 + seed)
    S, bs = 5, 16
    if variant == "qwen":
        Hq, Hkv, D, window, base, cap = 8, 2, 128, None, 1000000.0, 400
    else:
        Hq, Hkv, D, window, base, cap = 16, 2, 64, 40, 150000.0, 400
    max_blocks = cap // bs
    cache = PagedKVCache(num_blocks=70, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=max_blocks)
    cos, sin = O.rope_tables(D, cap, base)
    wq = O.round_to_bf16(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32)) if variant == "qwen" else None
    wk = O.round_to_bf16(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32)) if variant == "qwen" else None
    sinks = _rand(rng, Hq) if variant == "gpt_oss" else None
    layer = PagedAttention(cache, Hq, rope_base=base, max_positions=cap,
                           q_norm_weight=None if wq is None else bf16_to_dev(wq),
                           k_norm_weight=None if wk is None else bf16_to_dev(wk), norm_eps=1e-6,
                           sinks=None if sinks is None else bf16_to_dev(sinks), sliding_window=window)
    mirror = _Mirror(S, cos, sin, wq, wk, 1e-6, window=window, sinks=sinks)
    steps = 0
    for it in range(70):
        action = rng.choice(["prompt", "decode", "decode", "decode", "verify", "fork", "release"])
        live = [s for s in range(S) if cache.lens[s] > 0]
        idle = [s for s in range(S) if cache.lens[s] == 0]
        if action == "fork" and live and idle:
            src, dst = int(rng.choice(live)), int(rng.choice(idle))
            try:
                cache.fork(src, dst)
            except OutOfBlocks:
                continue
            mirror.k[dst], mirror.v[dst] = mirror.k[src].copy(), mirror.v[src].copy()
            continue
        if action == "release" and live:
            s = int(rng.choice(live))
            cache.release(s)
            mirror.k[s] = mirror.v[s] = None
            continue
        if action == "prompt":
            T = int(rng.integers(5, 90))
            qlens = [int(rng.integers(1, T + 1)) if (s in idle or rng.integers(0, 3) == 0) else 0 for s in range(S)]
        elif action == "verify":
            T = int(rng.integers(2, 6))
            qlens = [int(rng.integers(1, T + 1)) if s in live else 0 for s in range(S)]
        else:
            T = 1
            qlens = [1 if s in live else 0 for s in range(S)]
        qlens = [n if cache.lens[s] + n <= cap else 0 for s, n in enumerate(qlens)]
        if max(qlens) == 0:
            continue
        T = max(T, max(qlens))
        xq, xk, xv = _rand(rng, (S, T, Hq, D)), _rand(rng, (S, T, Hkv, D)), _rand(rng, (S, T, Hkv, D))
        try:
            got = dev_to_f32(layer.step(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv), qlens))
        except OutOfBlocks:
            victim = max(range(S), key=lambda s: cache.lens[s])        # make room: drop the longest sequence
            cache.release(victim)
            mirror.k[victim] = mirror.v[victim] = None
            continue
        want = mirror.step(xq, xk, xv, qlens, layer.scale)
        steps += 1
        for b in range(S):
            if qlens[b]:
                assert_close_abs(got[b, :qlens[b]], want[b, :qlens[b]], 3e-2)
    assert steps >= 25
    # bookkeeping stays consistent: every block is free or owned, shared ones counted once per owner
    owned = {}
    for s in range(S):
        for blk in cache.blocks[s]:
            owned[blk] = owned.get(blk, 0) + 1
    assert all(cache.allocator.refcount(blk) == n for blk, n in owned.items())
    assert cache.allocator.num_free + len(owned) == 70


@pytest.mark.parametrize("bias", [False, True])
def test_layer_with_output_projection(rng, bias):
    """A layer given `o_weight` returns the projected rows: the attention output in its stored bfloat16 rounding
    times o_weight, float32 accumulation, one rounding (qwen3 attention.py:143-147; with bias gpt_oss
    attention.py:155-163)."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    S, Hq, Hkv, D, bs, hidden = 3, 8, 2, 128, 16, 512
    cache = PagedKVCache(num_blocks=30, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=8)
    w = _rand(rng, (Hq * D, hidden), 0.05)
    b = _rand(rng, hidden) if bias else None
    layer = PagedAttention(cache, Hq, o_weight=bf16_to_dev(w), o_bias=None if b is None else bf16_to_dev(b))
    mirror = _Mirror(S, None, None, None, None, 1e-6)
    for T, qlens in ((19, [19, 7, 0]), (1, [1, 1, 0]), (1, [1, 1, 0])):
        cache.begin_step(qlens, T)
        xq, xk, xv = _rand(rng, (S, T, Hq, D)), _rand(rng, (S, T, Hkv, D)), _rand(rng, (S, T, Hkv, D))
        got = dev_to_f32(layer.attend(bf16_to_dev(xq), bf16_to_dev(xk), bf16_to_dev(xv)))
        assert got.shape == (S, T, hidden)
        attn = mirror.step(xq, xk, xv, qlens, layer.scale)
        want = O.o_proj(attn.reshape(S, T, Hq * D), w, b)
        for s in range(S):
            if qlens[s]:
                assert_close_abs(got[s, :qlens[s]], want[s, :qlens[s]], 4e-2)
    with pytest.raises(ValueError):
        PagedAttention(cache, Hq, o_weight=bf16_to_dev(_rand(rng, (Hq * D - 64, hidden))))


def test_decode_steps_replayed_from_one_graph_while_the_contexts_grow(rng):
    """The launch-bound part of serving: the decode step of a stack of layers (K norm + RoPE + KV write, decode
    attention with the Q transform on its load, output projection) captured once into a HIP graph and replayed
    every step with new inputs, while begin_step outside the graph extends the sequences across block borders
    and past the lengths they had at capture time.  Every replay is checked, bit for bit, against the same
    layers run eagerly on a twin cache, with eager work between the replays."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    from tests.pa_testlib import dev_bits
    S, L, Hq, Hkv, D, bs, hidden = 3, 2, 8, 2, 128, 16, 256
    wq = bf16_to_dev(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32))
    wk = bf16_to_dev(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32))
    ow = [bf16_to_dev((rng.standard_normal((Hq * D, hidden)) / 32).astype(np.float32)) for _ in range(L)]

    def stack():
        cache = PagedKVCache(num_blocks=64, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S, max_blocks_per_seq=10,
                             num_layers=L)
        layers = [PagedAttention(cache, Hq, layer=l, rope_base=10000.0, max_positions=10 * bs, q_norm_weight=wq,
                                 k_norm_weight=wk, o_weight=ow[l]) for l in range(L)]
        return cache, layers

    (ca, la), (cb, lb) = stack(), stack()
    T0 = 40
    prompt = [[_rand(rng, (S, T0, h, D)) for h in (Hq, Hkv, Hkv)] for _ in range(L)]
    plens = [40, 7, 23]
    for cache, layers in ((ca, la), (cb, lb)):
        cache.begin_step(plens, T0)
        for l in range(L):
            layers[l].attend(*[bf16_to_dev(t) for t in prompt[l]])
    # static inputs of the captured step, one set per layer
    xs = [[torch.zeros((S, 1, h, D), dtype=torch.bfloat16, device="cuda") for h in (Hq, Hkv, Hkv)] for _ in range(L)]

    def fill():
        for l in range(L):
            for t in xs[l]:
                t.copy_(bf16_to_dev(_rand(rng, tuple(t.shape))))

    def eager(cache, layers):
        cache.begin_step([1] * S, 1)
        return [layers[l].attend(*xs[l]) for l in range(L)]

    fill()
    want = [o.clone() for o in eager(cb, lb)]
    got = eager(ca, la)                      # one eager decode step first: buffers and workspaces exist before the capture
    torch.cuda.synchronize()
    for l in range(L):
        assert np.array_equal(dev_bits(got[l]), dev_bits(want[l]))
    fill()
    ca.begin_step([1] * S, 1)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        outs = [la[l].attend(*xs[l]) for l in range(L)]
    for step in range(45):                   # 41 -> 86 tokens in slot 0: five more blocks, twice the captured length
        if step:
            fill()
            ca.begin_step([1] * S, 1)
        print(f"replay {step}: lens {ca.lens}", flush=True)
        g.replay()
        want = eager(cb, lb)
        torch.cuda.synchronize()
        for l in range(L):
            assert np.array_equal(dev_bits(outs[l]), dev_bits(want[l])), (step, l)
    assert ca.lens == cb.lens == [86, 53, 69]


@pytest.mark.parametrize("bound", [None, 256])
def test_graph_replay_on_tables_longer_than_four_partitions(rng, bound):
    """Tables of 3 072 tokens per sequence: a decode step captured without a promise about the lengths must serve any
    of them and takes the balanced kernel, while the eager twin, which knows its contexts are short, takes the
    fixed-partition one; the two agree to the order of their float32 sums (tolerance, not bits).  With the same
    `max_seq_len` given to both, the captured step takes the small-call kernel too and every replay equals the eager
    step bit for bit; a context that would outgrow the promise is refused on the host."""
    from nkipy_amd.engine import PagedAttention, PagedKVCache
    from tests.pa_testlib import dev_bits
    S, L, Hq, Hkv, D, bs, hidden = 3, 2, 8, 2, 128, 16, 256
    ow = [bf16_to_dev((rng.standard_normal((Hq * D, hidden)) / 32).astype(np.float32)) for _ in range(L)]

    def stack():
        cache = PagedKVCache(num_blocks=96, block_size=bs, n_kv_heads=Hkv, head_dim=D, max_seqs=S,
                             max_blocks_per_seq=192, num_layers=L)
        layers = [PagedAttention(cache, Hq, layer=l, rope_base=10000.0, max_positions=192 * bs, o_weight=ow[l])
                  for l in range(L)]
        return cache, layers

    (ca, la), (cb, lb) = stack(), stack()
    T0 = 40
    prompt = [[_rand(rng, (S, T0, h, D)) for h in (Hq, Hkv, Hkv)] for _ in range(L)]
    for cache, layers in ((ca, la), (cb, lb)):
        cache.begin_step([40, 7, 23], T0)
        for l in range(L):
            layers[l].attend(*[bf16_to_dev(t) for t in prompt[l]])
    xs = [[torch.zeros((S, 1, h, D), dtype=torch.bfloat16, device="cuda") for h in (Hq, Hkv, Hkv)] for _ in range(L)]

    def fill():
        for l in range(L):
            for t in xs[l]:
                t.copy_(bf16_to_dev(_rand(rng, tuple(t.shape))))

    def eager(cache, layers):
        cache.begin_step([1] * S, 1)
        return [layers[l].attend(*xs[l], max_seq_len=bound) for l in range(L)]

    fill()
    eager(ca, la), eager(cb, lb)             # buffers and workspaces exist before the capture
    torch.cuda.synchronize()
    fill()
    ca.begin_step([1] * S, 1)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        outs = [la[l].attend(*xs[l], max_seq_len=bound) for l in range(L)]
    for step in range(12):
        if step:
            fill()
            ca.begin_step([1] * S, 1)
        print(f"bound {bound} replay {step}: lens {ca.lens}", flush=True)
        g.replay()
        want = eager(cb, lb)
        torch.cuda.synchronize()
        for l in range(L):
            if bound is None:
                a, b = outs[l].float().cpu().numpy(), want[l].float().cpu().numpy()
                assert np.abs(a - b).max() <= 2e-2 + 2 ** -7 * np.abs(b).max(), (step, l)
            else:
                assert np.array_equal(dev_bits(outs[l]), dev_bits(want[l])), (step, l)
    if bound is not None:
        ca.begin_step([bound] * S, bound)    # contexts beyond the promise
        with pytest.raises(ValueError):
            la[0].attend(*[torch.zeros((S, bound, h, D), dtype=torch.bfloat16, device="cuda") for h in (Hq, Hkv, Hkv)],
                         max_seq_len=bound)
