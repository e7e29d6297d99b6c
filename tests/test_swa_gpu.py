"""GPU parity of the sliding-window attention kernels (through the C ABI) against the oracle."""
import pytest
import torch

from conftest import rel_l2
from oracle import based_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2  # rel-L2, bf16


def _qkv(B, L, H, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    qkv = (torch.randn(B, L, 3, H, 64, generator=g) * scale).bfloat16()
    return qkv


@pytest.mark.parametrize("B,L,H,w", [(2, 256, 3, 64), (1, 1, 2, 64), (1, 65, 1, 64), (1, 100, 2, 64),
                                     (1, 130, 2, 17), (2, 64, 2, 0), (1, 333, 4, 64), (1, 1024, 16, 64),
                                     # left windows past 64 (three staged key blocks); lengths either side of 128/129/256
                                     (1, 128, 2, 128), (1, 129, 2, 128), (2, 130, 2, 128), (1, 256, 3, 128), (1, 257, 2, 128),
                                     (1, 300, 2, 65), (1, 200, 2, 100), (1, 1, 1, 128), (1, 700, 16, 128), (2, 2048, 4, 128)])
def test_prefill_matches_oracle(dev, B, L, H, w):
    from based_amd import ops

    print(f"swa prefill case B={B} L={L} H={H} w={w}", flush=True)
    qkv = _qkv(B, L, H, seed=3)
    ref = O.sliding_window_attn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=w)
    qkv_d = qkv.to(dev)  # packed layout: q, k, v are strided views, as the module passes them
    out = ops.swa_prefill(qkv_d[:, :, 0], qkv_d[:, :, 1], qkv_d[:, :, 2], w_left=w)
    torch.cuda.synchronize()
    assert out.shape == (B, L, H, 64) and out.dtype == torch.bfloat16
    assert torch.isfinite(out.float()).all()
    assert rel_l2(out.float(), ref.float()) < TOL


@pytest.mark.parametrize("B,L,H,w", [(8, 1500, 16, 64), (8, 1100, 16, 33), (4, 2000, 8, 64), (8, 2000, 6, 64),
                                     (8, 601, 16, 0)])
def test_prefill_runs_in_both_directions(dev, B, L, H, w):
    """Batches whose head groups come in multiples of eight and whose runs hold several tiles: even
    runs walk their tiles downwards, odd runs upwards (four heads per workgroup, and two for H = 6).
    The cache fill keeps every run upwards: both must give the oracle's rows, and each other's."""
    from based_amd import ops

    print(f"swa prefill, runs in both directions: B={B} L={L} H={H} w={w}", flush=True)
    qkv = _qkv(B, L, H, seed=11)
    ref = O.sliding_window_attn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=w)
    qkv_d = qkv.to(dev)
    out = ops.swa_prefill(qkv_d[:, :, 0], qkv_d[:, :, 1], qkv_d[:, :, 2], w_left=w)
    cache = torch.zeros(B, L, 2, H, 64, dtype=torch.bfloat16, device=dev)
    out_up = ops.swa_prefill(qkv_d[:, :, 0], qkv_d[:, :, 1], qkv_d[:, :, 2], w_left=w, kv_cache=cache)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert rel_l2(out.float(), ref.float()) < TOL
    for b in range(B):  # no run may have gone wrong alone
        assert rel_l2(out[b].float(), ref[b].float()) < TOL, f"batch entry {b}"
    assert torch.equal(out, out_up)
    assert torch.equal(cache[:, :, 0], qkv_d[:, :, 1]) and torch.equal(cache[:, :, 1], qkv_d[:, :, 2])


@pytest.mark.parametrize("w", [0, 1, 63, 64, 65, 100, 127, 128])
def test_window_edges_are_exact(dev, w):
    """q = 0 makes every visible key weigh the same, so the output is the plain mean of the V rows in
    [i - w, i]: one key too many or too few moves it by 1/(w+1) of a row, far above this bound."""
    from based_amd import ops

    B, L, H = 1, 400, 2
    qkv = _qkv(B, L, H, seed=7)
    qkv[:, :, 0] = 0
    v = qkv[:, :, 2].float()
    ref = torch.stack([v[:, max(0, i - w): i + 1].mean(dim=1) for i in range(L)], dim=1)
    qd = qkv.to(dev)
    out = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w)
    assert rel_l2(out.float(), ref) < 3e-3
    # and the decode step at positions around the window width
    cache = torch.zeros(B, L, 2, H, 64, dtype=torch.bfloat16, device=dev)
    cache[:, :, 0] = qd[:, :, 1]
    cache[:, :, 1] = qd[:, :, 2]
    for t in sorted({0, 1, max(w - 1, 0), w, w + 1, w + 2, 2 * w + 1, L - 1}):
        o = ops.swa_step(qd[:, t:t + 1, 0], qd[:, t:t + 1, 1], qd[:, t:t + 1, 2], cache, t, w_left=w)
        assert rel_l2(o.float(), ref[:, t:t + 1]) < 3e-3, f"step at {t}"


def test_prefill_large_scores(dev):
    """Scores with a wide dynamic range (|s| up to ~60): softmax must stay finite."""
    from based_amd import ops

    qkv = _qkv(1, 200, 2, seed=4, scale=3.0)
    ref = O.sliding_window_attn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=64)
    qd = qkv.to(dev)
    out = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=64)
    assert torch.isfinite(out.float()).all()
    assert rel_l2(out.float(), ref.float()) < TOL


@pytest.mark.parametrize("P,T,w", [(0, 70, 64), (60, 12, 64), (200, 5, 64), (10, 10, 7), (0, 140, 128), (120, 20, 128),
                                   (250, 10, 128), (60, 80, 100), (60, 10, 65)])
def test_decode_matches_prefill_oracle(dev, P, T, w):
    """Decode steps after a P-token prefill equal the parallel oracle at each position
    (the reference's own cached == uncached invariant)."""
    from based_amd import ops

    B, H = 2, 3
    L = P + T
    qkv = _qkv(B, L, H, seed=5)
    ref = O.sliding_window_attn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    cache = torch.zeros(B, L + 3, 2, H, 64, dtype=torch.bfloat16, device=dev)
    cache[:, :P] = qd[:, :P, 1:]
    cache_ref = torch.zeros(B, L + 3, 2, H, 64, dtype=torch.bfloat16)
    cache_ref[:, :P] = qkv[:, :P, 1:]
    for t in range(P, L):
        print(f"swa step case P={P} w={w} pos={t}", flush=True)
        q, kn, vn = qd[:, t:t + 1, 0], qd[:, t:t + 1, 1], qd[:, t:t + 1, 2]
        if t % 2 == 0:
            o = ops.swa_step(q, kn, vn, cache, t, w_left=w)
        else:  # device-side positions (graph-capturable variant)
            o = ops.swa_step(q, kn, vn, cache, torch.full((B,), t, dtype=torch.int32, device=dev), w_left=w)
        o_ref = O.sliding_window_step(qkv[:, t:t + 1, 0], qkv[:, t:t + 1, 1], qkv[:, t:t + 1, 2], cache_ref, t, w_left=w)
        assert rel_l2(o.float(), o_ref.float()) < TOL
        assert rel_l2(o.float(), ref[:, t:t + 1].float()) < TOL
    assert torch.equal(cache.cpu(), cache_ref)


def test_rejects(dev):
    from based_amd import ops

    x = torch.zeros(1, 4, 2, 12, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swa_prefill(x, x, x)  # head dim 12 (not a multiple of 8)
    x = torch.zeros(1, 4, 2, 32, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swa_prefill(x, x, x, rope=_rope_tables(4, dev))  # 64 rotated channels do not fit a head of 32
    y = torch.zeros(1, 4, 2, 64, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swa_prefill(y, y, y, w_left=129)
    cache = torch.zeros(1, 8, 2, 2, 64, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swa_step(y[:, :1], y[:, :1], y[:, :1], cache, 8)  # position outside the cache
    with pytest.raises(ValueError):
        ops.swa_step(y[:, :1], y[:, :1], y[:, :1], cache, 2, w_left=129)


def _rope_tables(n_pos, dev):
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, 64, 2, dtype=torch.float32) / 64))
    ang = torch.outer(torch.arange(n_pos).float(), inv_freq)
    return ang.cos().contiguous().to(dev), ang.sin().contiguous().to(dev)


@pytest.mark.parametrize("B,L,H,w", [(2, 256, 3, 64), (1, 1, 2, 64), (1, 100, 2, 64), (1, 333, 4, 20), (1, 1024, 8, 64),
                                     (2, 257, 3, 128), (1, 129, 2, 128), (1, 1024, 8, 128), (1, 333, 4, 90),
                                     # paired heads under the three-block ring, runs of 2+2+2+1, 3+3+3+3 and 5+4 tiles
                                     # (every exit of the loop that is unrolled over the ring's positions)
                                     (8, 448, 16, 128), (8, 709, 16, 128), (16, 576, 16, 100)])
def test_prefill_with_rotary_and_cache_output(dev, B, L, H, w):
    """Rotary inside the kernel == rotating q, k first (oracle RoPE, rounded to bf16 like the
    reference's rotated tensors); the optional cache output holds the rotated k and v."""
    from based_amd import ops

    print(f"swa prefill rotary case B={B} L={L} H={H} w={w}", flush=True)
    qkv = _qkv(B, L, H, seed=13)
    pos = torch.arange(L)
    q_r, k_r = O.rotary_embedding(qkv[:, :, 0], pos), O.rotary_embedding(qkv[:, :, 1], pos)
    ref = O.sliding_window_attn(q_r, k_r, qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    rope = _rope_tables(L + 5, dev)
    cache = torch.full((B, L + 2, 2, H, 64), 3.0, dtype=torch.bfloat16, device=dev)
    out = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w, rope=rope, kv_cache=cache)
    torch.cuda.synchronize()
    assert rel_l2(out.float(), ref.float()) < TOL
    out2 = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w, rope=rope)
    assert torch.equal(out, out2)
    # cache: v exact, rotated k to one bf16 rounding (fp32 contraction order may differ), rest untouched
    c = cache.cpu()
    assert torch.equal(c[:, :L, 1], qkv[:, :, 2])
    assert rel_l2(c[:, :L, 0].float(), k_r.float()) < 3e-3
    assert bool((c[:, L:] == 3.0).all())
    # without rotary the cache receives k as it is
    cache2 = torch.zeros_like(cache)
    ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w, kv_cache=cache2)
    assert torch.equal(cache2.cpu()[:, :L], qkv[:, :, 1:])


@pytest.mark.parametrize("P,T,w", [(0, 70, 64), (130, 6, 64), (10, 10, 7), (0, 135, 128), (200, 8, 128), (100, 40, 128)])
def test_decode_with_rotary_matches_parallel(dev, P, T, w):
    """Prefill P tokens into the cache with in-kernel rotary, then rotary decode steps (host and
    device positions): every step equals the parallel oracle on the rotated sequence."""
    from based_amd import ops

    B, H = 2, 3
    L = P + T
    qkv = _qkv(B, L, H, seed=17)
    pos = torch.arange(L)
    q_r, k_r = O.rotary_embedding(qkv[:, :, 0], pos), O.rotary_embedding(qkv[:, :, 1], pos)
    ref = O.sliding_window_attn(q_r, k_r, qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    rope = _rope_tables(L, dev)
    cache = torch.zeros(B, L, 2, H, 64, dtype=torch.bfloat16, device=dev)
    if P > 0:
        o0 = ops.swa_prefill(qd[:, :P, 0], qd[:, :P, 1], qd[:, :P, 2], w_left=w, rope=rope, kv_cache=cache)
        assert rel_l2(o0.float(), ref[:, :P].float()) < TOL
    for t in range(P, L):
        print(f"swa rotary step case P={P} w={w} pos={t}", flush=True)
        q, kn, vn = qd[:, t:t + 1, 0], qd[:, t:t + 1, 1], qd[:, t:t + 1, 2]
        p = t if t % 2 == 0 else torch.full((B,), t, dtype=torch.int32, device=dev)
        o = ops.swa_step(q, kn, vn, cache, p, w_left=w, rope=rope)
        assert rel_l2(o.float(), ref[:, t:t + 1].float()) < TOL
    assert rel_l2(cache[:, :, 0].float(), k_r.float()) < 3e-3
    assert torch.equal(cache[:, :, 1].cpu(), qkv[:, :, 2])


def _qkv_d(B, L, H, D, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, L, 3, H, D, generator=g).bfloat16()


@pytest.mark.parametrize("impl", [None, "plain"])
@pytest.mark.parametrize("B,L,H,D,w", [(2, 200, 3, 16, 64), (1, 300, 2, 32, 128), (1, 70, 2, 128, 17), (1, 1, 1, 8, 64),
                                       (2, 130, 4, 16, 0), (1, 257, 2, 96, 100), (2, 300, 3, 112, 128), (1, 1000, 16, 112, 128),
                                       (1, 129, 2, 128, 128), (1, 500, 2, 72, 64), (1, 333, 2, 112, 64)])
def test_other_head_dims_prefill_and_cache(dev, B, L, H, D, w, impl):
    """Head dims other than 64 (112 and 128: the released 1B / 1.3B models; 16: the reference's test
    models): the general MFMA kernel and the plain kernel against the oracle, with and without the
    cache output."""
    from based_amd import ops as ops_mod
    from types import SimpleNamespace

    ops = SimpleNamespace(swa_prefill=lambda *a, **kw: ops_mod.swa_prefill(*a, impl=impl, **kw))
    print(f"swa any-dim prefill case B={B} L={L} H={H} D={D} w={w} impl={impl}", flush=True)
    qkv = _qkv_d(B, L, H, D, seed=23)
    ref = O.sliding_window_attn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    cache = torch.full((B, L + 3, 2, H, D), 3.0, dtype=torch.bfloat16, device=dev)
    out = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w, kv_cache=cache)
    assert out.shape == (B, L, H, D) and rel_l2(out.float(), ref.float()) < 5e-3
    assert torch.equal(cache[:, :L].cpu(), qkv[:, :, 1:]) and bool((cache[:, L:] == 3.0).all())
    assert torch.equal(out, ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w))


@pytest.mark.parametrize("impl", [None, "plain"])
@pytest.mark.parametrize("D,P,T,w", [(16, 0, 70, 64), (16, 100, 40, 128), (32, 60, 10, 65), (128, 10, 6, 7),
                                     (112, 0, 140, 128), (112, 200, 6, 128), (128, 70, 5, 64), (72, 3, 70, 64)])
def test_other_head_dims_decode(dev, D, P, T, w, impl):
    from based_amd import ops as ops_mod
    from types import SimpleNamespace

    ops = SimpleNamespace(swa_prefill=lambda *a, **kw: ops_mod.swa_prefill(*a, impl=impl, **kw),
                          swa_step=lambda *a, **kw: ops_mod.swa_step(*a, impl=impl, **kw))
    B, H = 2, 3
    L = P + T
    qkv = _qkv_d(B, L, H, D, seed=29)
    ref = O.sliding_window_attn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    cache = torch.zeros(B, L + 2, 2, H, D, dtype=torch.bfloat16, device=dev)
    if P > 0:
        ops.swa_prefill(qd[:, :P, 0], qd[:, :P, 1], qd[:, :P, 2], w_left=w, kv_cache=cache)
    for t in range(P, L):
        print(f"swa any-dim step case D={D} P={P} w={w} pos={t}", flush=True)
        p = t if t % 2 == 0 else torch.full((B,), t, dtype=torch.int32, device=dev)
        o = ops.swa_step(qd[:, t:t + 1, 0], qd[:, t:t + 1, 1], qd[:, t:t + 1, 2], cache, p, w_left=w)
        assert rel_l2(o.float(), ref[:, t:t + 1].float()) < 5e-3
    assert torch.equal(cache[:, :L].cpu(), qkv[:, :, 1:])
    bad = ops.swa_step(qd[:, :1, 0], qd[:, :1, 1], qd[:, :1, 2], cache, torch.full((B,), L + 2, dtype=torch.int32, device=dev), w_left=w)
    assert bool(torch.isnan(bad.float()).all())        # device-side position outside the cache


def test_plain_kernel_agrees_with_mfma_kernel_at_head_dim_64(dev):
    """The plain kernels are a second statement of the attention: at head dim 64 they can be called
    through the C ABI next to the MFMA kernels."""
    from based_amd import _lib, ops

    B, L, H, w = 2, 333, 4, 128
    qkv = _qkv(B, L, H, seed=31).to(dev)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    fast = ops.swa_prefill(q, k, v, w_left=w)
    slow = torch.empty_like(fast)
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(_lib.lib().based_swa_prefill_anydim(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), slow.data_ptr(), B, H, L, 64, q.stride(0), q.stride(1), q.stride(2),
        k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2), slow.stride(0), slow.stride(1),
        slow.stride(2), w, 0.125, None, None, 0, 0, 0, 0, _lib.BASED_BF16, stream))
    assert rel_l2(fast.float(), slow.float()) < 4e-3


def _rope_tables_d(n_pos, rotary_dim, dev, interleaved=False, base=10000.0):
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    ang = torch.outer(torch.arange(n_pos).float(), inv_freq)
    return ang.cos().contiguous().to(dev), ang.sin().contiguous().to(dev), interleaved


@pytest.mark.parametrize("D,R,inter", [(112, 112, False), (128, 128, False), (112, 112, True), (128, 64, False),
                                       (112, 48, True), (64, 32, False), (64, 64, True), (64, 16, True),
                                       (32, 32, False), (96, 80, False)])
@pytest.mark.parametrize("B,L,H,w", [(2, 300, 3, 128), (1, 130, 2, 64)])
def test_wide_prefill_rotary_layouts_and_cache(dev, D, R, inter, B, L, H, w):
    """The rotary shapes of the reference's constructor (rotary_emb_dim a multiple of 16 up to the
    head dim, half-split or interleaved pairs; slide_attention.py:346-355) inside the general
    kernel == rotating q and k first with the oracle; the cache receives the rotated k and v."""
    from based_amd import ops

    print(f"swa wide rotary case D={D} R={R} interleaved={inter} B={B} L={L} H={H} w={w}", flush=True)
    qkv = _qkv_d(B, L, H, D, seed=37)
    pos = torch.arange(L)
    q_r = O.rotary_embedding(qkv[:, :, 0], pos, rotary_dim=R, interleaved=inter)
    k_r = O.rotary_embedding(qkv[:, :, 1], pos, rotary_dim=R, interleaved=inter)
    ref = O.sliding_window_attn(q_r, k_r, qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    rope = _rope_tables_d(L + 3, R, dev, inter)
    cache = torch.full((B, L + 2, 2, H, D), 3.0, dtype=torch.bfloat16, device=dev)
    out = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w, rope=rope, kv_cache=cache)
    torch.cuda.synchronize()
    assert rel_l2(out.float(), ref.float()) < TOL
    c = cache.cpu()
    assert torch.equal(c[:, :L, 1], qkv[:, :, 2])
    assert rel_l2(c[:, :L, 0].float(), k_r.float()) < 3e-3
    assert torch.equal(c[:, :L, 0][..., R:], qkv[:, :, 1][..., R:])   # channels past rotary_dim pass through
    assert bool((c[:, L:] == 3.0).all())


@pytest.mark.parametrize("D,R,inter,L", [(112, 0, False, 1100), (112, 112, False, 1100), (128, 64, True, 1237),
                                         (96, 96, False, 700)])
def test_wide_prefill_long_runs_of_tile_pairs(dev, D, R, inter, L):
    """128 heads and 128 keys to the left: every workgroup walks a run of many steps of two query
    tiles (both register sets of rows in flight, the four-block ring going round several times, a
    last step whose second tile is past the sequence)."""
    from based_amd import ops

    B, H, w = 8, 16, 128
    print(f"swa wide long-run case D={D} R={R} interleaved={inter} L={L}", flush=True)
    qkv = _qkv_d(B, L, H, D, seed=53)
    q_r, k_r = qkv[:, :, 0], qkv[:, :, 1]
    rope = None
    if R:
        pos = torch.arange(L)
        q_r = O.rotary_embedding(q_r, pos, rotary_dim=R, interleaved=inter)
        k_r = O.rotary_embedding(k_r, pos, rotary_dim=R, interleaved=inter)
        rope = _rope_tables_d(L, R, dev, inter)
    ref = O.sliding_window_attn(q_r, k_r, qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    cache = torch.full((B, L + 1, 2, H, D), 3.0, dtype=torch.bfloat16, device=dev)
    out = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w, rope=rope, kv_cache=cache, impl="wide")
    torch.cuda.synchronize()
    per_tile = (out.float().cpu() - ref.float()).flatten(2).norm(dim=2) / ref.float().flatten(2).norm(dim=2)
    assert float(per_tile.max()) < 1.5e-2, f"worst token at {int(per_tile.argmax()) % L}"
    assert rel_l2(out.float(), ref.float()) < TOL
    c = cache.cpu()
    assert torch.equal(c[:, :L, 1], qkv[:, :, 2]) and bool((c[:, L:] == 3.0).all())
    assert rel_l2(c[:, :L, 0].float(), k_r.float()) < 3e-3
    assert torch.equal(out, ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w, rope=rope, impl="wide"))


@pytest.mark.parametrize("D,R,inter,P,T,w", [(112, 112, False, 0, 140, 128), (112, 112, False, 200, 8, 128),
                                             (128, 128, False, 70, 6, 64), (112, 64, True, 50, 20, 128),
                                             (64, 32, False, 10, 10, 7), (64, 64, True, 100, 40, 128)])
def test_wide_decode_rotary_matches_parallel(dev, D, R, inter, P, T, w):
    """Prefill P tokens into the cache with in-kernel rotary, then rotary decode steps (host and
    device positions) through the general kernels: every step equals the parallel oracle."""
    from based_amd import ops

    B, H = 2, 3
    L = P + T
    qkv = _qkv_d(B, L, H, D, seed=41)
    pos = torch.arange(L)
    q_r = O.rotary_embedding(qkv[:, :, 0], pos, rotary_dim=R, interleaved=inter)
    k_r = O.rotary_embedding(qkv[:, :, 1], pos, rotary_dim=R, interleaved=inter)
    ref = O.sliding_window_attn(q_r, k_r, qkv[:, :, 2], w_left=w)
    qd = qkv.to(dev)
    rope = _rope_tables_d(L, R, dev, inter)
    cache = torch.zeros(B, L, 2, H, D, dtype=torch.bfloat16, device=dev)
    if P > 0:
        o0 = ops.swa_prefill(qd[:, :P, 0], qd[:, :P, 1], qd[:, :P, 2], w_left=w, rope=rope, kv_cache=cache)
        assert rel_l2(o0.float(), ref[:, :P].float()) < TOL
    for t in range(P, L):
        print(f"swa wide rotary step case D={D} R={R} P={P} w={w} pos={t}", flush=True)
        p = t if t % 2 == 0 else torch.full((B,), t, dtype=torch.int32, device=dev)
        o = ops.swa_step(qd[:, t:t + 1, 0], qd[:, t:t + 1, 1], qd[:, t:t + 1, 2], cache, p, w_left=w, rope=rope)
        assert rel_l2(o.float(), ref[:, t:t + 1].float()) < TOL
    assert rel_l2(cache[:, :, 0].float(), k_r.float()) < 3e-3
    assert torch.equal(cache[:, :, 1].cpu(), qkv[:, :, 2])
    bad = ops.swa_step(qd[:, :1, 0], qd[:, :1, 1], qd[:, :1, 2], cache, torch.full((B,), L, dtype=torch.int32, device=dev),
                       w_left=w, rope=rope)
    assert bool(torch.isnan(bad.float()).all())        # device-side position outside the cache


def test_wide_kernel_agrees_with_64_channel_kernel(dev):
    """At head dim 64 with whole-head half-split rotary both MFMA kernels apply; they agree to bf16
    noise on outputs and cache, prefill and step."""
    from based_amd import ops

    B, L, H, w = 2, 333, 4, 128
    qkv = _qkv(B, L + 1, H, seed=43).to(dev)
    rope = _rope_tables_d(L + 1, 64, dev)
    q, k, v = qkv[:, :L, 0], qkv[:, :L, 1], qkv[:, :L, 2]
    c1 = torch.zeros(B, L + 1, 2, H, 64, dtype=torch.bfloat16, device=dev)
    c2 = torch.zeros_like(c1)
    fast = ops.swa_prefill(q, k, v, w_left=w, rope=rope, kv_cache=c1)
    wide = ops.swa_prefill(q, k, v, w_left=w, rope=rope, kv_cache=c2, impl="wide")
    assert rel_l2(wide.float(), fast.float()) < 4e-3 and rel_l2(c2.float(), c1.float()) < 1e-3
    s1 = ops.swa_step(qkv[:, L:, 0], qkv[:, L:, 1], qkv[:, L:, 2], c1, L, w_left=w, rope=rope)
    s2 = ops.swa_step(qkv[:, L:, 0], qkv[:, L:, 1], qkv[:, L:, 2], c2, L, w_left=w, rope=rope, impl="wide")
    assert rel_l2(s2.float(), s1.float()) < 4e-3


@pytest.mark.parametrize("w", [0, 1, 64, 65, 127, 128])
def test_wide_window_edges_are_exact(dev, w):
    """The q = 0 mean test of the window edges on the general kernel (head dim 112)."""
    from based_amd import ops

    B, L, H, D = 1, 400, 2, 112
    qkv = _qkv_d(B, L, H, D, seed=47)
    qkv[:, :, 0] = 0
    v = qkv[:, :, 2].float()
    ref = torch.stack([v[:, max(0, i - w): i + 1].mean(dim=1) for i in range(L)], dim=1)
    qd = qkv.to(dev)
    out = ops.swa_prefill(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], w_left=w)
    assert rel_l2(out.float(), ref) < 3e-3
    cache = torch.zeros(B, L, 2, H, D, dtype=torch.bfloat16, device=dev)
    cache[:, :, 0] = qd[:, :, 1]
    cache[:, :, 1] = qd[:, :, 2]
    for t in sorted({0, 1, max(w - 1, 0), w, w + 1, w + 2, 2 * w + 1, L - 1}):
        o = ops.swa_step(qd[:, t:t + 1, 0], qd[:, t:t + 1, 1], qd[:, t:t + 1, 2], cache, t, w_left=w)
        assert rel_l2(o.float(), ref[:, t:t + 1]) < 3e-3, f"step at {t}"
