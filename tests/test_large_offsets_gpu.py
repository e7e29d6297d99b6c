"""Tensors of more than 2^31 elements: the rows that lie past that mark must come out exactly as
they do when the same rows are handed over on their own (a 32-bit product anywhere in a kernel's
addressing would send them elsewhere).  The oracle is not involved: these sizes are out of its
reach, and what the rows should be is pinned by the small-shape parity tests; here a kernel is
compared with itself, bit for bit, on a batch entry before and after the 2^31 mark.

Every case needs 5 - 30 GB of device memory and a few milliseconds of kernel time."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

MARK = 2 ** 31


def _need(dev, gib):
    free, _ = torch.cuda.mem_get_info(dev)
    if free < gib * 2 ** 30:
        pytest.skip(f"needs {gib} GiB of free device memory, {free / 2 ** 30:.0f} GiB free")


def _randn(shape, dev, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator(device=dev).manual_seed(seed)
    # generated on the device, in pieces along the first dimension (the fp32 source of one piece stays small)
    out = torch.empty(shape, dtype=dtype, device=dev)
    step = max(1, shape[0] // 16)
    for i in range(0, shape[0], step):
        n = min(step, shape[0] - i)
        out[i:i + n] = (torch.randn((n,) + tuple(shape[1:]), generator=g, device=dev) * scale).to(dtype)
    return out


@pytest.fixture(autouse=True)
def _release(dev):
    yield
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def test_linear_prefill_past_the_mark(dev):
    from based_amd import ops

    B, L, H, dv = 160, 8192, 16, 128
    assert (B - 1) * L * H * dv > MARK
    _need(dev, 16)
    print(f"large offsets: linear prefill B={B} L={L} H={H} dv={dv}", flush=True)
    q = _randn((B, L, H, 16), dev, 1).transpose(1, 2)
    k = _randn((B, L, H, 16), dev, 2).transpose(1, 2)
    v = _randn((B, L, H, dv), dev, 3).transpose(1, 2)
    y, kv, ks = ops.linear_attn_prefill(q, k, v, return_state=True)
    for b in (0, B - 1):
        y1, kv1, ks1 = ops.linear_attn_prefill(q[b:b + 1].clone(), k[b:b + 1].clone(), v[b:b + 1].clone(),
                                               return_state=True, split=False)
        torch.cuda.synchronize()
        assert torch.equal(y[b], y1[0]), f"batch entry {b}"
        assert torch.equal(kv[b], kv1[0]) and torch.equal(ks[b], ks1[0]), f"states of batch entry {b}"
    assert torch.isfinite(y[B - 1].float()).all()


def test_linear_step_state_past_the_mark(dev):
    from based_amd import ops

    B, H, dv = 4096, 16, 128
    assert (B - 1) * H * dv * 273 > MARK
    _need(dev, 14)
    print(f"large offsets: linear step B={B} H={H} dv={dv}", flush=True)
    kv = _randn((B, H, 1, dv, 273), dev, 4, dtype=torch.float32)
    ks = _randn((B, H, 1, 1, 273), dev, 5, dtype=torch.float32).abs_() + 1.0
    q = _randn((B, H, 1, 16), dev, 6)
    k = _randn((B, H, 1, 16), dev, 7)
    v = _randn((B, H, 1, dv), dev, 8)
    rows = (0, B // 2, B - 1)
    before = {b: (kv[b:b + 1].clone(), ks[b:b + 1].clone()) for b in rows}
    y = ops.linear_attn_step(q, k, v, kv, ks)
    for b in rows:
        kv1, ks1 = before[b]
        y1 = ops.linear_attn_step(q[b:b + 1].clone(), k[b:b + 1].clone(), v[b:b + 1].clone(), kv1, ks1)
        torch.cuda.synchronize()
        assert torch.equal(y[b], y1[0]), f"batch entry {b}"
        assert torch.equal(kv[b], kv1[0]) and torch.equal(ks[b], ks1[0]), f"states of batch entry {b}"


@pytest.mark.parametrize("D,B,w", [(64, 130, 64), (64, 130, 128), (112, 76, 128)])
def test_window_prefill_past_the_mark(dev, D, B, w):
    """Packed (B, L, 3, H, D) input, rotary, cache fill: q / k / v, the output and the cache all
    cross the mark."""
    from based_amd import ops

    L, H = 16384, 16
    assert (B - 1) * L * H * D > MARK  # the output, hence also the packed input and the cache
    _need(dev, 40)
    print(f"large offsets: window prefill D={D} B={B} L={L} w={w}", flush=True)
    qkv = _randn((B, L, 3, H, D), dev, 9)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32, device=dev) / D))
    ang = torch.outer(torch.arange(L, dtype=torch.float32, device=dev), inv)
    rope = (ang.cos().contiguous(), ang.sin().contiguous())
    cache = torch.zeros(B, L, 2, H, D, dtype=torch.bfloat16, device=dev)
    out = ops.swa_prefill(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=w, rope=rope, kv_cache=cache)
    for b in (0, B - 1):
        one = qkv[b:b + 1].clone()
        cache1 = torch.zeros(1, L, 2, H, D, dtype=torch.bfloat16, device=dev)
        out1 = ops.swa_prefill(one[:, :, 0], one[:, :, 1], one[:, :, 2], w_left=w, rope=rope, kv_cache=cache1)
        torch.cuda.synchronize()
        assert torch.equal(out[b], out1[0]), f"batch entry {b}"
        assert torch.equal(cache[b], cache1[0]), f"cache of batch entry {b}"
    assert torch.isfinite(out[B - 1].float()).all()
    # the step that follows reads and writes the cache past the mark as well
    pos = torch.full((B,), L - 1, dtype=torch.int32, device=dev)
    new = _randn((B, 1, 3, H, D), dev, 10)
    cache_b = cache[B - 1:B].clone()
    o = ops.swa_step(new[:, :, 0], new[:, :, 1], new[:, :, 2], cache, pos, w_left=w, rope=rope)
    o1 = ops.swa_step(new[B - 1:, :, 0], new[B - 1:, :, 1], new[B - 1:, :, 2], cache_b, pos[B - 1:], w_left=w, rope=rope)
    torch.cuda.synchronize()
    assert torch.equal(o[B - 1], o1[0]) and torch.equal(cache[B - 1], cache_b[0])


def test_gated_conv_past_the_mark(dev):
    from based_amd import ops

    B, L, D, K = 40, 16384, 2048, 3
    assert (B - 1) * L * 2 * D > MARK
    _need(dev, 12)
    print(f"large offsets: gated convolution B={B} L={L} D={D}", flush=True)
    u = _randn((B, L, 2 * D), dev, 11)
    wgt = _randn((D, 1, K), dev, 12)
    bias = _randn((D,), dev, 13)
    state = torch.zeros(B, D, K, dtype=torch.bfloat16, device=dev)
    y = ops.gated_conv_prefill(u, wgt, bias, state=state)
    for b in (0, B - 1):
        state1 = torch.zeros(1, D, K, dtype=torch.bfloat16, device=dev)
        y1 = ops.gated_conv_prefill(u[b:b + 1].clone(), wgt, bias, state=state1)
        torch.cuda.synchronize()
        assert torch.equal(y[b], y1[0]) and torch.equal(state[b], state1[0]), f"batch entry {b}"


def test_block_glue_past_the_mark(dev):
    from based_amd import ops

    N, D = 2_400_000, 1024
    assert (N - 1) * D > MARK
    _need(dev, 30)
    print(f"large offsets: add + RMS norm, SwiGLU, {N} rows", flush=True)
    x = _randn((N, D), dev, 14)
    res = _randn((N, D), dev, 15, dtype=torch.float32)
    wgt = _randn((D,), dev, 16)
    y, r = ops.add_rms_norm(x, res, wgt)
    tail = slice(N - 1000, N)
    y1, r1 = ops.add_rms_norm(x[tail].clone(), res[tail].clone(), wgt)
    torch.cuda.synchronize()
    assert torch.equal(y[tail], y1) and torch.equal(r[tail], r1)
    del y, r, res
    g = ops.swiglu(x.view(N // 2, 2 * D))
    g1 = ops.swiglu(x.view(N // 2, 2 * D)[N // 2 - 1000:].clone())
    torch.cuda.synchronize()
    assert torch.equal(g[N // 2 - 1000:], g1)
    # (the SwiGLU input above is 2.4e9 elements; its output stays below the mark, the norm's does not)
    assert math.prod(x.shape) > MARK
