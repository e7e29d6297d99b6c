"""Pins the CPU oracle against evidence that does not come from the oracle itself: closed
forms, brute force on tiny inputs, library routines, the reference's own compiled C++ causal
product (oracle/_ref), and the invariants the reference's test-suite relies on."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import based_oracle as O
from oracle import ref_loader


def _rand(*shape, seed=0, scale=1.0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float64) * scale).to(dtype)


# ---------------------------------------------------------------- TaylorExp
def test_taylor_shape_and_order():
    x = _rand(2, 3, 5, 16, seed=1)
    f = O.taylor_exp(x)
    assert f.shape == (2, 3, 5, 273)
    assert torch.all(f[..., 0] == 1)
    assert torch.allclose(f[..., 1:17], x / 2)                     # d^(1/4) = 2 for d = 16
    i, j = 3, 11
    assert torch.allclose(f[..., 17 + 16 * i + j], x[..., i] * x[..., j] / (math.sqrt(2) * 4))
    assert torch.allclose(f[..., 17 + 16 * j + i], f[..., 17 + 16 * i + j])  # full, not triangular


def test_taylor_zero_is_e0():
    f = O.taylor_exp(torch.zeros(1, 1, 1, 16, dtype=torch.float64))
    e0 = torch.zeros(273, dtype=torch.float64)
    e0[0] = 1
    assert torch.equal(f[0, 0, 0], e0)


def test_taylor_inner_product_closed_form():
    q, k = _rand(4, 2, 7, 16, seed=2), _rand(4, 2, 7, 16, seed=3)
    lhs = (O.taylor_exp(q) * O.taylor_exp(k)).sum(-1)
    s = (q * k).sum(-1) / 4
    assert torch.allclose(lhs, 1 + s + s * s / 2, rtol=1e-12, atol=1e-12)
    assert torch.allclose(lhs, O.taylor_dot(q, k), rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------- parallel linear attention
def _brute(q, k, v, eps):
    B, H, L, _ = q.shape
    y = torch.zeros(B, H, L, v.shape[-1], dtype=q.dtype)
    for b in range(B):
        for h in range(H):
            for i in range(L):
                num = torch.zeros(v.shape[-1], dtype=q.dtype)
                den = 0.0
                for j in range(i + 1):
                    s = float((q[b, h, i] * k[b, h, j]).sum()) / 4
                    w = 1 + s + s * s / 2
                    num += w * v[b, h, j]
                    den += w
                y[b, h, i] = num / (den + eps)
    return y


def test_quadratic_matches_brute_force():
    q, k, v = _rand(2, 2, 7, 16, seed=4), _rand(2, 2, 7, 16, seed=5), _rand(2, 2, 7, 5, seed=6)
    assert torch.allclose(O.linear_attn_quadratic(q, k, v, eps=1e-12), _brute(q, k, v, 1e-12), rtol=1e-10, atol=1e-12)


def test_cumsum_matches_quadratic():
    q, k, v = _rand(1, 3, 150, 16, seed=7), _rand(1, 3, 150, 16, seed=8), _rand(1, 3, 150, 8, seed=9)
    a = O.linear_attn_quadratic(q, k, v)
    for chunk in (1, 64, 1000):
        assert torch.allclose(O.linear_attn_cumsum(q, k, v, chunk=chunk), a, rtol=1e-9, atol=1e-11)


def test_zero_qk_is_running_mean():
    v = _rand(1, 1, 20, 4, seed=10)
    z = torch.zeros(1, 1, 20, 16, dtype=torch.float64)
    y = O.linear_attn_quadratic(z, z, v, eps=0.0)
    mean = v.cumsum(2) / torch.arange(1, 21, dtype=torch.float64)[None, None, :, None]
    assert torch.allclose(y, mean, rtol=1e-12, atol=1e-12)


def test_single_token_returns_v():
    q, k, v = _rand(1, 1, 1, 16, seed=11), _rand(1, 1, 1, 16, seed=12), _rand(1, 1, 1, 6, seed=13)
    w = O.taylor_dot(q, k)
    assert torch.allclose(O.linear_attn_quadratic(q, k, v), v * (w / (w + 1e-12))[..., None])


def test_causality():
    q, k, v = _rand(1, 2, 30, 16, seed=14), _rand(1, 2, 30, 16, seed=15), _rand(1, 2, 30, 4, seed=16)
    y0 = O.linear_attn_cumsum(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 17] += 1.0
    v2[:, :, 17] -= 2.0
    y1 = O.linear_attn_cumsum(q, k2, v2)
    assert torch.equal(y0[:, :, :17], y1[:, :, :17])
    assert not torch.allclose(y0[:, :, 17:], y1[:, :, 17:])


@pytest.mark.skipif(not ref_loader.available(), reason="oracle/_ref not built (make -C oracle)")
def test_numerator_matches_reference_cpp():
    """The reference's own CPU causal product, compiled unmodified, on E = 273, M = 64 fp32."""
    q, k = _rand(2, 3, 96, 16, seed=17, scale=0.5, dtype=torch.float32), _rand(2, 3, 96, 16, seed=18, scale=0.5, dtype=torch.float32)
    v = _rand(2, 3, 96, 64, seed=19, dtype=torch.float32)
    fq, fk = O.taylor_exp(q), O.taylor_exp(k)
    num_ref = ref_loader.causal_dot_product(fq, fk, v)
    z = torch.einsum("bhld,bhld->bhl", fq, fk.cumsum(2)) + 1e-12
    y_ref = num_ref / z[..., None]
    for y in (O.linear_attn_quadratic(q, k, v), O.linear_attn_cumsum(q, k, v)):
        assert float((y - y_ref).norm() / y_ref.norm()) < 1e-5


def test_golden_causal_product_fixture():
    """Committed output of the reference's compiled CPU causal product (written by
    tests/golden/make_causal_dot_golden.py): numerator and normaliser at E = 273, M = 64."""
    import os

    import numpy as np

    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "causal_dot_E273_M64.npz"))
    q, k, v = (torch.from_numpy(g[n]) for n in ("q", "k", "v"))
    num, den = torch.from_numpy(g["numerator"]), torch.from_numpy(g["normaliser"])
    y_gold = num / (den + 1e-12)
    for y in (O.linear_attn_quadratic(q, k, v), O.linear_attn_cumsum(q, k, v)):
        assert float((y - y_gold).norm() / y_gold.norm()) < 1e-5
    # the normaliser alone pins the closed form 1 + s + s^2/2 summed over the causal prefix
    s_ = torch.einsum("bhid,bhjd->bhij", q, k) / 4.0
    den_closed = torch.tril(1 + s_ + s_ * s_ / 2).sum(-1, keepdim=True)
    assert float((den - den_closed).norm() / den_closed.norm()) < 1e-5


def test_smoke_script_formulation():
    """The comparison the reference's causal-product smoke script makes (positive q, k, v;
    cumulative-sum form), whose recorded difference is 7.4e-05 in bf16: here in fp64 on the
    273-dim features the two forms agree to round-off."""
    q, k, v = _rand(1, 2, 40, 16, seed=20).abs(), _rand(1, 2, 40, 16, seed=21).abs(), _rand(1, 2, 40, 8, seed=22).abs()
    fq, fk = O.taylor_exp(q), O.taylor_exp(k)
    slow = (fq.unsqueeze(-2) * (fk.unsqueeze(-2) * v.unsqueeze(-1)).cumsum(dim=2)).sum(-1) / (
        (fq * fk.cumsum(dim=2)).sum(-1, keepdim=True) + 1e-12)
    assert torch.allclose(O.linear_attn_cumsum(q, k, v), slow, rtol=1e-10, atol=1e-12)


# ---------------------------------------------------------------- decode state and step
def test_state_closed_form():
    k, v = _rand(2, 2, 9, 16, seed=23), _rand(2, 2, 9, 5, seed=24)
    kv, ks = O.linear_attn_prefill_state(k, v)
    assert kv.shape == (2, 2, 1, 5, 273) and ks.shape == (2, 2, 1, 1, 273)
    fk = O.taylor_exp(k)
    e, f = 3, 140
    assert torch.allclose(kv[:, :, 0, e, f], (v[..., e] * fk[..., f]).sum(-1))
    assert torch.allclose(ks[:, :, 0, 0, f], fk[..., f].sum(-1))


def test_recurrent_equals_parallel():
    """prefill P then step T == parallel over P + T (the reference's test_generation invariant)."""
    P, T = 11, 6
    q, k, v = _rand(2, 2, P + T, 16, seed=25), _rand(2, 2, P + T, 16, seed=26), _rand(2, 2, P + T, 4, seed=27)
    y_par = O.linear_attn_quadratic(q, k, v)
    kv, ks = O.linear_attn_prefill_state(k[:, :, :P], v[:, :, :P])
    kv, ks = kv.clone(), ks.clone()
    ptr = kv.data_ptr()
    for t in range(P, P + T):
        y = O.linear_attn_step(kv, ks, q[:, :, t:t + 1], k[:, :, t:t + 1], v[:, :, t:t + 1])
        assert torch.allclose(y, y_par[:, :, t:t + 1], rtol=1e-9, atol=1e-11)
    assert kv.data_ptr() == ptr  # in place
    kv2, ks2 = O.linear_attn_prefill_state(k, v)
    assert torch.allclose(kv, kv2) and torch.allclose(ks, ks2)


# ---------------------------------------------------------------- sliding window
def test_window_covering_sequence_is_causal_sdpa():
    q, k, v = (_rand(2, 40, 3, 64, seed=s, dtype=torch.float32) for s in (28, 29, 30))
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True).transpose(1, 2)
    assert torch.allclose(O.sliding_window_attn(q, k, v, w_left=64), ref, rtol=1e-4, atol=1e-5)
    assert torch.allclose(O.sliding_window_attn(q, k, v, w_left=39), ref, rtol=1e-4, atol=1e-5)


def test_window_zero_returns_v():
    q, k, v = (_rand(1, 9, 2, 64, seed=s, dtype=torch.float32) for s in (31, 32, 33))
    assert torch.allclose(O.sliding_window_attn(q, k, v, w_left=0), v, atol=1e-6)


def test_zero_query_is_window_mean():
    L, w = 150, 64
    v = _rand(1, L, 1, 64, seed=34, dtype=torch.float32)
    z = torch.zeros_like(v)
    o = O.sliding_window_attn(z, _rand(1, L, 1, 64, seed=35, dtype=torch.float32), v, w_left=w)
    for i in (0, 5, 64, 65, 149):
        lo = max(0, i - w)
        assert torch.allclose(o[0, i, 0], v[0, lo:i + 1, 0].mean(0), atol=1e-5)


def test_window_brute_force_elements():
    L, w = 100, 64
    q, k, v = (_rand(1, L, 1, 64, seed=s, dtype=torch.float32) for s in (36, 37, 38))
    o = O.sliding_window_attn(q, k, v, w_left=w)
    for i in (0, 63, 64, 65, 99):
        lo = max(0, i - w)
        s = (k[0, lo:i + 1, 0] @ q[0, i, 0]) / 8.0
        p = torch.softmax(s, 0)
        assert torch.allclose(o[0, i, 0], p @ v[0, lo:i + 1, 0], atol=1e-5)
    assert (i - lo + 1) == 65  # 64 to the left plus the token itself


def test_window_decode_equals_prefill():
    L, w = 140, 64
    q, k, v = (_rand(2, L, 2, 64, seed=s, dtype=torch.float32) for s in (39, 40, 41))
    ref = O.sliding_window_attn(q, k, v, w_left=w)
    cache = torch.zeros(2, L, 2, 2, 64)
    P = 60
    cache[:, :P, 0], cache[:, :P, 1] = k[:, :P], v[:, :P]
    for t in range(P, L):  # crosses pos = 63, 64, 65, 128, 129
        o = O.sliding_window_step(q[:, t:t + 1], k[:, t:t + 1], v[:, t:t + 1], cache, t, w_left=w)
        assert torch.allclose(o, ref[:, t:t + 1], atol=1e-5)


# ---------------------------------------------------------------- stack glue
def test_rms_norm_swiglu_conv():
    x = _rand(2, 5, 8, seed=42, dtype=torch.float32)
    w = _rand(8, seed=43, dtype=torch.float32)
    assert torch.allclose(O.rms_norm(x, w, 1e-5), x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w, atol=1e-6)
    w1, w2 = _rand(12, 8, seed=44, dtype=torch.float32), _rand(8, 6, seed=45, dtype=torch.float32)
    h = x @ w1.T
    assert torch.allclose(O.swiglu_mlp(x, w1, w2), (h[..., :6] * F.silu(h[..., 6:])) @ w2.T, atol=1e-5)
    cw = _rand(8, 3, seed=46, dtype=torch.float32)
    ref = F.conv1d(x.transpose(1, 2), cw[:, None, :], padding=2, groups=8)[..., :5].transpose(1, 2)
    assert torch.allclose(O.short_conv(x, cw), ref, atol=1e-6)
    state = torch.zeros(2, 8, 3)
    for t in range(5):
        y = O.short_conv_step(x[:, t:t + 1], state, cw)
        assert torch.allclose(y, ref[:, t:t + 1], atol=1e-6)


def test_gated_short_conv_against_library_and_brute_force():
    """Gated short convolution: F.conv1d(groups=D, padding=K-1) truncated to L (the module form
    the reference uses), F.silu, per-element brute force on a tiny case, and step == parallel."""
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(5)
    B, L, D, K = 2, 11, 6, 3
    u = torch.randn(B, L, 2 * D, generator=g)
    w = torch.randn(D, K, generator=g)
    bias = torch.randn(D, generator=g)
    for b_ in (None, bias):
        y = O.gated_short_conv(u, w, b_)
        conv = F.conv1d(u[..., :D].transpose(1, 2), w[:, None, :], bias=b_, groups=D, padding=K - 1)[..., :L].transpose(1, 2)
        assert torch.allclose(y, F.silu(conv) * u[..., D:], atol=1e-6)
    # brute force: y[b,l,c] = silu(sum_j w[c,j] u1[b,l-K+1+j,c]) * u2[b,l,c]
    y = O.gated_short_conv(u, w)
    for (b, l, c) in [(0, 0, 0), (1, 1, 3), (0, 7, 5), (1, 10, 2)]:
        acc = sum(float(w[c, j]) * float(u[b, l - K + 1 + j, c]) for j in range(K) if l - K + 1 + j >= 0)
        ref = acc / (1 + math.exp(-acc)) * float(u[b, l, D + c])
        assert abs(float(y[b, l, c]) - ref) < 1e-5
    # step == parallel: prefix through the parallel form leaves the state, then single tokens
    P = 7
    state = torch.zeros(B, D, K)
    state[..., -min(K, P):] = u[:, P - min(K, P):P, :D].transpose(1, 2)
    for t in range(P, L):
        yt = O.gated_short_conv_step(u[:, t:t + 1], state, w, bias)
        assert torch.allclose(yt[:, 0], O.gated_short_conv(u, w, bias)[:, t], atol=1e-5)


def test_rotary_embedding_properties():
    """RoPE: identity at position 0, norm preservation, <R_m q, R_n k> depends on m - n only,
    and a brute-force complex multiplication (x_i + i x_{i+D/2}) * exp(i p w_i)."""
    g = torch.Generator().manual_seed(9)
    B, L, H, D = 2, 12, 3, 64
    x = torch.randn(B, L, H, D, generator=g)
    y = torch.randn(B, L, H, D, generator=g)
    pos = torch.arange(L)
    rx = O.rotary_embedding(x, pos)
    assert torch.allclose(rx[:, 0], x[:, 0], atol=1e-6)
    assert torch.allclose(rx.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)
    # relative-position property: shift both positions by 5
    ry = O.rotary_embedding(y, pos)
    rx5, ry5 = O.rotary_embedding(x, pos + 5), O.rotary_embedding(y, pos + 5)
    d0 = torch.einsum("bmhd,bnhd->bhmn", rx, ry)
    d5 = torch.einsum("bmhd,bnhd->bhmn", rx5, ry5)
    assert torch.allclose(d0, d5, atol=2e-4)
    # complex brute force on a few entries
    for (b, l, h, i) in [(0, 3, 1, 0), (1, 11, 2, 31), (0, 7, 0, 13)]:
        w = 10000.0 ** (-2.0 * i / D)
        z = complex(float(x[b, l, h, i]), float(x[b, l, h, i + D // 2])) * complex(math.cos(l * w), math.sin(l * w))
        assert abs(float(rx[b, l, h, i]) - z.real) < 1e-5 and abs(float(rx[b, l, h, i + D // 2]) - z.imag) < 1e-5


def test_rotary_embedding_partial_and_interleaved():
    """The two other rotary shapes the reference's constructor admits (rotary_emb_dim < head dim,
    rotary_emb_interleaved; slide_attention.py:346-355): each against a complex multiplication of
    ITS pairing, channels past rotary_dim untouched, and the interleaved layout as the half-split
    one under the channel permutation that maps pair (2i, 2i+1) to (i, i + R/2)."""
    g = torch.Generator().manual_seed(10)
    B, L, H, D, R = 2, 9, 2, 48, 32
    x = torch.randn(B, L, H, D, generator=g)
    pos = torch.arange(3, 3 + L)
    part = O.rotary_embedding(x, pos, rotary_dim=R)
    assert torch.equal(part[..., R:], x[..., R:])
    assert torch.allclose(part[..., :R], O.rotary_embedding(x[..., :R], pos), atol=1e-6)
    inter = O.rotary_embedding(x, pos, rotary_dim=R, interleaved=True)
    assert torch.equal(inter[..., R:], x[..., R:])
    for (b, l, h, i) in [(0, 0, 0, 0), (1, 8, 1, 15), (0, 4, 1, 7)]:
        w = 10000.0 ** (-2.0 * i / R)
        p = int(pos[l])
        z = complex(float(x[b, l, h, i]), float(x[b, l, h, i + R // 2])) * complex(math.cos(p * w), math.sin(p * w))
        assert abs(float(part[b, l, h, i]) - z.real) < 1e-5 and abs(float(part[b, l, h, i + R // 2]) - z.imag) < 1e-5
        z = complex(float(x[b, l, h, 2 * i]), float(x[b, l, h, 2 * i + 1])) * complex(math.cos(p * w), math.sin(p * w))
        assert abs(float(inter[b, l, h, 2 * i]) - z.real) < 1e-5 and abs(float(inter[b, l, h, 2 * i + 1]) - z.imag) < 1e-5
    perm = torch.cat([torch.arange(0, R, 2), torch.arange(1, R, 2)])          # half-split position -> interleaved channel
    half = O.rotary_embedding(x[..., :R][..., perm], pos)
    assert torch.allclose(half, inter[..., :R][..., perm], atol=1e-6)
    assert torch.allclose(inter.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)


def test_add_layer_norm_against_library_routine():
    """nn.LayerNorm glue of a config without rms_norm: F.layer_norm on the cast sum, the fp32 stream
    handed on unrounded, and one row by hand."""
    g = torch.Generator().manual_seed(12)
    x = torch.randn(3, 5, 32, generator=g)
    res = torch.randn(3, 5, 32, generator=g)
    w, b = torch.randn(32, generator=g), torch.randn(32, generator=g)
    y, r = O.add_layer_norm(x, res, w, b, eps=1e-5)
    assert torch.allclose(y, F.layer_norm(x + res, (32,), w, b, 1e-5), atol=1e-5) and torch.equal(r, x + res)
    y, r = O.add_layer_norm(x, None, w, None, eps=1e-5)
    assert torch.allclose(y, F.layer_norm(x, (32,), w, None, 1e-5), atol=1e-5) and torch.equal(r, x)
    # bf16 activations on an fp32 stream: normalised from the bf16-rounded sum, stream kept in fp32
    xb = x.bfloat16()
    y, r = O.add_layer_norm(xb, res, w.bfloat16(), b.bfloat16(), eps=1e-5)
    assert y.dtype == torch.bfloat16 and r.dtype == torch.float32 and torch.equal(r, xb.float() + res)
    want = F.layer_norm((xb.float() + res).bfloat16(), (32,), w.bfloat16(), b.bfloat16(), 1e-5)
    assert torch.allclose(y.float(), want.float(), atol=4e-2)
    # by hand: [1, 3] -> mean 2, var 1 -> [-1, 1] * w + b
    y, _ = O.add_layer_norm(torch.tensor([[1.0, 3.0]]), None, torch.tensor([2.0, 3.0]), torch.tensor([0.5, -0.5]), eps=0.0)
    assert torch.allclose(y, torch.tensor([[-1.5, 2.5]]), atol=1e-6)


def test_add_rms_norm_closed_form_cast_order_and_fp32_stream():
    """The prenorm glue (block.py:134-139): (i) closed form on hand-made rows; (ii) the sum is cast to
    the activation dtype BEFORE the norm (a bf16 activation plus an fp32 residual is normalised from
    the bf16-rounded sum); (iii) the residual stream that is handed on is the UNROUNDED fp32 sum."""
    # (i) r = [3, 4] + [0, 0]: mean(r^2) = 12.5, y = r / sqrt(12.5 + eps) * w
    x = torch.tensor([[3.0, 4.0]])
    w = torch.tensor([2.0, 0.5])
    y, r = O.add_rms_norm(x, None, w, eps=0.0, residual_in_fp32=True)
    assert torch.allclose(y, torch.tensor([[3.0 / math.sqrt(12.5) * 2.0, 4.0 / math.sqrt(12.5) * 0.5]]), atol=1e-6)
    assert torch.equal(r, x)
    y, r = O.add_rms_norm(x, torch.tensor([[1.0, -4.0]]), w, eps=0.0)
    assert torch.allclose(y, torch.tensor([[4.0 / math.sqrt(8.0) * 2.0, 0.0]]), atol=1e-6) and torch.equal(r, torch.tensor([[4.0, 0.0]]))
    # eps enters under the root
    y, _ = O.add_rms_norm(torch.tensor([[0.0, 0.0]]), None, w, eps=1e-5)
    assert torch.equal(y, torch.zeros(1, 2))
    y, _ = O.add_rms_norm(torch.tensor([[1e-3, 0.0]]), None, torch.ones(2), eps=1e-5)
    assert abs(float(y[0, 0]) - 1e-3 / math.sqrt(0.5e-6 + 1e-5)) < 1e-6
    # (ii) + (iii): x bf16, residual fp32 with bits below bf16 resolution
    xb = torch.tensor([[1.0, 2.0, -3.0, 0.5]], dtype=torch.bfloat16)
    res = torch.tensor([[0.001953125 * 0.37, 0.00390625 * 0.41, 0.0078125 * 0.3, 1.0 / 1024 * 0.45]])  # sub-ulp parts
    wb = torch.ones(4, dtype=torch.bfloat16)
    y, r = O.add_rms_norm(xb, res, wb, eps=1e-5, residual_in_fp32=True)
    exact_sum = xb.float() + res
    assert r.dtype == torch.float32 and torch.equal(r, exact_sum)           # stream: exact fp32 sum
    rounded = exact_sum.to(torch.bfloat16)
    assert not torch.equal(rounded.float(), exact_sum)                        # the case is discriminating
    expect = (rounded.float() * torch.rsqrt(rounded.float().square().mean(-1, keepdim=True) + 1e-5)).to(torch.bfloat16)
    assert y.dtype == torch.bfloat16 and torch.equal(y, expect)              # norm of the ROUNDED sum
    # without an fp32 stream the sum itself is what torch promotion gives, handed on as is
    y2, r2 = O.add_rms_norm(xb, res.to(torch.bfloat16), wb, eps=1e-5, residual_in_fp32=False)
    assert r2.dtype == torch.bfloat16


def test_gated_mlp_layouts():
    """mlp.py:141-157: F.glu for the sigmoid gate, y * act(gate) for base, act(fc1) * fc3 for alt."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(3, 5, 8, generator=g)
    w1, w2 = torch.randn(12, 8, generator=g), torch.randn(8, 6, generator=g)
    h = x @ w1.T
    assert torch.allclose(O.gated_mlp(x, w1, w2, activation="glu"), F.glu(h, dim=-1) @ w2.T, atol=1e-5)
    assert torch.allclose(O.gated_mlp(x, w1, w2, activation="swiglu"), O.swiglu_mlp(x, w1, w2), atol=1e-6)
    y, gate = h[..., :6], h[..., 6:]
    assert torch.allclose(O.gated_mlp(x, w1, w2, activation="geglu"), (y * 0.5 * gate * (1 + torch.erf(gate / math.sqrt(2)))) @ w2.T, atol=1e-5)
    w1a, w3a, w2a = torch.randn(6, 8, generator=g), torch.randn(6, 8, generator=g), torch.randn(8, 6, generator=g)
    a = x @ w1a.T
    ref = ((0.5 * a * (1 + torch.erf(a / math.sqrt(2)))) * (x @ w3a.T)) @ w2a.T
    assert torch.allclose(O.gated_mlp(x, w1a, w2a, w3a, activation="geglu"), ref, atol=1e-5)
    b1, b2 = torch.randn(12, generator=g), torch.randn(8, generator=g)
    assert torch.allclose(O.gated_mlp(x, w1, w2, activation="swiglu", fc1_b=b1, fc2_b=b2),
                          ((h + b1)[..., :6] * F.silu((h + b1)[..., 6:])) @ w2.T + b2, atol=1e-5)


def _tiny_stack_config(**over):
    cfg = dict(
        n_embd=128, n_head=2, n_layer=3, n_inner=256, vocab_size=96, pad_vocab_size_multiple=8, rms_norm=True,
        residual_in_fp32=True, activation_function="swiglu", mlp_type="base", layer_norm_epsilon=1e-5,
        mlp_fc1_bias=False, mlp_fc2_bias=False, qkv_proj_bias=False, out_proj_bias=False, max_position_embeddings=0,
        rotary_emb_fraction=0.0, scale_attn_weights=True,
        mixer={"_target_": "based.models.mixers.convolution.BaseConv", "l_max": 64, "use_bias": True, "expand_proj": 4,
               "kernel_size": 3},
        alt_mixer={"_target_": "based.models.mixers.linear_attention.LinearAttention", "l_max": 64,
                   "feature_map": {"_target_": "based.models.mixers.linear_attention.TaylorExp", "input_dim": 16},
                   "feature_dim": 16, "num_heads": 2},
        alt_mixer_layers=[1],
        alt_mixer_2={"_target_": "based.models.mixers.slide_attention.SlidingAttention", "window_size": 128,
                     "num_heads": 2, "causal": True},
        alt_mixer_2_layers=[2],
    )
    cfg.update(over)
    return cfg


def test_stack_forward_against_hand_unrolled_modules():
    """The composition (block.py:134-163, gpt.py:622-736) against the same stack unrolled by hand
    from torch building blocks that share no code with the oracle's functions: nn.Embedding,
    nn.Linear, nn.Conv1d (depthwise, padding K-1, truncated), F.scaled_dot_product_attention for
    a window that covers the sequence, and the Taylor weights 1 + s + s^2/2 written out."""
    import torch.nn as nn

    from based_amd.stack import GPTLMHeadModel, StackConfig

    torch.manual_seed(3)
    cfg = _tiny_stack_config(rotary_emb_fraction=0.0, max_position_embeddings=32)
    model = GPTLMHeadModel(StackConfig(**cfg))            # only used as a container of random weights
    sd = {k: v.detach().clone() for k, v in model.state_dict().items()}
    for k in sd:                                          # make every norm weight non-trivial
        if "norm" in k or "ln_f" in k:
            sd[k] = 1.0 + 0.1 * torch.randn_like(sd[k])
    B, L, D, H = 2, 20, 128, 2
    ids = torch.randint(0, 96, (B, L))
    got = O.stack_forward(ids, sd, cfg)

    def rms(x, w):
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w

    emb = nn.Embedding.from_pretrained(sd["transformer.embeddings.word_embeddings.weight"])
    h = emb(ids) + sd["transformer.embeddings.position_embeddings.weight"][:L]
    res = None
    for i in range(3):
        pre = f"transformer.layers.{i}."
        res = h if res is None else h + res
        x = rms(res, sd[pre + "norm1.weight"])
        m = pre + "mixer."
        if i == 0:
            u = x @ sd[m + "in_proj.weight"].T + sd[m + "in_proj.bias"]
            conv = nn.Conv1d(256, 256, 3, groups=256, padding=2, bias=False)
            conv.weight.data.copy_(sd[m + "conv.conv.weight"])
            c = conv(u[..., :256].transpose(1, 2))[..., :L].transpose(1, 2)
            h = (F.silu(c) * u[..., 256:]) @ sd[m + "out_proj.weight"].T + sd[m + "out_proj.bias"]
        elif i == 1:
            q = (x @ sd[m + "proj_q.weight"].T).view(B, L, H, 16).transpose(1, 2)
            k = (x @ sd[m + "proj_k.weight"].T).view(B, L, H, 16).transpose(1, 2)
            v = (x @ sd[m + "proj_v.weight"].T).view(B, L, H, 64).transpose(1, 2)
            s = q @ k.transpose(-1, -2) / 4.0
            a = torch.tril(1 + s + s * s / 2)
            y = (a @ v) / (a.sum(-1, keepdim=True) + 1e-12)
            h = y.transpose(1, 2).reshape(B, L, D) @ sd[m + "out_proj.weight"].T
        else:
            qkv = (x @ sd[m + "Wqkv.weight"].T).view(B, L, 3, H, 64)
            o = F.scaled_dot_product_attention(qkv[:, :, 0].transpose(1, 2), qkv[:, :, 1].transpose(1, 2),
                                               qkv[:, :, 2].transpose(1, 2), is_causal=True)   # window 64 >= L
            h = o.transpose(1, 2).reshape(B, L, D) @ sd[m + "out_proj.weight"].T
        res = h + res
        x = rms(res, sd[pre + "norm2.weight"])
        yv, gate = (x @ sd[pre + "mlp.fc1.weight"].T).chunk(2, -1)
        h = (yv * F.silu(gate)) @ sd[pre + "mlp.fc2.weight"].T
    x = rms(h + res, sd["transformer.ln_f.weight"])
    ref = x @ sd["lm_head.weight"].T
    assert got.shape == ref.shape == (B, L, 96)
    assert torch.allclose(got, ref, atol=2e-5, rtol=1e-5)
    # causality of the whole stack: changing the last token leaves earlier logits alone
    ids2 = ids.clone()
    ids2[:, -1] = (ids2[:, -1] + 1) % 96
    assert torch.equal(O.stack_forward(ids2, sd, cfg)[:, :-1], got[:, :-1])


def test_stack_forward_layer_norm_config_against_nn_modules():
    """A reference-format config that omits rms_norm (nn.LayerNorm, gpt.py:352,537) and rotates a
    part of the head in the interleaved layout: the composition against nn.LayerNorm /
    nn.Linear building blocks, the mixer (one window layer) unrolled by hand."""
    import torch.nn as nn

    from based_amd.stack import GPTLMHeadModel, StackConfig

    torch.manual_seed(5)
    cfg = _tiny_stack_config(n_layer=1, alt_mixer_layers=[], alt_mixer_2_layers=[0], rotary_emb_fraction=0.5,
                             rotary_emb_interleaved=True, qkv_proj_bias=True, out_proj_bias=True)
    del cfg["rms_norm"]
    full = vars(StackConfig.from_reference_dict(cfg))
    assert full["rms_norm"] is False
    model = GPTLMHeadModel(StackConfig.from_reference_dict(cfg))
    assert isinstance(model.transformer.ln_f, nn.LayerNorm)
    sd = {k: v.detach().clone() for k, v in model.state_dict().items()}
    for k in sd:
        if "norm" in k or "ln_f" in k or k.endswith("bias"):
            sd[k] = (1.0 if k.endswith("weight") else 0.0) + 0.1 * torch.randn_like(sd[k])
    B, L, D, H = 2, 12, 128, 2
    ids = torch.randint(0, 96, (B, L))
    got = O.stack_forward(ids, sd, full)

    def ln(x, name):
        m = nn.LayerNorm(D, eps=1e-5)
        m.weight.data.copy_(sd[name + ".weight"])
        m.bias.data.copy_(sd[name + ".bias"])
        return m(x)

    pre = "transformer.layers.0."
    res = F.embedding(ids, sd["transformer.embeddings.word_embeddings.weight"])
    x = ln(res, pre + "norm1")
    qkv = (x @ sd[pre + "mixer.Wqkv.weight"].T + sd[pre + "mixer.Wqkv.bias"]).view(B, L, 3, H, 64)
    q, k, v = qkv[:, :, 0].clone(), qkv[:, :, 1].clone(), qkv[:, :, 2]
    for t in (q, k):            # interleaved rotary of the first 32 channels, pair by pair
        for l in range(L):
            for i in range(16):
                a = l * 10000.0 ** (-2.0 * i / 32)
                x0, x1 = t[:, l, :, 2 * i].clone(), t[:, l, :, 2 * i + 1].clone()
                t[:, l, :, 2 * i] = x0 * math.cos(a) - x1 * math.sin(a)
                t[:, l, :, 2 * i + 1] = x0 * math.sin(a) + x1 * math.cos(a)
    o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True)
    h = o.transpose(1, 2).reshape(B, L, D) @ sd[pre + "mixer.out_proj.weight"].T + sd[pre + "mixer.out_proj.bias"]
    res = h + res
    x = ln(res, pre + "norm2")
    yv, gate = (x @ sd[pre + "mlp.fc1.weight"].T).chunk(2, -1)
    h = (yv * F.silu(gate)) @ sd[pre + "mlp.fc2.weight"].T
    ref = ln(h + res, "transformer.ln_f") @ sd["lm_head.weight"].T
    assert torch.allclose(got, ref, atol=3e-5, rtol=1e-5)
