"""GPU parity of the linear-attention prefill kernels (through the C ABI) against the oracle."""
import math

import pytest
import torch

from conftest import rel_l2
from oracle import based_oracle as O

pytestmark = pytest.mark.gpu
TOL = {torch.bfloat16: 1e-2, torch.float32: 1e-4}  # rel-L2 bounds of the build target


def _qkv(B, H, L, dv, dtype, seed, qk_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, H, L, 16, generator=g) * qk_scale).to(dtype)
    k = (torch.randn(B, H, L, 16, generator=g) * qk_scale).to(dtype)
    v = torch.randn(B, H, L, dv, generator=g).to(dtype)
    return q, k, v


def _check(dev, q, k, v, dtype, with_state=True):
    from based_amd import ops

    y_ref = O.linear_attn_cumsum(q.float(), k.float(), v.float())
    y, kv, ks = ops.linear_attn_prefill(q.to(dev), k.to(dev), v.to(dev), return_state=with_state)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == y_ref.shape
    assert torch.isfinite(y.float()).all()
    assert rel_l2(y.float(), y_ref) < TOL[dtype]
    if with_state:
        kv_ref, ks_ref = O.linear_attn_prefill_state(k.float(), v.float())
        assert kv.shape == kv_ref.shape and ks.shape == ks_ref.shape
        # states accumulate products of bf16 operands in fp32: bf16-level agreement for the
        # MFMA path, fp32-level for the fp32 path
        stol = 5e-3 if dtype == torch.bfloat16 else 1e-5
        assert rel_l2(kv, kv_ref) < stol
        assert rel_l2(ks, ks_ref) < stol
        # the constant feature's entry of the normaliser state counts the tokens exactly
        assert torch.all(ks[..., 0] == q.shape[2])
    return y


@pytest.mark.parametrize("B,H,L,dv", [(1, 2, 64, 64), (2, 3, 1, 64), (1, 2, 5, 64), (1, 1, 65, 64),
                                      (1, 2, 100, 64), (2, 2, 128, 64), (1, 2, 200, 128), (1, 16, 1024, 64),
                                      (1, 2, 333, 128)])
def test_bf16_mfma_matches_oracle(dev, B, H, L, dv):
    print(f"prefill bf16 case B={B} H={H} L={L} dv={dv}", flush=True)
    q, k, v = _qkv(B, H, L, dv, torch.bfloat16, seed=7)
    _check(dev, q, k, v, torch.bfloat16)


@pytest.mark.parametrize("B,H,L,dv", [(1, 2, 200, 112), (2, 3, 65, 112), (1, 2, 130, 16), (1, 2, 100, 48),
                                      (1, 1, 77, 80), (1, 2, 64, 96), (1, 1, 150, 176), (1, 2, 1, 112)])
def test_bf16_mfma_head_dims_that_are_no_multiple_of_64(dev, B, H, L, dv):
    """Head dims in whole 16-channel tiles: the last 64-channel block of a workgroup grid runs with
    fewer live tiles (112 = 64 + 48 is the released 1B / 1.3B shape: n_embd 1792 over 16 heads).
    Outputs AND states against the oracle; the channels past dv must not leak into anything (the
    output and state tensors are exactly dv wide, so an out-of-range store would corrupt a
    neighbouring head, which the comparison would show)."""
    print(f"prefill bf16 odd-dv case B={B} H={H} L={L} dv={dv}", flush=True)
    q, k, v = _qkv(B, H, L, dv, torch.bfloat16, seed=23)
    _check(dev, q, k, v, torch.bfloat16)


def test_bf16_mfma_dv112_projection_layout_split_and_steps(dev):
    """dv = 112 in the layout the module hands over ((B, L, H*112) projections viewed (B, H, L, 112)),
    scanned in one pass and as segments, then decoded on: every step equals the parallel form."""
    from based_amd import ops

    B, H, L, T, dv = 2, 16, 700, 5, 112
    g = torch.Generator().manual_seed(24)
    qp = torch.randn(B, L + T, H * 16, generator=g).bfloat16()
    kp = torch.randn(B, L + T, H * 16, generator=g).bfloat16()
    vp = torch.randn(B, L + T, H * dv, generator=g).bfloat16()
    view = lambda t, d: t.view(B, L + T, H, d).transpose(1, 2)
    y_ref = O.linear_attn_cumsum(view(qp, 16).float(), view(kp, 16).float(), view(vp, dv).float())
    qd, kd, vd = view(qp.to(dev), 16), view(kp.to(dev), 16), view(vp.to(dev), dv)
    y1, kv1, ks1 = ops.linear_attn_prefill(qd[:, :, :L], kd[:, :, :L], vd[:, :, :L], return_state=True, split=False)
    y2, kv2, ks2 = ops.linear_attn_prefill(qd[:, :, :L], kd[:, :, :L], vd[:, :, :L], return_state=True, split=3)
    assert y1.transpose(1, 2).is_contiguous()
    assert rel_l2(y1.float(), y_ref[:, :, :L]) < 1e-2 and rel_l2(y2.float(), y_ref[:, :, :L]) < 1e-2
    kv_ref, ks_ref = O.linear_attn_prefill_state(view(kp, 16)[:, :, :L].float(), view(vp, dv)[:, :, :L].float())
    for kv, ks in ((kv1, ks1), (kv2, ks2)):
        assert rel_l2(kv, kv_ref) < 5e-3 and rel_l2(ks, ks_ref) < 5e-3
    for t in range(L, L + T):
        y = ops.linear_attn_step(qd[:, :, t:t + 1], kd[:, :, t:t + 1], vd[:, :, t:t + 1], kv1, ks1)
        assert rel_l2(y.float(), y_ref[:, :, t:t + 1]) < 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_golden_reference_causal_product(dev, dtype):
    """Both prefill kernels against the committed output of the reference's compiled CPU causal
    product (tests/golden/causal_dot_E273_M64.npz; inputs are bf16-representable)."""
    import os

    import numpy as np
    from based_amd import ops

    print(f"prefill golden case dtype={dtype}", flush=True)
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "causal_dot_E273_M64.npz"))
    q, k, v = (torch.from_numpy(g[n]).to(dtype) for n in ("q", "k", "v"))
    y_gold = torch.from_numpy(g["numerator"]) / (torch.from_numpy(g["normaliser"]) + 1e-12)
    y, _, _ = ops.linear_attn_prefill(q.to(dev), k.to(dev), v.to(dev), return_state=False)
    torch.cuda.synchronize()
    assert rel_l2(y.float(), y_gold) < TOL[dtype]


def test_bf16_small_qk_scale(dev):
    """q, k scaled by 1/sqrt(16) as in the reference's CPU-runnable configuration."""
    q, k, v = _qkv(1, 4, 512, 64, torch.bfloat16, seed=8, qk_scale=0.25)
    _check(dev, q, k, v, torch.bfloat16)


def test_config1_fp32(dev):
    """B=1, H=16, L=1024, d=16, dv=64 fp32, q,k ~ N(0,1)/sqrt(16), eps 1e-12: rel-L2 <= 1e-4."""
    print("prefill fp32 config-1 case", flush=True)
    q, k, v = _qkv(1, 16, 1024, 64, torch.float32, seed=0, qk_scale=1 / math.sqrt(16))
    _check(dev, q, k, v, torch.float32)


@pytest.mark.parametrize("B,H,L,dv,dtype", [(1, 2, 37, 64, torch.float32), (2, 1, 9, 32, torch.float32),
                                            (1, 2, 70, 24, torch.bfloat16), (1, 1, 50, 192, torch.float32)])
def test_fp32_kernel_shapes(dev, B, H, L, dv, dtype):
    print(f"prefill f32-kernel case B={B} H={H} L={L} dv={dv} {dtype}", flush=True)
    q, k, v = _qkv(B, H, L, dv, dtype, seed=9)
    _check(dev, q, k, v, dtype)


def test_strided_projection_views(dev):
    """Inputs as the module produces them: (B, L, H*d) projections viewed (B, H, L, d)."""
    from based_amd import ops

    B, H, L, dv = 2, 4, 150, 64
    g = torch.Generator().manual_seed(10)
    qp = torch.randn(B, L, H * 16, generator=g).bfloat16()
    kp = torch.randn(B, L, H * 16, generator=g).bfloat16()
    vp = torch.randn(B, L, H * dv, generator=g).bfloat16()
    view = lambda t, d: t.view(B, L, H, d).transpose(1, 2)
    y_ref = O.linear_attn_cumsum(view(qp, 16).float(), view(kp, 16).float(), view(vp, dv).float())
    y, _, _ = ops.linear_attn_prefill(view(qp.to(dev), 16), view(kp.to(dev), 16), view(vp.to(dev), dv))
    assert rel_l2(y.float(), y_ref) < 1e-2
    # output is laid out (B, L, H, dv): the 'b h l d -> b l (h d)' rearrange is a free view
    assert y.transpose(1, 2).is_contiguous()


def test_no_state_variant(dev):
    q, k, v = _qkv(1, 2, 96, 64, torch.bfloat16, seed=11)
    _check(dev, q, k, v, torch.bfloat16, with_state=False)


def test_prefill_then_steps_equal_parallel(dev):
    """The reference's own invariant (recurrent == parallel): prefill P tokens, decode T more
    with the step kernel, compare every decoded position with a prefill over P + T tokens."""
    from based_amd import ops

    B, H, dv, P, T = 2, 4, 64, 130, 6
    q, k, v = _qkv(B, H, P + T, dv, torch.bfloat16, seed=12)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y_all, _, _ = ops.linear_attn_prefill(qd, kd, vd)
    _, kv, ks = ops.linear_attn_prefill(qd[:, :, :P], kd[:, :, :P], vd[:, :, :P], return_state=True)
    y_ref = O.linear_attn_cumsum(q.float(), k.float(), v.float())
    for t in range(P, P + T):
        y = ops.linear_attn_step(qd[:, :, t:t + 1], kd[:, :, t:t + 1], vd[:, :, t:t + 1], kv, ks)
        assert rel_l2(y.float(), y_all[:, :, t:t + 1].float()) < 1e-2
        assert rel_l2(y.float(), y_ref[:, :, t:t + 1]) < 1e-2


def test_mfma_vs_fp32_kernel_long(dev):
    """Two independent GPU implementations agree on a sequence the CPU oracle would take
    minutes on (L = 4096, B = 2): bf16 MFMA scan vs fp32 recurrent kernel on the same
    bf16-rounded inputs."""
    from based_amd import ops

    q, k, v = _qkv(2, 16, 4096, 64, torch.bfloat16, seed=13)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, kv1, ks1 = ops.linear_attn_prefill(qd, kd, vd, return_state=True)
    y2, kv2, ks2 = ops.linear_attn_prefill(qd.float(), kd.float(), vd.float(), return_state=True)
    assert rel_l2(y1.float(), y2) < 1e-2
    assert rel_l2(kv1, kv2) < 5e-3
    assert rel_l2(ks1, ks2) < 5e-3


@pytest.mark.parametrize("scale", [0.25, 3.0, 8.0])
@pytest.mark.parametrize("split", [False, 4])
def test_input_magnitudes(dev, scale, split):
    """q, k well below and well above unit scale (scores up to a few hundred: the second-order term
    dominates; the normaliser's second-moment operand is split into two bf16 halves): the MFMA
    scan stays finite and agrees with the fp32 recurrent kernel, single pass and segmented."""
    from based_amd import ops

    q, k, v = _qkv(1, 4, 2048, 64, torch.bfloat16, seed=17)
    qd, kd, vd = (q.float() * scale).bfloat16().to(dev), (k.float() * scale).bfloat16().to(dev), v.to(dev)
    y1, kv1, ks1 = ops.linear_attn_prefill(qd, kd, vd, return_state=True, split=split)
    y2, kv2, ks2 = ops.linear_attn_prefill(qd.float(), kd.float(), vd.float(), return_state=True)
    assert bool(torch.isfinite(y1.float()).all())
    assert rel_l2(y1.float(), y2) < 5e-3 and rel_l2(kv1, kv2) < 5e-3 and rel_l2(ks1, ks2) < 1e-5


@pytest.mark.parametrize("B,H,L,dv,split", [(1, 2, 1000, 64, 4), (1, 2, 1200, 64, 5), (1, 1, 128, 64, 2), (2, 2, 700, 128, 3),
                                            (1, 3, 4096, 64, 64), (1, 16, 4096, 64, None),
                                            # 8 and 16 segments summed by the second pass itself, 32 through the prefix launch
                                            (2, 2, 2048, 64, 8), (1, 2, 4096, 112, 16), (1, 2, 4096, 128, 32)])
def test_segmented_scan_matches_single_pass(dev, B, H, L, dv, split):
    """Sequences scanned as concurrent segments (small-batch path) against the single-pass kernel
    and the oracle, outputs and decode states; split=None lets the library plan the segments."""
    from based_amd import ops

    print(f"prefill split case B={B} H={H} L={L} dv={dv} split={split}", flush=True)
    q, k, v = _qkv(B, H, L, dv, torch.bfloat16, seed=21)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, kv1, ks1 = ops.linear_attn_prefill(qd, kd, vd, return_state=True, split=False)
    y2, kv2, ks2 = ops.linear_attn_prefill(qd, kd, vd, return_state=True, split=split)
    torch.cuda.synchronize()
    assert rel_l2(y2.float(), y1.float()) < 5e-3
    assert rel_l2(kv2, kv1) < 2e-3 and rel_l2(ks2, ks1) < 2e-3
    n = min(L, 1024)
    y_ref = O.linear_attn_cumsum(q[:, :, :n].float(), k[:, :, :n].float(), v[:, :, :n].float())
    assert rel_l2(y2[:, :, :n].float(), y_ref) < 1e-2
    y3, _, _ = ops.linear_attn_prefill(qd, kd, vd, return_state=False, split=split)
    assert torch.equal(y3, y2)  # deterministic, with or without the state outputs


def test_split_plan(dev):
    import ctypes
    from based_amd import _lib

    lib = _lib.lib()
    n, w = ctypes.c_int64(), ctypes.c_int64()
    assert lib.based_linear_attn_prefill_plan(64, 16, 4096, 64, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value == 1 and w.value == 0                     # plenty of chains: single pass
    assert lib.based_linear_attn_prefill_plan(1, 16, 4096, 64, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert 2 <= n.value <= 64 and w.value == 16 * n.value * 43008
    assert lib.based_linear_attn_prefill_plan(8, 16, 4096, 64, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value == 4                                      # few enough segments for the pass without a prefix launch
    assert lib.based_linear_attn_prefill_plan(12, 16, 4096, 64, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value == 1                                      # 192 chains: the single pass is faster
    assert lib.based_linear_attn_prefill_plan(1, 16, 32768, 128, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value == 16 and w.value == 32 * 16 * 43008      # long sequence: segments of 32 chunks
    assert lib.based_linear_attn_prefill_plan(1, 16, 4096, 64, 1, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value == 1                                      # fp32 path is never split
    assert lib.based_linear_attn_prefill_plan(1, 16, 64, 64, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value == 1                                      # a single chunk cannot be split
    assert lib.based_linear_attn_prefill_plan(1, 16, 4096, 112, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value >= 2 and w.value == 32 * n.value * 43008  # dv 112: two channel blocks per (batch, head)
    assert lib.based_linear_attn_prefill_plan(1, 16, 4096, 72, 0, ctypes.byref(n), ctypes.byref(w)) == 0
    assert n.value == 1 and w.value == 0                     # not whole 16-channel tiles: the fp32 kernel, never split


@pytest.mark.parametrize("B", [32, 96])
def test_full_size_prefill_properties(dev, B):
    """The bench's prefill sizes (H=16, L=4096, dv=64, bf16; B=96 is the 1536-chain launch) through
    properties that need no CPU pass: the first half of every sequence does not depend on the
    second (bit-exact: same chunks, same order), a sequence does not depend on its place in the
    batch (bit-exact), the output is linear in v (the normaliser does not see v), the states equal
    those of the fp32 recurrent kernel on four sequences, and the segmented small-batch scan agrees
    with the single pass on the same rows."""
    from based_amd import ops

    H, L, dv = 16, 4096, 64
    g = torch.Generator(device="cpu").manual_seed(1000 + B)
    print(f"full-size prefill properties B={B}", flush=True)
    q = torch.randn(B, L, H, 16, generator=g).bfloat16().to(dev).transpose(1, 2)
    k = torch.randn(B, L, H, 16, generator=g).bfloat16().to(dev).transpose(1, 2)
    v = torch.randn(B, L, H, dv, generator=g).bfloat16().to(dev).transpose(1, 2)
    y, kv, ks = ops.linear_attn_prefill(q, k, v, return_state=True, split=False)
    assert bool(torch.isfinite(y.float()).all())
    assert torch.all(ks[..., 0] == L)
    # causality: the first half alone
    y_half, _, _ = ops.linear_attn_prefill(q[:, :, :L // 2], k[:, :, :L // 2], v[:, :, :L // 2], split=False)
    assert torch.equal(y_half, y[:, :, :L // 2])
    # batch order: reversed batch
    y_rev, kv_rev, _ = ops.linear_attn_prefill(q.flip(0), k.flip(0), v.flip(0), return_state=True, split=False)
    assert torch.equal(y_rev.flip(0), y) and torch.equal(kv_rev.flip(0), kv)
    del y_rev, kv_rev, y_half
    # linearity in v: y(v) + y(v2) = y(v + v2) up to the bf16 rounding of the three outputs
    v2 = torch.randn(B, L, H, dv, generator=g).bfloat16().to(dev).transpose(1, 2)
    vs = (v.float() + v2.float()).bfloat16()
    y2, _, _ = ops.linear_attn_prefill(q, k, v2, split=False)
    y_sum, _, _ = ops.linear_attn_prefill(q, k, vs, split=False)
    assert rel_l2(y_sum.float(), y.float() + y2.float()) < 1e-2
    del v2, vs, y2, y_sum
    # four sequences against the fp32 recurrent kernel (outputs and states) and through the segmented scan
    rows = [0, 1, B // 2, B - 1]
    qs, ks_, vs_ = q[rows], k[rows], v[rows]
    y32, kv32, ks32 = ops.linear_attn_prefill(qs.float(), ks_.float(), vs_.float(), return_state=True)
    assert rel_l2(y[rows].float(), y32) < 1e-2
    assert rel_l2(kv[rows], kv32) < 5e-3 and rel_l2(ks[rows], ks32) < 5e-3
    y_seg, kv_seg, ks_seg = ops.linear_attn_prefill(qs, ks_, vs_, return_state=True, split=4)
    assert rel_l2(y_seg.float(), y[rows].float()) < 5e-3
    assert rel_l2(kv_seg, kv[rows]) < 2e-3 and rel_l2(ks_seg, ks[rows]) < 2e-3
