"""GPU parity of the decode step kernel (through the C ABI) against the CPU oracle."""
import pytest
import torch

from conftest import rel_l2
from oracle import based_oracle as O

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 1e-2, torch.float32: 1e-4}  # rel-L2 bounds of the build target


def _inputs(B, H, dv, dtype, seed, P=32):
    g = torch.Generator().manual_seed(seed)
    kp = torch.randn(B, H, P, 16, generator=g)
    vp = torch.randn(B, H, P, dv, generator=g)
    kv, ks = O.linear_attn_prefill_state(kp, vp)
    return kv.contiguous(), ks.contiguous(), g


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,H,dv", [(2, 16, 64), (1, 3, 128), (3, 2, 16), (1, 1, 256), (2, 2, 48)])
def test_step_matches_oracle(dev, B, H, dv, dtype):
    from based_amd import ops

    kv, ks, g = _inputs(B, H, dv, dtype, seed=1)
    kv_d, ks_d = kv.to(dev), ks.to(dev)
    kv_ptr = kv_d.data_ptr()
    for step in range(3):
        print(f"step case B={B} H={H} dv={dv} {dtype} step={step}", flush=True)
        q = torch.randn(B, H, 1, 16, generator=g).to(dtype)
        k = torch.randn(B, H, 1, 16, generator=g).to(dtype)
        v = torch.randn(B, H, 1, dv, generator=g).to(dtype)
        y_ref = O.linear_attn_step(kv, ks, q.float(), k.float(), v.float())
        y = ops.linear_attn_step(q.to(dev), k.to(dev), v.to(dev), kv_d, ks_d)
        torch.cuda.synchronize()
        assert y.dtype == dtype and tuple(y.shape) == (B, H, 1, dv)
        assert rel_l2(y.float(), y_ref) < TOL[dtype]
        assert rel_l2(kv_d, kv) < 1e-5
        assert rel_l2(ks_d, ks) < 1e-5
    assert kv_d.data_ptr() == kv_ptr  # state is updated in place


def test_step_strided_inputs(dev):
    """q, k, v arrive as (B,1,H,d) projections viewed as (B,H,1,d): non-contiguous."""
    from based_amd import ops

    B, H, dv = 4, 16, 64
    kv, ks, g = _inputs(B, H, dv, torch.bfloat16, seed=2)
    kv_d, ks_d = kv.to(dev), ks.to(dev)
    q = torch.randn(B, 1, H * 16, generator=g).bfloat16()
    k = torch.randn(B, 1, H * 16, generator=g).bfloat16()
    v = torch.randn(B, 1, H * dv, generator=g).bfloat16()
    view = lambda t, d: t.view(B, 1, H, d).transpose(1, 2)
    y_ref = O.linear_attn_step(kv, ks, view(q, 16).float(), view(k, 16).float(), view(v, dv).float())
    y = ops.linear_attn_step(view(q.to(dev), 16), view(k.to(dev), 16), view(v.to(dev), dv), kv_d, ks_d)
    assert rel_l2(y.float(), y_ref) < 1e-2
    assert rel_l2(kv_d, kv) < 1e-5


def test_step_rejects_bad_shapes(dev):
    from based_amd import ops

    q = torch.zeros(1, 1, 1, 16, device=dev, dtype=torch.bfloat16)
    v = torch.zeros(1, 1, 1, 40, device=dev, dtype=torch.bfloat16)
    kv = torch.zeros(1, 1, 1, 40, 273, device=dev)
    ks = torch.zeros(1, 1, 1, 1, 273, device=dev)
    with pytest.raises(ValueError):
        ops.linear_attn_step(q, q, v, kv, ks)  # dv not a multiple of 16
