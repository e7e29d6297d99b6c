"""GPU parity of the gated short-convolution kernels (through the C ABI) against the oracle."""
import pytest
import torch

from conftest import rel_l2
from oracle import based_oracle as O

pytestmark = pytest.mark.gpu
TOL = {torch.bfloat16: 1e-2, torch.float32: 1e-4}  # rel-L2 bounds of the build target


def _inputs(B, L, D, K, dtype, seed, bias):
    g = torch.Generator().manual_seed(seed)
    u = torch.randn(B, L, 2 * D, generator=g).to(dtype)
    w = (torch.randn(D, 1, K, generator=g) * 0.5).to(dtype)
    b = torch.randn(D, generator=g).to(dtype) if bias else None
    return u, w, b


@pytest.mark.parametrize("B,L,D,K,dtype,bias", [
    (2, 37, 64, 3, torch.bfloat16, False), (1, 1, 8, 3, torch.bfloat16, False), (3, 2, 16, 3, torch.bfloat16, True),
    (1, 16, 2048, 3, torch.bfloat16, False), (2, 100, 264, 4, torch.bfloat16, True), (2, 17, 24, 2, torch.bfloat16, False),
    (2, 33, 20, 3, torch.float32, True), (1, 300, 2048, 3, torch.float32, False)])
def test_prefill_matches_oracle(dev, B, L, D, K, dtype, bias):
    from based_amd import ops

    print(f"gated conv prefill case B={B} L={L} D={D} K={K} {dtype} bias={bias}", flush=True)
    u, w, b = _inputs(B, L, D, K, dtype, seed=3, bias=bias)
    y_ref = O.gated_short_conv(u.float(), w[:, 0].float(), None if b is None else b.float())
    for sdtype in (dtype, torch.float32):
        state = torch.full((B, D, K), 7.0, dtype=sdtype, device=dev)
        y = ops.gated_conv_prefill(u.to(dev), w.to(dev), None if b is None else b.to(dev), state=state)
        torch.cuda.synchronize()
        assert y.shape == (B, L, D) and y.dtype == dtype
        assert rel_l2(y.float(), y_ref) < TOL[dtype]
        # state = the last K inputs, oldest first, zeros where the sequence is shorter (exact copies)
        kk = min(K, L)
        state_ref = torch.zeros(B, D, K)
        state_ref[..., -kk:] = u[:, -kk:, :D].float().transpose(1, 2)
        assert torch.equal(state.float().cpu(), state_ref)
    y2 = ops.gated_conv_prefill(u.to(dev), w.to(dev), None if b is None else b.to(dev))
    assert torch.equal(y2, y)


@pytest.mark.parametrize("B,D,K,dtype,bias", [(4, 2048, 3, torch.bfloat16, False), (3, 24, 4, torch.bfloat16, True),
                                              (128, 2048, 3, torch.bfloat16, False), (2, 16, 2, torch.float32, True)])
def test_steps_match_parallel(dev, B, D, K, dtype, bias):
    """Prefill P tokens (leaving the state), then single-token steps: every step equals the
    parallel form on the whole sequence (the reference's recurrent == parallel invariant)."""
    from based_amd import ops

    print(f"gated conv step case B={B} D={D} K={K} {dtype} bias={bias}", flush=True)
    P, T = 5, 6
    u, w, b = _inputs(B, P + T, D, K, dtype, seed=11, bias=bias)
    y_ref = O.gated_short_conv(u.float(), w[:, 0].float(), None if b is None else b.float())
    ud, wd, bd = u.to(dev), w.to(dev), None if b is None else b.to(dev)
    state = torch.zeros(B, D, K, dtype=dtype, device=dev)
    y0 = ops.gated_conv_prefill(ud[:, :P], wd, bd, state=state)
    assert rel_l2(y0.float(), y_ref[:, :P]) < TOL[dtype]
    ptr = state.data_ptr()
    for t in range(P, P + T):
        yt = ops.gated_conv_step(ud[:, t:t + 1], state, wd, bd)
        assert yt.shape == (B, 1, D)
        assert rel_l2(yt[:, 0].float(), y_ref[:, t]) < TOL[dtype]
    assert state.data_ptr() == ptr
    assert torch.equal(state.float().cpu(), u[:, -K:, :D].float().transpose(1, 2))


def test_strided_rows_and_errors(dev):
    from based_amd import ops

    g = torch.Generator().manual_seed(2)
    big = torch.randn(2, 9, 3 * 64, generator=g).bfloat16().to(dev)
    u = big[..., :64]                      # rows 192 elements apart, 2D = 64
    w = (torch.randn(32, 1, 3, generator=g) * 0.5).bfloat16().to(dev)
    y = ops.gated_conv_prefill(u, w)
    y_ref = O.gated_short_conv(u.float().cpu(), w[:, 0].float().cpu())
    assert rel_l2(y.float(), y_ref) < 1e-2
    with pytest.raises(ValueError):
        ops.gated_conv_prefill(u, torch.zeros(32, 1, 5, dtype=torch.bfloat16, device=dev))   # kernel size 5
    with pytest.raises(ValueError):
        ops.gated_conv_prefill(big[..., :24], torch.zeros(12, 1, 3, dtype=torch.bfloat16, device=dev))  # D % 8
    with pytest.raises(ValueError):
        ops.gated_conv_prefill(u.float(), w)                                                   # dtype mismatch


@pytest.mark.parametrize("shape,dtype", [((4, 1, 4096), torch.bfloat16), ((2, 37, 1024), torch.bfloat16),
                                         ((3, 48), torch.float32), ((2, 5, 272), torch.bfloat16)])
def test_swiglu_matches_torch_statement(dev, shape, dtype):
    """out = y * silu(gate), y, gate = u.chunk(2) -- the statement of mlp.py:147-151, evaluated by
    torch on the host in the same dtype (so the intermediate rounding of silu(gate) is the same)."""
    import torch.nn.functional as F
    from based_amd import ops

    g = torch.Generator().manual_seed(8)
    u = (torch.randn(*shape, generator=g) * 2).to(dtype)
    y, gate = u.chunk(2, dim=-1)
    ref = y * F.silu(gate)
    out = ops.swiglu(u.to(dev))
    assert out.shape == ref.shape and out.dtype == dtype
    assert rel_l2(out.float(), ref.float()) < (4e-3 if dtype == torch.bfloat16 else 1e-6)
    # against fp32 arithmetic as well (the bound of the build target)
    ref32 = y.float() * F.silu(gate.float())
    assert rel_l2(out.float(), ref32) < TOL[dtype]


@pytest.mark.parametrize("K,dtype", [(3, torch.bfloat16), (4, torch.float32), (2, torch.bfloat16)])
def test_convolution_alone_prefill_and_steps(dev, K, dtype):
    """The ungated form (ShortConvolution as a mixer of its own): prefill, exact state, decode steps."""
    from based_amd import ops

    B, L, D, T = 2, 77, 64, 5
    g = torch.Generator().manual_seed(41)
    x = torch.randn(B, L + T, D, generator=g).to(dtype)
    w = (torch.randn(D, 1, K, generator=g) * 0.5).to(dtype)
    ref = O.short_conv(x.float(), w[:, 0].float())
    tol = 5e-3 if dtype == torch.bfloat16 else 1e-5
    xd, wd = x.to(dev), w.to(dev)
    state = torch.zeros(B, D, K, dtype=dtype, device=dev)
    y = ops.gated_conv_prefill(xd[:, :L], wd, None, state=state, gated=False)
    assert y.shape == (B, L, D) and rel_l2(y.float(), ref[:, :L]) < tol
    assert torch.equal(state.cpu(), x[:, L - K:L].transpose(1, 2))
    for t in range(L, L + T):
        yt = ops.gated_conv_step(xd[:, t:t + 1], state, wd, None, gated=False)
        assert rel_l2(yt.float(), ref[:, t:t + 1]) < tol
