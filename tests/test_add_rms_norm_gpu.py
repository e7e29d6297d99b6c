"""GPU parity of the fused residual-add + RMSNorm kernel (through the C ABI) against the oracle."""
import pytest
import torch

from conftest import rel_l2
from oracle import based_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,dtype,res,res_fp32", [
    ((4, 1, 1024), torch.bfloat16, True, True), ((2, 37, 1024), torch.bfloat16, True, True),
    ((3, 5, 1024), torch.bfloat16, False, True), ((2, 9, 256), torch.bfloat16, True, False),
    ((1, 7, 4096), torch.bfloat16, True, True), ((2, 3, 520), torch.bfloat16, True, True),
    ((5, 8), torch.float32, True, True), ((2, 4, 1536), torch.float32, False, True)])
def test_matches_oracle(dev, shape, dtype, res, res_fp32):
    from based_amd import ops

    print(f"add_rms_norm case {shape} {dtype} residual={res} fp32_stream={res_fp32}", flush=True)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(*shape, generator=g).to(dtype)
    r_dtype = torch.float32 if res_fp32 else dtype
    r = (torch.randn(*shape, generator=g) * 3).to(r_dtype) if res else None
    w = (1 + 0.1 * torch.randn(shape[-1], generator=g)).to(dtype)
    y_ref, r_ref = O.add_rms_norm(x, r, w, eps=1e-5, residual_in_fp32=res_fp32)
    y, r_out = ops.add_rms_norm(x.to(dev), None if r is None else r.to(dev), w.to(dev), eps=1e-5,
                                residual_in_fp32=res_fp32)
    torch.cuda.synchronize()
    assert y.shape == x.shape and y.dtype == dtype and r_out.dtype == r_dtype
    assert rel_l2(y.float(), y_ref.float()) < (5e-3 if dtype == torch.bfloat16 else 1e-5)
    # the residual stream is a plain sum: exact in fp32, one rounding in bf16
    if r_dtype == torch.float32:
        assert torch.equal(r_out.cpu(), r_ref)
    else:
        assert rel_l2(r_out.float(), r_ref.float()) < 4e-3
    y2, none = ops.add_rms_norm(x.to(dev), None if r is None else r.to(dev), w.to(dev), eps=1e-5,
                                residual_in_fp32=res_fp32, want_residual=False)
    assert none is None and torch.equal(y2, y)


def test_strided_rows_and_errors(dev):
    from based_amd import ops

    g = torch.Generator().manual_seed(6)
    big = torch.randn(6, 2048, generator=g).bfloat16().to(dev)
    x = big[:, :1024]            # rows 2048 elements apart
    w = torch.ones(1024, dtype=torch.bfloat16, device=dev)
    y, r = ops.add_rms_norm(x, None, w)
    y_ref, _ = O.add_rms_norm(x.cpu(), None, w.cpu())
    assert rel_l2(y.float(), y_ref.float()) < 5e-3 and torch.equal(r.cpu(), x.float().cpu())
    with pytest.raises(ValueError):
        ops.add_rms_norm(torch.zeros(2, 12, dtype=torch.bfloat16, device=dev), None, torch.ones(12, dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError):
        ops.add_rms_norm(torch.zeros(2, 8192, dtype=torch.bfloat16, device=dev), None, torch.ones(8192, dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError):
        ops.add_rms_norm(x, None, w.float())
