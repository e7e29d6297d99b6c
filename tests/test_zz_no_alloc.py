"""The allocation-free segmented prefill (based_linear_attn_prefill_split_static, static device
scratch) against based_linear_attn_prefill_split with a caller-owned workspace: same kernels,
same launch order, so the outputs and decode states must be bit-identical.  Two calls in a row,
the second smaller, so that stale scratch contents of the first would show."""
import ctypes

import pytest
import torch

from conftest import rel_l2
from oracle import based_oracle as O

pytestmark = pytest.mark.gpu


def _run(dev, B, H, L, dv, n_seg, seed, static):
    from based_amd import _lib

    lib = _lib.lib()
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, L, 16, generator=g).bfloat16().to(dev)
    k = torch.randn(B, H, L, 16, generator=g).bfloat16().to(dev)
    v = torch.randn(B, H, L, dv, generator=g).bfloat16().to(dev)
    y = torch.full((B, H, L, dv), float("nan"), dtype=torch.bfloat16, device=dev)
    kv = torch.full((B, H, 1, dv, 273), float("nan"), dtype=torch.float32, device=dev)
    ks = torch.full((B, H, 1, 1, 273), float("nan"), dtype=torch.float32, device=dev)
    args = [q.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(), kv.data_ptr(), ks.data_ptr(), B, H, L, dv]
    for t in (q, k, v, y):
        args += [t.stride(0), t.stride(1), t.stride(2)]
    args += [1e-12, _lib.BASED_BF16, n_seg]
    stream = torch.cuda.current_stream(dev).cuda_stream
    if static:
        _lib.check(lib.based_linear_attn_prefill_split_static(*args, stream))
    else:
        ws_bytes = B * H * (dv // 64) * n_seg * _lib.PREFILL_SEGMENT_STATE_BYTES
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        _lib.check(lib.based_linear_attn_prefill_split(*args, ws.data_ptr(), ws_bytes, stream))
    torch.cuda.synchronize()
    return (q, k, v), y, kv, ks


def test_static_scratch_matches_workspace_variant(dev):
    # first call: 2*4 chains x 24 segments (the prefix launch between the two passes); then fewer segments (the second
    # pass sums them itself), then fewer chains, shorter, ragged
    for (B, H, L, dv, n_seg, seed) in [(2, 4, 1536, 64, 24, 11), (2, 4, 1536, 64, 6, 13), (1, 2, 700, 128, 3, 12)]:
        print(f"no-alloc prefill case B={B} H={H} L={L} dv={dv} n_seg={n_seg}", flush=True)
        (q, k, v), y_s, kv_s, ks_s = _run(dev, B, H, L, dv, n_seg, seed, static=True)
        _, y_w, kv_w, ks_w = _run(dev, B, H, L, dv, n_seg, seed, static=False)
        assert torch.isfinite(y_s.float()).all() and torch.isfinite(kv_s).all() and torch.isfinite(ks_s).all()
        assert torch.equal(y_s, y_w) and torch.equal(kv_s, kv_w) and torch.equal(ks_s, ks_w)
        y_ref = O.linear_attn_cumsum(q.float().cpu(), k.float().cpu(), v.float().cpu())
        assert rel_l2(y_s.float(), y_ref) < 1e-2


def test_static_scratch_rejects_oversized_requests(dev):
    from based_amd import _lib

    lib = _lib.lib()
    buf = torch.zeros(64, dtype=torch.bfloat16, device=dev)
    p = buf.data_ptr()
    # 4096 chains x 4 segments x 43,008 B = 672 MiB > 64 MiB: refused before anything is launched
    rc = lib.based_linear_attn_prefill_split_static(p, p, p, p, None, None, 256, 16, 4096, 64,
                                                    0, 0, 16, 0, 0, 16, 0, 0, 64, 0, 0, 64, 1e-12, 0, 4, None)
    assert rc == 1 and b"scratch" in lib.based_hip_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)
    torch.cuda.synchronize()
