"""The benchmark's streaming probes (bench_probes.hip, a library of their own) do what they say
(bit-exact: they only move bytes)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,H,L,g", [(2, 4, 200, 1), (2, 4, 200, 2), (1, 8, 64, 4), (3, 2, 1, 2), (1, 16, 4096, 2)])
def test_stream_probe_combines_q_k_v_pieces(dev, B, H, L, g):
    import bench

    print(f"probe stream case B={B} H={H} L={L} heads/group={g}", flush=True)
    x = torch.randint(-2**15, 2**15, (B, L, 3, H, 64), dtype=torch.int16, device=dev)
    o = torch.zeros(B, L, H, 64, dtype=torch.int16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    assert bench.probes().bench_probe_stream_qkv(x.data_ptr(), o.data_ptr(), B, H, L, g, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(o, x[:, :, 0] ^ x[:, :, 1] ^ x[:, :, 2])


def test_rmw_and_copy_probes(dev):
    import bench

    lib = bench.probes()
    stream = torch.cuda.current_stream().cuda_stream
    n = 16 * 100003   # not a multiple of the grid
    a = torch.arange(n // 4, dtype=torch.int32, device=dev)
    assert lib.bench_probe_rmw(a.data_ptr(), n, stream) == 0
    assert torch.equal(a, torch.arange(n // 4, dtype=torch.int32, device=dev) + 1)
    b = torch.zeros_like(a)
    assert lib.bench_probe_copy(b.data_ptr(), a.data_ptr(), n, stream) == 0
    assert torch.equal(a, b)
    assert lib.bench_probe_rmw(a.data_ptr(), 24, stream) == 1        # not a multiple of 16: refused
    assert lib.bench_probe_stream_qkv(a.data_ptr(), b.data_ptr(), 1, 6, 8, 4, stream) == 1   # H % group: refused
