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


def test_stream_prefill_probe_moves_what_it_says(dev):
    """The prefill memory probe reads every q, k, v row of its (batch, head) and writes every y row:
    y piece (token 64 c + t / 8, piece t % 8) = v piece ^ the q or k piece thread t < 256 fetched."""
    import bench

    B, H, L = 2, 8, 256
    q = torch.randint(-2**15, 2**15, (B, L, H, 16), dtype=torch.int16, device=dev)
    k = torch.randint(-2**15, 2**15, (B, L, H, 16), dtype=torch.int16, device=dev)
    v = torch.randint(-2**15, 2**15, (B, L, H, 64), dtype=torch.int16, device=dev)
    y = torch.zeros(B, L, H, 64, dtype=torch.int16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    assert bench.probes().bench_probe_stream_prefill(q.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(), B, H, L, stream) == 0
    torch.cuda.synchronize()
    t = torch.arange(512, device=dev)
    src_row, src_pc = (t & 127) >> 1, t & 1
    want = torch.empty_like(y)
    pick = lambda x, rows, n_pc, pc: x[:, rows].view(B, 512, H, n_pc, 8)[:, t, :, pc].permute(1, 0, 2, 3)   # (B, 512, H, 8)
    for c in range(L // 64):
        qk = torch.where((t < 128)[None, :, None, None], pick(q, 64 * c + src_row, 2, src_pc), pick(k, 64 * c + src_row, 2, src_pc))
        qk = torch.where((t < 256)[None, :, None, None], qk, torch.zeros_like(qk))   # threads 256..511 fetch v only
        vv = pick(v, 64 * c + (t >> 3), 8, t & 7)
        blk = (qk ^ vv).view(B, 64, 8, H, 8).permute(0, 1, 3, 2, 4).reshape(B, 64, H, 64)    # thread t = (row t / 8, piece t % 8)
        want[:, 64 * c: 64 * c + 64] = blk
    assert torch.equal(y, want)


def test_mfma_probe_counts_its_flops_and_runs(dev):
    """The MFMA-rate probe reports 32 MFMA 16x16x32 per iteration and wavefront, writes one finite
    sum per lane (every lane's operands differ, the sums are not all equal) and refuses bad sizes."""
    import ctypes as C
    import bench

    lib = bench.probes()
    wgs, iters = 8, 3
    out = torch.zeros(wgs * 256, dtype=torch.float32, device=dev)
    flops = C.c_double(0.0)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.bench_probe_mfma(out.data_ptr(), wgs, iters, C.byref(flops), stream) == 0
    torch.cuda.synchronize()
    assert flops.value == wgs * 4 * iters * 32 * 2 * 16 * 16 * 32
    assert torch.isfinite(out).all() and out.unique().numel() > wgs
    assert lib.bench_probe_mfma(out.data_ptr(), 0, iters, C.byref(flops), stream) == 1
    assert lib.bench_probe_mfma(None, wgs, iters, C.byref(flops), stream) == 1


def test_timestamp_probe_agrees_with_events(dev):
    """Two timestamp launches around a run of copy launches, recorded in a graph: their difference in
    ticks of the device clock is the run's duration as HIP events around the replay see it (events
    also see the launch of the graph: they may read a little more, never less than the stamps by
    more than the resolution)."""
    import bench

    lib = bench.probes()
    khz = lib.bench_probe_clock_khz()
    assert khz > 0
    n = 64 << 20
    a = torch.zeros(n // 4, dtype=torch.int32, device=dev)
    b = torch.zeros_like(a)
    stamps = torch.zeros(2, dtype=torch.int64, device=dev)
    assert lib.bench_probe_timestamp(stamps.data_ptr() + 4, torch.cuda.current_stream().cuda_stream) == 1   # misaligned: refused
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            sp = torch.cuda.current_stream().cuda_stream
            assert lib.bench_probe_copy(b.data_ptr(), a.data_ptr(), n, sp) == 0
            assert lib.bench_probe_timestamp(stamps.data_ptr(), sp) == 0
            for _ in range(40):
                assert lib.bench_probe_copy(b.data_ptr(), a.data_ptr(), n, sp) == 0
            assert lib.bench_probe_timestamp(stamps.data_ptr() + 8, sp) == 0
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        t0, t1 = stamps.cpu().tolist()
        ms_stamps = (t1 - t0) / khz
        ms_events = e0.elapsed_time(e1) * 40 / 41
        print(f"timestamp probe: {ms_stamps:.4f} ms by the stamps, {ms_events:.4f} ms by events (scaled to 40 of 41 copies)", flush=True)
        assert t1 > t0
        assert 0.9 * ms_events < ms_stamps < 1.05 * ms_events
