"""The benchmark's command line and its committed constants, without a GPU: more than one GPU is
refused with a message, the probe library exports what bench.py binds, and the HBM traffic figures
bench.py reports are the ones the committed counter summaries hold."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "5", "--warmup", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr)


def test_traffic_constants_match_the_committed_profiles():
    sys.path.insert(0, ROOT)
    import bench

    def total(name, pattern):
        text = open(os.path.join(ROOT, "profiles", name)).read()
        m = re.search(pattern, text)
        assert m, (name, pattern)
        return int(m.group(1).replace(",", ""))

    t = bench.MEASURED_TRAFFIC_BYTES
    assert t["lin_step_kernel"] == total("lin_step_kernel_decode_B128_hbm_traffic.md",
                                         r"B=128 dv=64, total HBM traffic per launch\*\* \| \| \| \*\*([\d,]+)\*\*")
    assert t["lin_step_kernel_B64_dv128"] == total("lin_step_kernel_decode_B128_hbm_traffic.md", r"B=64 dv=128, total \| \| \| ([\d,]+)")
    assert t["lin_prefill_mfma_kernel"][96] == total("lin_prefill_mfma_kernel_B96_L4096_hbm_traffic.md",
                                                     r"total HBM traffic per launch \| \| \| \*\*([\d,]+)\*\*")
    assert t["swa_prefill_kernel"] == total("swa_prefill_kernel_B8_L4096_hbm_traffic.md",
                                            r"swa_prefill_kernel<false, 2, 4>`[^\n]*?\*\*([\d,]+)\*\*")


def test_probe_library_exports_what_the_bench_binds():
    import ctypes

    path = os.path.join(ROOT, "libbench_probes.so")
    if not os.path.exists(path):
        import pytest

        pytest.skip("libbench_probes.so not built (python -c 'import __graft_entry__ as g; g.build()')")
    lib = ctypes.CDLL(path)  # loading needs no GPU; nothing is launched
    for name in ("bench_probe_stream_qkv", "bench_probe_rmw", "bench_probe_copy", "bench_probe_stream_prefill",
                 "bench_probe_mfma", "bench_probe_timestamp", "bench_probe_clock_khz"):
        assert hasattr(lib, name), name
