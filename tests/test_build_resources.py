"""What the compiler reports for the kernels of the last build (based_amd/build.py keeps it beside
the objects): the hot kernels must not spill vector registers.  A change that pushes one of them
over its register budget costs a few per cent without any other sign, so it is caught here."""
import json
import os

import pytest

from based_amd import build

# 1024-thread forms of the decode step (head dims above 128) run at 64 registers per lane and spill
KNOWN_SPILLS = ("lin_step_kernelIDF16bLi1024E", "lin_step_kernelIfLi1024E",
                "lin_step_deferred_kernelIDF16bLi1024E", "lin_step_deferred_kernelIfLi1024E")


def test_hot_kernels_do_not_spill_vector_registers():
    if not os.path.exists(build.RESOURCES):
        pytest.skip("no build in this tree yet (python -m based_amd.build writes the report)")
    usage = json.load(open(build.RESOURCES))
    seen = 0
    for src, kernels in usage.items():
        for name, u in kernels.items():
            seen += 1
            if any(k in name for k in KNOWN_SPILLS):
                continue
            assert u.get("VGPRs Spill", 0) == 0, f"{src}: {name} spills {u['VGPRs Spill']} vector registers"
    assert seen > 50   # the report covers every source
