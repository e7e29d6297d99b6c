"""The C-ABI library loads and exports every symbol include/based_hip.h declares, the ctypes
binding covers exactly that set, and argument validation works without a GPU (validation
happens before any HIP call)."""
import ctypes
import os
import re

import pytest

from based_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "based_hip.h")).read()
    return set(re.findall(r"BASED_API\s+[\w\s\*]+?\b(based_\w+)\s*\(", text))


def test_header_symbols_are_exported_and_bound():
    declared = _declared()
    assert {"based_linear_attn_step", "based_linear_attn_prefill", "based_swa_prefill", "based_swa_step",
            "based_hip_version", "based_hip_last_error"} <= declared
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m based_amd.build"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in the header but not exported"
    assert set(_lib.SIGNATURES) == declared


def test_header_constants_match_binding():
    text = open(os.path.join(ROOT, "include", "based_hip.h")).read()
    m = re.search(r"#define\s+BASED_PREFILL_SEGMENT_STATE_BYTES\s+(\d+)", text)
    assert m and int(m.group(1)) == _lib.PREFILL_SEGMENT_STATE_BYTES


def test_version_and_error_string():
    lib = _lib.lib()
    assert lib.based_hip_version() >= 1
    assert isinstance(lib.based_hip_last_error(), bytes)


def test_argument_validation_without_gpu():
    lib = _lib.lib()
    # null pointers -> BASED_ERR_ARG (4), nothing launched
    rc = lib.based_linear_attn_step(None, None, None, None, None, None, 1, 1, 64, 0, 0, 0, 0, 0, 0, 0, 0, 1e-12, 0, None)
    assert rc == 4 and b"null" in lib.based_hip_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)
    buf = (ctypes.c_float * 64)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    # unsupported head dim -> BASED_ERR_SHAPE (1)
    rc = lib.based_linear_attn_step(p, p, p, p, p, p, 1, 1, 40, 0, 0, 0, 0, 0, 0, 0, 0, 1e-12, 0, None)
    assert rc == 1
    # window too wide -> BASED_ERR_SHAPE
    rc = lib.based_swa_prefill(p, p, p, p, 1, 1, 8, 0, 64, 64, 0, 64, 64, 0, 64, 64, 0, 64, 64, 129, 0.125, None, None, 0, None, None, 0, 0, 0, 0, 0, None)
    assert rc == 1
    # fp32 is not a sliding-window element type -> BASED_ERR_DTYPE (2)
    rc = lib.based_swa_prefill(p, p, p, p, 1, 1, 8, 0, 64, 64, 0, 64, 64, 0, 64, 64, 0, 64, 64, 64, 0.125, None, None, 0, None, None, 0, 0, 0, 0, 1, None)
    assert rc == 2
    # misaligned stride -> BASED_ERR_ALIGN (3)
    rc = lib.based_linear_attn_prefill(p, p, p, p, None, None, 1, 1, 8, 64, 0, 0, 20, 0, 0, 16, 0, 0, 64, 0, 0, 64, 1e-12, 0, None)
    assert rc == 3
    # one state pointer without the other -> BASED_ERR_ARG
    rc = lib.based_linear_attn_prefill(p, p, p, p, p, None, 1, 1, 8, 64, 0, 0, 16, 0, 0, 16, 0, 0, 64, 0, 0, 64, 1e-12, 0, None)
    assert rc == 4
    # empty batch is a no-op success
    rc = lib.based_swa_prefill(p, p, p, p, 0, 1, 8, 0, 64, 64, 0, 64, 64, 0, 64, 64, 0, 64, 64, 64, 0.125, None, None, 0, None, None, 0, 0, 0, 0, 0, None)
    assert rc == 0
    # one rotary table without the other -> BASED_ERR_ARG
    rc = lib.based_swa_prefill(p, p, p, p, 1, 1, 8, 0, 64, 64, 0, 64, 64, 0, 64, 64, 0, 64, 64, 64, 0.125, p, None, 8, None, None, 0, 0, 0, 0, 0, None)
    assert rc == 4
    # gated convolution: kernel size outside 2..4 -> BASED_ERR_SHAPE
    rc = lib.based_gated_conv_prefill(p, p, None, p, None, 1, 4, 8, 5, 64, 16, 32, 8, 0, 0, None)
    assert rc == 1
    # allocation-free segmented prefill: more scratch than the static array holds -> BASED_ERR_SHAPE,
    # refused before any HIP call
    rc = lib.based_linear_attn_prefill_split_static(p, p, p, p, None, None, 256, 16, 4096, 64, 0, 0, 16, 0, 0, 16,
                                                    0, 0, 64, 0, 0, 64, 1e-12, 0, 4, None)
    assert rc == 1 and b"scratch" in lib.based_hip_last_error()
