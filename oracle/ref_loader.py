"""Loads the reference's own CPU causal product, built by oracle/Makefile into oracle/_ref/.

TEST INFRASTRUCTURE ONLY.  The module is the reference's
train/csrc/causal_dot_prod/causal_attention.cpp compiled unmodified; it is used to
cross-check the restated oracle and never ships with the product.
"""
from __future__ import annotations

import importlib.util
import os

_SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref", "causal_attention_ref.so")


def available() -> bool:
    return os.path.exists(_SO)


def load():
    """Returns the extension module exposing causal_dot_product(q, k, v, out)."""
    import torch  # noqa: F401  (libtorch must be loaded before the extension)

    spec = importlib.util.spec_from_file_location("causal_attention_ref", _SO)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def causal_dot_product(q, k, v):
    """sum_{j<=i} (q_i . k_j) v_j for fp32 (N, H, L, E) q, k and (N, H, L, M) v, calling
    convention of train/csrc/causal_dot_prod/causal_attention.py:35-68 (zero-filled output)."""
    import torch

    out = torch.zeros(*q.shape[:3], v.shape[-1], dtype=torch.float32)
    load().causal_dot_product(q.contiguous().float(), k.contiguous().float(), v.contiguous().float(), out)
    return out
