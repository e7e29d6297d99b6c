"""Writes tests/golden/causal_dot_E273_M64.npz with the reference's own CPU causal product.

Run in the build container after `make -C oracle` (needs oracle/_ref, i.e. the reference's
train/csrc/causal_dot_prod/causal_attention.cpp compiled by oracle/Makefile):

    python tests/golden/make_causal_dot_golden.py

Inputs: seeded raw q, k (rounded to bf16-representable values so that the bf16 kernels see
exactly these numbers) and v.  Expected output: the un-normalised numerator
sum_{j<=i} (phi(q_i) . phi(k_j)) v_j computed by the reference C++ on the 273-dim feature maps
(call convention of train/csrc/causal_dot_prod/causal_attention.py:35-68), and the normaliser
sum_{j<=i} phi(q_i) . phi(k_j) obtained from the same routine with a column of ones as v.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import based_oracle as O  # noqa: E402
from oracle import ref_loader  # noqa: E402


def main():
    assert ref_loader.available(), "build oracle/_ref first: make -C oracle"
    g = torch.Generator().manual_seed(20240229)
    B, H, L, dv = 1, 2, 96, 64
    q = (torch.randn(B, H, L, 16, generator=g) * 0.5).bfloat16().float()
    k = (torch.randn(B, H, L, 16, generator=g) * 0.5).bfloat16().float()
    v = torch.randn(B, H, L, dv, generator=g).bfloat16().float()
    fq, fk = O.taylor_exp(q), O.taylor_exp(k)
    num = ref_loader.causal_dot_product(fq, fk, v)
    den = ref_loader.causal_dot_product(fq, fk, torch.ones(B, H, L, 1))
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "causal_dot_E273_M64.npz")
    np.savez_compressed(out, q=q.numpy(), k=k.numpy(), v=v.numpy(), numerator=num.numpy(), normaliser=den.numpy())
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
