"""CPU restatement of the Based sequence-mixer arithmetic.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory; it exists so that the HIP kernels can be checked against an
independent, slow, obviously-correct statement of the reference semantics.
Allowed importers: the test-suite, the smoke check and the CPU-baseline leg of
the benchmark.
"""
from .based_oracle import (  # noqa: F401
    taylor_exp,
    taylor_dot,
    linear_attn_quadratic,
    linear_attn_cumsum,
    linear_attn_prefill_state,
    linear_attn_step,
    sliding_window_attn,
    sliding_window_step,
    rms_norm,
    swiglu_mlp,
    short_conv,
    short_conv_step,
)
