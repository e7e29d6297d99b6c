"""based_amd — MI355X (gfx950) kernels and drop-in mixers for the Based sequence-mixer hot path."""
from .generation import InferenceParams, decode, sample  # noqa: F401
from .mixers import BaseConv, FeatureMap, LinearAttention, ShortConvolution, SlidingAttention, TaylorExp  # noqa: F401

__version__ = "0.1.0"
