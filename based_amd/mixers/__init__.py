from .linear_attention import FeatureMap, LinearAttention, TaylorExp  # noqa: F401
from .slide_attention import SlidingAttention  # noqa: F401
from .convolution import BaseConv, ShortConvolution  # noqa: F401
