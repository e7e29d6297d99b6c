"""Short convolution mixers; mirror the interface of based/models/mixers/convolution.py:16-218:
BaseConv = in_proj -> depthwise causal conv (kernel 3) -> SiLU -> gate -> out_proj, with a rolling
(B, D, K) state for decoding; everything between the two projections is one kernel
(`ops.gated_conv_prefill` / `ops.gated_conv_step`).  ShortConvolution on its own is the same
kernel without activation and gate.  There is no host-tensor path."""
from __future__ import annotations

import torch
import torch.nn as nn


class ShortConvolution(nn.Module):
    def __init__(self, d_model: int, kernel_size: int, layer_idx=None, conv_bias: bool = False,
                 device=None, dtype=None, **kwargs):
        super().__init__()
        self.d_model = d_model
        self.kernel_size = kernel_size
        self.layer_idx = layer_idx
        self.conv = nn.Conv1d(d_model, d_model, kernel_size=kernel_size, groups=d_model,
                              padding=kernel_size - 1, bias=conv_bias, device=device, dtype=dtype)

    def forward(self, x: torch.Tensor, inference_params=None, **kwargs):
        """x (b, l, d) -> (b, l, d): the depthwise causal convolution alone (no activation), with the
        rolling state of ShortConvolution.forward / step (convolution.py:47-109).  Inside BaseConv
        this method is not used: conv, SiLU and gate are one kernel there."""
        from .. import ops

        weight, bias = self.conv.weight, self.conv.bias
        if inference_params is None:
            return ops.gated_conv_prefill(x, weight, bias, gated=False)
        if inference_params.seqlen_offset > 0:
            state = self._get_state(inference_params)
            return ops.gated_conv_step(x, state[: x.shape[0]], weight, bias, gated=False)
        self._init_state(inference_params)
        state = self._get_state(inference_params)
        return ops.gated_conv_prefill(x, weight, bias, state=state[: x.shape[0]], gated=False)

    def allocate_inference_cache(self, batch_size: int, max_seqlen: int, dtype=None, **kwargs):
        return torch.zeros(batch_size, self.d_model, self.kernel_size, device=self.conv.weight.device,
                           dtype=self.conv.weight.dtype if dtype is None else dtype)

    def _init_state(self, inference_params):
        """Creates the state if it does not exist, zeroes it otherwise (a pre-allocated state may
        be larger than the running batch; it is cleared whole)."""
        outer, inner = self.layer_idx if isinstance(self.layer_idx, tuple) else (self.layer_idx, None)
        d = inference_params.key_value_memory_dict
        if inner is not None:
            d = d.setdefault(outer, {})
        key = outer if inner is None else inner
        if key in d:
            d[key].zero_()
        else:
            d[key] = self.allocate_inference_cache(inference_params.max_batch_size, inference_params.max_seqlen)

    def _get_state(self, inference_params):
        d = inference_params.key_value_memory_dict
        if isinstance(self.layer_idx, tuple):
            return d[self.layer_idx[0]][self.layer_idx[1]]
        return d[self.layer_idx]


class BaseConv(nn.Module):
    def __init__(self, d_model: int, l_max: int = 2048, kernel_size: int = 3, layer_idx=None, use_bias=True,
                 expand_proj: int = 2, device=None, dtype=None, **kwargs):
        super().__init__()
        self.d_model = d_model
        self.l_max = l_max
        self.layer_idx = layer_idx
        self.d_inner = expand_proj * d_model // 2
        self.in_proj = nn.Linear(d_model, expand_proj * d_model, bias=use_bias, device=device, dtype=dtype)
        self.out_proj = nn.Linear(self.d_inner, d_model, bias=use_bias, device=device, dtype=dtype)
        self.conv = ShortConvolution(self.d_inner, kernel_size=kernel_size, layer_idx=(layer_idx, "conv"),
                                     device=device, dtype=dtype)

    def forward(self, u, position_ids=None, inference_params=None, *args, **kwargs):
        return self.out_proj(self._gated_conv_hip(self.in_proj(u), inference_params))

    def supports_decode_step(self) -> bool:
        from .. import ops

        return ops.decode_linear_weight_ok(self.in_proj.weight) and ops.decode_linear_weight_ok(self.out_proj.weight)

    def decode_step(self, u, inference_params, **prologue):
        """One token per sequence with the projections as `ops.decode_linear` launches: u (b, d_model)
        bf16 -> (b, d_model).  `prologue` goes to in_proj (the block's residual add + norm,
        possibly the embedding gather)."""
        from .. import ops

        state = self.conv._get_state(inference_params)
        rows = prologue["row_index"].numel() if prologue.get("row_index") is not None else u.shape[0]
        if self.in_proj.weight.shape[1] <= 2048 and self.conv.kernel_size <= 4:
            # in_proj with the convolution step in its tail: one launch
            y = ops.decode_linear(u, self.in_proj.weight, self.in_proj.bias, epilogue=ops.EPILOGUE_GATED_CONV_STEP,
                                  conv_state=state[:rows], conv_weight=self.conv.conv.weight,
                                  conv_bias=self.conv.conv.bias, **prologue)
        else:
            x = ops.decode_linear(u, self.in_proj.weight, self.in_proj.bias, **prologue)
            y = ops.gated_conv_step(x, state[:rows], self.conv.conv.weight, self.conv.conv.bias)
        return ops.decode_linear(y, self.out_proj.weight, self.out_proj.bias)

    def _gated_conv_hip(self, u, inference_params):
        """silu(conv(u1)) * u2 and the state handling of ShortConvolution.forward/step in one launch."""
        from .. import ops

        weight, bias = self.conv.conv.weight, self.conv.conv.bias
        if inference_params is None:
            return ops.gated_conv_prefill(u, weight, bias)
        if inference_params.seqlen_offset > 0:
            state = self.conv._get_state(inference_params)
            return ops.gated_conv_step(u, state[: u.shape[0]], weight, bias)
        self.conv._init_state(inference_params)
        state = self.conv._get_state(inference_params)
        return ops.gated_conv_prefill(u, weight, bias, state=state[: u.shape[0]])

    def allocate_inference_cache(self, batch_size: int, max_seqlen: int, dtype=None, **kwargs):
        return {"conv": self.conv.allocate_inference_cache(batch_size, max_seqlen, dtype=dtype, **kwargs)}
