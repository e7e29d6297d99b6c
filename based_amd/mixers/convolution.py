"""Gated short convolution mixer; mirrors based/models/mixers/convolution.py:16-218 (non-CUDA
branch): depthwise causal conv (kernel 3) -> SiLU -> gate -> out_proj, with a rolling (B, D, K)
state for decoding.  On a HIP device everything between the two projections is one kernel
(`ops.gated_conv_prefill` / `ops.gated_conv_step`); host tensors take the literal torch
statement of the same arithmetic, which is what the module-level CPU tests exercise."""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F


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
        """x (b, l, d) -> (b, l, d)."""
        b, l, d = x.shape
        if inference_params is not None:
            if inference_params.seqlen_offset > 0:
                return self.step(x, self._get_state(inference_params))
            self._init_state(inference_params)
            state = self._get_state(inference_params)
            kk = min(self.kernel_size, l)
            state[:b, :, -kk:] = x[:, -kk:].transpose(1, 2)
        return self.conv(x.transpose(1, 2))[..., :l].transpose(1, 2)

    def step(self, x: torch.Tensor, state: torch.Tensor):
        state = state[: x.shape[0]]
        state.copy_(torch.roll(state, shifts=-1, dims=-1))
        state[:, :, -1] = x.squeeze(1)
        y = torch.einsum("bdk,dgk->bd", state, self.conv.weight).to(x.dtype)
        if self.conv.bias is not None:
            y = y + self.conv.bias
        return y.unsqueeze(1)

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
        u = self.in_proj(u)
        if u.is_cuda:
            return self.out_proj(self._gated_conv_hip(u, inference_params))
        u1, u2 = torch.split(u, self.d_inner, dim=-1)
        u_conv = F.silu(self.conv(u1, inference_params=inference_params))
        return self.out_proj(u_conv * u2)

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
