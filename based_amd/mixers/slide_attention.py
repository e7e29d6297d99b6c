"""Sliding-window softmax attention mixer backed by the gfx950 kernels.

Drop-in for SlidingAttention of based/models/mixers/slide_attention.py:284-600: same
constructor arguments, parameter names (Wqkv / out_proj), forward and
allocate_inference_cache signatures and the reference's linear (B, max_seqlen, 2, H, D) KV
cache.  `window_size=W` means query i attends keys [i - W//2, i] (flash-attn's
`window_size=(W//2, 0)` with causal=True, slide_attention.py:332-336).
In scope: self-attention, num_heads_kv == num_heads, head dims that are multiples of 8 up to 128
(64, 112 and 128 are the released models'), rotary over any leading multiple of 16 channels in
either pair layout, applied inside the kernels, window_size up to 256 (128 keys to the left, what
the released checkpoints use), no dropout / padding / varlen; other arguments raise
NotImplementedError.  Non-half inputs are computed in bf16
(the reference casts to bf16 for prefill, slide_attention.py:76-78).
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ops


class RotaryEmbedding(nn.Module):
    """Standard (non-interleaved or interleaved) rotary position embedding applied to the first
    `dim` channels of q and k; stands in for flash_attn.layers.rotary.RotaryEmbedding as used
    at slide_attention.py:346-355,553-556 (no xPos scaling)."""

    def __init__(self, dim: int, base: float = 10000.0, interleaved: bool = False, device=None):
        super().__init__()
        self.dim = dim
        self.base = float(base)
        self.interleaved = interleaved
        inv_freq = 1.0 / (self.base ** (torch.arange(0, dim, 2, device=device, dtype=torch.float32) / dim))
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    def _cos_sin(self, positions: torch.Tensor):
        freqs = torch.outer(positions.float(), self.inv_freq.to(positions.device))
        return freqs.cos(), freqs.sin()

    def tables(self, n_pos: int, device):
        """(cos, sin, interleaved): fp32 (>= n_pos, dim/2) tables for the kernels' in-flight rotation
        and the pair layout; grown on demand and kept (a captured decode graph holds their addresses)."""
        cached = getattr(self, "_tables", None)
        if cached is None or cached[0].shape[0] < n_pos or cached[0].device != device:
            if cached is not None:
                # a recorded graph may still point at the smaller tables: they stay alive (and
                # stay correct for the positions they cover)
                self._retired_tables = getattr(self, "_retired_tables", []) + [cached]
            cos, sin = self._cos_sin(torch.arange(n_pos, device=device))
            self._tables = (cos.contiguous(), sin.contiguous(), self.interleaved)
        return self._tables

    def _rotate(self, x, cos, sin):
        # x: (B, L, H, D); cos/sin: (L, dim/2)
        ro = x[..., : self.dim].float()
        cos, sin = cos[None, :, None, :], sin[None, :, None, :]
        if self.interleaved:
            x1, x2 = ro[..., 0::2], ro[..., 1::2]
            out = torch.stack([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).flatten(-2)
        else:
            x1, x2 = ro[..., : self.dim // 2], ro[..., self.dim // 2:]
            out = torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1)
        return torch.cat([out.to(x.dtype), x[..., self.dim:]], dim=-1)

    def forward(self, qkv: torch.Tensor, seqlen_offset: int = 0):
        """qkv (B, L, 3, H, D): rotates q and k at positions seqlen_offset .. seqlen_offset+L-1."""
        L = qkv.shape[1]
        pos = torch.arange(seqlen_offset, seqlen_offset + L, device=qkv.device)
        cos, sin = self._cos_sin(pos)
        q = self._rotate(qkv[:, :, 0], cos, sin)
        k = self._rotate(qkv[:, :, 1], cos, sin)
        return torch.stack([q, k, qkv[:, :, 2]], dim=2)


class SlidingAttention(nn.Module):
    def __init__(
        self,
        embed_dim,
        num_heads,
        num_heads_kv=None,
        cross_attn=False,
        qkv_proj_bias=True,
        out_proj_bias=True,
        dropout=0.0,
        softmax_scale=None,
        causal=True,
        layer_idx=None,
        rotary_emb_dim=0,
        rotary_emb_base=10000.0,
        rotary_emb_scale_base=None,
        rotary_emb_interleaved=False,
        fused_bias_fc=False,
        use_flash_attn=True,
        return_residual=False,
        checkpointing=False,
        window_size=128,
        device=None,
        dtype=None,
    ) -> None:
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        if cross_attn or (num_heads_kv is not None and num_heads_kv != num_heads):
            raise NotImplementedError("cross-attention / grouped KV heads are outside the HIP path")
        if dropout != 0.0:
            raise NotImplementedError("attention dropout is outside the HIP path (inference only)")
        if rotary_emb_scale_base is not None:
            raise NotImplementedError("xPos rotary scaling is not supported")
        if window_size is None:
            raise NotImplementedError("SlidingAttention needs a window (the reference asserts the same)")
        self.embed_dim = embed_dim
        self.cross_attn = False
        self.causal = True
        self.layer_idx = layer_idx
        self.rotary_emb_dim = rotary_emb_dim
        self.use_flash_attn = True
        self.return_residual = return_residual
        self.checkpointing = checkpointing
        self.window = (window_size // 2, 0)
        if self.window[0] > 128:
            raise NotImplementedError(f"left window {self.window[0]} > 128 is not built into the kernels")

        self.num_heads = num_heads
        self.num_heads_kv = num_heads
        assert self.embed_dim % num_heads == 0, "embed_dim must be divisible by num_heads"
        self.head_dim = self.embed_dim // num_heads
        if self.head_dim % 8 != 0 or self.head_dim > 128:
            raise NotImplementedError("the HIP kernels take head dims that are multiples of 8 up to 128")
        if self.rotary_emb_dim > 0 and (self.rotary_emb_dim % 16 != 0 or self.rotary_emb_dim > self.head_dim):
            # flash-attn's rotary kernels ask for the same (a multiple of 16, at most the head dim)
            raise NotImplementedError(f"rotary_emb_dim {self.rotary_emb_dim}: a multiple of 16 up to head_dim {self.head_dim}")
        self.softmax_scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(self.head_dim)
        if self.rotary_emb_dim > 0:
            self.rotary_emb = RotaryEmbedding(self.rotary_emb_dim, base=rotary_emb_base,
                                              interleaved=rotary_emb_interleaved, device=device)
        qkv_dim = self.head_dim * 3 * self.num_heads
        self.Wqkv = nn.Linear(embed_dim, qkv_dim, bias=qkv_proj_bias, **factory_kwargs)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=out_proj_bias, **factory_kwargs)

    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None):
        dtype = self.out_proj.weight.dtype if dtype is None else dtype
        if dtype not in (torch.bfloat16,):
            dtype = torch.bfloat16  # the kernels attend in bf16
        device = self.out_proj.weight.device
        return torch.empty(batch_size, max_seqlen, 2, self.num_heads_kv, self.head_dim, dtype=dtype, device=device)

    def _cache(self, inference_params, like: torch.Tensor):
        assert self.layer_idx is not None, "Generation requires layer_idx in the constructor"
        d = inference_params.key_value_memory_dict
        if self.layer_idx not in d:
            d[self.layer_idx] = torch.empty(inference_params.max_batch_size, inference_params.max_seqlen, 2,
                                            self.num_heads_kv, self.head_dim, dtype=torch.bfloat16, device=like.device)
        return d[self.layer_idx]

    def supports_decode_step(self) -> bool:
        return ops.decode_linear_weight_ok(self.Wqkv.weight) and ops.decode_linear_weight_ok(self.out_proj.weight)

    def decode_step(self, x, inference_params, **prologue):
        """One token per sequence with the projections as `ops.decode_linear` launches: x (b, hidden)
        bf16 -> (b, hidden).  `prologue` goes to the first projection (the block's residual add +
        norm, possibly the embedding gather)."""
        qkv = ops.decode_linear(x, self.Wqkv.weight, self.Wqkv.bias, **prologue)
        b = qkv.shape[0]
        qkv = qkv.view(b, 1, 3, self.num_heads, self.head_dim)
        offset = inference_params.seqlen_offset
        rope = None
        if self.rotary_emb_dim > 0:
            rope = self.rotary_emb.tables(max(inference_params.max_seqlen, offset + 1), qkv.device)
        cache = self._cache(inference_params, qkv)
        b0 = inference_params.batch_size_offset
        pos = offset
        if inference_params.lengths_per_sample is not None:
            pos = inference_params.lengths_per_sample[b0:b0 + b]
        context = ops.swa_step(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], cache[b0:b0 + b], pos,
                               w_left=self.window[0], scale=self.softmax_scale, rope=rope)
        return ops.decode_linear(context.view(b, self.embed_dim), self.out_proj.weight, self.out_proj.bias)

    def forward(self, x, x_kv=None, key_padding_mask=None, cu_seqlens=None, max_seqlen=None,
                mixer_subset=None, inference_params=None, **kwargs):
        """x (batch, seqlen, hidden) -> (batch, seqlen, hidden)."""
        if x_kv is not None or mixer_subset is not None:
            raise NotImplementedError("cross-attention inputs are outside the HIP path")
        if key_padding_mask is not None or cu_seqlens is not None or max_seqlen is not None:
            raise NotImplementedError("padding masks / variable-length batches are outside the HIP path")
        in_dtype = x.dtype
        batch, seqlen = x.shape[:2]
        qkv = self.Wqkv(x)
        qkv = qkv.view(batch, seqlen, 3, self.num_heads, self.head_dim)
        if qkv.dtype != torch.bfloat16:
            qkv = qkv.to(torch.bfloat16)
        offset = 0 if inference_params is None else inference_params.seqlen_offset
        # the rotation (whole head or a leading part, either pair layout) happens inside the kernels,
        # at positions they take from the host or, for a recorded decode step, from the device
        rope = None
        if self.rotary_emb_dim > 0:
            n_pos = seqlen if inference_params is None else max(inference_params.max_seqlen, offset + seqlen)
            rope = self.rotary_emb.tables(n_pos, qkv.device)
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]

        if inference_params is None:
            context = ops.swa_prefill(q, k, v, w_left=self.window[0], scale=self.softmax_scale, rope=rope)
        elif offset == 0:
            cache = self._cache(inference_params, qkv)
            b0 = inference_params.batch_size_offset
            assert b0 + batch <= cache.shape[0] and seqlen <= cache.shape[1]
            # the kernel also files the (rotated) k and the v rows in the cache
            context = ops.swa_prefill(q, k, v, w_left=self.window[0], scale=self.softmax_scale, rope=rope,
                                      kv_cache=cache[b0:b0 + batch])
        else:
            assert seqlen == 1, "decoding feeds one token at a time"
            cache = self._cache(inference_params, qkv)
            b0 = inference_params.batch_size_offset
            pos = offset
            if inference_params.lengths_per_sample is not None:
                pos = inference_params.lengths_per_sample[b0:b0 + batch]
            context = ops.swa_step(q, k, v, cache[b0:b0 + batch], pos, w_left=self.window[0],
                                   scale=self.softmax_scale, rope=rope)
        out = self.out_proj(context.reshape(batch, seqlen, self.embed_dim).to(in_dtype))
        return out if not self.return_residual else (out, x)
