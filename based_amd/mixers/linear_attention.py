"""Taylor linear attention mixer backed by the gfx950 kernels.

Drop-in for based/models/mixers/linear_attention.py of the reference: same constructor
arguments, parameter names (proj_q / proj_k / proj_v / out_proj), forward /
recurrent_forward / allocate_inference_cache signatures and cache layout.  The q/k/v and
output projections stay ordinary nn.Linear GEMMs; everything between them (feature map,
causal product, normaliser, decode-state construction and update) is one HIP kernel call.
There is no non-HIP path: tensors must live on the GPU.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..generation import InferenceParams


class FeatureMap(nn.Module):
    """Parent feature map; identity (linear_attention.py:37-50)."""

    def __init__(self, input_dim: int, **kwargs):
        super().__init__()
        self.input_dim = input_dim

    def forward(self, x: torch.Tensor):
        return x


class TaylorExp(FeatureMap):
    """2nd-order Taylor feature map, 16 -> 273 dims (linear_attention.py:52-75).

    Kept as a module so configs and callers that name it keep working.  The mixer's kernels
    evaluate the map on the fly from the raw 16-dim vectors and never call forward(); forward()
    is the explicit expansion for callers that want phi(x) itself (e.g. to hand
    recurrent_forward its pre-mapped arguments)."""

    def __init__(self, input_dim: int, **kwargs):
        super().__init__(input_dim, **kwargs)
        self.r2 = math.sqrt(2)
        self.rd = math.sqrt(input_dim)
        self.rrd = math.sqrt(self.rd)

    def forward(self, x: torch.Tensor):
        x2 = (x.unsqueeze(-1) * x.unsqueeze(-2)).flatten(start_dim=-2) / self.r2
        return torch.cat([x[..., :1] ** 0, x / self.rrd, x2 / self.rd], dim=-1)

    def raw_from_mapped(self, fx: torch.Tensor) -> torch.Tensor:
        """Inverse on the linear block: phi(x)[1:1+d] = x / d^(1/4)."""
        return fx[..., 1:1 + self.input_dim] * self.rrd


class LinearAttention(nn.Module):
    def __init__(
        self,
        d_model: int,
        feature_map: FeatureMap = None,
        l_max: int = 2048,
        feature_dim: int = 16,
        head_dim: int = None,
        num_heads: int = 16,
        eps: float = 1e-12,
        layer_idx: int = None,
        parallel_implementation: str = "quadratic",
        deferred_state_steps: int = 0,
        device=None,
        dtype=None,
        **kwargs,
    ):
        super().__init__()
        factory_kwargs = {"device": device, "dtype": dtype}
        self.layer_idx = layer_idx
        self.d_model = d_model
        self.l_max = l_max
        # Accepted for config compatibility; there is exactly one implementation here.  The one
        # thing the name changes is the regulariser of the denominator: the reference's "fla_*"
        # paths use 1e-6 instead of `eps`, in the parallel kernel they call and in the recurrent
        # step (linear_attention.py:199-212,245-249); so does this module.
        self.parallel_implementation = parallel_implementation
        self.eps = 1e-6 if "fla" in parallel_implementation else eps
        # Not in the reference.  2..8: a decode step only reads kv_state and parks the token's k and v
        # in a small ring; every that-many-th step writes the state (`ops.linear_attn_step_deferred`:
        # same outputs, about 40 % less memory traffic per step at period 8).  The inference cache
        # then carries the ring after the two states, and kv_state is current only after such a step
        # or after `flush_deferred_state`.  0 or 1: the reference's behaviour, kv_state rewritten by
        # every step.
        if not 0 <= int(deferred_state_steps) <= ops.DEFERRED_MAX_STEPS:
            raise ValueError(f"deferred_state_steps must be in [0, {ops.DEFERRED_MAX_STEPS}]")
        self.deferred_state_steps = int(deferred_state_steps)

        self.num_heads = num_heads
        self.head_dim = self.d_model // self.num_heads if head_dim is None else head_dim
        self.feature_dim = feature_dim
        if feature_map is None or isinstance(feature_map, type):
            feature_map = TaylorExp(input_dim=feature_dim)
        if not isinstance(feature_map, TaylorExp) or feature_map.input_dim != ops.FEATURE_DIM or feature_dim != ops.FEATURE_DIM:
            raise NotImplementedError(
                "the HIP kernels implement the TaylorExp feature map with feature_dim=16 only")
        self.feature_map = feature_map

        self.proj_q = nn.Linear(self.d_model, self.feature_dim * self.num_heads, bias=False, **factory_kwargs)
        self.proj_k = nn.Linear(self.d_model, self.feature_dim * self.num_heads, bias=False, **factory_kwargs)
        self.proj_v = nn.Linear(self.d_model, self.num_heads * self.head_dim, bias=False, **factory_kwargs)
        self.out_proj = nn.Linear(self.num_heads * self.head_dim, self.d_model, bias=False, **factory_kwargs)

    def forward(self, hidden_states: torch.Tensor, inference_params: InferenceParams = None, *args, **kwargs):
        """hidden_states (b, l, d_model) -> (b, l, d_model)."""
        b, l, _ = hidden_states.size()
        if l == 1 and inference_params is not None and not torch.is_grad_enabled():
            # a decode step is bound by launches, not by arithmetic: one GEMM over the stacked
            # projection weights instead of three
            nq = self.feature_dim * self.num_heads
            qkv = F.linear(hidden_states, self._stacked_qkv_weight())
            q, k, v = qkv[..., :nq], qkv[..., nq:2 * nq], qkv[..., 2 * nq:]
        else:
            q, k, v = self.proj_q(hidden_states), self.proj_k(hidden_states), self.proj_v(hidden_states)
        q = q.view(b, l, self.num_heads, self.feature_dim).transpose(1, 2)
        k = k.view(b, l, self.num_heads, self.feature_dim).transpose(1, 2)
        v = v.view(b, l, self.num_heads, self.head_dim).transpose(1, 2)

        self.is_inference = inference_params is not None
        if inference_params is None:
            return self.parallel_forward(hidden_states, q, k, v)
        if inference_params.seqlen_offset > 0:
            y = self._cache_step(self._get_inference_cache(inference_params), q, k, v)
            return self.out_proj(y.transpose(1, 2).reshape(b, l, self.num_heads * self.head_dim))
        y, kv_state, k_state = self.parallel_forward(hidden_states, q, k, v)
        if self.layer_idx in inference_params.key_value_memory_dict:
            # pre-allocated caches (graph-style decoding) are filled in place
            cache = inference_params.key_value_memory_dict[self.layer_idx]
            cache[0][:b].copy_(kv_state)
            cache[1][:b].copy_(k_state)
            if len(cache) > 2:
                cache[4][:b].zero_()  # the ring of a deferred-update cache starts empty
        else:
            cache = (kv_state, k_state)
            if self.deferred_state_steps > 1:
                cache += ops.deferred_step_buffers(b, self.num_heads, self.head_dim, kv_state.device)
            inference_params.key_value_memory_dict[self.layer_idx] = cache
        return y

    def _cache_step(self, cache, q, k, v):
        """One decode step on an inference cache, (kv_state, k_state) or that plus the ring of the
        deferred update: q, k (b, h, 1, 16), v (b, h, 1, head_dim) -> y (b, h, 1, head_dim).  Caches
        allocated for a larger batch serve a smaller one through their leading rows."""
        b = q.shape[0]
        if len(cache) > 2 and self.deferred_state_steps > 1:
            return ops.linear_attn_step_deferred(q, k, v, cache[0][:b], cache[1][:b], tuple(t[:b] for t in cache[2:]),
                                                 self.deferred_state_steps, eps=self.eps)
        if len(cache) > 2:
            # a cache with a ring, but the option has been switched off since: bring the state up to date
            ops.linear_attn_flush_deferred(cache[0], cache[2:])
        return ops.linear_attn_step(q, k, v, cache[0][:b], cache[1][:b], eps=self.eps)

    def flush_deferred_state(self, inference_params: InferenceParams) -> None:
        """Applies the tokens still parked in the ring to kv_state (for whoever reads kv_state
        itself: the decode steps do not need it).  Nothing to do without the deferred update."""
        cache = inference_params.key_value_memory_dict.get(self.layer_idx)
        if cache is not None and len(cache) > 2:
            ops.linear_attn_flush_deferred(cache[0], cache[2:])

    def decode_step(self, x: torch.Tensor, inference_params: InferenceParams, **prologue) -> torch.Tensor:
        """One token per sequence with the projections as `ops.decode_linear` launches: x (b, d_model)
        bf16 -> (b, d_model).  `prologue` goes to the first projection (the block's residual add +
        norm, possibly the embedding gather, fused in front of it); with a `row_index` in it, x is
        the table the rows are gathered from."""
        qkv = ops.decode_linear(x, self._stacked_qkv_weight(), **prologue)
        b = qkv.shape[0]
        nq = self.feature_dim * self.num_heads
        q = qkv[:, :nq].view(b, self.num_heads, 1, self.feature_dim)
        k = qkv[:, nq:2 * nq].view(b, self.num_heads, 1, self.feature_dim)
        v = qkv[:, 2 * nq:].view(b, self.num_heads, 1, self.head_dim)
        y = self._cache_step(self._get_inference_cache(inference_params), q, k, v)
        return ops.decode_linear(y.view(b, self.num_heads * self.head_dim), self.out_proj.weight, self.out_proj.bias)

    def supports_decode_step(self) -> bool:
        return all(ops.decode_linear_weight_ok(w) for w in
                   (self.proj_q.weight, self.proj_k.weight, self.proj_v.weight, self.out_proj.weight))

    def _stacked_qkv_weight(self) -> torch.Tensor:
        """[proj_q; proj_k; proj_v] weights as one matrix for the single-token step.  The first call
        moves the three weights into one tensor and turns each `weight.data` into a view of its
        rows, so there is no second copy that could go stale: writes through `weight.data`,
        optimizers and `load_state_dict` all land in the shared storage.  Only a weight whose
        tensor is replaced (`.to()`, a new Parameter, `weight.data = other`) changes the key below
        (storage address, version counter), and the stack is then rebuilt from the live weights."""
        ws = (self.proj_q.weight, self.proj_k.weight, self.proj_v.weight)
        key = tuple((w.data_ptr(), w._version) for w in ws)
        cached = getattr(self, "_qkv_cache", None)
        if cached is None or cached[0] != key:
            with torch.inference_mode(False), torch.no_grad():
                stacked = torch.cat([w.detach() for w in ws], dim=0)
                row = 0
                for w in ws:
                    w.data = stacked[row:row + w.shape[0]]
                    row += w.shape[0]
            cached = (tuple((w.data_ptr(), w._version) for w in ws), stacked)
            self._qkv_cache = cached
        return cached[1]

    def invalidate_stacked_weights(self) -> None:
        """Forgets the stacked projection matrix (it is rebuilt from proj_q / proj_k / proj_v at the
        next single-token step).  Never needed for in-place writes; for callers that swap weight
        tensors behind the module's back in ways the key above cannot see."""
        self._qkv_cache = None

    def parallel_forward(self, x: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        """q, k: (b, h, l, 16) raw; v: (b, h, l, head_dim).  Returns out_proj(y), plus the decode
        states when called on the inference path."""
        is_inference = getattr(self, "is_inference", False)
        y, kv_state, k_state = ops.linear_attn_prefill(q, k, v, eps=self.eps, return_state=is_inference)
        b, h, l, d = y.shape
        y = y.transpose(1, 2).reshape(b, l, h * d)  # 'b h l d -> b l (h d)', a view of the kernel output
        out = self.out_proj(y.to(x.dtype))
        if is_inference:
            return out, kv_state, k_state
        return out

    def _step(self, kv_state, k_state, q, k, v):
        y = ops.linear_attn_step(q, k, v, kv_state, k_state, eps=self.eps)
        b, h, l, d = y.shape
        return self.out_proj(y.transpose(1, 2).reshape(b, l, h * d))

    def recurrent_forward(self, hidden_states: torch.Tensor, kv_state: torch.Tensor, k_state: torch.Tensor,
                          q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor = None):
        """Reference signature: q, k arrive ALREADY feature-mapped, shape (b, h, 1, 273); v is
        (b, h, 1, head_dim).  The kernel fuses the map, so the raw vectors are recovered from
        the linear block of phi (exact: a multiplication by 2)."""
        b, h, l, d = q.shape
        assert l == 1, f"q.shape is {q.shape} but should be ({b}, {h}, 1, {d})"
        if d == self.feature_map.input_dim:
            raw_q, raw_k = q, k
        else:
            raw_q, raw_k = self.feature_map.raw_from_mapped(q), self.feature_map.raw_from_mapped(k)
        return self._step(kv_state, k_state, raw_q, raw_k, v)

    def expanded_size(self):
        return self.feature_dim ** 2 + self.feature_dim + 1

    def allocate_inference_cache(self, batch_size: int, max_seqlen: int, dtype=None, **kwargs):
        """(kv_state (B,H,1,head_dim,273), k_state (B,H,1,1,273)).  The states are carried in
        fp32 whatever `dtype` asks for: the decode kernel accumulates in place in fp32.  With
        `deferred_state_steps` > 1 the ring of the deferred update follows: keys (B,H,8,16), values
        (B,H,8,head_dim), fill count (B,H).  Such a cache is a 5-tuple and its kv_state lacks the
        tokens still parked in the ring: whoever reads, copies or reorders kv_state itself (beam
        search, cache export) must call `flush_deferred_state` first; unpacking it as
        `(kv_state, k_state)` is only valid for the default 2-tuple."""
        device = self.out_proj.weight.device
        kv_state = torch.zeros(batch_size, self.num_heads, 1, self.head_dim, self.expanded_size(),
                               dtype=torch.float32, device=device)
        k_state = torch.zeros(batch_size, self.num_heads, 1, 1, self.expanded_size(),
                              dtype=torch.float32, device=device)
        if self.deferred_state_steps > 1:
            return (kv_state, k_state) + ops.deferred_step_buffers(batch_size, self.num_heads, self.head_dim, device)
        return (kv_state, k_state)

    def _get_inference_cache(self, inference_params: InferenceParams):
        return inference_params.key_value_memory_dict[self.layer_idx]
