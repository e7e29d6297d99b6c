"""Minimal Based language-model stack around the HIP mixers (plain PyTorch glue).

Just enough of based/models/gpt.py (create_mixer_cls :64-96, create_block :347-394, _init_weights
:463-485, GPTModel :510-736, GPTLMHeadModel :739-827), block.py (:114-163), mlp.py (GatedMlp
:99-157) and the RMSNorm closed form (based/ops/triton/layer_norm.py:117-118) to run the
27-layer Based-360m shape end to end: embeddings -> [prenorm Block(mixer, SwiGLU MLP)] x N ->
final norm -> tied LM head, with the generation cache threaded through.  The GEMMs and the
embedding lookup are ordinary torch (hipBLASLt); mixers, add + RMSNorm and the SwiGLU gate are
the HIP kernels, and there is no host-tensor path.
"""
from __future__ import annotations

import math
from collections import namedtuple
from functools import partial
from types import SimpleNamespace
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

from .generation import GenerationMixin
from .mixers.convolution import BaseConv, ShortConvolution
from .mixers.linear_attention import LinearAttention, TaylorExp
from .mixers.slide_attention import SlidingAttention

# `_target_` strings accepted in mixer config dicts: the reference's own paths and this package's.
_TARGETS = {
    "based.models.mixers.linear_attention.LinearAttention": LinearAttention,
    "based.models.mixers.linear_attention.TaylorExp": TaylorExp,
    "based.models.mixers.slide_attention.SlidingAttention": SlidingAttention,
    "based.models.mixers.convolution.BaseConv": BaseConv,
    "based.models.mixers.convolution.ShortConvolution": ShortConvolution,
    "based_amd.mixers.linear_attention.LinearAttention": LinearAttention,
    "based_amd.mixers.linear_attention.TaylorExp": TaylorExp,
    "based_amd.mixers.slide_attention.SlidingAttention": SlidingAttention,
    "based_amd.mixers.convolution.BaseConv": BaseConv,
    "based_amd.mixers.convolution.ShortConvolution": ShortConvolution,
}


def _instantiate(spec: dict, *args, **extra):
    """Tiny stand-in for hydra.utils.instantiate: nested dicts with `_target_` become objects."""
    spec = dict(spec)
    cls = _TARGETS[spec.pop("_target_")]
    kwargs = {k: (_instantiate(v) if isinstance(v, dict) and "_target_" in v else v) for k, v in spec.items()}
    kwargs.update(extra)
    return cls(*args, **kwargs)


class StackConfig(SimpleNamespace):
    """Attribute bag with the GPT2Config fields the stack reads (gpt.py:58-61 lets the config
    carry arbitrary attributes; so does this)."""

    def __init__(self, **kw):
        defaults = dict(
            n_embd=1024, n_layer=27, n_head=16, n_inner=None, vocab_size=50277, pad_vocab_size_multiple=8,
            layer_norm_epsilon=1e-5, rms_norm=True, residual_in_fp32=True, initializer_range=0.02,
            tie_word_embeddings=True, activation_function="swiglu", mlp_fc1_bias=False, mlp_fc2_bias=False,
            mlp_type="base", ff_mult=2,
            qkv_proj_bias=False, out_proj_bias=False, rotary_emb_fraction=0.0, rotary_emb_base=10000.0,
            rotary_emb_interleaved=False, scale_attn_weights=True, max_position_embeddings=0,
            mixer=None, alt_mixer=None, alt_mixer_layers=None, alt_mixer_2=None, alt_mixer_2_layers=None,
        )
        defaults.update(kw)
        super().__init__(**defaults)

    # What the reference assumes for a key that a config dictionary does not carry: transformers'
    # GPT2Config constructor defaults plus the getattr defaults of based/models/gpt.py:100-113,
    # 206-208, 254, 262, 352, 359, 529, 745.  They differ from the defaults above (which describe
    # the released Based configurations): a config.json written by the reference's training code
    # that omits a key must mean here what it means there.
    REFERENCE_DEFAULTS = dict(
        n_embd=768, n_layer=12, n_head=12, n_inner=None, vocab_size=50257, pad_vocab_size_multiple=1,
        layer_norm_epsilon=1e-5, rms_norm=False, residual_in_fp32=False, initializer_range=0.02,
        tie_word_embeddings=True, activation_function="gelu_new", mlp_fc1_bias=True, mlp_fc2_bias=True,
        mlp_type="base", ff_mult=2, qkv_proj_bias=True, out_proj_bias=True, rotary_emb_fraction=0.0,
        rotary_emb_base=10000.0, rotary_emb_interleaved=False, scale_attn_weights=True,
        max_position_embeddings=0, n_positions=1024,
    )

    @classmethod
    def from_reference_dict(cls, d: dict) -> "StackConfig":
        """Config from a dictionary in the reference's format (the content of a checkpoint's
        config.json, or the keyword arguments its tests pass to GPT2MixerConfig), missing keys
        filled with the reference's defaults.  GPT2Config's `n_positions` feeds
        `max_position_embeddings` (its attribute map), as the reference's model reads it."""
        cfg = dict(cls.REFERENCE_DEFAULTS)
        cfg.update(d)
        if "max_position_embeddings" not in d:
            cfg["max_position_embeddings"] = cfg["n_positions"]
        return cls(**cfg)

    @property
    def hidden_size(self):
        return self.n_embd

    @property
    def num_hidden_layers(self):
        return self.n_layer

    @property
    def num_attention_heads(self):
        return self.n_head


def based_360m_config(**overrides) -> StackConfig:
    """The 360M-scale benchmark stack: the layer plan of the released Based-360m (BaseConv everywhere
    except Taylor linear attention at layers {1,6,11,16,21} and sliding-window attention at
    {2,7,12,17,22}; train/configs/experiment/reference/based-360m.yaml:53-65) with window_size 128,
    i.e. 64 keys to the left, and no rotary.  The released checkpoint itself uses window_size 256
    and rotary over the whole head: `based_360m_released_config`."""
    cfg = dict(
        n_embd=1024, n_layer=27, n_head=16, n_inner=2048, vocab_size=50277,
        mixer={"_target_": "based.models.mixers.convolution.BaseConv", "l_max": 2048, "use_bias": True,
               "expand_proj": 4, "kernel_size": 3},
        alt_mixer={"_target_": "based.models.mixers.linear_attention.LinearAttention", "l_max": 2048,
                   "feature_map": {"_target_": "based.models.mixers.linear_attention.TaylorExp", "input_dim": 16},
                   "feature_dim": 16, "num_heads": 16},
        alt_mixer_layers=[1, 6, 11, 16, 21],
        alt_mixer_2={"_target_": "based.models.mixers.slide_attention.SlidingAttention", "window_size": 128,
                     "num_heads": 16, "causal": True},
        alt_mixer_2_layers=[2, 7, 12, 17, 22],
    )
    cfg.update(overrides)
    return StackConfig(**cfg)


def based_360m_released_config(**overrides) -> StackConfig:
    """The model section of train/configs/experiment/reference/based-360m.yaml:49-115 as written:
    window_size 256 (128 keys to the left), rotary_emb_fraction 1, parallel_implementation
    "fla_parallel" on the linear-attention layers, everything else as `based_360m_config`."""
    cfg = vars(based_360m_config())
    cfg = {k: (dict(v) if isinstance(v, dict) else v) for k, v in cfg.items()}
    cfg["alt_mixer"]["parallel_implementation"] = "fla_parallel"
    cfg["alt_mixer_2"]["window_size"] = 256
    cfg.update(rotary_emb_fraction=1, n_positions=2048, max_position_embeddings=0)
    cfg.update(overrides)
    return StackConfig(**cfg)


def create_mixer_cls(config, layer_idx=None, device=None, dtype=None):
    """Layer -> mixer routing of gpt.py:64-96."""
    value = config.mixer
    if config.alt_mixer_2_layers is not None and layer_idx in config.alt_mixer_2_layers:
        value = config.alt_mixer_2
    elif config.alt_mixer_layers is not None and layer_idx in config.alt_mixer_layers:
        value = config.alt_mixer
    if value is None:
        raise NotImplementedError("plain multi-head attention layers are outside this build")
    value = dict(value)
    if "slide" in value["_target_"]:
        head_dim = config.hidden_size // config.num_attention_heads
        value.update({
            "num_heads": config.num_attention_heads,
            "qkv_proj_bias": config.qkv_proj_bias,
            "out_proj_bias": config.out_proj_bias,
            "softmax_scale": head_dim ** (-0.5) if config.scale_attn_weights else 1.0,
            "causal": True,
            "rotary_emb_dim": int(config.rotary_emb_fraction * head_dim),
            "rotary_emb_base": config.rotary_emb_base,
            "rotary_emb_interleaved": config.rotary_emb_interleaved,
        })
    return partial(_instantiate, value, device=device, dtype=dtype, layer_idx=layer_idx)


def _norm_kernel_takes(x, residual, weight) -> bool:
    """Whether `ops.add_rms_norm` accepts these device tensors: rows of a multiple of 8 up to 4096
    elements, bf16 or fp32 activations with a weight of the same dtype, a residual
    stream in bf16 or fp32 (fp32 for fp32 activations)."""
    D = x.shape[-1]
    if not (x.is_cuda and weight.is_cuda):
        raise ValueError("based_amd runs on HIP device tensors only (no CPU path)")
    if not (x.dtype in (torch.bfloat16, torch.float32) and weight.dtype == x.dtype
            and D % 8 == 0 and D <= ops.ADD_RMS_NORM_MAX_DIM and weight.is_contiguous()):
        return False
    if residual is None:
        return True
    return (residual.shape == x.shape and residual.dtype in (torch.bfloat16, torch.float32)
            and not (x.dtype == torch.float32 and residual.dtype != torch.float32))


class RMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) * weight (based/ops/triton/layer_norm.py:117-118), no bias."""

    def __init__(self, hidden_size, eps=1e-5, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, device=device, dtype=dtype))

    def forward(self, x):
        if _norm_kernel_takes(x, None, self.weight):
            return ops.add_rms_norm(x, None, self.weight, self.eps, want_residual=False)[0]
        # shapes, dtypes or devices the kernel is not built for: the closed form as the reference states it
        rstd = 1 / torch.sqrt(x.square().mean(dim=-1, keepdim=True) + self.eps)
        return (x * rstd * self.weight).to(x.dtype)


def add_norm(norm, hidden_states, residual, residual_in_fp32: bool, want_residual: bool = True):
    """residual + hidden, the norm of the sum, and the sum itself for the next block
    (block.py:134-139; gpt.py:676-694 for the closing norm).  RMSNorm on tensors the kernel takes
    is one launch; nn.LayerNorm (`rms_norm: False`, the reference's default) and everything the
    kernel refuses run the reference's own torch statement."""
    if isinstance(norm, RMSNorm) and _norm_kernel_takes(hidden_states, residual, norm.weight):
        if residual is None:
            return ops.add_rms_norm(hidden_states, None, norm.weight, norm.eps, residual_in_fp32, want_residual)
        return ops.add_rms_norm(hidden_states, residual, norm.weight, norm.eps,
                                residual.dtype == torch.float32, want_residual)
    residual = (hidden_states + residual) if residual is not None else hidden_states
    hidden_states = norm(residual.to(dtype=norm.weight.dtype))
    if not want_residual:
        return hidden_states, None
    if residual_in_fp32:
        residual = residual.to(torch.float32)
    return hidden_states, residual


_GATE_ACTIVATIONS = {"glu": torch.sigmoid, "swiglu": F.silu, "geglu": F.gelu}


class GatedMlp(nn.Module):
    """Gated MLP of based/models/mlp.py:99-157.  Layout 'base': fc2(y * act(gate)) with
    y, gate = fc1(x).chunk(2).  Layout 'alt' (the NeoX-style MLP of the reference's test
    configuration): fc2(act(fc1(x)) * fc3(x)) with a hidden size derived from ff_mult.
    activation: "swiglu" (silu; the released models), "geglu" (gelu) or "glu" (sigmoid),
    chosen as in gpt.py:238-243.  The released combination (base + swiglu) gates in one HIP
    kernel; the others are two element-wise torch operations."""

    def __init__(self, in_features, hidden_features=None, activation="swiglu", bias1=False, bias2=False,
                 multiple_of=256, mlp_type="base", ff_mult=2, device=None, dtype=None):
        super().__init__()
        if activation not in _GATE_ACTIVATIONS:
            raise NotImplementedError(f"activation_function {activation!r}: only gated MLPs (glu / swiglu / geglu)")
        fk = {"device": device, "dtype": dtype}
        self.activation = activation
        self.mlp_type = mlp_type
        if mlp_type == "base":
            hidden_features = hidden_features if hidden_features is not None else int(8 * in_features / 3)
            hidden_features = (hidden_features + multiple_of - 1) // multiple_of * multiple_of
            self.fc1 = nn.Linear(in_features, 2 * hidden_features, bias=bias1, **fk)
        else:
            hidden_features = int(2 * in_features * ff_mult / 3)
            hidden_features = (hidden_features + multiple_of - 1) // multiple_of * multiple_of
            self.fc1 = nn.Linear(in_features, hidden_features, bias=bias1, **fk)
            self.fc3 = nn.Linear(in_features, hidden_features, bias=bias1, **fk)
        self.fc2 = nn.Linear(hidden_features, in_features, bias=bias2, **fk)

    def forward(self, x):
        if self.mlp_type != "base":
            return self.fc2(_GATE_ACTIVATIONS[self.activation](self.fc1(x)) * self.fc3(x))
        if self.activation == "swiglu":
            return self.fc2(ops.swiglu(self.fc1(x)))
        y, gate = self.fc1(x).chunk(2, dim=-1)
        return self.fc2(y * _GATE_ACTIVATIONS[self.activation](gate))


class Block(nn.Module):
    """Prenorm block: add -> norm1 -> mixer -> add -> norm2 -> mlp, returning (hidden, residual)
    (block.py:134-163, dropout-free)."""

    def __init__(self, dim, mixer_cls, mlp_cls, norm_cls, residual_in_fp32=True, layer_idx=None):
        super().__init__()
        self.residual_in_fp32 = residual_in_fp32
        self.layer_idx = layer_idx
        self.mixer = mixer_cls(dim)
        self.norm1 = norm_cls(dim)
        self.mlp = mlp_cls(dim)
        self.norm2 = norm_cls(dim)

    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None, **kwargs):
        return self.mixer.allocate_inference_cache(batch_size, max_seqlen, dtype=dtype, **kwargs)

    def _add_norm(self, norm, hidden_states, residual):
        """residual + hidden, the norm of the sum, and the sum kept for the next block
        (block.py:134-139)."""
        return add_norm(norm, hidden_states, residual, self.residual_in_fp32)

    def supports_decode_step(self) -> bool:
        mlp = self.mlp
        return (getattr(self.mixer, "supports_decode_step", lambda: False)()
                and mlp.mlp_type == "base" and mlp.activation == "swiglu"
                and ops.decode_linear_weight_ok(mlp.fc1.weight) and ops.decode_linear_weight_ok(mlp.fc2.weight)
                and isinstance(self.norm1, RMSNorm) and isinstance(self.norm2, RMSNorm)
                and self.norm1.weight.dtype == torch.bfloat16 and self.residual_in_fp32)

    def decode_step(self, hidden_states, residual, spare, inference_params, row_index=None):
        """The block for one token per sequence in four to five launches: both norms run inside the
        projection that consumes them (`ops.decode_linear`), the SwiGLU gate in the tail of fc1.
        hidden_states (b, dim) bf16 (or the embedding table with `row_index`), residual fp32
        (b, dim) or None; `spare` is a second fp32 (b, dim) buffer: the two take turns as the
        input and the output of the residual stream.  Returns (hidden, residual, spare)."""
        if residual is None:
            residual_in, mid, last = None, spare[0], spare[1]
        else:
            residual_in, mid, last = residual, spare, residual
        norm = dict(prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=residual_in, residual_out=mid,
                    norm_weight=self.norm1.weight, eps=self.norm1.eps)
        if row_index is not None:
            norm["row_index"] = row_index
        hidden_states = self.mixer.decode_step(hidden_states, inference_params, **norm)
        norm = dict(prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=mid, residual_out=last,
                    norm_weight=self.norm2.weight, eps=self.norm2.eps)
        fc1, fc2 = self.mlp.fc1, self.mlp.fc2
        if fc1.weight.shape[1] <= 2048:
            # the gate in the tail of fc1
            gated = ops.decode_linear(hidden_states, fc1.weight, fc1.bias, epilogue=ops.EPILOGUE_SWIGLU, **norm)
            hidden_states = ops.decode_linear(gated, fc2.weight, fc2.bias)
        else:
            # wider models: the gate in front of fc2
            gate_in = ops.decode_linear(hidden_states, fc1.weight, fc1.bias, **norm)
            hidden_states = ops.decode_linear(gate_in, fc2.weight, fc2.bias, prologue=ops.PROLOGUE_SWIGLU)
        return hidden_states, last, mid

    def forward(self, hidden_states, residual=None, mixer_kwargs=None, position_ids=None, decay=None):
        hidden_states, residual = self._add_norm(self.norm1, hidden_states, residual)
        mixer_kwargs = mixer_kwargs or {}
        if position_ids is not None or decay is not None:
            hidden_states = self.mixer(hidden_states, position_ids=position_ids, decay=decay, **mixer_kwargs)
        else:
            hidden_states = self.mixer(hidden_states, **mixer_kwargs)
        hidden_states, residual = self._add_norm(self.norm2, hidden_states, residual)
        return self.mlp(hidden_states), residual


def _init_weights(module, n_layer, initializer_range=0.02):
    if isinstance(module, nn.Linear):
        nn.init.normal_(module.weight, std=initializer_range)
        if module.bias is not None:
            nn.init.zeros_(module.bias)
    elif isinstance(module, nn.Embedding):
        nn.init.normal_(module.weight, std=initializer_range)
    for name, p in module.named_parameters():
        if name in ["out_proj.weight", "fc2.weight"]:
            nn.init.normal_(p, mean=0.0, std=initializer_range / math.sqrt(2 * n_layer))


class GPTModel(nn.Module):
    def __init__(self, config: StackConfig, device=None, dtype=None):
        super().__init__()
        fk = {"device": device, "dtype": dtype}
        self.config = config
        self.residual_in_fp32 = config.residual_in_fp32
        vocab = math.ceil(config.vocab_size / config.pad_vocab_size_multiple) * config.pad_vocab_size_multiple
        self.embeddings = nn.Module()
        self.embeddings.word_embeddings = nn.Embedding(vocab, config.hidden_size, **fk)
        if config.max_position_embeddings > 0:
            self.embeddings.position_embeddings = nn.Embedding(config.max_position_embeddings, config.hidden_size, **fk)
        # rms_norm absent from a reference config means nn.LayerNorm (gpt.py:352,537)
        norm_cls = partial(RMSNorm if config.rms_norm else nn.LayerNorm, eps=config.layer_norm_epsilon, **fk)
        mlp_cls = partial(GatedMlp, hidden_features=config.n_inner, activation=config.activation_function,
                          bias1=config.mlp_fc1_bias, bias2=config.mlp_fc2_bias, mlp_type=config.mlp_type,
                          ff_mult=config.ff_mult, **fk)
        self.layers = nn.ModuleList([
            Block(config.hidden_size, create_mixer_cls(config, layer_idx=i, **fk), mlp_cls, norm_cls,
                  residual_in_fp32=config.residual_in_fp32, layer_idx=i)
            for i in range(config.num_hidden_layers)
        ])
        self.ln_f = norm_cls(config.hidden_size)
        self.apply(partial(_init_weights, n_layer=config.num_hidden_layers,
                           initializer_range=config.initializer_range))

    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None, **kwargs):
        return {i: layer.allocate_inference_cache(batch_size, max_seqlen, dtype=dtype, **kwargs)
                for i, layer in enumerate(self.layers)}

    # Single-token steps of a bf16 model run through `decode_layers`: every projection is an
    # `ops.decode_linear` launch with the element-wise work in front of it folded in.  Set to False
    # to send them through the general path (torch GEMMs + stand-alone norm and gate kernels).
    fused_decode = True

    def decode_layers_ok(self, input_ids, inference_params) -> bool:
        if not (self.fused_decode and inference_params is not None and inference_params.seqlen_offset > 0
                and input_ids.shape[1] == 1 and input_ids.shape[0] <= ops.DECODE_LINEAR_MAX_ROWS
                and input_ids.is_cuda and not torch.is_grad_enabled()
                and self.config.max_position_embeddings == 0):
            return False
        # the answer depends on dtypes and devices of the parameters only: worked out once per
        # (dtype, device) of the embedding table
        table = self.embeddings.word_embeddings.weight
        cached = self.__dict__.get("_decode_layers_supported")
        if cached is None or cached[0] != (table.dtype, table.device):
            ok = (ops.decode_linear_weight_ok(table) and isinstance(self.ln_f, RMSNorm)
                  and self.ln_f.weight.dtype == torch.bfloat16
                  and all(layer.supports_decode_step() for layer in self.layers))
            cached = ((table.dtype, table.device), ok)
            self.__dict__["_decode_layers_supported"] = cached
        return cached[1]

    def decode_layers(self, input_ids, inference_params):
        """All blocks for one token per sequence.  Returns (hidden (b, dim) bf16, residual (b, dim)
        fp32): the inputs of the closing add + norm, which the caller folds into what follows."""
        b = input_ids.shape[0]
        table = self.embeddings.word_embeddings.weight
        key = (b, table.device)
        buffers = self.__dict__.setdefault("_decode_residuals", {}).get(key)
        if buffers is None:
            buffers = tuple(torch.empty(b, table.shape[1], dtype=torch.float32, device=table.device) for _ in range(2))
            self._decode_residuals[key] = buffers
        ids = input_ids.reshape(-1).contiguous()  # a column of a wider id tensor is a strided view
        hidden_states, residual, spare = self.layers[0].decode_step(table, None, buffers, inference_params, row_index=ids)
        for layer in self.layers[1:]:
            hidden_states, residual, spare = layer.decode_step(hidden_states, residual, spare, inference_params)
        return hidden_states, residual

    def forward(self, input_ids, position_ids=None, inference_params=None, stream=None):
        if self.decode_layers_ok(input_ids, inference_params):
            hidden_states, residual = self.decode_layers(input_ids, inference_params)
            return add_norm(self.ln_f, hidden_states, residual, True, want_residual=False)[0].unsqueeze(1)
        hidden_states = self.embeddings.word_embeddings(input_ids)
        if self.config.max_position_embeddings > 0:
            if position_ids is None:
                position_ids = torch.arange(input_ids.shape[1], dtype=torch.long, device=input_ids.device)
            hidden_states = hidden_states + self.embeddings.position_embeddings(position_ids)
        residual = None
        mixer_kwargs = {}
        if inference_params is not None:
            mixer_kwargs["inference_params"] = inference_params
            mixer_kwargs["stream"] = stream
        for layer in self.layers:
            hidden_states, residual = layer(hidden_states, residual=residual, position_ids=position_ids,
                                            mixer_kwargs=mixer_kwargs)
        return add_norm(self.ln_f, hidden_states, residual, self.residual_in_fp32, want_residual=False)[0]


class GPTLMHeadModel(nn.Module, GenerationMixin):
    def __init__(self, config: StackConfig, device=None, dtype=None):
        super().__init__()
        self.config = config
        self.transformer = GPTModel(config, device=device, dtype=dtype)
        vocab = self.transformer.embeddings.word_embeddings.num_embeddings
        self.lm_head = nn.Linear(config.n_embd, vocab, bias=False, device=device, dtype=dtype)
        self.apply(partial(_init_weights, n_layer=config.num_hidden_layers,
                           initializer_range=config.initializer_range))
        if config.tie_word_embeddings:
            self.lm_head.weight = self.transformer.embeddings.word_embeddings.weight

    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None, **kwargs):
        return self.transformer.allocate_inference_cache(batch_size, max_seqlen, dtype=dtype, **kwargs)

    @classmethod
    def from_pretrained_local(cls, directory, device=None, dtype=None, strict=True):
        """Builds the model from a LOCAL directory laid out like the released checkpoints:
        `config.json` (the GPT2Config dictionary) and `pytorch_model.bin` or `model.safetensors`.
        Counterpart of from_pretrained_hf (gpt.py:446-459) without the hub: same key clean-up
        (leading "model." stripped, training-metric entries dropped).  The weights file is read
        with a loader that executes nothing from it."""
        import json
        import os
        import re

        with open(os.path.join(directory, "config.json")) as f:
            config = StackConfig.from_reference_dict(json.load(f))
        model = cls(config, device=device, dtype=dtype)
        st_path = os.path.join(directory, "model.safetensors")
        if os.path.exists(st_path):
            from safetensors.torch import load_file

            state = load_file(st_path, device="cpu")
        else:
            state = torch.load(os.path.join(directory, "pytorch_model.bin"), map_location="cpu", weights_only=True)
        state = {re.sub(r"^model\.", "", k): v for k, v in state.items() if "metrics" not in k}
        if config.tie_word_embeddings and "lm_head.weight" not in state:
            state["lm_head.weight"] = state["transformer.embeddings.word_embeddings.weight"]
        model.load_state_dict(state, strict=strict)
        return model

    def load_state_dict(self, state_dict, strict=True, **kwargs):
        """Also accepts checkpoints written with the older order of the layers in a block (norm
        after the mixer / MLP, a leading `transformer.ln_0`): their norm parameters are moved to
        the current prenorm slots exactly as the reference does (gpt.py:829-853); norms without
        a bias (RMSNorm) simply have no bias entries to move."""
        if "transformer.ln_0.weight" in state_dict:
            state_dict = dict(state_dict)
            n_layers = len(self.transformer.layers)

            def move(src, dst):
                for suffix in ("weight", "bias"):
                    if f"{src}.{suffix}" in state_dict:
                        state_dict[f"{dst}.{suffix}"] = state_dict.pop(f"{src}.{suffix}")

            move(f"transformer.layers.{n_layers - 1}.norm2", "transformer.ln_f")
            for l in reversed(range(n_layers)):
                move(f"transformer.layers.{l}.norm1", f"transformer.layers.{l}.norm2")
                if l > 0:
                    move(f"transformer.layers.{l - 1}.norm2", f"transformer.layers.{l}.norm1")
            move("transformer.ln_0", "transformer.layers.0.norm1")
        return super().load_state_dict(state_dict, strict=strict, **kwargs)

    def forward(self, input_ids, position_ids=None, inference_params=None, num_last_tokens=0, stream=None, **kwargs):
        assert input_ids.ndim == 2, f"Expected `input_ids` to have shape [b, slen], but got shape {input_ids.shape}"
        CausalLMOutput = namedtuple("CausalLMOutput", ["logits"])
        if (self.transformer.decode_layers_ok(input_ids, inference_params)
                and ops.decode_linear_weight_ok(self.lm_head.weight)):
            # closing add + norm inside the LM head's projection
            hidden_states, residual = self.transformer.decode_layers(input_ids, inference_params)
            ln_f = self.transformer.ln_f
            logits = ops.decode_linear(hidden_states, self.lm_head.weight, self.lm_head.bias,
                                       prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=residual,
                                       norm_weight=ln_f.weight, eps=ln_f.eps)
            return CausalLMOutput(logits=logits.unsqueeze(1))
        hidden_states = self.transformer(input_ids, position_ids=position_ids, inference_params=inference_params,
                                         stream=stream)
        if num_last_tokens > 0:
            hidden_states = hidden_states[:, -num_last_tokens:]
        return CausalLMOutput(logits=self.lm_head(hidden_states))
