"""Pure-PyTorch CPU restatement of the Based sequence-mixer arithmetic.

TEST INFRASTRUCTURE ONLY: the shipped package never imports this file.  Each
function states, as plainly as possible, what the reference computes; the
citations are into the reference tree (paths relative to its root).

Pinning status (what independent evidence each function is checked against in
tests/test_oracle.py):

  taylor_exp              closed form  phi(q).phi(k) == 1 + s + s^2/2, element order,
                          phi(0) == e_0                                   -> pinned
  linear_attn_quadratic   brute-force per-element formula on tiny inputs, running-mean
                          special case, causality, the compiled reference C++ causal
                          product (oracle/_ref) for the numerator         -> pinned
  linear_attn_cumsum      equality with linear_attn_quadratic + reference C++ -> pinned
  linear_attn_prefill_state / linear_attn_step
                          recurrent == parallel invariant (the reference's own
                          test), closed-form state sums                   -> pinned
  sliding_window_attn     reduction to F.scaled_dot_product_attention(is_causal) when
                          the window covers the sequence, w=0 => o=v, q=0 => running
                          window mean, per-element brute force            -> pinned
                          against the textbook definition; the reference delegates
                          this arithmetic to flash-attn 2.5.2 (absent from the tree),
                          so agreement with THAT library is "parity unpinned".
  sliding_window_step     decode == prefill invariant                     -> pinned (same caveat)
  rms_norm / swiglu_mlp / short_conv(_step)
                          closed forms + F.conv1d + step == parallel      -> pinned
  rotary_embedding        position 0 == identity, norm preservation, relative-position
                          property of the rotated dot product, complex-number brute
                          force                                            -> pinned against
                          the published RoPE formula (GPT-NeoX half-split layout, the
                          GPT-J interleaved layout, rotation of a leading part of the head
                          only: each as a complex multiplication of its own pairing); the
                          reference takes it from flash-attn's rotary layer (absent), so
                          agreement with THAT library is "parity unpinned".
  gated_short_conv(_step) F.conv1d(groups=D, padding=K-1)[..., :L] + F.silu, per-element
                          brute force, step == parallel                   -> pinned
  add_rms_norm            closed form on hand-made rows, the cast BEFORE the norm (a bf16
                          sum rounded first), the fp32 residual stream     -> pinned
  add_layer_norm          F.layer_norm (library routine), hand-made rows   -> pinned
  gated_mlp               F.glu / explicit products for the four (activation, layout)
                          combinations                                      -> pinned
  stack_forward           composition of the functions above in the order of
                          block.py:134-163 and gpt.py:622-736; checked against a
                          hand-unrolled one-layer case and against nn.Module building
                          blocks (nn.Linear, nn.Embedding, F.conv1d, SDPA) -> pinned
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------------------------
# TaylorExp feature map  (based/models/mixers/linear_attention.py:52-75)
# ----------------------------------------------------------------------------------------------
def taylor_exp(x: torch.Tensor) -> torch.Tensor:
    """phi(x) = [1, x / d^(1/4), vec(x x^T) / (sqrt(2) sqrt(d))]  ->  (..., 1 + d + d*d).

    Second-order block is the FULL outer product in row-major order (index 1+d+i*d+j),
    exactly as `(x.unsqueeze(-1) * x.unsqueeze(-2)).flatten(-2)` at linear_attention.py:69.
    Arithmetic is done in the dtype of `x` (the reference does not upcast).
    """
    d = x.shape[-1]
    rd = math.sqrt(d)
    rrd = math.sqrt(rd)
    r2 = math.sqrt(2.0)
    outer = x[..., :, None] * x[..., None, :]
    second = outer.reshape(*x.shape[:-1], d * d) / r2
    ones = torch.ones_like(x[..., :1])
    return torch.cat([ones, x / rrd, second / rd], dim=-1)


def taylor_dot(q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """Closed form of phi(q).phi(k):  1 + s + s^2/2 with s = q.k / sqrt(d)."""
    s = (q * k).sum(-1) / math.sqrt(q.shape[-1])
    return 1.0 + s + 0.5 * s * s


# ----------------------------------------------------------------------------------------------
# Causal linear attention, parallel forms
# ----------------------------------------------------------------------------------------------
def linear_attn_quadratic(q, k, v, eps: float = 1e-12):
    """Reference "quadratic" branch (linear_attention.py:169-183) without the out_proj.

    q, k: (B, H, L, d) raw (un-mapped);  v: (B, H, L, dv).  Returns y (B, H, L, dv) with
        y_i = sum_{j<=i} (phi(q_i).phi(k_j)) v_j / (phi(q_i) . sum_{j<=i} phi(k_j) + eps)
    """
    fq, fk = taylor_exp(q), taylor_exp(k)
    a = torch.einsum("bhnd,bhmd->bhnm", fq, fk)
    a = torch.tril(a)
    y = torch.einsum("bhnm,bhme->bhne", a, v)
    z = 1.0 / (torch.einsum("bhld,bhld->bhl", fq, fk.cumsum(2)) + eps)
    return y * z[..., None]


def linear_attn_cumsum(q, k, v, eps: float = 1e-12, chunk: int = 64):
    """O(L) form: running kv = sum phi(k) (x) v, as in the reference's C++ causal product
    (train/csrc/causal_dot_prod/causal_attention.cpp:82-124) and its smoke script
    (train/csrc/causal_dot_prod/test.py:22-27).  Evaluated chunk-wise so the
    (L, D, dv) cumulative tensor is never materialised.
    """
    fq, fk = taylor_exp(q), taylor_exp(k)
    B, H, L, D = fq.shape
    dv = v.shape[-1]
    kv = torch.zeros(B, H, D, dv, dtype=fq.dtype)
    ks = torch.zeros(B, H, D, dtype=fq.dtype)
    out = torch.empty(B, H, L, dv, dtype=fq.dtype)
    for s in range(0, L, chunk):
        e = min(L, s + chunk)
        kvc = kv[:, :, None] + torch.cumsum(fk[:, :, s:e, :, None] * v[:, :, s:e, None, :], dim=2)
        ksc = ks[:, :, None] + torch.cumsum(fk[:, :, s:e], dim=2)
        num = torch.einsum("bhld,bhlde->bhle", fq[:, :, s:e], kvc)
        den = torch.einsum("bhld,bhld->bhl", fq[:, :, s:e], ksc) + eps
        out[:, :, s:e] = num / den[..., None]
        kv, ks = kvc[:, :, -1], ksc[:, :, -1]
    return out


def linear_attn_prefill_state(k, v):
    """Decode state left behind by a prefill (linear_attention.py:220-222).

    Returns kv_state (B, H, 1, dv, D) with kv_state[b,h,0,e,f] = sum_n v[n,e] phi(k)[n,f]
    and k_state (B, H, 1, 1, D) = sum_n phi(k)[n].
    """
    fk = taylor_exp(k)
    kv_state = torch.einsum("bhnd,bhnf->bhfd", fk, v)[:, :, None]
    k_state = fk.sum(dim=2)[:, :, None, None]
    return kv_state, k_state


def linear_attn_step(kv_state, k_state, q, k, v, eps: float = 1e-12):
    """One recurrent decode step (linear_attention.py:230-252) without the out_proj.

    q, k: (B, H, 1, d) raw;  v: (B, H, 1, dv).  Mutates kv_state (B,H,1,dv,D) and
    k_state (B,H,1,1,D) IN PLACE, returns y (B, H, 1, dv) in the dtype of the states.
    """
    fq, fk = taylor_exp(q), taylor_exp(k)
    fq, fk, vv = fq.unsqueeze(-2), fk.unsqueeze(-2), v.unsqueeze(-1)
    kv_state += (fk[:, :, -1:] * vv[:, :, -1:]).to(kv_state.dtype)
    k_state += fk[:, :, -1:].to(k_state.dtype)
    num = (fq.to(kv_state.dtype) * kv_state).sum(dim=-1)
    den = (fq.to(k_state.dtype) * k_state).sum(dim=-1) + eps
    return num / den


# ----------------------------------------------------------------------------------------------
# Sliding-window causal softmax attention
# ----------------------------------------------------------------------------------------------
def sliding_window_attn(q, k, v, w_left: int = 64, scale: float | None = None):
    """Textbook masked softmax with the flash-attn window convention the reference passes
    (`window_size=(W//2, 0)`, causal: slide_attention.py:97-106,332-336): query i attends
    keys j in [i - w_left, i].  Statement follows the in-tree textbook attention
    (based/models/mixers/mha.py:243-275) with the band mask added.

    q, k, v: (B, L, H, D).  Returns (B, L, H, D) in fp32 arithmetic, cast to q.dtype.
    """
    B, L, H, D = q.shape
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    qf, kf, vf = q.float(), k.float(), v.float()
    scores = torch.einsum("bthd,bshd->bhts", qf, kf) * scale
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    keep = (j <= i) & (j >= i - w_left)
    scores = scores.masked_fill(~keep, float("-inf"))
    p = torch.softmax(scores, dim=-1)
    return torch.einsum("bhts,bshd->bthd", p, vf).to(q.dtype)


def sliding_window_step(q, k_new, v_new, kv_cache, pos: int, w_left: int = 64, scale: float | None = None):
    """Decode step with a linear KV cache (slide_attention.py:430-481): write the new k, v at
    row `pos` of kv_cache (B, max_seqlen, 2, H, D), then attend keys [pos - w_left, pos].

    q, k_new, v_new: (B, 1, H, D).  Mutates kv_cache in place.  Returns (B, 1, H, D).
    """
    B, _, H, D = q.shape
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    kv_cache[:, pos, 0] = k_new[:, 0].to(kv_cache.dtype)
    kv_cache[:, pos, 1] = v_new[:, 0].to(kv_cache.dtype)
    lo = max(0, pos - w_left)
    kf = kv_cache[:, lo:pos + 1, 0].float()
    vf = kv_cache[:, lo:pos + 1, 1].float()
    scores = torch.einsum("bthd,bshd->bhts", q.float(), kf) * scale
    p = torch.softmax(scores, dim=-1)
    return torch.einsum("bhts,bshd->bthd", p, vf).to(q.dtype)


# ----------------------------------------------------------------------------------------------
# Stack glue used only by the 27-layer configuration
# ----------------------------------------------------------------------------------------------
def rms_norm(x, weight, eps: float = 1e-5):
    """x * rsqrt(mean(x^2) + eps) * w  (based/ops/triton/layer_norm.py:117-118), fp32 math."""
    xf = x.float()
    rstd = torch.rsqrt(xf.square().mean(dim=-1, keepdim=True) + eps)
    return (xf * rstd * weight.float()).to(x.dtype)


def swiglu_mlp(x, w1, w2):
    """fc2( y * silu(gate) ) with y, gate = fc1(x).chunk(2)  (based/models/mlp.py:141-157)."""
    y, gate = F.linear(x, w1).chunk(2, dim=-1)
    return F.linear(y * F.silu(gate), w2)


def short_conv(x, weight):
    """Depthwise causal convolution (based/models/mixers/convolution.py:47-83, non-CUDA path):
    y[b, t, c] = sum_{i<K} weight[c, i] * x[b, t - (K-1) + i, c], zero left padding.
    x: (B, L, C); weight: (C, K).
    """
    B, L, C = x.shape
    K = weight.shape[-1]
    y = torch.zeros_like(x)
    for i in range(K):
        shift = K - 1 - i
        if shift == 0:
            y += x * weight[:, i]
        elif shift < L:
            y[:, shift:] += x[:, : L - shift] * weight[:, i]
    return y


def short_conv_step(x, state, weight):
    """Single-token update of the rolling (B, C, K) state (convolution.py:85-109, non-CUDA
    path): shift left, append x (B, 1, C), return sum_k state * weight as (B, 1, C)."""
    state.copy_(torch.roll(state, shifts=-1, dims=-1))
    state[:, :, -1] = x[:, 0]
    return torch.einsum("bck,ck->bc", state, weight).to(x.dtype).unsqueeze(1)


def gated_short_conv(u, weight, bias=None):
    """BaseConv between its projections (convolution.py:201-208, non-CUDA branch): split
    u (B, L, 2D) into u1 | u2, y = silu(short_conv(u1) + bias) * u2.  weight: (D, K)."""
    D = u.shape[-1] // 2
    u1, u2 = u[..., :D].float(), u[..., D:].float()
    c = short_conv(u1, weight.float())
    if bias is not None:
        c = c + bias.float()
    return (F.silu(c) * u2).to(u.dtype)


def gated_short_conv_step(u, state, weight, bias=None):
    """Single-token form (convolution.py:104-108 + :204-207): roll the (B, D, K) state, append
    u1, contract with the weight, SiLU, gate.  u: (B, 1, 2D).  The state is updated in place."""
    D = u.shape[-1] // 2
    c = short_conv_step(u[..., :D].float(), state, weight.float())
    if bias is not None:
        c = c + bias.float()
    return (F.silu(c.float()) * u[..., D:].float()).to(u.dtype)


def rotary_embedding(x, positions, base: float = 10000.0, rotary_dim: int = None, interleaved: bool = False):
    """Rotary position embedding of the first `rotary_dim` channels (default: all of them) of the
    last dimension, as the reference applies to q and k of the sliding-window mixer through
    flash-attn's RotaryEmbedding (slide_attention.py:346-355,553-556); channels past rotary_dim
    pass through.  With R = rotary_dim and w_i = base^(-2i/R), i < R/2:
      non-interleaved ("half-split", rotary_emb_interleaved=False), pairs (i, i + R/2):
        out[..., i]       = x[..., i] cos(p w_i) - x[..., i + R/2] sin(p w_i)
        out[..., i + R/2] = x[..., i] sin(p w_i) + x[..., i + R/2] cos(p w_i)
      interleaved (GPT-J style), pairs (2i, 2i + 1):
        out[..., 2i]      = x[..., 2i] cos(p w_i) - x[..., 2i + 1] sin(p w_i)
        out[..., 2i + 1]  = x[..., 2i] sin(p w_i) + x[..., 2i + 1] cos(p w_i).
    x: (B, L, H, D); positions: (L,) integer tensor.  fp32 arithmetic, cast back to x.dtype."""
    D = x.shape[-1]
    R = D if rotary_dim is None else int(rotary_dim)
    assert 0 < R <= D and R % 2 == 0
    inv_freq = 1.0 / (base ** (torch.arange(0, R, 2, dtype=torch.float32) / R))
    ang = torch.outer(positions.float(), inv_freq)            # (L, R/2)
    cos, sin = ang.cos()[None, :, None, :], ang.sin()[None, :, None, :]
    if interleaved:
        x1, x2 = x[..., 0:R:2].float(), x[..., 1:R:2].float()
        rot = torch.stack([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).flatten(-2)
    else:
        x1, x2 = x[..., : R // 2].float(), x[..., R // 2: R].float()
        rot = torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1)
    return torch.cat([rot.to(x.dtype), x[..., R:]], dim=-1)


def add_rms_norm(x, residual, weight, eps: float = 1e-5, residual_in_fp32: bool = True):
    """Prenorm block glue (based/models/block.py:134-139): r = x + residual (torch promotion: fp32
    when the residual stream is fp32), y = rms_norm(r.to(x.dtype)), r kept in fp32 if asked.
    Returns (y, r)."""
    r = x if residual is None else x + residual
    y = rms_norm(r.to(x.dtype), weight, eps)
    return y, (r.float() if residual_in_fp32 else r)


def add_layer_norm(x, residual, weight, bias, eps: float = 1e-5, residual_in_fp32: bool = True):
    """The same glue with nn.LayerNorm, the norm of a reference config without `rms_norm`
    (gpt.py:352,537; block.py:134-139): r = x + residual, y = (c - mean(c)) / sqrt(var(c) + eps) *
    weight + bias with c = r cast to the norm's dtype and the biased variance.  Returns (y, r)."""
    r = x if residual is None else x + residual
    c = r.to(weight.dtype)
    mu = c.mean(dim=-1, keepdim=True)
    var = (c - mu).square().mean(dim=-1, keepdim=True)
    y = (c - mu) / torch.sqrt(var + eps) * weight
    if bias is not None:
        y = y + bias
    return y.to(weight.dtype), (r.float() if residual_in_fp32 else r)


# ----------------------------------------------------------------------------------------------
# Model assembly (only what the stack-level parity tests need), CPU, any float dtype
# ----------------------------------------------------------------------------------------------
def gated_mlp(x, fc1_w, fc2_w, fc3_w=None, activation: str = "swiglu", fc1_b=None, fc2_b=None, fc3_b=None):
    """GatedMlp.forward (based/models/mlp.py:141-157).  Layout 'base' (fc3_w is None):
    y, gate = fc1(x).chunk(2); fc2(y * act(gate)), with F.glu for the sigmoid case.  Layout
    'alt' (fc3_w given): fc2(act(fc1(x)) * fc3(x)).  act: glu -> sigmoid, swiglu -> silu,
    geglu -> gelu (based/models/gpt.py:238-243)."""
    act = {"glu": torch.sigmoid, "swiglu": F.silu, "geglu": F.gelu}[activation]
    if fc3_w is None:
        y, gate = F.linear(x, fc1_w, fc1_b).chunk(2, dim=-1)
        return F.linear(y * act(gate), fc2_w, fc2_b)
    return F.linear(act(F.linear(x, fc1_w, fc1_b)) * F.linear(x, fc3_w, fc3_b), fc2_w, fc2_b)


def mixer_kind(config, layer_idx: int) -> tuple:
    """(kind, spec) of a layer's mixer following create_mixer_cls (based/models/gpt.py:64-96):
    alt_mixer_2 wins over alt_mixer wins over mixer; kind from the `_target_` string."""
    spec = config["mixer"]
    if config.get("alt_mixer_2_layers") is not None and layer_idx in config["alt_mixer_2_layers"]:
        spec = config["alt_mixer_2"]
    elif config.get("alt_mixer_layers") is not None and layer_idx in config["alt_mixer_layers"]:
        spec = config["alt_mixer"]
    target = spec["_target_"]
    kind = ("linear" if "linear_attention" in target else "slide" if "slide" in target
            else "short_conv" if target.endswith("ShortConvolution") else "conv")
    return kind, spec


def stack_forward(input_ids, sd: dict, config: dict, dtype=torch.float32):
    """Parallel forward of the Based stack: embeddings (+ learned positions) ->
    [add + norm -> mixer -> add + norm -> gated MLP] x n_layer -> add + final norm -> LM head;
    norm = RMSNorm with `rms_norm`, nn.LayerNorm without (gpt.py:352,537) (GPTModel.forward gpt.py:622-736, Block.forward block.py:134-163, dropout-free,
    prenorm, residual stream in fp32 when residual_in_fp32).  `sd` is a state dict with the
    reference's parameter names; `config` a plain dict with the reference's keys.  Activations are
    kept in `dtype` between the operations exactly where the model would hold them in its own
    dtype (every projection output is rounded to `dtype`); the mixers' inner arithmetic is fp32 on
    those rounded inputs.  With dtype=float32 this is the exact-arithmetic statement of the model;
    with dtype=bfloat16 it shows how far a bf16 model may sit from it through rounding alone."""
    g = lambda name: sd[name].to(dtype) if name in sd else None
    n_embd, n_head, eps = config["n_embd"], config["n_head"], config.get("layer_norm_epsilon", 1e-5)
    res_fp32 = config.get("residual_in_fp32", False)
    B, L = input_ids.shape

    def norm(x, residual, name):
        if config.get("rms_norm", False):
            return add_rms_norm(x, residual, g(name + ".weight"), eps, res_fp32)
        return add_layer_norm(x, residual, g(name + ".weight"), g(name + ".bias"), eps, res_fp32)

    hidden = F.embedding(input_ids, g("transformer.embeddings.word_embeddings.weight"))
    if config.get("max_position_embeddings", 0) > 0:
        hidden = hidden + g("transformer.embeddings.position_embeddings.weight")[:L]
    residual = None
    for i in range(config["n_layer"]):
        pre = f"transformer.layers.{i}."
        hidden, residual = norm(hidden, residual, pre + "norm1")
        kind, spec = mixer_kind(config, i)
        m = pre + "mixer."
        if kind == "conv":
            u = F.linear(hidden, g(m + "in_proj.weight"), g(m + "in_proj.bias"))
            y = gated_short_conv(u, g(m + "conv.conv.weight")[:, 0], g(m + "conv.conv.bias"))
            hidden = F.linear(y, g(m + "out_proj.weight"), g(m + "out_proj.bias"))
        elif kind == "short_conv":   # the convolution alone as the mixer (convolution.py:47-87)
            hidden = short_conv(hidden.float(), g(m + "conv.weight")[:, 0].float()).to(dtype)
            if g(m + "conv.bias") is not None:
                hidden = (hidden.float() + g(m + "conv.bias").float()).to(dtype)
        elif kind == "linear":
            H = spec.get("num_heads", 16)
            fd = spec.get("feature_dim", 16)
            q = F.linear(hidden, g(m + "proj_q.weight")).view(B, L, H, fd).transpose(1, 2)
            k = F.linear(hidden, g(m + "proj_k.weight")).view(B, L, H, fd).transpose(1, 2)
            v = F.linear(hidden, g(m + "proj_v.weight")).view(B, L, H, -1).transpose(1, 2)
            # fp32 arithmetic on the (dtype-rounded) projections, like the kernels (module header, F9)
            # the reference's "fla_*" implementations regularise with 1e-6 (linear_attention.py:199-212,245-249)
            lin_eps = 1e-6 if "fla" in spec.get("parallel_implementation", "") else spec.get("eps", 1e-12)
            y = linear_attn_quadratic(q.float(), k.float(), v.float(), eps=lin_eps)
            y = y.transpose(1, 2).reshape(B, L, -1)
            hidden = F.linear(y.to(dtype), g(m + "out_proj.weight"))
        else:
            hd = n_embd // n_head
            qkv = F.linear(hidden, g(m + "Wqkv.weight"), g(m + "Wqkv.bias")).view(B, L, 3, n_head, hd)
            q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
            rot = int(config.get("rotary_emb_fraction", 0.0) * hd)
            if rot > 0:
                pos = torch.arange(L)
                inter = config.get("rotary_emb_interleaved", False)
                q = rotary_embedding(q, pos, config.get("rotary_emb_base", 10000.0), rot, inter)
                k = rotary_embedding(k, pos, config.get("rotary_emb_base", 10000.0), rot, inter)
            scale = hd ** -0.5 if config.get("scale_attn_weights", True) else 1.0
            o = sliding_window_attn(q, k, v, w_left=spec.get("window_size", 128) // 2, scale=scale)
            hidden = F.linear(o.reshape(B, L, n_embd).to(dtype), g(m + "out_proj.weight"), g(m + "out_proj.bias"))
        hidden, residual = norm(hidden, residual, pre + "norm2")
        p = pre + "mlp."
        hidden = gated_mlp(hidden, g(p + "fc1.weight"), g(p + "fc2.weight"), g(p + "fc3.weight"),
                           config.get("activation_function", "swiglu"), g(p + "fc1.bias"), g(p + "fc2.bias"),
                           g(p + "fc3.bias"))
    hidden, _ = norm(hidden, residual, "transformer.ln_f")
    return F.linear(hidden, g("lm_head.weight"))
