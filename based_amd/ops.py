"""Tensor-level wrappers over the C ABI: validate, take pointers/strides, enqueue on torch's
current stream.  PyTorch is used for device memory and streams only."""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Tuple

import torch

from . import _lib

FEATURE_DIM = 16
EXPANDED_DIM = 273


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.BASED_BF16
    if t.dtype == torch.float32:
        return _lib.BASED_F32
    raise ValueError(f"unsupported dtype {t.dtype} (bfloat16 or float32)")


# torch's current stream on a device as a raw hipStream_t.  The private accessor skips building a
# Stream object (several microseconds per call, which a single-token step notices); where a torch
# build lacks it the public route is taken.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(t: torch.Tensor) -> int:
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _on_device:
    """Enters `torch.cuda.device(dev)` only when dev is not already current (entering the context
    costs microseconds, which matters for single-token steps)."""

    __slots__ = ("ctx",)

    def __init__(self, dev: torch.device):
        self.ctx = None if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


# Argument checks of the single-token entry points are done once per distinct combination of
# shapes, strides, dtypes and device (a decode loop presents the same combination every step).
_CHECKED: dict = {}


def _require_cuda(*ts: torch.Tensor) -> None:
    dev = ts[0].device
    for t in ts:
        if not t.is_cuda:
            raise ValueError("based_amd kernels need tensors on a HIP device (no CPU path)")
        if t.device != dev:
            raise ValueError("all tensors must live on the same device")


def linear_attn_step(q, k, v, kv_state, k_state, eps: float = 1e-12, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One decode step.  q, k: (B, H, 1, 16) raw; v: (B, H, 1, dv); kv_state (B,H,1,dv,273)
    and k_state (B,H,1,1,273) fp32 contiguous, updated in place.  Returns y (B, H, 1, dv)
    (written into `out` when given)."""
    key = ("lin_step", q.shape, q.stride(), k.shape, k.stride(), v.shape, v.stride(), kv_state.shape, kv_state.stride(),
           k_state.shape, k_state.stride(), q.dtype, k.dtype, v.dtype, kv_state.dtype, k_state.dtype, q.device,
           k.device, v.device, kv_state.device, k_state.device)
    if key not in _CHECKED:
        _require_cuda(q, k, v, kv_state, k_state)
        B, H, l, d = q.shape
        assert l == 1, f"q.shape is {tuple(q.shape)} but should be ({B}, {H}, 1, {d})"
        dv = v.shape[-1]
        if d != FEATURE_DIM or k.shape != q.shape or v.shape[:3] != q.shape[:3]:
            raise ValueError(f"bad shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
        if kv_state.dtype != torch.float32 or k_state.dtype != torch.float32:
            raise ValueError("decode states must be float32")
        if tuple(kv_state.shape) != (B, H, 1, dv, EXPANDED_DIM) or tuple(k_state.shape) != (B, H, 1, 1, EXPANDED_DIM):
            raise ValueError(f"bad state shapes {tuple(kv_state.shape)} {tuple(k_state.shape)}")
        if not (kv_state.is_contiguous() and k_state.is_contiguous()):
            raise ValueError("decode states must be contiguous")
        if not (q.dtype == k.dtype == v.dtype):
            raise ValueError("q, k, v must share a dtype")
        for t in (q, k, v):
            if t.stride(-1) != 1:
                raise ValueError("innermost dimension must be contiguous")
        _dtype_code(q)
        _CHECKED[key] = True
    B, H, _, _ = q.shape
    dv = v.shape[-1]
    if out is None:
        y = torch.empty(B, H, 1, dv, dtype=q.dtype, device=q.device)
    else:
        y = out
        if tuple(y.shape) != (B, H, 1, dv) or y.dtype != q.dtype or y.device != q.device or y.stride(-1) != 1:
            raise ValueError(f"out must be a ({B}, {H}, 1, {dv}) {q.dtype} tensor on {q.device}")
    with _on_device(q.device):
        _lib.check(_lib.lib().based_linear_attn_step(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), kv_state.data_ptr(), k_state.data_ptr(), y.data_ptr(),
            B, H, dv,
            q.stride(0), q.stride(1), k.stride(0), k.stride(1),
            v.stride(0), v.stride(1), y.stride(0), y.stride(1),
            float(eps), _dtype_code(q), _stream_ptr(q)))
    return y


DEFERRED_MAX_STEPS = 8  # BASED_DEFERRED_MAX_STEPS


def deferred_step_buffers(batch: int, heads: int, dv: int, device) -> tuple:
    """The ring of `linear_attn_step_deferred` for (batch, heads) states: keys (B, H, 8, 16) and
    values (B, H, 8, dv) in fp32, and the per-(batch, head) fill count (B, H) int32, all zero."""
    return (torch.zeros(batch, heads, DEFERRED_MAX_STEPS, FEATURE_DIM, dtype=torch.float32, device=device),
            torch.zeros(batch, heads, DEFERRED_MAX_STEPS, dv, dtype=torch.float32, device=device),
            torch.zeros(batch, heads, dtype=torch.int32, device=device))


def _check_deferred(kv_state, pending):
    pend_k, pend_v, pend_n = pending
    B, H, _, dv, _ = kv_state.shape
    _require_cuda(kv_state, pend_k, pend_v, pend_n)
    if (tuple(pend_k.shape) != (B, H, DEFERRED_MAX_STEPS, FEATURE_DIM) or tuple(pend_v.shape) != (B, H, DEFERRED_MAX_STEPS, dv)
            or tuple(pend_n.shape) != (B, H)):
        raise ValueError(f"bad ring shapes {tuple(pend_k.shape)} {tuple(pend_v.shape)} {tuple(pend_n.shape)} for a "
                         f"state {tuple(kv_state.shape)}")
    if pend_k.dtype != torch.float32 or pend_v.dtype != torch.float32 or pend_n.dtype != torch.int32:
        raise ValueError("the ring is float32 keys and values and an int32 count")
    if not (pend_k.is_contiguous() and pend_v.is_contiguous() and pend_n.is_contiguous()):
        raise ValueError("the ring must be contiguous")


def linear_attn_step_deferred(q, k, v, kv_state, k_state, pending, period: int, eps: float = 1e-12,
                              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`linear_attn_step` with the write-back of kv_state deferred: the step reads kv_state, updates
    k_state and parks the token's raw k and v in `pending` (from `deferred_step_buffers`); every
    `period`-th step (1..8) applies the parked tokens and its own to kv_state in one pass.  The
    output is the one of `linear_attn_step` up to fp32 summation order; kv_state is current only
    after such a step or after `linear_attn_flush_deferred`.  Leading rows of larger states and
    rings may be passed (views of the first B rows)."""
    key = ("lin_step_deferred", q.shape, q.stride(), k.shape, k.stride(), v.shape, v.stride(), kv_state.shape,
           kv_state.stride(), k_state.shape, k_state.stride(), q.dtype, k.dtype, v.dtype, kv_state.dtype, k_state.dtype,
           q.device, k.device, v.device, kv_state.device, k_state.device,
           tuple((t.shape, t.stride(), t.dtype, t.device) for t in pending), int(period))
    if key not in _CHECKED:
        _require_cuda(q, k, v, kv_state, k_state)
        B, H, l, d = q.shape
        assert l == 1, f"q.shape is {tuple(q.shape)} but should be ({B}, {H}, 1, {d})"
        dv = v.shape[-1]
        if d != FEATURE_DIM or k.shape != q.shape or v.shape[:3] != q.shape[:3]:
            raise ValueError(f"bad shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
        if kv_state.dtype != torch.float32 or k_state.dtype != torch.float32:
            raise ValueError("decode states must be float32")
        if tuple(kv_state.shape) != (B, H, 1, dv, EXPANDED_DIM) or tuple(k_state.shape) != (B, H, 1, 1, EXPANDED_DIM):
            raise ValueError(f"bad state shapes {tuple(kv_state.shape)} {tuple(k_state.shape)}")
        if not (kv_state.is_contiguous() and k_state.is_contiguous()):
            raise ValueError("decode states must be contiguous")
        if not (q.dtype == k.dtype == v.dtype):
            raise ValueError("q, k, v must share a dtype")
        for t in (q, k, v):
            if t.stride(-1) != 1:
                raise ValueError("innermost dimension must be contiguous")
        if not 1 <= int(period) <= DEFERRED_MAX_STEPS:
            raise ValueError(f"period must be in [1, {DEFERRED_MAX_STEPS}], got {period}")
        _check_deferred(kv_state, pending)
        _dtype_code(q)
        _CHECKED[key] = True
    B, H, _, _ = q.shape
    dv = v.shape[-1]
    if out is None:
        y = torch.empty(B, H, 1, dv, dtype=q.dtype, device=q.device)
    else:
        y = out
        if tuple(y.shape) != (B, H, 1, dv) or y.dtype != q.dtype or y.device != q.device or y.stride(-1) != 1:
            raise ValueError(f"out must be a ({B}, {H}, 1, {dv}) {q.dtype} tensor on {q.device}")
    pend_k, pend_v, pend_n = pending
    with _on_device(q.device):
        _lib.check(_lib.lib().based_linear_attn_step_deferred(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), kv_state.data_ptr(), k_state.data_ptr(), pend_k.data_ptr(),
            pend_v.data_ptr(), pend_n.data_ptr(), y.data_ptr(), B, H, dv,
            q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), y.stride(0), y.stride(1),
            float(eps), int(period), _dtype_code(q), _stream_ptr(q)))
    return y


def linear_attn_flush_deferred(kv_state, pending) -> None:
    """Applies the tokens parked by `linear_attn_step_deferred` to kv_state (B,H,1,dv,273) and
    empties the ring."""
    if kv_state.dtype != torch.float32 or kv_state.dim() != 5 or not kv_state.is_contiguous():
        raise ValueError("kv_state must be a contiguous float32 (B, H, 1, dv, 273) tensor")
    _check_deferred(kv_state, pending)
    B, H, _, dv, _ = kv_state.shape
    pend_k, pend_v, pend_n = pending
    with _on_device(kv_state.device):
        _lib.check(_lib.lib().based_linear_attn_flush_deferred(kv_state.data_ptr(), pend_k.data_ptr(), pend_v.data_ptr(),
                                                               pend_n.data_ptr(), B, H, dv, _stream_ptr(kv_state)))


def _rope_tables(rope, device, need_rows, head_dim):
    """rope = (cos, sin) or (cos, sin, interleaved): fp32 (n_pos, rotary_dim / 2) contiguous device
    tables -> (cos_ptr, sin_ptr, n_pos, rotary_dim, interleaved), or Nones / zeros without rotary."""
    if rope is None:
        return None, None, 0, 0, False
    cos, sin = rope[0], rope[1]
    interleaved = bool(rope[2]) if len(rope) > 2 else False
    for t in (cos, sin):
        if not t.is_cuda or t.device != device or t.dtype != torch.float32 or t.dim() != 2 or not t.is_contiguous():
            raise ValueError("rotary tables must be contiguous fp32 (n_pos, rotary_dim / 2) tensors on the device of q")
    rotary_dim = 2 * cos.shape[1]
    if cos.shape != sin.shape or cos.shape[0] < need_rows:
        raise ValueError(f"rotary tables hold {cos.shape[0]} positions, need {need_rows}")
    if rotary_dim % 16 != 0 or not 0 < rotary_dim <= head_dim:
        raise ValueError(f"rotary_dim {rotary_dim} must be a multiple of 16 and at most the head dim {head_dim}")
    return cos.data_ptr(), sin.data_ptr(), cos.shape[0], rotary_dim, interleaved


def _swa_fast64(D: int, rotary_dim: int, interleaved: bool, impl) -> bool:
    """Head dim 64 without rotary, or rotated over the whole head in half-split pairs, runs the
    kernels built for exactly that (two heads per workgroup, 128-byte rows)."""
    return impl is None and D == 64 and (rotary_dim == 0 or (rotary_dim == 64 and not interleaved))


def swa_prefill(q, k, v, w_left: int = 64, scale: Optional[float] = None, rope=None, kv_cache=None,
                out: Optional[torch.Tensor] = None, impl: Optional[str] = None) -> torch.Tensor:
    """Sliding-window causal attention.  q, k, v: (B, L, H, D) bf16 (any strides with the
    last dim contiguous, e.g. slices of a packed qkv), D a multiple of 8 up to 128.  Query i sees
    keys [i - w_left, i], 0 <= w_left <= 128.
    rope: None, or (cos, sin[, interleaved]) with fp32 (n_pos >= L, rotary_dim / 2) tables: the
    first rotary_dim channels of q and k are rotated in the kernel at positions 0..L-1, in
    half-split pairs (c, c + rotary_dim / 2) or, interleaved, pairs (2i, 2i + 1).
    kv_cache: None or a (B, max_seqlen >= L, 2, H, D) bf16 cache whose rows 0..L-1 receive the
    (rotated) k and v.  out: None or a (B, L, H, D) tensor (last dim contiguous) to write into.
    impl: None (MFMA kernels), "wide" (the general MFMA kernel also where the 64-channel one would
    do) or "plain" (the one-wavefront-per-query kernel, no rotary: a second statement for tests)."""
    _require_cuda(q, k, v)
    B, L, H, D = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"bad shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
    for t in (q, k, v):
        if t.stride(-1) != 1:
            raise ValueError("innermost dimension must be contiguous")
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    cos_ptr, sin_ptr, n_pos, rotary_dim, interleaved = _rope_tables(rope, q.device, L, D)
    if impl == "plain" and rope is not None:
        raise ValueError("the plain kernel has no in-kernel rotary")
    kc_ptr = vc_ptr = None
    c_strides, max_seqlen = (0, 0, 0), 0
    if kv_cache is not None:
        _require_cuda(q, kv_cache)
        if (kv_cache.dim() != 5 or kv_cache.shape[0] != B or kv_cache.shape[2] != 2
                or tuple(kv_cache.shape[3:]) != (H, D) or kv_cache.dtype != q.dtype or kv_cache.stride(-1) != 1):
            raise ValueError(f"bad cache {tuple(kv_cache.shape)} {kv_cache.dtype}")
        kc, vc = kv_cache[:, :, 0], kv_cache[:, :, 1]
        kc_ptr, vc_ptr = kc.data_ptr(), vc.data_ptr()
        c_strides, max_seqlen = (kc.stride(0), kc.stride(1), kc.stride(2)), kv_cache.shape[1]
    if out is None:
        o = torch.empty(B, L, H, D, dtype=q.dtype, device=q.device)
    else:
        o = out
        if tuple(o.shape) != (B, L, H, D) or o.dtype != q.dtype or o.device != q.device or o.stride(-1) != 1:
            raise ValueError(f"out must be a ({B}, {L}, {H}, {D}) {q.dtype} tensor on {q.device}")
    strides = (q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
               v.stride(0), v.stride(1), v.stride(2), o.stride(0), o.stride(1), o.stride(2))
    with _on_device(q.device):
        if _swa_fast64(D, rotary_dim, interleaved, impl):
            _lib.check(_lib.lib().based_swa_prefill(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, H, L, *strides,
                int(w_left), scale, cos_ptr, sin_ptr, n_pos, kc_ptr, vc_ptr, *c_strides, max_seqlen,
                _dtype_code(q), _stream_ptr(q)))
        elif impl == "plain":
            _lib.check(_lib.lib().based_swa_prefill_anydim(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, H, L, D, *strides,
                int(w_left), scale, kc_ptr, vc_ptr, *c_strides, max_seqlen, _dtype_code(q), _stream_ptr(q)))
        else:
            _lib.check(_lib.lib().based_swa_prefill_wide(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, H, L, D, *strides,
                int(w_left), scale, cos_ptr, sin_ptr, n_pos, rotary_dim, int(interleaved), kc_ptr, vc_ptr, *c_strides,
                max_seqlen, _dtype_code(q), _stream_ptr(q)))
    return o


def swa_step(q, k_new, v_new, kv_cache, pos, w_left: int = 64, scale: Optional[float] = None, rope=None,
             out: Optional[torch.Tensor] = None, impl: Optional[str] = None) -> torch.Tensor:
    """Decode step.  q, k_new, v_new: (B, 1, H, D) bf16; kv_cache (B, max_seqlen, 2, H, D)
    bf16, row `pos` is written in place, then rows [pos - w_left, pos] are attended.  D a multiple
    of 8 up to 128.
    pos: int (same for the whole batch) or an int32 device tensor of B positions.
    rope: None or (cos, sin[, interleaved]) tables as for swa_prefill: q and k_new are rotated at `pos` first.
    out: None or a (B, 1, H, D) tensor (last dim contiguous) to write into.  impl: as for swa_prefill."""
    key = ("swa_step", q.shape, q.stride(), k_new.shape, k_new.stride(), v_new.shape, v_new.stride(), kv_cache.shape,
           kv_cache.stride(), q.dtype, k_new.dtype, v_new.dtype, kv_cache.dtype, q.device, k_new.device, v_new.device,
           kv_cache.device)
    if key not in _CHECKED:
        _require_cuda(q, k_new, v_new, kv_cache)
        B, one, H, D = q.shape
        if one != 1 or k_new.shape != q.shape or v_new.shape != q.shape:
            raise ValueError(f"bad shapes q{tuple(q.shape)} k{tuple(k_new.shape)} v{tuple(v_new.shape)}")
        if kv_cache.dim() != 5 or kv_cache.shape[0] < B or kv_cache.shape[2] != 2 or tuple(kv_cache.shape[3:]) != (H, D):
            raise ValueError(f"bad cache shape {tuple(kv_cache.shape)}")
        if kv_cache.dtype != q.dtype or kv_cache.stride(-1) != 1:
            raise ValueError("cache must share q's dtype and have a contiguous last dim")
        for t in (q, k_new, v_new):
            if t.stride(-1) != 1:
                raise ValueError("innermost dimension must be contiguous")
        _dtype_code(q)
        _CHECKED[key] = True
    B, _, H, D = q.shape
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    if impl == "plain" and rope is not None:
        raise ValueError("the plain kernel has no in-kernel rotary")
    if isinstance(pos, torch.Tensor):
        if pos.dtype != torch.int32 or not pos.is_cuda or pos.numel() < B or not pos.is_contiguous():
            raise ValueError("cache_seqlens must be a contiguous int32 device tensor with B entries")
        seq_ptr, pos_host = pos.data_ptr(), 0
        cos_ptr, sin_ptr, n_pos, rotary_dim, interleaved = _rope_tables(rope, q.device, 1, D)
    else:
        seq_ptr, pos_host = None, int(pos)
        cos_ptr, sin_ptr, n_pos, rotary_dim, interleaved = _rope_tables(rope, q.device, pos_host + 1, D)
    if out is None:
        o = torch.empty(B, 1, H, D, dtype=q.dtype, device=q.device)
    else:
        o = out
        if tuple(o.shape) != (B, 1, H, D) or o.dtype != q.dtype or o.device != q.device or o.stride(-1) != 1:
            raise ValueError(f"out must be a ({B}, 1, {H}, {D}) {q.dtype} tensor on {q.device}")
    c_sb, c_st, _, c_sh, _ = kv_cache.stride()
    kc_ptr = kv_cache.data_ptr()
    vc_ptr = kc_ptr + kv_cache.stride(2) * kv_cache.element_size()
    strides = (q.stride(0), q.stride(2), k_new.stride(0), k_new.stride(2),
               v_new.stride(0), v_new.stride(2), o.stride(0), o.stride(2), c_sb, c_st, c_sh)
    with _on_device(q.device):
        if _swa_fast64(D, rotary_dim, interleaved, impl):
            _lib.check(_lib.lib().based_swa_step(
                q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), kc_ptr, vc_ptr, o.data_ptr(),
                seq_ptr, pos_host, B, H, kv_cache.shape[1], *strides,
                int(w_left), scale, cos_ptr, sin_ptr, n_pos, _dtype_code(q), _stream_ptr(q)))
        elif impl == "plain":
            _lib.check(_lib.lib().based_swa_step_anydim(
                q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), kc_ptr, vc_ptr, o.data_ptr(),
                seq_ptr, pos_host, B, H, D, kv_cache.shape[1], *strides, int(w_left), scale, _dtype_code(q),
                _stream_ptr(q)))
        else:
            _lib.check(_lib.lib().based_swa_step_wide(
                q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), kc_ptr, vc_ptr, o.data_ptr(),
                seq_ptr, pos_host, B, H, D, kv_cache.shape[1], *strides, int(w_left), scale,
                cos_ptr, sin_ptr, n_pos, rotary_dim, int(interleaved), _dtype_code(q), _stream_ptr(q)))
    return o


def linear_attn_prefill(q, k, v, eps: float = 1e-12, return_state: bool = False, split=None
                        ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Causal Taylor linear attention.  q, k: (B, H, L, 16) raw; v: (B, H, L, dv); any strides
    with the last dim contiguous (e.g. `(B, L, H, d).transpose(1, 2)` views).

    Returns (y, kv_state, k_state): y (B, H, L, dv) in q's dtype, stored so that
    `y.transpose(1, 2).reshape(B, L, H*dv)` is a free view; states are fp32
    (B, H, 1, dv, 273) / (B, H, 1, 1, 273), or None unless return_state.

    split: None = let the library decide whether to scan each sequence in concurrent segments
    (small batches); False = never; an int > 1 = that many segments."""
    _require_cuda(q, k, v)
    B, H, L, d = q.shape
    dv = v.shape[-1]
    if d != FEATURE_DIM or k.shape != q.shape or tuple(v.shape[:3]) != (B, H, L):
        raise ValueError(f"bad shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)} (feature dim 16)")
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share a dtype")
    for t in (q, k, v):
        if t.stride(-1) != 1:
            raise ValueError("innermost dimension must be contiguous")
    y = torch.empty(B, L, H, dv, dtype=q.dtype, device=q.device).transpose(1, 2)
    kv_state = k_state = None
    if return_state:
        kv_state = torch.empty(B, H, 1, dv, EXPANDED_DIM, dtype=torch.float32, device=q.device)
        k_state = torch.empty(B, H, 1, 1, EXPANDED_DIM, dtype=torch.float32, device=q.device)
    lib = _lib.lib()
    n_seg, ws_bytes = ctypes.c_int64(1), ctypes.c_int64(0)
    if split is not False:
        _lib.check(lib.based_linear_attn_prefill_plan(B, H, L, dv, _dtype_code(q), ctypes.byref(n_seg),
                                                      ctypes.byref(ws_bytes)))
    if isinstance(split, int) and not isinstance(split, bool) and split > 1:
        n_seg = ctypes.c_int64(split)  # explicit segment count (tests)
        ws_bytes = ctypes.c_int64(B * H * ((dv + 63) // 64) * split * _lib.PREFILL_SEGMENT_STATE_BYTES)
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(),
            kv_state.data_ptr() if return_state else None, k_state.data_ptr() if return_state else None,
            B, H, L, dv,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            v.stride(0), v.stride(1), v.stride(2), y.stride(0), y.stride(1), y.stride(2),
            float(eps), _dtype_code(q))
    with _on_device(q.device):
        if n_seg.value > 1:
            # scratch for the per-segment states; torch's caching allocator makes this cheap
            ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=q.device)
            _lib.check(lib.based_linear_attn_prefill_split(*args, n_seg.value, ws.data_ptr(), ws_bytes.value,
                                                           _stream_ptr(q)))
        else:
            _lib.check(lib.based_linear_attn_prefill(*args, _stream_ptr(q)))
    return y, kv_state, k_state


def gated_conv_prefill(u, weight, bias=None, state=None, gated: bool = True) -> torch.Tensor:
    """y = silu(causal depthwise conv(u[..., :D]) + bias) * u[..., D:].  u: (B, L, 2D) with a
    contiguous last dimension; weight: the (D, 1, K) nn.Conv1d weight; bias (D) or None; state
    None or (B, D, K) contiguous, overwritten with the last K inputs.  Returns y (B, L, D).
    gated=False: the convolution alone, y = conv(u) + bias with u (B, L, D)."""
    _require_cuda(u, weight)
    if u.dim() != 3 or (gated and u.shape[-1] % 2 != 0):
        raise ValueError(f"u must be (B, L, 2D), got {tuple(u.shape)}")
    B, L, D2 = u.shape
    D = D2 // 2 if gated else D2
    if weight.dim() != 3 or weight.shape[0] != D or weight.shape[1] != 1:
        raise ValueError(f"weight must be ({D}, 1, K), got {tuple(weight.shape)}")
    K = weight.shape[2]
    if weight.dtype != u.dtype or (bias is not None and bias.dtype != u.dtype):
        raise ValueError("weight and bias must have the dtype of u")
    if u.stride(-1) != 1:
        raise ValueError("innermost dimension must be contiguous")
    weight = weight.contiguous()
    if bias is not None:
        _require_cuda(u, bias)
        bias = bias.contiguous()
        if tuple(bias.shape) != (D,):
            raise ValueError(f"bias must be ({D},), got {tuple(bias.shape)}")
    state_code = _lib.BASED_BF16
    if state is not None:
        _require_cuda(u, state)
        if tuple(state.shape) != (B, D, K) or not state.is_contiguous():
            raise ValueError(f"state must be a contiguous ({B}, {D}, {K}) tensor, got {tuple(state.shape)}")
        state_code = _dtype_code(state)
    y = torch.empty(B, L, D, dtype=u.dtype, device=u.device)
    fn = _lib.lib().based_gated_conv_prefill if gated else _lib.lib().based_short_conv_prefill
    with _on_device(u.device):
        _lib.check(fn(
            u.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None, y.data_ptr(),
            state.data_ptr() if state is not None else None, B, L, D, K,
            u.stride(0), u.stride(1), y.stride(0), y.stride(1), _dtype_code(u), state_code, _stream_ptr(u)))
    return y


def gated_conv_step(u, state, weight, bias=None, gated: bool = True) -> torch.Tensor:
    """Single-token gated short convolution.  u: (B, 1, 2D) or (B, 2D); state (B, D, K)
    contiguous, rolled and updated in place.  Returns y with u's leading shape and D channels.
    gated=False: the convolution alone on u (B, 1, D) or (B, D)."""
    _require_cuda(u, state, weight)
    squeeze = u.dim() == 3
    if squeeze:
        if u.shape[1] != 1:
            raise ValueError(f"step takes one token, got {tuple(u.shape)}")
        u2d = u[:, 0]
    else:
        u2d = u
    B, D2 = u2d.shape
    D = D2 // 2 if gated else D2
    K = weight.shape[-1]
    if tuple(weight.shape) != (D, 1, K) or tuple(state.shape) != (B, D, K) or not state.is_contiguous():
        raise ValueError(f"bad shapes u{tuple(u.shape)} weight{tuple(weight.shape)} state{tuple(state.shape)}")
    if weight.dtype != u.dtype or (bias is not None and bias.dtype != u.dtype):
        raise ValueError("weight and bias must have the dtype of u")
    if u2d.stride(-1) != 1:
        raise ValueError("innermost dimension must be contiguous")
    weight = weight.contiguous()
    if bias is not None:
        _require_cuda(u, bias)
        bias = bias.contiguous()
    y = torch.empty(B, D, dtype=u.dtype, device=u.device)
    fn = _lib.lib().based_gated_conv_step if gated else _lib.lib().based_short_conv_step
    with _on_device(u.device):
        _lib.check(fn(
            u2d.data_ptr(), state.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None,
            y.data_ptr(), B, D, K, u2d.stride(0), y.stride(0), _dtype_code(u), _dtype_code(state), _stream_ptr(u)))
    return y.unsqueeze(1) if squeeze else y


ADD_RMS_NORM_MAX_DIM = 4096  # widest row based_add_rms_norm takes


def add_rms_norm(x, residual, weight, eps: float = 1e-5, residual_in_fp32: bool = True, want_residual: bool = True):
    """Prenorm block glue in one launch: r = x + residual (r = x when residual is None),
    y = rms_norm(r cast to x.dtype) * weight, and r itself (fp32 when residual_in_fp32, else
    x.dtype).  x: (..., D) with contiguous rows; returns (y, r) with r None if not wanted."""
    D = x.shape[-1]
    key = ("add_rms_norm", x.shape, x.stride(), x.dtype, x.device, weight.shape, weight.dtype, weight.device,
           None if residual is None else (residual.shape, residual.stride(), residual.dtype, residual.device))
    if key not in _CHECKED:
        _require_cuda(x, weight)
        if weight.shape != (D,) or weight.dtype != x.dtype or not weight.is_contiguous():
            raise ValueError(f"weight must be a contiguous ({D},) of {x.dtype}, got {tuple(weight.shape)} {weight.dtype}")
        if residual is not None:
            _require_cuda(x, residual)
            if residual.shape != x.shape:
                raise ValueError(f"residual {tuple(residual.shape)} does not match x {tuple(x.shape)}")
            if x.dtype == torch.float32 and residual.dtype != torch.float32:
                raise ValueError("fp32 activations need an fp32 residual stream")
            if residual.dtype not in (torch.float32, torch.bfloat16):
                raise ValueError(f"unsupported residual dtype {residual.dtype}")
        _dtype_code(x)
        _CHECKED[key] = True
    x2 = x if x.dim() == 2 else x.reshape(-1, D)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    res_dtype = torch.float32 if residual_in_fp32 else x.dtype
    r2 = None
    if residual is not None:
        # a residual stream of another dtype (first block with residual_in_fp32=False, ...) keeps its own
        res_dtype = residual.dtype
        r2 = residual if residual.dim() == 2 else residual.reshape(-1, D)
        if r2.stride(-1) != 1:
            r2 = r2.contiguous()
    if x.dtype == torch.float32 and res_dtype != torch.float32:
        raise ValueError("fp32 activations need an fp32 residual stream")
    y = torch.empty(rows, D, dtype=x.dtype, device=x.device)
    out = torch.empty(rows, D, dtype=res_dtype, device=x.device) if want_residual else None
    res_code = _lib.BASED_F32 if res_dtype == torch.float32 else _lib.BASED_BF16
    with _on_device(x.device):
        _lib.check(_lib.lib().based_add_rms_norm(
            x2.data_ptr(), r2.data_ptr() if r2 is not None else None, weight.data_ptr(), y.data_ptr(),
            out.data_ptr() if out is not None else None, rows, D, x2.stride(0),
            r2.stride(0) if r2 is not None else 0, D, D if out is not None else 0,
            float(eps), _dtype_code(x), res_code, _stream_ptr(x)))
    return y.view(x.shape), (out.view(x.shape) if out is not None else None)


def swiglu(u) -> torch.Tensor:
    """u (..., 2F) -> u[..., :F] * silu(u[..., F:]), one pass."""
    _require_cuda(u)
    F2 = u.shape[-1]
    if F2 % 2 != 0:
        raise ValueError(f"last dimension must be even, got {F2}")
    F = F2 // 2
    u2 = u.reshape(-1, F2)
    if u2.stride(-1) != 1:
        u2 = u2.contiguous()
    out = torch.empty(u2.shape[0], F, dtype=u.dtype, device=u.device)
    with _on_device(u.device):
        _lib.check(_lib.lib().based_swiglu(u2.data_ptr(), out.data_ptr(), u2.shape[0], F, u2.stride(0), out.stride(0),
                                           _dtype_code(u), _stream_ptr(u)))
    return out.view(*u.shape[:-1], F)


def greedy_step(logits, next_ids, lengths, sequences=None, position_ids=None, vocab_size=None) -> None:
    """Greedy sampling of one decoding step plus the loop's bookkeeping, in one launch (recordable
    in the decode graph): per row b, tok = argmax(logits[b, :vocab_size]) (first index of the
    maximum, NaN largest, as torch.argmax), written to next_ids[b] and to
    sequences[b, lengths[b] + 1]; lengths[b] and position_ids[b] advance by one.

    logits (B, V) bf16 / fp32 with contiguous rows; next_ids (B,) or (B, 1) int64; lengths (B,)
    int32; sequences (B, max_length) int64 or None; position_ids (B,) or (B, 1) int64 or None."""
    _require_cuda(logits, next_ids, lengths)
    if logits.ndim != 2 or logits.stride(-1) != 1:
        raise ValueError("logits must be (B, V) with contiguous rows")
    B, V = logits.shape
    V = V if vocab_size is None else int(vocab_size)
    if not 0 < V <= logits.shape[1]:
        raise ValueError(f"vocab_size {V} outside (0, {logits.shape[1]}]")
    if next_ids.dtype != torch.int64 or next_ids.numel() != B or lengths.dtype != torch.int32 or lengths.numel() != B \
            or not lengths.is_contiguous():
        raise ValueError("next_ids must hold B int64 values, lengths B contiguous int32 values")
    for t, name in ((sequences, "sequences"), (position_ids, "position_ids")):
        if t is not None and (t.dtype != torch.int64 or t.shape[0] != B or not t.is_cuda):
            raise ValueError(f"{name} must be an int64 device tensor with B rows")
    if sequences is not None and (sequences.ndim != 2 or sequences.stride(1) != 1):
        raise ValueError("sequences must be (B, max_length) with contiguous rows")
    if position_ids is not None and position_ids.numel() != B:
        raise ValueError("position_ids must hold B values")
    with _on_device(logits.device):
        _lib.check(_lib.lib().based_greedy_step(
            logits.data_ptr(), B, V, logits.stride(0), next_ids.data_ptr(), next_ids.stride(0),
            sequences.data_ptr() if sequences is not None else None,
            sequences.stride(0) if sequences is not None else 0,
            sequences.shape[1] if sequences is not None else 0, lengths.data_ptr(),
            position_ids.data_ptr() if position_ids is not None else None,
            position_ids.stride(0) if position_ids is not None else 0, _dtype_code(logits), _stream_ptr(logits)))


DECODE_LINEAR_MAX_ROWS = 32  # BASED_DECODE_LINEAR_MAX_ROWS of include/based_hip.h
PROLOGUE_NONE, PROLOGUE_ADD_RMS_NORM, PROLOGUE_SWIGLU = 0, 1, 2
EPILOGUE_NONE, EPILOGUE_SWIGLU, EPILOGUE_GATED_CONV_STEP = 0, 1, 2


def decode_linear_weight_ok(weight: torch.Tensor) -> bool:
    """Whether `decode_linear` takes projections through this weight: bf16 (N, K) on the GPU with
    contiguous rows, K a multiple of 8 up to 4096."""
    return (weight.is_cuda and weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.stride(1) == 1
            and weight.stride(0) % 8 == 0 and weight.shape[1] % 8 == 0 and weight.shape[1] <= 4096)


def decode_linear(x, weight, bias=None, *, prologue: int = PROLOGUE_NONE, residual_in=None, residual_out=None,
                  norm_weight=None, eps: float = 1e-5, row_index=None, epilogue: int = EPILOGUE_NONE,
                  conv_state=None, conv_weight=None, conv_bias=None, out: Optional[torch.Tensor] = None
                  ) -> torch.Tensor:
    """y = epi(pro(x) @ weight.T (+ bias)) for the few rows of a single-token step, one launch.

    x: (M, K) bf16 rows (M <= 32; any leading shape is flattened), or for PROLOGUE_SWIGLU (M, 2K):
    value | gate.  weight: (N, K) bf16; bias None or (N).  PROLOGUE_ADD_RMS_NORM first forms
    r = x + residual_in (fp32, residual_in may be None), writes r to residual_out (fp32, may be
    None, never residual_in itself) and projects rms_norm(r) * norm_weight.  row_index: None, or an
    int64 device vector of M row numbers into x (the embedding table).
    EPILOGUE_SWIGLU: weight is (2F, K), y[:, f] = p[:, f] * silu(p[:, F + f]).
    EPILOGUE_GATED_CONV_STEP: weight is (2F, K); the gated short-convolution step on p with
    conv_state (M, F, k) rolled in place, conv_weight the (F, 1, k) or (F, k) Conv1d weight,
    conv_bias None or (F).  Returns y (M, N) or (M, F), written into `out` when given."""
    N, K = weight.shape
    x2 = x if x.dim() == 2 else x.reshape(-1, x.shape[-1])
    M = x2.shape[0] if row_index is None else row_index.numel()
    n_out = N if epilogue == EPILOGUE_NONE else N // 2
    key = ("decode_linear", x2.shape, x2.stride(), x2.dtype, x2.device, weight.shape, weight.stride(), weight.dtype,
           weight.device, prologue, epilogue,
           None if bias is None else (bias.shape, bias.dtype, bias.device, bias.stride()),
           None if residual_in is None else (residual_in.shape, residual_in.stride(), residual_in.dtype, residual_in.device),
           None if residual_out is None else (residual_out.shape, residual_out.stride(), residual_out.dtype, residual_out.device),
           None if norm_weight is None else (norm_weight.shape, norm_weight.dtype, norm_weight.device, norm_weight.stride()),
           None if row_index is None else (row_index.shape, row_index.dtype, row_index.device, row_index.stride()),
           None if conv_state is None else (conv_state.shape, conv_state.stride(), conv_state.dtype, conv_state.device),
           None if conv_weight is None else (conv_weight.shape, conv_weight.stride(), conv_weight.dtype, conv_weight.device),
           None if conv_bias is None else (conv_bias.shape, conv_bias.stride(), conv_bias.dtype, conv_bias.device))
    if key not in _CHECKED:
        _require_cuda(x2, weight)
        if x2.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            raise ValueError("decode_linear takes bfloat16 activations and weights")
        if weight.dim() != 2 or weight.stride(1) != 1 or x2.stride(1) != 1:
            raise ValueError("weight must be (N, K) and rows of x and weight contiguous")
        if x2.shape[1] != (2 * K if prologue == PROLOGUE_SWIGLU else K):
            raise ValueError(f"x {tuple(x.shape)} does not match weight {tuple(weight.shape)} (prologue {prologue})")
        if M > DECODE_LINEAR_MAX_ROWS:
            raise ValueError(f"decode_linear takes at most {DECODE_LINEAR_MAX_ROWS} rows, got {M}")
        if bias is not None:
            _require_cuda(x2, bias)
            if tuple(bias.shape) != (N,) or bias.dtype != torch.bfloat16 or not bias.is_contiguous():
                raise ValueError(f"bias must be a contiguous bfloat16 ({N},)")
        if prologue == PROLOGUE_ADD_RMS_NORM:
            if norm_weight is None:
                raise ValueError("the norm prologue needs norm_weight")
            _require_cuda(x2, norm_weight)
            if tuple(norm_weight.shape) != (K,) or norm_weight.dtype != torch.bfloat16 or not norm_weight.is_contiguous():
                raise ValueError(f"norm_weight must be a contiguous bfloat16 ({K},)")
            for r in (residual_in, residual_out):
                if r is not None:
                    _require_cuda(x2, r)
                    if r.dtype != torch.float32 or r.dim() != 2 or tuple(r.shape) != (M, K) or r.stride(1) != 1:
                        raise ValueError(f"residuals must be float32 ({M}, {K}) with contiguous rows")
        elif residual_in is not None or residual_out is not None or norm_weight is not None:
            raise ValueError("residual and norm arguments belong to PROLOGUE_ADD_RMS_NORM")
        if row_index is not None:
            _require_cuda(x2, row_index)
            if row_index.dtype != torch.int64 or row_index.dim() != 1 or not row_index.is_contiguous():
                raise ValueError("row_index must be a contiguous int64 device vector")
        if epilogue != EPILOGUE_NONE and N % 2 != 0:
            raise ValueError("a paired epilogue needs an even number of weight rows")
        if epilogue == EPILOGUE_GATED_CONV_STEP:
            if conv_state is None or conv_weight is None:
                raise ValueError("the convolution epilogue needs conv_state and conv_weight")
            _require_cuda(x2, conv_state, conv_weight)
            k = conv_weight.shape[-1]
            if (conv_weight.numel() != n_out * k or conv_weight.shape[0] != n_out or not conv_weight.is_contiguous()
                    or conv_weight.dtype != torch.bfloat16):
                raise ValueError(f"conv_weight must be a contiguous bfloat16 ({n_out}, 1, k), got {tuple(conv_weight.shape)}")
            if tuple(conv_state.shape) != (M, n_out, k) or not conv_state.is_contiguous():
                raise ValueError(f"conv_state must be a contiguous ({M}, {n_out}, {k}) tensor, got {tuple(conv_state.shape)}")
            _dtype_code(conv_state)
            if conv_bias is not None:
                _require_cuda(x2, conv_bias)
                if tuple(conv_bias.shape) != (n_out,) or conv_bias.dtype != torch.bfloat16 or not conv_bias.is_contiguous():
                    raise ValueError(f"conv_bias must be a contiguous bfloat16 ({n_out},)")
        elif conv_state is not None or conv_weight is not None or conv_bias is not None:
            raise ValueError("convolution arguments belong to EPILOGUE_GATED_CONV_STEP")
        _CHECKED[key] = True
    if out is None:
        y = torch.empty(M, n_out, dtype=torch.bfloat16, device=x2.device)
    else:
        y = out
        if tuple(y.shape) != (M, n_out) or y.dtype != torch.bfloat16 or y.device != x2.device or y.stride(1) != 1:
            raise ValueError(f"out must be a ({M}, {n_out}) bfloat16 tensor on {x2.device} with contiguous rows")
    conv = epilogue == EPILOGUE_GATED_CONV_STEP
    with _on_device(x2.device):
        _lib.check(_lib.lib().based_decode_linear(
            x2.data_ptr(), x2.stride(0), None if row_index is None else row_index.data_ptr(),
            x2.shape[0] if row_index is not None else 0,
            weight.data_ptr(), weight.stride(0), None if bias is None else bias.data_ptr(),
            y.data_ptr(), y.stride(0), M, N, K, prologue,
            None if residual_in is None else residual_in.data_ptr(), 0 if residual_in is None else residual_in.stride(0),
            None if residual_out is None else residual_out.data_ptr(), 0 if residual_out is None else residual_out.stride(0),
            None if norm_weight is None else norm_weight.data_ptr(), float(eps), epilogue,
            conv_state.data_ptr() if conv else None, _dtype_code(conv_state) if conv else 0,
            conv_weight.data_ptr() if conv else None,
            conv_bias.data_ptr() if conv and conv_bias is not None else None,
            conv_weight.shape[-1] if conv else 0, _stream_ptr(x2)))
    return y
