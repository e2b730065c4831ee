"""Per-head RMS normalisation on AMD MI355X, gated and plain: host side of the operators.

Mirrors ``group_norm_gated`` / ``LayerNormGatedFunction`` of the reference's
``src/forgetting_transformer/model/forgetting_transformer/fuse_norm_gate.py`` (``:726-823``,
``:977-1002``) for the configuration the FoX layer uses on the attention output
(``modeling_forgetting_transformer.py:243, 417-420``): RMS norm per group, a weight, no bias, no
residual, sigmoid (or swish) gate; and ``group_norm`` / ``rms_norm`` / ``LayerNormFunction`` of
``layernorm.py`` (``:706-860``) for the plain form the layer applies to queries and keys
(``modeling_forgetting_transformer.py:258-265, 314-325``) and as its ungated output norm (``:245``).
The device work is done by the gfx950 kernels behind ``fox_norm_gate_fwd`` / ``fox_norm_gate_bwd``;
there is no fallback path, and the options of the reference that the layer never uses raise
``NotImplementedError``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib
from .forgetting_attention import _DTYPES, _stream

__all__ = ["group_norm_gated", "GroupNormGated", "group_norm", "rms_norm", "GroupNormPlain"]

_ACTS = {"sigmoid": _lib.ACT_SIGMOID, "swish": _lib.ACT_SWISH, "silu": _lib.ACT_SWISH}
_GROUP_SIZES = {16, 32, 64, 128}


def _rows(t: torch.Tensor, width: int) -> torch.Tensor:
    """(rows, width) view with unit inner stride, 16-byte aligned, row stride a multiple of 8."""
    t = t.reshape(-1, width)
    ok = t.stride(1) == 1 and t.data_ptr() % 16 == 0 and t.stride(0) % 8 == 0
    return t if ok else t.contiguous()


def _norm_forward(ctx, x, g, weight, act, eps, num_groups):
    """Shared forward: validates, launches ``fox_norm_gate_fwd`` and fills ``ctx``.  ``g`` is None for the plain norm."""
    assert x.dtype in _DTYPES, "x must be bfloat16 or float16"
    if g is not None:
        assert x.shape == g.shape, "x and g must have the same shape"
        assert g.dtype == x.dtype, "x and g must both be bfloat16 or both float16"
    width = x.shape[-1]
    if width % num_groups != 0:
        raise ValueError("num_channels must be divisible by num_groups")
    D = width // num_groups
    assert D in _GROUP_SIZES, "group size must be one of 16, 32, 64, 128"
    assert weight is not None and weight.shape == (width,), "weight must have shape (num_groups * group size,)"
    if not x.is_cuda:
        raise RuntimeError("the normalisation needs tensors on an AMD GPU (there is no CPU path)")
    lib = _lib.load()
    x2 = _rows(x, width)
    g2 = _rows(g, width) if g is not None else None
    rows = x2.shape[0]
    w32 = weight.detach().float().contiguous()
    y = torch.empty((rows, width), dtype=x.dtype, device=x.device)
    rstd = torch.empty((rows, num_groups), dtype=torch.float32, device=x.device)
    args = _lib.NormGateArgs(rows, num_groups, D, _DTYPES[x.dtype], act, float(eps),
                             x2.data_ptr(), x2.stride(0), g2.data_ptr() if g2 is not None else None,
                             g2.stride(0) if g2 is not None else 0, w32.data_ptr(),
                             y.data_ptr(), y.stride(0), rstd.data_ptr(), None, 0, None, 0, None, 0, None, None)
    with torch.cuda.device(x.device):
        _lib.check(lib.fox_norm_gate_fwd(C.byref(args), _stream(x.device)), "fox_norm_gate_fwd")
    if g2 is not None:
        ctx.save_for_backward(x2, w32, rstd, g2)
    else:
        ctx.save_for_backward(x2, w32, rstd)
    ctx.meta = (x.shape, num_groups, D, act, float(eps), weight.dtype)
    return y.reshape(x.shape)


def _norm_backward(ctx, dy):
    """Shared backward: returns (dx, dg or None, dweight)."""
    x2, w32, rstd, *rest = ctx.saved_tensors
    g2 = rest[0] if rest else None
    x_shape, G, D, act, eps, w_dtype = ctx.meta
    width = G * D
    rows = x2.shape[0]
    dy2 = _rows(dy, width)
    lib = _lib.load()
    dx = torch.empty((rows, width), dtype=x2.dtype, device=x2.device)
    dg = torch.empty((rows, width), dtype=x2.dtype, device=x2.device) if g2 is not None else None
    dw = torch.empty((width,), dtype=torch.float32, device=x2.device)
    ws_bytes = C.c_int64(0)
    _lib.check(lib.fox_norm_gate_workspace_bytes(rows, G, D, C.byref(ws_bytes)), "fox_norm_gate_workspace_bytes")
    ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=x2.device)
    args = _lib.NormGateArgs(rows, G, D, _DTYPES[x2.dtype], act, eps, x2.data_ptr(), x2.stride(0),
                             g2.data_ptr() if g2 is not None else None, g2.stride(0) if g2 is not None else 0,
                             w32.data_ptr(), None, 0, rstd.data_ptr(), dy2.data_ptr(), dy2.stride(0),
                             dx.data_ptr(), dx.stride(0), dg.data_ptr() if dg is not None else None,
                             dg.stride(0) if dg is not None else 0, dw.data_ptr(), ws.data_ptr())
    with torch.cuda.device(x2.device):
        _lib.check(lib.fox_norm_gate_bwd(C.byref(args), _stream(x2.device)), "fox_norm_gate_bwd")
    return dx.reshape(x_shape), (dg.reshape(x_shape) if dg is not None else None), dw.to(w_dtype)


class GroupNormGated(torch.autograd.Function):
    """Autograd node with the reference's argument list (``fuse_norm_gate.py:730-743``)."""

    @staticmethod
    def forward(ctx, x, g, weight, bias, activation, residual=None, eps=1e-6, prenorm=False, residual_in_fp32=False,
                is_rms_norm=False, num_groups=1):
        if bias is not None or residual is not None or prenorm or residual_in_fp32 or not is_rms_norm:
            raise NotImplementedError("only the FoX output-norm configuration is built: RMS norm, weight, no bias, "
                                      "no residual")
        if activation not in _ACTS:
            raise ValueError(f"Unsupported activation: {activation}")
        assert g is not None, "the gated norm needs a gate tensor"
        return _norm_forward(ctx, x, g, weight, _ACTS[activation], eps, num_groups)

    @staticmethod
    def backward(ctx, dy, *ignored):
        dx, dg, dw = _norm_backward(ctx, dy)
        return (dx, dg, dw, None, None, None, None, None, None, None, None)


class GroupNormPlain(torch.autograd.Function):
    """Ungated norm with the argument list of the reference's ``LayerNormFunction`` (``layernorm.py:706-721``)."""

    @staticmethod
    def forward(ctx, x, weight, bias, residual=None, eps=1e-5, prenorm=False, residual_in_fp32=False,
                is_rms_norm=False, num_groups=1):
        if bias is not None or residual is not None or prenorm or residual_in_fp32 or not is_rms_norm:
            raise NotImplementedError("only the FoX QK-norm / output-norm configuration is built: RMS norm, weight, "
                                      "no bias, no residual")
        return _norm_forward(ctx, x, None, weight, _lib.ACT_NONE, eps, num_groups)

    @staticmethod
    def backward(ctx, dy, *ignored):
        dx, _, dw = _norm_backward(ctx, dy)
        return (dx, dw, None, None, None, None, None, None, None)


def group_norm_gated(x: torch.Tensor, g: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     activation: str = "swish", residual: Optional[torch.Tensor] = None, prenorm: bool = False,
                     residual_in_fp32: bool = False, is_rms_norm: bool = False, num_groups: int = 1, eps: float = 1e-6):
    """``rms_norm_per_group(x) * weight * act(g)`` with the reference's signature (``fuse_norm_gate.py:977-1002``).

    x, g: (..., num_groups * D) bfloat16/float16; weight: (num_groups * D,).  The FoX layer calls it with
    ``is_rms_norm=True, activation="sigmoid", num_groups=heads``.
    """
    return GroupNormGated.apply(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, is_rms_norm,
                                num_groups)


def group_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               residual: Optional[torch.Tensor] = None, eps: float = 1e-5, prenorm: bool = False,
               residual_in_fp32: bool = False, is_rms_norm: bool = False, num_groups: int = 1):
    """``rms_norm_per_group(x) * weight`` with the reference's signature (``layernorm.py:817-838``).

    The FoX layer's QK-norm: ``GroupNorm(num_groups=heads, hidden_size, is_rms_norm=True)`` on the (B, T, H*D)
    projections (``modeling_forgetting_transformer.py:264-265, 314-316``).
    """
    return GroupNormPlain.apply(x, weight, bias, residual, eps, prenorm, residual_in_fp32, is_rms_norm, num_groups)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
             residual: Optional[torch.Tensor] = None, eps: float = 1e-5, prenorm: bool = False,
             residual_in_fp32: bool = False):
    """RMS norm over the last dimension with the reference's signature (``layernorm.py:841-859``).

    The FoX layer's QK-norm with weights shared across heads: ``RMSNorm(head_dim)`` on (B, T, H, D)
    (``modeling_forgetting_transformer.py:261-262, 323-325``); the last dimension must be 16, 32, 64 or 128.
    """
    return GroupNormPlain.apply(x, weight, bias, residual, eps, prenorm, residual_in_fp32, True, 1)
