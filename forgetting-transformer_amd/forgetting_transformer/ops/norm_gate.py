"""Gated per-head RMS normalisation on AMD MI355X: host side of the operator.

Mirrors ``group_norm_gated`` / ``LayerNormGatedFunction`` of the reference's
``src/forgetting_transformer/model/forgetting_transformer/fuse_norm_gate.py`` (``:726-823``,
``:977-1002``) for the configuration the FoX layer uses on the attention output
(``modeling_forgetting_transformer.py:243, 417-420``): RMS norm per group, a weight, no bias, no
residual, sigmoid (or swish) gate.  The device work is done by the gfx950 kernels behind
``fox_norm_gate_fwd`` / ``fox_norm_gate_bwd``; there is no fallback path, and the options of the
reference that the layer never uses raise ``NotImplementedError``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib
from .forgetting_attention import _DTYPES, _stream

__all__ = ["group_norm_gated", "GroupNormGated"]

_ACTS = {"sigmoid": _lib.ACT_SIGMOID, "swish": _lib.ACT_SWISH, "silu": _lib.ACT_SWISH}


def _rows(t: torch.Tensor, width: int) -> torch.Tensor:
    """(rows, width) view with unit inner stride, 16-byte aligned, row stride a multiple of 8."""
    t = t.reshape(-1, width)
    ok = t.stride(1) == 1 and t.data_ptr() % 16 == 0 and t.stride(0) % 8 == 0
    return t if ok else t.contiguous()


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
        assert x.shape == g.shape, "x and g must have the same shape"
        assert x.dtype in _DTYPES and g.dtype == x.dtype, "x and g must both be bfloat16 or both float16"
        width = x.shape[-1]
        assert width % num_groups == 0, "num_channels must be divisible by num_groups"
        D = width // num_groups
        assert D in {16, 32, 64, 128}, "group size must be one of 16, 32, 64, 128"
        assert weight is not None and weight.shape == (width,)
        if not x.is_cuda:
            raise RuntimeError("group_norm_gated needs tensors on an AMD GPU (there is no CPU path)")
        lib = _lib.load()
        x2, g2 = _rows(x, width), _rows(g, width)
        rows = x2.shape[0]
        w32 = weight.detach().float().contiguous()
        y = torch.empty((rows, width), dtype=x.dtype, device=x.device)
        rstd = torch.empty((rows, num_groups), dtype=torch.float32, device=x.device)
        args = _lib.NormGateArgs(rows, num_groups, D, _DTYPES[x.dtype], _ACTS[activation], float(eps),
                                 x2.data_ptr(), x2.stride(0), g2.data_ptr(), g2.stride(0), w32.data_ptr(),
                                 y.data_ptr(), y.stride(0), rstd.data_ptr(), None, 0, None, 0, None, 0, None, None)
        with torch.cuda.device(x.device):
            _lib.check(lib.fox_norm_gate_fwd(C.byref(args), _stream(x.device)), "fox_norm_gate_fwd")
        ctx.save_for_backward(x2, g2, w32, rstd)
        ctx.meta = (x.shape, g.shape, num_groups, D, _ACTS[activation], float(eps), weight.dtype)
        return y.reshape(x.shape)

    @staticmethod
    def backward(ctx, dy, *ignored):
        x2, g2, w32, rstd = ctx.saved_tensors
        x_shape, g_shape, G, D, act, eps, w_dtype = ctx.meta
        width = G * D
        rows = x2.shape[0]
        dy2 = _rows(dy, width)
        lib = _lib.load()
        dx = torch.empty((rows, width), dtype=x2.dtype, device=x2.device)
        dg = torch.empty((rows, width), dtype=g2.dtype, device=x2.device)
        dw = torch.empty((width,), dtype=torch.float32, device=x2.device)
        ws_bytes = C.c_int64(0)
        _lib.check(lib.fox_norm_gate_workspace_bytes(rows, G, D, C.byref(ws_bytes)), "fox_norm_gate_workspace_bytes")
        ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=x2.device)
        args = _lib.NormGateArgs(rows, G, D, _DTYPES[x2.dtype], act, eps, x2.data_ptr(), x2.stride(0), g2.data_ptr(),
                                 g2.stride(0), w32.data_ptr(), None, 0, rstd.data_ptr(), dy2.data_ptr(), dy2.stride(0),
                                 dx.data_ptr(), dx.stride(0), dg.data_ptr(), dg.stride(0), dw.data_ptr(), ws.data_ptr())
        with torch.cuda.device(x2.device):
            _lib.check(lib.fox_norm_gate_bwd(C.byref(args), _stream(x2.device)), "fox_norm_gate_bwd")
        return (dx.reshape(x_shape), dg.reshape(g_shape), dw.to(w_dtype), None, None, None, None, None, None, None, None)


def group_norm_gated(x: torch.Tensor, g: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     activation: str = "swish", residual: Optional[torch.Tensor] = None, prenorm: bool = False,
                     residual_in_fp32: bool = False, is_rms_norm: bool = False, num_groups: int = 1, eps: float = 1e-6):
    """``rms_norm_per_group(x) * weight * act(g)`` with the reference's signature (``fuse_norm_gate.py:977-1002``).

    x, g: (..., num_groups * D) bfloat16/float16; weight: (num_groups * D,).  The FoX layer calls it with
    ``is_rms_norm=True, activation="sigmoid", num_groups=heads``.
    """
    return GroupNormGated.apply(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, is_rms_norm,
                                num_groups)
