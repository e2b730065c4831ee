"""Token shift on AMD MI355X: host side of the operator.

Mirrors ``token_shift`` / ``TokenShift`` of the reference's
``src/forgetting_transformer/model/forgetting_transformer/token_shift.py``
(``:158-236``): same arguments, checks and error types.  The FoX layer calls it as
``token_shift(out_per_head, alpha, 1.0 - alpha)`` on the key and value projections
right before the attention (``modeling_forgetting_transformer.py:68-95``).  The
device work is done by the gfx950 kernels behind ``fox_token_shift_fwd`` /
``fox_token_shift_bwd``; there is no fallback path.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from .forgetting_attention import _DTYPES, _stream, maybe_contiguous

__all__ = ["token_shift", "TokenShift"]


def _args(x, prev_weight, curr_weight, **ptrs):
    B, T, H, D = x.shape
    a = _lib.ShiftArgs(B, T, H, D, _DTYPES[x.dtype], x.data_ptr(), x.stride(0), x.stride(1), x.stride(2),
                       prev_weight.data_ptr(), curr_weight.data_ptr(), curr_weight.stride(0), curr_weight.stride(1),
                       curr_weight.stride(2), None, None, None, None, None)
    for name, t in ptrs.items():
        setattr(a, name, t.data_ptr())
    return a


def _check(x, prev_weight, curr_weight):
    assert x.ndim == 4, "x must be (B, T, H, D)"
    B, T, H, D = x.size()
    assert D in {16, 32, 64, 128}
    assert prev_weight.size() == curr_weight.size() == (B, T, H)
    assert prev_weight.stride() == curr_weight.stride()
    assert x.dtype in _DTYPES, "x must be bfloat16 or float16"
    assert prev_weight.dtype == curr_weight.dtype == torch.float32, "the shift weights must be float32"
    if not x.is_cuda or not prev_weight.is_cuda or not curr_weight.is_cuda:
        raise RuntimeError("token_shift needs tensors on an AMD GPU (there is no CPU path)")


class TokenShift(torch.autograd.Function):
    """Autograd node with the reference's argument list (``token_shift.py:160-162``)."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, prev_weight: torch.Tensor, curr_weight: torch.Tensor):
        _check(x, prev_weight, curr_weight)
        x = maybe_contiguous(x)
        out = torch.empty_like(x)
        if x.stride() != out.stride():
            # x and out share one set of strides in the kernels; empty_like only keeps the strides of a
            # dense tensor (the reference asserts here, token_shift.py:169), so a strided view is copied
            x = x.contiguous()
            out = torch.empty_like(x)
        lib = _lib.load()
        with torch.cuda.device(x.device):
            _lib.check(lib.fox_token_shift_fwd(C.byref(_args(x, prev_weight, curr_weight, out=out)), _stream(x.device)),
                       "fox_token_shift_fwd")
        ctx.save_for_backward(x, prev_weight, curr_weight)
        return out

    @staticmethod
    def backward(ctx, dout: torch.Tensor):
        x, prev_weight, curr_weight = ctx.saved_tensors
        dout = dout if dout.stride() == x.stride() and dout.data_ptr() % 16 == 0 else _restride(dout, x)
        dx = torch.empty_like(x)
        dcurr_weight = torch.empty_like(curr_weight)
        dprev_weight = torch.empty_like(prev_weight)
        assert prev_weight.stride() == curr_weight.stride() == dcurr_weight.stride() == dprev_weight.stride()
        assert dout.stride() == x.stride() == dx.stride()
        lib = _lib.load()
        with torch.cuda.device(x.device):
            _lib.check(lib.fox_token_shift_bwd(
                C.byref(_args(x, prev_weight, curr_weight, dout=dout, dx=dx, dprev_weight=dprev_weight,
                              dcurr_weight=dcurr_weight)), _stream(x.device)), "fox_token_shift_bwd")
        return dx, dprev_weight, dcurr_weight


def _restride(t: torch.Tensor, like: torch.Tensor) -> torch.Tensor:
    """Copy ``t`` into memory laid out like ``like`` (the kernels share one set of strides)."""
    out = torch.empty_like(like)
    out.copy_(t)
    return out


def token_shift(x: torch.Tensor, prev_weight: torch.Tensor, curr_weight: torch.Tensor) -> torch.Tensor:
    """``out[b,t] = x[b,t] * curr_weight[b,t] + x[b,t-1] * prev_weight[b,t]`` per head, with ``x[b,-1] = 0``.

    x: ``(B, T, H, D)`` bfloat16/float16; weights: ``(B, T, H)`` float32.  Differentiable
    with respect to all three arguments.
    """
    return TokenShift.apply(x, prev_weight, curr_weight)
