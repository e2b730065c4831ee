"""Forgetting Attention on AMD MI355X: host side of the operator.

This module mirrors the public surface of the reference's
``src/forgetting_transformer/ops/forgetting_attention.py`` -- the function
``forgetting_attention`` (``:403-455``) and the ``torch.autograd.Function``
``ForgettingAttention`` (``:44-400``) with the same argument order, checks and
error types -- but every device computation is done by hand-written gfx950 HIP
kernels reached through the flat C ABI of ``libfox_attn.so``.  PyTorch only
provides device memory, the current stream and autograd bookkeeping.  There is no
fallback path: without the library, or with tensors that are not on a GPU, the
call raises.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import functools
import math
from collections import defaultdict
from typing import Literal, Optional, Union

import torch

from . import _lib

__all__ = ["forgetting_attention", "forgetting_attention_from_logits", "forgetting_attention_norm_gate",
           "qk_norm_threshold", "record_pruning_bounds", "ForgettingAttention", "ForgettingAttentionFromLogits",
           "ForgettingAttentionNormGate"]

_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_FP16}


def maybe_contiguous(x: torch.Tensor) -> torch.Tensor:
    """Make ``x`` usable by the kernels without copying when possible.

    The reference only requires a unit innermost stride (``:35-38``); the HIP
    kernels read 16-byte vectors, so the base pointer must also be 16-byte aligned
    and the outer strides multiples of 8 elements.  Anything else is copied.
    """
    ok = x.stride(-1) == 1 and x.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in x.stride()[:-1])
    return x if ok else x.contiguous()


def _is_dense(shape, strides) -> bool:
    """True when the strides describe a permutation of a contiguous tensor (no gaps, no overlap)."""
    expect = 1
    for size, stride in sorted(zip(shape, strides), key=lambda p: p[1]):
        if size == 1:
            continue
        if stride != expect:
            return False
        expect *= size
    return True


def _view(x: torch.Tensor) -> _lib.View:
    return _lib.View(x.data_ptr(), x.stride(0), x.stride(1), x.stride(2))


def _ptr(x: Optional[torch.Tensor]):
    return None if x is None else C.c_void_p(x.data_ptr())


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()

_bound_records = None   # list that collects the pruning bounds of every call while record_pruning_bounds() is active


@contextlib.contextmanager
def record_pruning_bounds():
    """Collect the pruning bounds the kernels work with, for every call made inside the ``with`` block.

    The reference computes them with kernels of their own (``_find_start_index_kernel`` ``:695-745``,
    ``_find_end_index_kernel`` ``:747-795``) whose results only ``return_start_index`` exposes, and only for the
    forward.  Here the searches run inside the attention kernels; this context asks all three for what they found.
    Yields a list that receives one dict per call with a threshold: ``{"fwd_first_block": (B,H,ceil(M/block_m))}``
    from a forward, ``{"dq_first_block": (B,H,ceil(M/block_m)), "kv_end_row": (B,H,ceil(N/64))}`` from a backward
    (int32 tensors: first key block, in blocks of ``block_n`` keys, that each query block visits, and per 64 keys the
    query row where the dK/dV walk below them stops).  Not thread-safe; meant for tests and diagnostics."""
    global _bound_records
    prev, _bound_records = _bound_records, []
    try:
        yield _bound_records
    finally:
        _bound_records = prev


_current_device = getattr(torch._C, "_cuda_getDevice", torch.cuda.current_device)   # the binding without its Python wrappers


def _on_device(device: torch.device):
    """Context that makes ``device`` current; nothing to do (and nothing to pay) when it already is."""
    return _NO_SWITCH if _current_device() == device.index else torch.cuda.device(device)


# The raw handle of the current stream without building a torch.cuda.Stream object around it (about 9 us per call
# through the public accessor, a tenth of a small-shape step); the public accessor when this torch lacks the binding.
_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device: torch.device):
    if _raw_current_stream is not None and device.index is not None:
        return C.c_void_p(_raw_current_stream(device.index))
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class ForgettingAttention(torch.autograd.Function):
    """Autograd node; argument list identical to the reference's (``:72-73``).

    ``record_time_key`` / ``record_attention_time`` / ``record_find_index_time`` are the
    reference's in-op timers (``:45-70, 176-181, 217-222, 301-306, 358-363, 394-399``):
    with ``record_attention_time`` the forward and the backward are bracketed by events on
    the current stream, the host waits for the end event (as the reference synchronises)
    and the milliseconds are added to ``ForgettingAttention.info[record_time_key]``
    (``fwd_time`` / ``fwd_count`` / ``bwd_time`` / ``bwd_count``).  The pruning bounds are
    searched inside the attention kernels here, not by kernels of their own, so
    ``record_find_index_time`` only counts calls (``*_find_index_count``); the
    ``*_find_index_time`` entries stay 0.0.
    """

    info = defaultdict(lambda: {
        "fwd_time": 0.0, "fwd_count": 0, "bwd_time": 0.0, "bwd_count": 0,
        "fwd_find_index_time": 0.0, "fwd_find_index_count": 0,
        "bwd_find_index_kv_time": 0.0, "bwd_find_index_kv_count": 0,
        "bwd_find_index_q_time": 0.0, "bwd_find_index_q_count": 0,
    })
    events = defaultdict(lambda: {name: torch.cuda.Event(enable_timing=True)
                                  for name in ("fwd_start_event", "fwd_end_event", "bwd_start_event", "bwd_end_event")})

    @staticmethod
    def forward(ctx, q, k, v, log_fgate, seq_start, causal, sm_scale, adaptive_threshold,
                return_log_normalizer=False, return_start_index=False, record_time_key=None,
                record_attention_time=False, record_find_index_time=False):
        cls = ForgettingAttention
        if record_attention_time:
            cls.events[record_time_key]["fwd_start_event"].record()
        outs = _forward(ctx, False, q, k, v, log_fgate, seq_start, causal, sm_scale, adaptive_threshold,
                        return_log_normalizer, return_start_index)
        ctx.record_time_key = record_time_key
        ctx.record_attention_time = record_attention_time
        ctx.record_find_index_time = record_find_index_time
        if record_find_index_time and adaptive_threshold is not None:
            cls.info[record_time_key]["fwd_find_index_count"] += 1
        if record_attention_time:
            ev = cls.events[record_time_key]
            ev["fwd_end_event"].record()
            ev["fwd_end_event"].synchronize()
            cls.info[record_time_key]["fwd_time"] += ev["fwd_start_event"].elapsed_time(ev["fwd_end_event"])
            cls.info[record_time_key]["fwd_count"] += 1
        return outs

    @staticmethod
    def backward(ctx, do, *ignored):
        cls = ForgettingAttention
        key = ctx.record_time_key
        if ctx.record_attention_time:
            cls.events[key]["bwd_start_event"].record()
        grads = _backward(ctx, do)
        if ctx.record_find_index_time and ctx.saved_tensors[7] is not None:
            cls.info[key]["bwd_find_index_kv_count"] += 1
            cls.info[key]["bwd_find_index_q_count"] += 1
        if ctx.record_attention_time:
            ev = cls.events[key]
            ev["bwd_end_event"].record()
            ev["bwd_end_event"].synchronize()
            cls.info[key]["bwd_time"] += ev["bwd_start_event"].elapsed_time(ev["bwd_end_event"])
            cls.info[key]["bwd_count"] += 1
        return grads + (None,) * 9


class ForgettingAttentionFromLogits(torch.autograd.Function):
    """The same operator fed with the forget-gate *logits*: ``logsigmoid`` (fp32) is fused into the
    cumulative-sum kernel and its derivative into the reverse scan of the backward, which removes the
    layer's separate ``logsigmoid(fgate_logit.float())`` pass
    (``modeling_forgetting_transformer.py:343-346``).  Returns ``(out, log_fgate)``; ``log_fgate``
    (fp32, what the decode cache stores) is not differentiable here."""

    @staticmethod
    def forward(ctx, q, k, v, fgate_logit, seq_start, sm_scale, adaptive_threshold):
        out = _forward(ctx, True, q, k, v, fgate_logit, seq_start, True, sm_scale, adaptive_threshold,
                       False, False)
        ctx.mark_non_differentiable(ctx.log_fgate)
        return out, ctx.log_fgate

    @staticmethod
    def backward(ctx, do, *ignored):
        return _backward(ctx, do) + (None,) * 3


class ForgettingAttentionNormGate(torch.autograd.Function):
    """The operator followed by the layer's per-head RMS norm and output gate
    (``modeling_forgetting_transformer.py:417-422``), with that norm applied in the epilogue of the
    forward kernel: the attention output is normalised while it leaves the kernel instead of being
    read back by a kernel of its own.  The backward runs the norm's backward kernel on ``dy`` and
    feeds its ``dx`` to the operator's backward.  ``gate`` is None for the ungated norm."""

    @staticmethod
    def forward(ctx, q, k, v, log_fgate, gate, weight, seq_start, sm_scale, adaptive_threshold, activation, eps,
                fgate_is_logit=False):
        B, H, M, D = q.shape
        assert weight.shape == (H * D,), "weight must have shape (heads * head_dim,)"
        if gate is not None:
            assert gate.shape == q.shape, "gate must have the shape of q"
            assert gate.dtype == q.dtype, "gate must have the dtype of q"
            gate = _heads_adjacent(gate)
        w32 = weight.detach().float().contiguous()
        y = _forward(ctx, fgate_is_logit, q, k, v, log_fgate, seq_start, True, sm_scale, adaptive_threshold, False, False,
                     epilogue=(gate, w32, activation, float(eps)))
        ctx.norm_meta = (activation, float(eps), weight.dtype, gate is not None)
        if fgate_is_logit:  # the fp32 log gates are a by-product of the fused scan (see ForgettingAttentionFromLogits)
            ctx.mark_non_differentiable(ctx.log_fgate)
            return y, ctx.log_fgate
        return y

    @staticmethod
    def backward(ctx, dy, *ignored):
        q, o = ctx.saved_tensors[0], ctx.saved_tensors[3]
        gate, w32, rstd = ctx.saved_tensors[9:12]
        act, eps, w_dtype, gated = ctx.norm_meta
        B, H, M, D = q.shape
        rows, width = B * M, H * D
        lib = _lib.load()
        dy = _heads_adjacent(dy)
        do = torch.empty((B, M, H, D), dtype=q.dtype, device=q.device).transpose(1, 2)
        dgate = torch.empty((B, M, H, D), dtype=q.dtype, device=q.device).transpose(1, 2) if gated else None
        dw = torch.empty((width,), dtype=torch.float32, device=q.device)
        ws_bytes = C.c_int64(0)
        _lib.check(lib.fox_norm_gate_workspace_bytes(rows, H, D, C.byref(ws_bytes)), "fox_norm_gate_workspace_bytes")
        ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=q.device)
        args = _lib.NormGateArgs(rows, H, D, _DTYPES[q.dtype], act, eps, o.data_ptr(), o.stride(2),
                                 gate.data_ptr() if gated else None, gate.stride(2) if gated else 0,
                                 w32.data_ptr(), None, 0, rstd.data_ptr(), dy.data_ptr(), dy.stride(2),
                                 do.data_ptr(), do.stride(2), dgate.data_ptr() if gated else None,
                                 dgate.stride(2) if gated else 0, dw.data_ptr(), ws.data_ptr())
        with _on_device(q.device):
            _lib.check(lib.fox_norm_gate_bwd(C.byref(args), _stream(q.device)), "fox_norm_gate_bwd")
        dq, dk, dv, dlog_fgate = _backward(ctx, do)
        return dq, dk, dv, dlog_fgate, dgate, dw.to(w_dtype), None, None, None, None, None, None


def _heads_adjacent(x: torch.Tensor) -> torch.Tensor:
    """(B, H, M, D) tensor whose memory is (B, M, H, D) contiguous, 16-byte aligned: one row of heads * head_dim
    elements per token, the layout of the layer's (batch, time, hidden) tensors.  Copies only when needed."""
    B, H, M, D = x.shape
    ok = x.stride() == (M * H * D, D, H * D, 1) and x.data_ptr() % 16 == 0
    return x if ok else x.transpose(1, 2).contiguous().transpose(1, 2)


_GATE_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_FP16, torch.float32: _lib.DTYPE_FP32}


@functools.lru_cache(maxsize=256)
def _fwd_workspace_bytes(B, H, M, N, D, dtype_code):
    """Bytes of key-split scratch the forward wants for a shape (0 = the shape is not split); asked once per shape."""
    need = C.c_int64(0)
    _lib.check(_lib.load().fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(B, H, M, N, D, dtype_code)), C.byref(need)),
               "fox_attn_fwd_workspace_bytes")
    return need.value


@functools.lru_cache(maxsize=64)
def _cached_constant_threshold(value, B, H, device):
    t = torch.full((B, H), value, dtype=torch.float, device=device)
    # the fill has finished before the tensor enters the cache: whichever stream reads it later needs no ordering
    torch.cuda.current_stream(device).synchronize()
    return t


def _constant_threshold(value, B, H, device):
    """(B, H) fp32 tensor holding one float threshold: the same values as as_tensor + broadcast_to of the reference
    (:104-109), filled on the device once per (value, shape, device) instead of once per call.  Read-only.
    Under stream capture the tensor is filled by a kernel of the captured graph instead (a tensor created during
    capture lives in the graph's memory pool and holds nothing until the graph runs, so it must not be cached)."""
    if device.type != "cuda" or torch.cuda.is_current_stream_capturing():   # (CPU tensors are rejected further down)
        return torch.full((B, H), value, dtype=torch.float, device=device)
    return _cached_constant_threshold(value, B, H, device)


def _forward(ctx, gate_is_logit, q, k, v, log_fgate, seq_start, causal, sm_scale, adaptive_threshold,
             return_log_normalizer, return_start_index, epilogue=None):
    assert causal, "Only causal attention is supported"
    Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Dq == Dk == Dv, "feature size of q, k, v should be equal"
    assert Dk in {16, 32, 64, 128}, "We only support head dims in {16, 32, 64, 128}"
    assert q.dtype == k.dtype == v.dtype, "q, k, v must share one dtype"

    B, H, M, D = q.shape
    N = k.shape[2]
    assert log_fgate.shape == (B, H, N)
    if gate_is_logit:
        assert log_fgate.dtype in _GATE_DTYPES, "the gate logits must be bfloat16, float16 or float32"
    else:
        assert log_fgate.dtype == torch.float32, (
            "log_fgate must be in torch.float32. It is best to do this cast before logsigmoid, "
            "e.g., torch.nn.functional.logsigmoid(fgate_logit.float()).")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    sm_scale = float(sm_scale)

    Hk, Hv = k.shape[1], v.shape[1]
    assert Hk == Hv, "num of heads in k and v should be equal"
    assert H == Hk, "groupped query attention has not been tested. You can uncomment this if you know what you are doing."
    assert k.shape == (B, Hk, N, D) and v.shape == (B, Hv, N, D)
    assert not (M > N), "The key/value tensors must be longer than the query tensor"

    # threshold: validate on the host first (:91-109), compute "auto" on the device later
    auto_threshold = False
    if adaptive_threshold is not None:
        if isinstance(adaptive_threshold, str):
            assert adaptive_threshold == "auto", (
                'adaptive_threshold must be either the string "auto", a float, or a Tensor, '
                f"but got {adaptive_threshold}.")
            auto_threshold = True
        elif isinstance(adaptive_threshold, (int, float)):
            # same values as as_tensor + broadcast_to below, filled on the device: no host-to-device copy to wait for
            adaptive_threshold = _constant_threshold(float(adaptive_threshold), B, H, q.device)
        else:
            adaptive_threshold = torch.as_tensor(adaptive_threshold, dtype=torch.float, device=q.device)
            try:
                adaptive_threshold = torch.broadcast_to(adaptive_threshold, (B, H))
            except RuntimeError:
                raise RuntimeError(
                    'adaptive_threshold must be either the string "auto" or broadcastable to '
                    f"(batch_size, num_heads) = ({B}, {H}), but got {adaptive_threshold.size()}.")
            assert adaptive_threshold.size() == (B, H)
            adaptive_threshold = adaptive_threshold.contiguous()

    if seq_start is not None:
        has_seq_start = True
        assert seq_start.shape == (B,)
    else:
        has_seq_start = False

    if q.device.type != "cuda":
        raise RuntimeError("forgetting_attention runs only on an AMD GPU (HIP device); "
                           f"got tensors on '{q.device}'. There is no CPU implementation.")
    lib = _lib.load()
    device = q.device
    dims = _lib.Dims(B, H, M, N, D, _DTYPES[q.dtype])
    if has_seq_start:
        seq_start = seq_start.to(device=device, dtype=torch.long).contiguous()

    q, k, v = maybe_contiguous(q), maybe_contiguous(k), maybe_contiguous(v)

    with _on_device(device):
        stream = _stream(device)

        if auto_threshold:
            adaptive_threshold = torch.empty((B, H), dtype=torch.float32, device=device)
            scratch = torch.empty((B, H, 3), dtype=torch.int32, device=device)
            qv, kv = _view(q), _view(k)
            _lib.check(lib.fox_auto_threshold(C.byref(dims), C.byref(qv), C.byref(kv), sm_scale,
                                              _ptr(adaptive_threshold), _ptr(scratch), stream), "fox_auto_threshold")

        # log_lambda (B,H,N), the log-normaliser L (B,H,M) and the key-split scratch come from one allocation
        ws_bytes = _fwd_workspace_bytes(B, H, M, N, D, dims.dtype)
        n_c, n_l = (B * H * N + 3) // 4 * 4, (B * H * M + 3) // 4 * 4    # floats; the scratch behind them stays 16-byte aligned
        buf = torch.empty(n_c + n_l + ws_bytes // 4, dtype=torch.float32, device=device)
        log_lambda = buf[:B * H * N].view(B, H, N)
        L = buf[n_c:n_c + B * H * M].view(B, H, M)
        workspace = buf[n_c + n_l:] if ws_bytes > 0 else None

        # c = cumsum(log_fgate) with gates left of seq_start zeroed, one fused kernel
        if gate_is_logit:  # logsigmoid fused into the scan; the fp32 log gates are a by-product
            ctx.log_fgate = torch.empty((B, H, N), dtype=torch.float32, device=device)
            _lib.check(lib.fox_gate_cumsum_fwd(_ptr(log_fgate), _GATE_DTYPES[log_fgate.dtype], log_fgate.stride(0),
                                               log_fgate.stride(1), log_fgate.stride(2), _ptr(seq_start),
                                               _ptr(ctx.log_fgate), _ptr(log_lambda), B, H, N, stream),
                       "fox_gate_cumsum_fwd")
        else:
            _lib.check(lib.fox_cumsum_fwd(_ptr(log_fgate), log_fgate.stride(0), log_fgate.stride(1),
                                          log_fgate.stride(2), _ptr(seq_start), _ptr(log_lambda), B, H, N, stream),
                       "fox_cumsum_fwd")

        y = rstd = None
        if epilogue is None:
            o = torch.empty_like(q)
        else:  # o and y as rows of heads * head_dim per token: what the norm's backward and the output projection read
            o = torch.empty((B, M, H, D), dtype=q.dtype, device=device).transpose(1, 2)
            y = torch.empty((B, M, H, D), dtype=q.dtype, device=device).transpose(1, 2)
            rstd = torch.empty((B, M, H), dtype=torch.float32, device=device)
        first_block = None
        if return_start_index or (_bound_records is not None and adaptive_threshold is not None):
            block_m, _, _, _ = _lib.tile_config(D)
            first_block = torch.zeros((B, H, (M + block_m - 1) // block_m), dtype=torch.int32, device=device)
        args = _lib.FwdArgs(dims, _view(q), _view(k), _view(v), _view(o), log_lambda.data_ptr(), L.data_ptr(),
                            None if seq_start is None else seq_start.data_ptr(),
                            None if adaptive_threshold is None else adaptive_threshold.data_ptr(),
                            sm_scale, None if first_block is None else first_block.data_ptr(),
                            None if workspace is None else workspace.data_ptr(), ws_bytes)
        if epilogue is None:
            _lib.check(lib.fox_attn_fwd(C.byref(args), stream), "fox_attn_fwd")
        else:
            gate, w32, act, eps = epilogue
            epi = _lib.FwdEpilogue(_view(gate) if gate is not None else _lib.View(), _view(y), w32.data_ptr(),
                                   rstd.data_ptr(), eps, act)
            _lib.check(lib.fox_attn_fwd_norm_gate(C.byref(args), C.byref(epi), stream), "fox_attn_fwd_norm_gate")

    if _bound_records is not None and adaptive_threshold is not None:
        _bound_records.append({"fwd_first_block": first_block})
    saved = (q, k, v, o, L, log_lambda, seq_start, adaptive_threshold, log_fgate if gate_is_logit else None)
    if epilogue is not None:
        saved += (epilogue[0], epilogue[1], rstd)
    ctx.save_for_backward(*saved)
    ctx.sm_scale = sm_scale
    ctx.causal = causal
    ctx.has_seq_start = has_seq_start
    ctx.gate_strides = tuple(log_fgate.stride())

    if return_log_normalizer or return_start_index:
        start_index = None
        if return_start_index:
            _, block_n, _, _ = _lib.tile_config(D)
            start_index = first_block.to(torch.long) * block_n
        outs = (o, L if return_log_normalizer else None, start_index)
        ctx.mark_non_differentiable(*[t for t in outs[1:] if t is not None])
        return outs
    return o if epilogue is None else y


def _backward(ctx, do):
    q, k, v, o, L, log_lambda, seq_start, adaptive_threshold, gate_logit = ctx.saved_tensors[:9]
    B, H, M, D = q.shape
    N = k.shape[2]
    device = q.device
    lib = _lib.load()
    do = maybe_contiguous(do)
    with _on_device(device):
        stream = _stream(device)
        # one allocation for the fp32 temporaries: rowsum(o * do) and the row sums of dS (B,H,M each), then dlog_lambda (B,H,N)
        tmp = torch.empty(2 * B * H * M + B * H * N, dtype=torch.float32, device=device)
        delta, drow, dlog_lambda = tmp[:B * H * M], tmp[B * H * M:2 * B * H * M], tmp[2 * B * H * M:]
        q_first = kv_end = None
        if _bound_records is not None and adaptive_threshold is not None:
            block_m, _, _, _ = _lib.tile_config(D)
            q_first = torch.zeros((B, H, (M + block_m - 1) // block_m), dtype=torch.int32, device=device)
            kv_end = torch.full((B, H, (N + 63) // 64), -1, dtype=torch.int32, device=device)
            _bound_records.append({"dq_first_block": q_first, "kv_end_row": kv_end})
        dlog_fgate = None
        if gate_logit is None:
            # in the layout of the caller's log_fgate when that is a permuted dense tensor (the (B,H,T) view of
            # (B,T,H) memory the FoX layer passes): autograd then takes the gradient as it is, without a copy
            gs = ctx.gate_strides if _is_dense((B, H, N), ctx.gate_strides) else (H * N, N, 1)
            dlog_fgate = torch.empty_strided((B, H, N), gs, dtype=torch.float32, device=device)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        args = _lib.BwdArgs(
            _lib.Dims(B, H, M, N, D, _DTYPES[q.dtype]),
            _view(q), _view(k), _view(v), _view(o), _view(do), _view(dq), _view(dk), _view(dv),
            log_lambda.data_ptr(), L.data_ptr(),
            None if seq_start is None else seq_start.data_ptr(),
            None if adaptive_threshold is None else adaptive_threshold.data_ptr(),
            ctx.sm_scale, delta.data_ptr(), drow.data_ptr(), dlog_lambda.data_ptr(),
            None if dlog_fgate is None else dlog_fgate.data_ptr(),
            *(dlog_fgate.stride() if dlog_fgate is not None else (0, 0, 0)),
            None if q_first is None else q_first.data_ptr(), None if kv_end is None else kv_end.data_ptr())
        if gate_logit is None:
            _lib.check(lib.fox_attn_bwd(C.byref(args), stream), "fox_attn_bwd")
            dgate = dlog_fgate
        else:  # same stages, the last one fused with the derivative of logsigmoid
            _lib.check(lib.fox_attn_bwd_dq(C.byref(args), stream), "fox_attn_bwd_dq")
            _lib.check(lib.fox_attn_bwd_dkdv(C.byref(args), stream), "fox_attn_bwd_dkdv")
            dgate = torch.empty_like(gate_logit)
            _lib.check(lib.fox_gate_cumsum_bwd(_ptr(dlog_lambda), _ptr(gate_logit), _GATE_DTYPES[gate_logit.dtype],
                                               gate_logit.stride(0), gate_logit.stride(1), gate_logit.stride(2),
                                               _ptr(seq_start), _ptr(dgate), dgate.stride(0), dgate.stride(1), dgate.stride(2), B, H, N,
                                               stream), "fox_gate_cumsum_bwd")
    return dq, dk, dv, dgate


def forgetting_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    log_fgate: torch.Tensor,
    *,
    head_first: bool = False,
    seq_start: Optional[torch.Tensor] = None,
    sm_scale: Optional[float] = None,
    adaptive_threshold: Optional[Union[Literal["auto"], float, torch.Tensor]] = None,
):
    """Causal softmax attention with a data-dependent forget-gate decay bias.

    Same contract as the reference (``:403-455``):

    - q, k, v are bfloat16/float16, log_fgate is float32
    - seqlen_q <= seqlen_k; query ``i`` sits at key position ``i + seqlen_k - seqlen_q``
    - head dim in {16, 32, 64, 128}

    Arguments:
        q: (batch, seqlen_q, heads, head_dim) unless head_first=True.
        k, v: (batch, seqlen_k, heads, head_dim) unless head_first=True.
        log_fgate: (batch, seqlen_k, heads) unless head_first=True; the log of the
            forget gates, typically ``logsigmoid(logits.float())``.
        head_first: heads axis before the sequence axis in all inputs and the output.
        seq_start: optional LongTensor (batch,); keys before ``seq_start[b]`` get no
            attention (left padding).
        sm_scale: score scale, default ``1/sqrt(head_dim)``.
        adaptive_threshold: Adaptive Computation Pruning threshold: ``"auto"``, a
            float, or a tensor broadcastable to (batch, heads).  Key blocks whose
            decay bias is below it for a whole query block are skipped.

    Returns:
        out: same shape, layout and dtype as q.
    """
    for name, entry in dict(q=q, k=k, v=v).items():
        assert entry.dtype in [torch.float16, torch.bfloat16], (
            f"Only torch.float16 or torch.bfloat16 are supported for q/k/v, but got {entry.dtype} for {name}.")
    if not head_first:
        q, k, v = [item.transpose(1, 2) for item in (q, k, v)]  # b t h d -> b h t d, views
        log_fgate = log_fgate.transpose(1, 2)                   # b t h -> b h t
    out = ForgettingAttention.apply(q, k, v, log_fgate, seq_start, True, sm_scale, adaptive_threshold,
                                    False, False, None, False, False)
    if not head_first:
        out = out.transpose(1, 2)
    return out


def forgetting_attention_from_logits(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    fgate_logit: torch.Tensor,
    *,
    head_first: bool = False,
    seq_start: Optional[torch.Tensor] = None,
    sm_scale: Optional[float] = None,
    adaptive_threshold: Optional[Union[Literal["auto"], float, torch.Tensor]] = None,
):
    """``forgetting_attention(q, k, v, logsigmoid(fgate_logit.float()), ...)`` with the log-sigmoid fused into
    the operator's scan kernels (forward and backward).

    ``fgate_logit`` is the output of the layer's gate projection, (batch, seqlen_k, heads) unless
    head_first=True, in bfloat16, float16 or float32; every other argument is as in
    ``forgetting_attention``.  Returns ``(out, log_fgate)`` where ``log_fgate`` is the float32
    ``logsigmoid(fgate_logit)`` in the layout of ``fgate_logit`` (what the layer's decode cache
    stores, ``modeling_forgetting_transformer.py:356-357``); gradients flow to q, k, v and
    fgate_logit through ``out`` only.
    """
    for name, entry in dict(q=q, k=k, v=v).items():
        assert entry.dtype in [torch.float16, torch.bfloat16], (
            f"Only torch.float16 or torch.bfloat16 are supported for q/k/v, but got {entry.dtype} for {name}.")
    if not head_first:
        q, k, v = [item.transpose(1, 2) for item in (q, k, v)]
        fgate_logit = fgate_logit.transpose(1, 2)
    out, log_fgate = ForgettingAttentionFromLogits.apply(q, k, v, fgate_logit, seq_start, sm_scale, adaptive_threshold)
    if not head_first:
        out, log_fgate = out.transpose(1, 2), log_fgate.transpose(1, 2)
    return out, log_fgate


_NORM_ACTS = {"sigmoid": _lib.ACT_SIGMOID, "swish": _lib.ACT_SWISH, "silu": _lib.ACT_SWISH}


def forgetting_attention_norm_gate(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    log_fgate: torch.Tensor,
    gate: Optional[torch.Tensor],
    norm_weight: torch.Tensor,
    *,
    activation: str = "sigmoid",
    eps: float = 1e-6,
    head_first: bool = False,
    seq_start: Optional[torch.Tensor] = None,
    sm_scale: Optional[float] = None,
    adaptive_threshold: Optional[Union[Literal["auto"], float, torch.Tensor]] = None,
    fgate_is_logit: bool = False,
):
    """``group_norm_gated(forgetting_attention(q, k, v, log_fgate, ...), gate, norm_weight, is_rms_norm=True,
    num_groups=heads)`` in one forward kernel: what the FoX layer computes between the attention and its output
    projection (``modeling_forgetting_transformer.py:396-422``).

    ``gate`` has the shape and dtype of q (the layer's ``ogate_proj(hidden_states)`` viewed per head), or is None
    for the ungated output norm (``:245, :422``); ``norm_weight`` is ``(heads * head_dim,)``; every other argument
    is as in ``forgetting_attention``.  Returns the normalised, gated output in the shape of q; with
    head_first=False it is contiguous, so ``.reshape(batch, seqlen, heads * head_dim)`` is a view.  Gradients
    flow to q, k, v, log_fgate, gate and norm_weight.

    With ``fgate_is_logit=True`` the fourth argument is the gate *logits* (bfloat16, float16 or float32) as in
    ``forgetting_attention_from_logits`` and the result is ``(y, log_fgate)``: the whole chain from the layer's
    gate projection to the input of its output projection in one scan kernel and one attention kernel.
    """
    for name, entry in dict(q=q, k=k, v=v).items():
        assert entry.dtype in [torch.float16, torch.bfloat16], (
            f"Only torch.float16 or torch.bfloat16 are supported for q/k/v, but got {entry.dtype} for {name}.")
    if gate is not None and activation not in _NORM_ACTS:
        raise ValueError(f"Unsupported activation: {activation}")
    if not head_first:
        q, k, v = [item.transpose(1, 2) for item in (q, k, v)]
        log_fgate = log_fgate.transpose(1, 2)
        gate = gate.transpose(1, 2) if gate is not None else None
    act = _NORM_ACTS[activation] if gate is not None else _lib.ACT_NONE
    out = ForgettingAttentionNormGate.apply(q, k, v, log_fgate, gate, norm_weight, seq_start, sm_scale,
                                            adaptive_threshold, act, eps, fgate_is_logit)
    if fgate_is_logit:
        y, lg = out
        return (y, lg) if head_first else (y.transpose(1, 2), lg.transpose(1, 2))
    return out if head_first else out.transpose(1, 2)


@torch.no_grad()
def qk_norm_threshold(q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor, num_heads: int, head_dim: int,
                      seq_len: int, log_pruning_tolerance: float, share_param_across_head: bool = False) -> torch.Tensor:
    """``adaptive_threshold`` for queries and keys that went through an RMS QK-norm, from the norm weights alone.

    The caller-side rule of the FoX layer (``modeling_forgetting_transformer.py:366-380``): a normalised row has
    L2 norm at most ``max|w| * sqrt(head_dim)``, so with ``sm_scale = 1/sqrt(head_dim)`` no logit exceeds
    ``max|w_q| * max|w_k| * sqrt(head_dim)``; the threshold is ``-(2 * bound + log(seq_len)) + log_pruning_tolerance``.
    Weights of shape ``(num_heads * head_dim,)`` give one threshold per head, shape ``(num_heads,)``, which
    ``forgetting_attention`` broadcasts over the batch; with ``share_param_across_head`` the weights are
    ``(head_dim,)`` and the result is a 0-d tensor.  No pass over q and k is needed (unlike ``"auto"``).
    """
    if share_param_across_head:
        assert q_norm_weight.shape == k_norm_weight.shape == (head_dim,)
        bound = q_norm_weight.abs().max() * k_norm_weight.abs().max() * math.sqrt(head_dim)
    else:
        assert q_norm_weight.shape == k_norm_weight.shape == (num_heads * head_dim,)
        bound = (q_norm_weight.view(num_heads, head_dim).abs().max(dim=-1).values
                 * k_norm_weight.view(num_heads, head_dim).abs().max(dim=-1).values * math.sqrt(head_dim))
    return -(2 * bound + math.log(seq_len)) + log_pruning_tolerance
