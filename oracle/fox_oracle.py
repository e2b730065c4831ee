"""TEST INFRASTRUCTURE ONLY -- not part of the shipped operator.

A plain-PyTorch restatement of the reference's materialised-mask Forgetting
Attention, used as the checker for the HIP kernels.  Only tests, the smoke
check and the CPU-baseline leg of the benchmark may import this module; the
operator itself never does.

Reference lines restated here (paths relative to the reference checkout):

* ``src/forgetting_transformer/ops/forgetting_attention.py:1380-1404``
  -- the pure-PyTorch Forgetting Attention inside ``test_op``: scores
  ``q k^T * sm_scale`` plus the decay bias ``c[i + P_SEQ] - c[j]`` with
  ``c = cumsum(log_fgate)``, a ``tril(diagonal=P_SEQ)`` causal mask, a
  ``seq_start`` column mask, fp32 softmax, NaN -> 0 for rows with no valid
  column, ``p @ v``, and gradients through ``torch.autograd``.
* ``:111-127`` -- the operator's prologue: zero ``log_fgate`` left of
  ``seq_start`` on a clone, then ``cumsum`` in fp32.
* ``:91-102``  -- the ``"auto"`` pruning threshold.
* ``:695-795`` -- the two block-boundary scans of Adaptive Computation Pruning
  (restated in pure Python for small cases; the C restatement covers the
  same scans for larger ones).
* ``:902-943, 956-1143, 1156-1344, 390-392`` -- the manual backward
  (``manual_backward`` below), written from the kernels' arithmetic.

* ``src/forgetting_transformer/model/forgetting_transformer/token_shift.py:264-270``
  -- the pure-PyTorch token shift inside its ``test_op`` (``token_shift_ref``):
  roll by one step, zero the first step, weighted sum in fp32, cast.  Pinned by
  the identity / pure-shift special cases, an explicit loop, ``gradcheck`` in
  fp64 and the C restatement.

* ``src/forgetting_transformer/model/forgetting_transformer/fuse_norm_gate.py:18-53``
  -- ``group_norm_gated_ref`` for the RMS / no bias / no residual case
  (``group_norm_gated_ref`` here): per-group ``x / sqrt(mean(x^2) + eps) * weight``
  times ``sigmoid(g)`` (or ``g * sigmoid(g)``), evaluated in the upcast dtype.
  Pinned by ``torch.nn.functional.rms_norm`` per group, ``gradcheck`` in fp64 and
  the C restatement.  ``group_norm_ref`` is the same without a gate
  (``layernorm.py:77-110``), pinned the same way; ``qk_norm_threshold_ref``
  (``modeling_forgetting_transformer.py:371-380``) is pinned by the bound it
  states: no logit of normalised q, k exceeds it (brute force).

Pinned by (see tests/test_oracle_cpu.py): ``scaled_dot_product_attention`` with
an additive mask, ``torch.logsumexp``, the ``g == 0`` and constant-``g``
closed forms, ``torch.autograd.gradcheck`` in fp64, the identities
``sum_n dc_n == 0`` and ``dg_l == sum_{i>=l} sum_{j<l} dS_ij``, brute force for
the pruning boundaries, and the independent C restatement in ``fox_oracle.c``.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple, Union

import torch

__all__ = [
    "group_norm_gated_ref",
    "group_norm_ref",
    "qk_norm_threshold_ref",
    "token_shift_ref",
    "cumulative_log_decay",
    "auto_threshold",
    "forgetting_attention_ref",
    "forgetting_attention_ref_grads",
    "manual_backward",
    "find_start_index_ref",
    "find_end_index_ref",
]


def cumulative_log_decay(log_fgate: torch.Tensor, seq_start: Optional[torch.Tensor],
                         dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``c = cumsum(g)`` over the key axis with ``g[n < seq_start] = 0``.

    ``log_fgate`` is head-first ``(B, H, N)``.  Follows
    ``ops/forgetting_attention.py:117-127``.
    """
    g = log_fgate.to(dtype)
    if seq_start is not None:
        n = torch.arange(g.shape[-1], device=g.device)
        g = torch.where(n[None, None, :] < seq_start[:, None, None], torch.zeros((), dtype=dtype, device=g.device), g)
    return torch.cumsum(g, dim=-1)


def auto_threshold(q: torch.Tensor, k: torch.Tensor, sm_scale: float) -> torch.Tensor:
    """The ``"auto"`` threshold, ``(B, H)`` fp32, for head-first ``q``/``k``.

    ``ops/forgetting_attention.py:95-102``: row L2 norms are taken in the
    input dtype, the bound uses ``log(N)`` (keys, not queries) and a fixed
    tolerance of ``-10``.
    """
    n_keys = k.shape[2]
    max_q = torch.linalg.vector_norm(q, dim=-1).max(dim=-1).values
    max_k = torch.linalg.vector_norm(k, dim=-1).max(dim=-1).values
    ub = max_q * max_k * sm_scale
    return (-(2 * ub + math.log(n_keys)) - 10).float()


def _scores(q, k, c, seq_start, sm_scale, row_lo=None):
    """Masked scores ``(B, H, M, N)`` in the dtype of ``c``; -inf where invalid."""
    M, N = q.shape[2], k.shape[2]
    p_seq = N - M
    s = torch.matmul(q, k.transpose(2, 3)) * sm_scale
    s = s + (c[..., p_seq:, None] - c[..., None, :])
    i = torch.arange(M, device=q.device)[:, None]
    j = torch.arange(N, device=q.device)[None, :]
    valid = (j <= i + p_seq)[None, None]
    if seq_start is not None:
        valid = valid & (j[None, None] >= seq_start[:, None, None, None])
    if row_lo is not None:
        valid = valid & (j[None, None] >= row_lo[..., None])
    return s.masked_fill(~valid, float("-inf")), valid


def forgetting_attention_ref(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, log_fgate: torch.Tensor, *,
    head_first: bool = False, seq_start: Optional[torch.Tensor] = None,
    sm_scale: Optional[float] = None, compute_dtype: torch.dtype = torch.float32,
    return_lse: bool = False, zero_gates_before_seq_start: bool = True, row_lo: Optional[torch.Tensor] = None,
) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """Materialised-mask Forgetting Attention (differentiable).

    Mirrors ``ops/forgetting_attention.py:1380-1399`` with everything upcast
    to ``compute_dtype`` (fp32 by default, fp64 for the tightest checks).
    Rows with no valid column give ``out = 0`` and ``lse = -inf`` (``:1395-1397``
    and the kernel's epilogue ``:679-685``).  ``row_lo`` ``(B, H, M)`` optionally
    drops, per query row, every key column left of it: this is what Adaptive
    Computation Pruning does when it starts a query block's key loop at
    ``start_index`` (``:608-613``).  The result is returned in
    ``compute_dtype`` in the layout of the inputs.
    """
    if not head_first:
        q, k, v = (x.transpose(1, 2) for x in (q, k, v))
        log_fgate = log_fgate.transpose(1, 2)
    B, H, M, D = q.shape
    N = k.shape[2]
    assert M <= N and log_fgate.shape == (B, H, N)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    qf, kf, vf = (x.to(compute_dtype) for x in (q, k, v))
    c = cumulative_log_decay(log_fgate, seq_start if zero_gates_before_seq_start else None, compute_dtype)
    s, valid = _scores(qf, kf, c, seq_start, sm_scale, row_lo)
    any_valid = valid.any(dim=-1, keepdim=True)
    # softmax with the NaN -> 0 convention for empty rows
    s_safe = torch.where(any_valid, s, torch.zeros((), dtype=compute_dtype, device=s.device))
    p = torch.softmax(s_safe, dim=-1)
    p = torch.where(valid & any_valid, p, torch.zeros((), dtype=compute_dtype, device=s.device))
    out = torch.matmul(p, vf)
    if not head_first:
        out = out.transpose(1, 2)
    if return_lse:
        lse = torch.logsumexp(s_safe, dim=-1)
        lse = torch.where(any_valid[..., 0], lse, torch.full((), float("-inf"), dtype=compute_dtype, device=s.device))
        return out, lse
    return out


def forgetting_attention_ref_grads(
    q, k, v, log_fgate, dout, *, head_first=False, seq_start=None, sm_scale=None,
    compute_dtype=torch.float32, bh_chunk: int = 0,
):
    """``(out, dq, dk, dv, dlog_fgate)`` through ``torch.autograd``
    (``ops/forgetting_attention.py:1400-1404``), evaluated in chunks of
    ``bh_chunk`` heads per batch element so long sequences fit in memory.
    All results are in ``compute_dtype`` and in the layout of the inputs.
    """
    if not head_first:
        q, k, v, dout = (x.transpose(1, 2) for x in (q, k, v, dout))
        log_fgate = log_fgate.transpose(1, 2)
    B, H = q.shape[:2]
    step = bh_chunk if bh_chunk > 0 else H
    outs, dqs, dks, dvs, dgs = [], [], [], [], []
    for b in range(B):
        ro, rq, rk, rv, rg = [], [], [], [], []
        for h0 in range(0, H, step):
            sl = slice(h0, min(H, h0 + step))
            qq, kk, vv = (x[b:b + 1, sl].detach().to(compute_dtype).requires_grad_() for x in (q, k, v))
            gg = log_fgate[b:b + 1, sl].detach().to(compute_dtype).requires_grad_()
            ss = None if seq_start is None else seq_start[b:b + 1]
            o = forgetting_attention_ref(qq, kk, vv, gg, head_first=True, seq_start=ss, sm_scale=sm_scale,
                                         compute_dtype=compute_dtype)
            o.backward(dout[b:b + 1, sl].to(compute_dtype))
            ro.append(o.detach()); rq.append(qq.grad); rk.append(kk.grad); rv.append(vv.grad); rg.append(gg.grad)
            del o, qq, kk, vv, gg
        outs.append(torch.cat(ro, 1)); dqs.append(torch.cat(rq, 1)); dks.append(torch.cat(rk, 1))
        dvs.append(torch.cat(rv, 1)); dgs.append(torch.cat(rg, 1))
    out, dq, dk, dv, dg = (torch.cat(x, 0) for x in (outs, dqs, dks, dvs, dgs))
    if not head_first:
        out, dq, dk, dv = (x.transpose(1, 2) for x in (out, dq, dk, dv))
        dg = dg.transpose(1, 2)
    return out, dq, dk, dv, dg


def manual_backward(q, k, v, log_fgate, dout, *, seq_start=None, sm_scale=None,
                    compute_dtype=torch.float64, out_round_dtype: Optional[torch.dtype] = None,
                    row_lo: Optional[torch.Tensor] = None, col_end: Optional[torch.Tensor] = None,
                    kv_keep: Optional[torch.Tensor] = None):
    """The kernels' hand-derived backward, head-first tensors only.

    ``delta = rowsum(o * do)``            (``_bwd_preprocess`` ``:902-943``)
    ``p = exp(s - lse)``; ``dp = do v^T``; ``ds = p (dp - delta)``
    ``dv = p^T do``; ``dk = sm_scale ds^T q``   (``_bwd_kv_kernel`` ``:1073-1129``)
    ``dq = sm_scale ds k``                       (``_bwd_q_kernel`` ``:1290-1333``)
    ``dc[n] = -sum_i ds[i, n]`` (``:1122``) ``+ sum_j ds[n - P_SEQ, j]`` (``:1326, 1334-1344``)
    ``dg = reverse inclusive cumsum(dc)``        (``:390-392``)

    ``out_round_dtype`` optionally rounds ``o`` the way the operator stores it
    before ``delta`` is formed.

    Adaptive Computation Pruning restricts each of the three kernels to its own set of entries
    (``:600-613``, ``:1038-1049``, ``:1239-1261``):

    * ``row_lo`` ``(B, H, M)``: the forward (``out``, ``lse``) and the query-side backward (``dq`` and
      the row sums that enter ``dc``) see, for query row ``i``, only the keys ``j >= row_lo[i]``;
    * ``col_end`` ``(B, H, N)``: the key-side backward (``dk``, ``dv`` and the column sums that enter
      ``dc``) sees, for key ``j``, only the query rows ``i < col_end[j]``; ``kv_keep`` ``(B, H, M, N)``
      bool gives that set entry by entry instead.

    Probabilities are ``exp(s - lse)`` with the pruned forward's ``lse`` everywhere, also for entries the
    forward itself dropped (the key-side kernel rebuilds them from the stored ``lse``, ``:1079-1087``).
    Returns ``(out, lse, dq, dk, dv, dc, dg)``.
    """
    B, H, M, D = q.shape
    N = k.shape[2]
    p_seq = N - M
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    assert col_end is None or kv_keep is None
    qf, kf, vf, dof = (x.to(compute_dtype) for x in (q, k, v, dout))
    c = cumulative_log_decay(log_fgate, seq_start, compute_dtype)
    s, valid = _scores(qf, kf, c, seq_start, sm_scale)
    zero = torch.zeros((), dtype=compute_dtype, device=s.device)
    q_keep = valid
    if row_lo is not None:
        j = torch.arange(N, device=q.device)
        q_keep = valid & (j[None, None, None, :] >= row_lo[..., None])
    any_valid = q_keep.any(dim=-1, keepdim=True)
    s_fwd = torch.where(any_valid, s.masked_fill(~q_keep, float("-inf")), zero)
    lse = torch.logsumexp(s_fwd, dim=-1, keepdim=True)
    p = torch.where(valid & any_valid, torch.exp(torch.where(any_valid, s, zero) - lse), zero)
    del s_fwd
    out = torch.where(q_keep, p, zero) @ vf
    o_used = out if out_round_dtype is None else out.to(out_round_dtype).to(compute_dtype)
    delta = (o_used * dof).sum(-1, keepdim=True)
    ds = p * (dof @ vf.transpose(2, 3) - delta)
    ds_q = torch.where(q_keep, ds, zero)
    dq = sm_scale * (ds_q @ kf)
    drow = ds_q.sum(dim=3)
    del ds_q
    if col_end is not None:
        i = torch.arange(M, device=q.device)
        kv_keep = i[None, None, :, None] < col_end[:, :, None, :]
    if kv_keep is not None:
        ds = torch.where(kv_keep, ds, zero)
        p = torch.where(kv_keep, p, zero)
    elif row_lo is not None:
        raise ValueError("a pruned forward needs the key-side set as well (col_end or kv_keep)")
    dv = p.transpose(2, 3) @ dof
    dk = sm_scale * (ds.transpose(2, 3) @ qf)
    dc = -ds.sum(dim=2)
    dc[..., p_seq:] += drow
    dg = torch.flip(torch.cumsum(torch.flip(dc, dims=[-1]), dim=-1), dims=[-1])
    lse_out = torch.where(any_valid[..., 0], lse[..., 0], torch.full((), float("-inf"), dtype=compute_dtype, device=s.device))
    return out, lse_out, dq, dk, dv, dc, dg


def find_start_index_ref(c_row, threshold: float, M: int, N: int, block_m: int, block_n: int):
    """Pure-Python restatement of ``_find_start_index_kernel`` (``:695-745``) for one
    ``(b, h)`` row of ``c`` (a 1-D sequence of fp32 values): for each query block
    the first key column (a multiple of ``block_n``) that may not be pruned.
    """
    p_seq = N - M
    out = []
    start = 0
    c = [float(x) for x in c_row]
    f32 = torch.float32
    for m0 in range(0, M, block_m):
        c_out = c[p_seq + m0]
        while True:
            col = min(N - 1, start + block_n - 1)
            decay = float(torch.tensor(c_out, dtype=f32) - torch.tensor(c[col], dtype=f32))
            if decay < threshold:
                start += block_n
            else:
                break
        out.append(start)
    return out


def find_end_index_ref(c_row, threshold: float, M: int, N: int, block_m: int, block_n: int, tight: bool = False):
    """Pure-Python restatement of ``_find_end_index_kernel`` (``:747-795``): for each
    key block the first query row (a multiple of ``block_m``, clamped to ``M``) from
    which on the block may be pruned.  The reference reads ``c[row]`` without the
    ``P_SEQ`` offset (``:783,789``); ``tight=True`` applies the offset, which prunes
    more when ``M < N`` and is still safe.
    """
    p_seq = N - M if tight else 0
    out = []
    end = 0
    c = [float(x) for x in c_row]
    f32 = torch.float32
    for n0 in range(0, N, block_n):
        col = min(N - 1, n0 + block_n - 1)
        while end < M:
            row = min(end, M - 1) + p_seq
            decay = float(torch.tensor(c[row], dtype=f32) - torch.tensor(c[col], dtype=f32))
            if decay >= threshold:
                end = min(end + block_m, M)
            else:
                break
        out.append(end)
    return out


def token_shift_ref(x: torch.Tensor, prev_weight: torch.Tensor, curr_weight: torch.Tensor) -> torch.Tensor:
    """``x[b,t-1] * prev_weight[b,t] + x[b,t] * curr_weight[b,t]`` per head with ``x[b,-1] = 0``
    (reference ``token_shift.py:264-270``).  x: (B, T, H, D); weights: (B, T, H).  The sum is formed
    in the promoted dtype of x and the weights and cast back to x's dtype; differentiable."""
    x_prev = torch.roll(x, shifts=1, dims=1)
    keep = torch.ones(x.shape[1], dtype=torch.bool, device=x.device)
    keep[0] = False
    x_prev = torch.where(keep[None, :, None, None], x_prev, torch.zeros_like(x_prev))
    return (x_prev * prev_weight[..., None] + x * curr_weight[..., None]).to(x.dtype)


def group_norm_gated_ref(x: torch.Tensor, g: Optional[torch.Tensor], weight: torch.Tensor, num_groups: int,
                         eps: float = 1e-6, activation: str = "sigmoid", upcast: bool = True) -> torch.Tensor:
    """Per-group RMS norm with weight, times the gate activation (reference
    ``fuse_norm_gate.py:18-53`` with ``is_rms_norm=True``, no bias, no residual).  x, g: (..., G*D).
    ``activation="none"`` (``g`` unused) is the plain per-group RMS norm of ``layernorm.py:77-110``."""
    dtype = x.dtype
    if upcast and dtype in (torch.float16, torch.bfloat16):
        x, weight = x.float(), weight.float()
        g = g.float() if g is not None else None
    shape = x.shape
    xg = x.reshape(*shape[:-1], num_groups, shape[-1] // num_groups)
    wg = weight.reshape(num_groups, shape[-1] // num_groups)
    rstd = 1 / torch.sqrt(xg.square().mean(dim=-1, keepdim=True) + eps)
    out = (xg * rstd * wg).reshape(shape)
    if activation != "none":
        s = torch.sigmoid(g)
        out = out * (s if activation == "sigmoid" else g * s)
    return out.to(dtype)


def group_norm_ref(x: torch.Tensor, weight: torch.Tensor, num_groups: int, eps: float = 1e-5,
                   upcast: bool = True) -> torch.Tensor:
    """Plain per-group RMS norm with weight (reference ``layernorm.py:77-110`` with ``is_rms_norm=True``, no
    bias, no residual): what the FoX layer applies to queries and keys (``modeling_forgetting_transformer.py:
    258-265, 314-325``)."""
    return group_norm_gated_ref(x, None, weight, num_groups, eps, "none", upcast)


def qk_norm_threshold_ref(q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor, num_heads: int, head_dim: int,
                          seq_len: int, log_pruning_tolerance: float, share_param_across_head: bool = False) -> torch.Tensor:
    """Pruning threshold from the QK-norm weights (``modeling_forgetting_transformer.py:371-380``): after an RMS
    norm every query/key row has L2 norm at most ``max|w| * sqrt(D)``, so with ``sm_scale = 1/sqrt(D)`` the logits are
    bounded by ``max|w_q| * max|w_k| * sqrt(D)``; the threshold is ``-(2 * bound + log T) + tolerance``, one per head
    (a scalar when the heads share their weights)."""
    if share_param_across_head:
        bound = q_norm_weight.abs().max() * k_norm_weight.abs().max() * math.sqrt(head_dim)
    else:
        bound = (q_norm_weight.view(num_heads, head_dim).abs().max(dim=-1).values
                 * k_norm_weight.view(num_heads, head_dim).abs().max(dim=-1).values * math.sqrt(head_dim))
    return -(2 * bound + math.log(seq_len)) + log_pruning_tolerance
