"""Pins the oracle (oracle/fox_oracle.py and oracle/fox_oracle.c) on the CPU.

The reference ships no golden vectors for this path, so every oracle function is
pinned by something that does not share its code: a library routine it must
reduce to, a closed form, an identity of the mathematics, brute force, or the
other (independently written) restatement.
"""
import ctypes as C
import math
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import ROOT, make_inputs
from oracle import fox_oracle as O

torch.set_num_threads(4)


# --------------------------------------------------------------------------------------
# C restatement, loaded through ctypes
# --------------------------------------------------------------------------------------
@pytest.fixture(scope="session")
def c_oracle():
    so = ROOT / "oracle" / "libfox_oracle.so"
    if not so.exists() or so.stat().st_mtime < (ROOT / "oracle" / "fox_oracle.c").stat().st_mtime:
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    lib = C.CDLL(str(so))
    return lib


def _dptr(a):
    return a.ctypes.data_as(C.c_void_p)


def c_forward_backward(lib, q, k, v, g, do, seq_start, sm_scale):
    """Run the C restatement on head-first tensors; returns numpy arrays."""
    B, H, M, D = q.shape
    N = k.shape[2]
    qd, kd, vd, dod = (np.ascontiguousarray(x.double().numpy()) for x in (q, k, v, do))
    gf = np.ascontiguousarray(g.float().numpy())
    ss = None if seq_start is None else np.ascontiguousarray(seq_start.numpy().astype(np.int64))
    c = np.empty((B, H, N), np.float32)
    lib.fox_oracle_cumsum(_dptr(gf), None if ss is None else _dptr(ss), _dptr(c), B, H, N)
    out = np.empty((B, H, M, D)); lse = np.empty((B, H, M))
    lib.fox_oracle_fwd.argtypes = [C.c_void_p] * 5 + [C.c_double] + [C.c_int] * 5 + [C.c_void_p] * 2
    rc = lib.fox_oracle_fwd(_dptr(qd), _dptr(kd), _dptr(vd), _dptr(c), None if ss is None else _dptr(ss),
                            sm_scale, B, H, M, N, D, _dptr(out), _dptr(lse))
    assert rc == 0
    dq = np.empty_like(qd); dk = np.empty_like(kd); dv = np.empty_like(vd)
    dc = np.empty((B, H, N)); dg = np.empty((B, H, N))
    lib.fox_oracle_bwd.argtypes = [C.c_void_p] * 5 + [C.c_double] + [C.c_int] * 5 + [C.c_void_p] * 8
    rc = lib.fox_oracle_bwd(_dptr(qd), _dptr(kd), _dptr(vd), _dptr(c), None if ss is None else _dptr(ss), sm_scale,
                            B, H, M, N, D, _dptr(out), _dptr(lse), _dptr(dod), _dptr(dq), _dptr(dk), _dptr(dv),
                            _dptr(dc), _dptr(dg))
    assert rc == 0
    return dict(c=c, out=out, lse=lse, dq=dq, dk=dk, dv=dv, dc=dc, dg=dg)


# --------------------------------------------------------------------------------------
# forward: library pins
# --------------------------------------------------------------------------------------
@pytest.mark.parametrize("B,H,M,N,D,ss", [(2, 4, 256, 256, 64, None), (2, 2, 37, 101, 16, None), (3, 2, 50, 80, 32, [0, 17, 60]),
                                           (1, 1, 1, 33, 64, None)])
def test_forward_matches_sdpa_with_additive_mask(B, H, M, N, D, ss):
    q, k, v, g, _, seq = make_inputs(B, H, M, N, D, dtype=torch.float64, seed=1, seq_start=ss)
    sm = 0.37
    out, lse = O.forgetting_attention_ref(q, k, v, g, head_first=True, seq_start=seq, sm_scale=sm,
                                          compute_dtype=torch.float64, return_lse=True)
    # independent construction of the bias: explicit loops over the gate sums
    c = torch.zeros(B, H, N, dtype=torch.float64)
    for b in range(B):
        s0 = 0 if seq is None else int(seq[b])
        run = torch.zeros(H, dtype=torch.float64)
        for n in range(N):
            if n >= s0:
                run = run + g[b, :, n]
            c[b, :, n] = run
    P = N - M
    bias = torch.full((B, H, M, N), float("-inf"), dtype=torch.float64)
    for i in range(M):
        for b in range(B):
            s0 = 0 if seq is None else int(seq[b])
            lo, hi = s0, i + P
            if lo <= hi:
                bias[b, :, i, lo:hi + 1] = c[b, :, i + P, None] - c[b, :, lo:hi + 1]
    empty = torch.isinf(bias).all(-1)
    bias_safe = bias.clone()
    bias_safe[empty] = 0.0
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=bias_safe, scale=sm)
    ref[empty] = 0.0
    assert torch.allclose(out, ref, atol=1e-12, rtol=1e-10)
    ref_lse = torch.logsumexp(q @ k.transpose(2, 3) * sm + bias, dim=-1)
    assert torch.equal(torch.isinf(lse), empty)
    assert torch.allclose(lse[~empty], ref_lse[~empty], atol=1e-12, rtol=1e-10)
    assert (out[empty] == 0).all()


def test_zero_gates_reduce_to_plain_causal_attention():
    q, k, v, _, _, _ = make_inputs(2, 3, 64, 64, 32, dtype=torch.float64, seed=2)
    g = torch.zeros(2, 3, 64, dtype=torch.float64)
    out = O.forgetting_attention_ref(q, k, v, g, head_first=True, compute_dtype=torch.float64)
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert torch.allclose(out, ref, atol=1e-12)


def test_constant_gate_is_alibi():
    B, H, M, N, D = 1, 2, 40, 72, 16
    q, k, v, _, _, _ = make_inputs(B, H, M, N, D, dtype=torch.float64, seed=3)
    slope = 0.3
    g = torch.full((B, H, N), -slope, dtype=torch.float64)
    out = O.forgetting_attention_ref(q, k, v, g, head_first=True, compute_dtype=torch.float64)
    i = torch.arange(M)[:, None] + (N - M)
    j = torch.arange(N)[None, :]
    bias = torch.where(j <= i, -slope * (i - j).double(), torch.tensor(float("-inf"), dtype=torch.float64))
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=bias)
    assert torch.allclose(out, ref, atol=1e-12)


def test_layouts_agree():
    q, k, v, g, _, ss = make_inputs(2, 3, 20, 31, 16, dtype=torch.float64, seed=4, seq_start=[3, 0])
    a = O.forgetting_attention_ref(q, k, v, g, head_first=True, seq_start=ss, compute_dtype=torch.float64)
    b = O.forgetting_attention_ref(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), g.transpose(1, 2),
                                   head_first=False, seq_start=ss, compute_dtype=torch.float64)
    assert torch.equal(a, b.transpose(1, 2))


def test_gates_left_of_seq_start_do_not_matter():
    q, k, v, g, _, ss = make_inputs(2, 2, 24, 40, 16, dtype=torch.float64, seed=5, seq_start=[7, 19])
    a = O.forgetting_attention_ref(q, k, v, g, head_first=True, seq_start=ss, compute_dtype=torch.float64)
    b = O.forgetting_attention_ref(q, k, v, g, head_first=True, seq_start=ss, compute_dtype=torch.float64,
                                   zero_gates_before_seq_start=False)  # the reference's test oracle does not zero them (:1386)
    assert torch.allclose(a, b, atol=1e-12)


# --------------------------------------------------------------------------------------
# backward
# --------------------------------------------------------------------------------------
def test_gradcheck_fp64():
    q, k, v, g, _, ss = make_inputs(1, 2, 5, 8, 16, dtype=torch.float64, seed=6, seq_start=[2], requires_grad=True)
    fn = lambda q_, k_, v_, g_: O.forgetting_attention_ref(q_, k_, v_, g_, head_first=True, seq_start=ss, sm_scale=0.5,
                                                           compute_dtype=torch.float64)
    assert torch.autograd.gradcheck(fn, (q, k, v, g), eps=1e-6, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("M,N,ss", [(48, 48, None), (30, 77, None), (30, 77, [0, 50, 76]), (1, 19, None)])
def test_manual_backward_matches_autograd(M, N, ss):
    B = 3 if ss else 2
    q, k, v, g, do, seq = make_inputs(B, 2, M, N, 16, dtype=torch.float64, seed=7, seq_start=ss)
    out, dq, dk, dv, dg = O.forgetting_attention_ref_grads(q, k, v, g, do, head_first=True, seq_start=seq, sm_scale=0.7,
                                                           compute_dtype=torch.float64)
    mo, ml, mdq, mdk, mdv, mdc, mdg = O.manual_backward(q, k, v, g, do, seq_start=seq, sm_scale=0.7)
    for a, b in ((out, mo), (dq, mdq), (dk, mdk), (dv, mdv), (dg, mdg)):
        assert torch.allclose(a, b, atol=1e-11, rtol=1e-9)
    # identities of the mathematics
    assert mdc.sum(-1).abs().max() < 1e-10          # sum_n dc_n = 0
    if seq is not None:
        for b in range(B):
            assert mdg[b, :, : int(seq[b]) + 1].abs().max() < 1e-10   # dg_l = 0 for l <= seq_start
    else:
        assert mdg[..., 0].abs().max() < 1e-10


@pytest.mark.parametrize("M,N,ss", [(40, 40, None), (24, 61, [0, 30])])
def test_pruned_manual_backward(M, N, ss):
    """The three entry sets of a pruned backward.  (1) When the key side keeps exactly the entries the forward
    kept, everything is the gradient of the pruned forward: autograd through ``forgetting_attention_ref(row_lo=...)``
    pins out, dq, dk, dv and dg.  (2) A key-side set of its own (``col_end``): dk, dv and dc from element loops that
    rebuild every probability from the pruned forward's lse."""
    B, H, D, sm = (2 if ss else 1), 2, 8, 0.6
    q, k, v, g, do, seq = make_inputs(B, H, M, N, D, dtype=torch.float64, seed=21, seq_start=ss, gate_mean=0.5)
    P = N - M
    gen = torch.Generator().manual_seed(3)
    # per-row lower bounds, block-shaped as the kernels' are (8 rows share a bound, a multiple of 4, never right of the row)
    blk = torch.randint(0, N // 4 + 1, (B, H, (M + 7) // 8), generator=gen) * 4
    row_lo = torch.minimum(blk.repeat_interleave(8, dim=-1)[..., :M], (torch.arange(M) + P) // 4 * 4)
    qq, kk, vv, gg = (x.clone().requires_grad_() for x in (q, k, v, g))
    out = O.forgetting_attention_ref(qq, kk, vv, gg, head_first=True, seq_start=seq, sm_scale=sm, compute_dtype=torch.float64,
                                     row_lo=row_lo)
    out.backward(do)
    i, j = torch.arange(M)[:, None], torch.arange(N)[None, :]
    kept = (j <= i + P)[None, None] & (j[None, None] >= row_lo[..., None])
    if seq is not None:
        kept = kept & (j[None, None] >= seq[:, None, None, None])
    mo, ml, mdq, mdk, mdv, mdc, mdg = O.manual_backward(q, k, v, g, do, seq_start=seq, sm_scale=sm, row_lo=row_lo, kv_keep=kept)
    for name, a, b in (("out", out, mo), ("dq", qq.grad, mdq), ("dk", kk.grad, mdk), ("dv", vv.grad, mdv), ("dg", gg.grad, mdg)):
        assert torch.allclose(a.detach(), b, atol=1e-11, rtol=1e-9), name
    full = O.forgetting_attention_ref(q, k, v, g, head_first=True, seq_start=seq, sm_scale=sm, compute_dtype=torch.float64)
    assert (full - mo).abs().max() > 1e-4          # the bounds did change the result
    # (2) key-side bound per key, block-shaped, independent of the forward's set
    col_end = (torch.randint(0, M // 8 + 2, (B, H, (N + 3) // 4), generator=gen) * 8).clamp(max=M).repeat_interleave(4, dim=-1)[..., :N]
    _, ml2, mdq2, mdk2, mdv2, mdc2, _ = O.manual_backward(q, k, v, g, do, seq_start=seq, sm_scale=sm, row_lo=row_lo, col_end=col_end)
    assert torch.equal(ml, ml2) and torch.equal(mdq, mdq2)   # the query side does not see the key side's set
    c = O.cumulative_log_decay(g, seq, torch.float64)
    delta = (mo * do).sum(-1)
    for b in range(B):
        s0 = 0 if seq is None else int(seq[b])
        for h in range(H):
            dk_ = torch.zeros(N, D, dtype=torch.float64); dv_ = torch.zeros(N, D, dtype=torch.float64)
            dc_ = torch.zeros(N, dtype=torch.float64)
            for n in range(N):
                for m in range(M):
                    if n > m + P or n < s0 or ml[b, h, m] == float("-inf"):
                        continue
                    p = math.exp(float(q[b, h, m] @ k[b, h, n]) * sm + float(c[b, h, m + P] - c[b, h, n]) - float(ml[b, h, m]))
                    ds = p * (float(do[b, h, m] @ v[b, h, n]) - float(delta[b, h, m]))
                    if n >= row_lo[b, h, m]:
                        dc_[m + P] += ds
                    if m < col_end[b, h, n]:
                        dv_[n] += p * do[b, h, m]
                        dk_[n] += sm * ds * q[b, h, m]
                        dc_[n] -= ds
            assert torch.allclose(mdk2[b, h], dk_, atol=1e-10) and torch.allclose(mdv2[b, h], dv_, atol=1e-10)
            assert torch.allclose(mdc2[b, h], dc_, atol=1e-10)


def test_gate_gradient_closed_form():
    """dg_l = sum over (rows at or after l) x (columns before l) of dS: only score
    pairs that straddle position l contribute."""
    B, H, M, N, D = 1, 2, 12, 20, 16
    q, k, v, g, do, _ = make_inputs(B, H, M, N, D, dtype=torch.float64, seed=8)
    P = N - M
    _, _, _, _, _, _, mdg = O.manual_backward(q, k, v, g, do, sm_scale=0.4)
    # dS by brute force
    c = torch.cumsum(g, -1)
    s = q @ k.transpose(2, 3) * 0.4 + (c[..., P:, None] - c[..., None, :])
    i = torch.arange(M)[:, None] + P
    j = torch.arange(N)[None, :]
    s = s.masked_fill(j > i, float("-inf"))
    p = torch.softmax(s, -1)
    dp = do @ v.transpose(2, 3)
    ds = p * (dp - (p * dp).sum(-1, keepdim=True))
    for l in range(N):
        rows = (torch.arange(M) + P) >= l
        expect = ds[:, :, rows][..., :l].sum((-1, -2))
        assert torch.allclose(mdg[..., l], expect, atol=1e-11)


# --------------------------------------------------------------------------------------
# the two restatements must agree
# --------------------------------------------------------------------------------------
@pytest.mark.parametrize("B,H,M,N,D,ss", [(2, 4, 256, 256, 64, None), (2, 2, 61, 130, 32, [5, 100]), (1, 2, 1, 40, 16, None)])
def test_c_restatement_matches_torch_restatement(c_oracle, B, H, M, N, D, ss):
    q, k, v, g, do, seq = make_inputs(B, H, M, N, D, dtype=torch.float32, seed=9, seq_start=ss)
    sm = 1.0 / math.sqrt(D)
    r = c_forward_backward(c_oracle, q, k, v, g, do, seq, sm)
    # cumsum: same fp32 running sum as torch on the CPU
    c_t = O.cumulative_log_decay(g, seq, torch.float32)
    assert np.allclose(r["c"], c_t.numpy(), atol=2e-5, rtol=1e-6)
    g64 = torch.from_numpy(r["c"]).double()
    g64 = torch.diff(g64, dim=-1, prepend=torch.zeros(B, H, 1, dtype=torch.float64))  # gates that reproduce the C cumsum exactly
    out, lse = O.forgetting_attention_ref(q, k, v, g64, head_first=True, seq_start=None if seq is None else seq,
                                          sm_scale=sm, compute_dtype=torch.float64, return_lse=True,
                                          zero_gates_before_seq_start=False)
    assert np.allclose(r["out"], out.numpy(), atol=1e-9)
    fin = ~torch.isinf(lse)
    assert np.array_equal(np.isinf(r["lse"]), ~fin.numpy())
    assert np.allclose(r["lse"][fin.numpy()], lse[fin].numpy(), atol=1e-9)
    _, dq, dk, dv, dg = O.forgetting_attention_ref_grads(q, k, v, g64, do, head_first=True, seq_start=seq, sm_scale=sm,
                                                         compute_dtype=torch.float64)
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert np.allclose(r[name], t.numpy(), atol=1e-9), name
    # gate gradient: compare where gates matter (right of seq_start); left of it both are 0
    assert np.allclose(r["dg"], dg.numpy(), atol=1e-8)
    assert abs(r["dc"].sum(-1)).max() < 1e-9


# --------------------------------------------------------------------------------------
# Adaptive Computation Pruning bounds
# --------------------------------------------------------------------------------------
def _brute_start(c, thr, M, N, bm, bn):
    """First key block of each query block that holds an entry with decay >= thr (causal part only)."""
    P = N - M
    out = []
    for m0 in range(0, M, bm):
        rows = range(m0, min(M, m0 + bm))
        first = None
        for t in range(0, (P + m0) // bn + 1):
            cols = range(t * bn, min(N, t * bn + bn))
            if any(np.float32(c[P + i]) - np.float32(c[j]) >= np.float32(thr) for i in rows for j in cols):
                first = t
                break
        out.append((first if first is not None else (P + m0) // bn) * bn)
    return out


@pytest.mark.parametrize("M,N,bm,bn,thr", [(64, 64, 16, 8, -3.0), (50, 120, 16, 16, -6.0), (128, 128, 128, 64, -10.0),
                                            (33, 97, 8, 32, -1.0), (40, 40, 8, 8, 0.0)])
def test_start_index_scan_is_exact(c_oracle, M, N, bm, bn, thr):
    g = torch.Generator().manual_seed(M * 1000 + N)
    c = torch.cumsum(F.logsigmoid(torch.randn(N, generator=g) * 2 - 1), 0).float()
    py = O.find_start_index_ref(c, thr, M, N, bm, bn)
    out = np.zeros(len(py), np.int64)
    cn = np.ascontiguousarray(c.numpy())
    c_oracle.fox_oracle_find_start_index.argtypes = [C.c_void_p, C.c_float] + [C.c_int] * 4 + [C.c_void_p]
    c_oracle.fox_oracle_find_start_index(_dptr(cn), thr, M, N, bm, bn, _dptr(out))
    assert list(out) == py
    # because c is non-increasing the scan equals brute force over every entry of every rectangle
    assert py == _brute_start(cn, thr, M, N, bm, bn)
    # safety: everything left of the bound is below the threshold
    P = N - M
    for blk, start in enumerate(py):
        for i in range(blk * bm, min(M, blk * bm + bm)):
            for j in range(0, min(start, P + i + 1)):
                assert cn[P + i] - cn[j] < thr


@pytest.mark.parametrize("M,N,bm,bn,thr", [(64, 64, 16, 8, -3.0), (50, 120, 16, 16, -6.0), (128, 128, 32, 128, -10.0)])
def test_end_index_scan_is_safe(c_oracle, M, N, bm, bn, thr):
    g = torch.Generator().manual_seed(M * 77 + N)
    c = torch.cumsum(F.logsigmoid(torch.randn(N, generator=g) * 2 - 1), 0).float()
    cn = np.ascontiguousarray(c.numpy())
    P = N - M
    c_oracle.fox_oracle_find_end_index.argtypes = [C.c_void_p, C.c_float] + [C.c_int] * 5 + [C.c_void_p]
    for tight in (0, 1):
        py = O.find_end_index_ref(c, thr, M, N, bm, bn, tight=bool(tight))
        out = np.zeros(len(py), np.int64)
        c_oracle.fox_oracle_find_end_index(_dptr(cn), thr, M, N, bm, bn, tight, _dptr(out))
        assert list(out) == py
        for blk, end in enumerate(py):
            for j in range(blk * bn, min(N, blk * bn + bn)):
                for i in range(end, M):
                    if j <= P + i:
                        assert cn[P + i] - cn[j] < thr
    loose = O.find_end_index_ref(c, thr, M, N, bm, bn, tight=False)
    tight_ = O.find_end_index_ref(c, thr, M, N, bm, bn, tight=True)
    assert all(t <= l for t, l in zip(tight_, loose))   # the reference's bound only ever prunes less
    # minimality of the tight form, by brute force over every entry of every (query block x key block) rectangle
    # (causal mask ignored, as in the scan): `end` is the end of the last query block that still holds an entry at or
    # above the threshold, and never moves back from one key block to the next.  An off-by-one in either direction
    # (a block too many kept, or one too many dropped) fails here.
    floor = 0
    for blk, end in enumerate(tight_):
        cols = range(blk * bn, min(N, blk * bn + bn))
        exact = floor
        for e0 in range(0, M, bm):
            if any(cn[P + i] - cn[j] >= np.float32(thr) for i in range(e0, min(M, e0 + bm)) for j in cols):
                exact = max(exact, min(M, e0 + bm))
        assert end == exact, (blk, end, exact)
        floor = end


def test_pruned_mass_is_bounded_by_the_auto_threshold():
    """With thr = -(2 ub + log N) - 10 the attention mass of pruned entries is <= e^-10 per row."""
    B, H, T, D = 1, 2, 96, 16
    q, k, v, g, _, _ = make_inputs(B, H, T, T, D, dtype=torch.float64, seed=11, gate_mean=-1.0, gate_std=2.0)
    sm = 1 / math.sqrt(D)
    thr = O.auto_threshold(q, k, sm).double()
    c = torch.cumsum(g, -1)
    decay = c[..., :, None] - c[..., None, :]
    s = q @ k.transpose(2, 3) * sm + decay
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    s = s.masked_fill(~mask, float("-inf"))
    p = torch.softmax(s, -1)
    pruned = (decay < thr[..., None, None]) & mask
    assert pruned.any()
    assert (p * pruned).sum(-1).max() <= math.exp(-10)
    out_full = p @ v
    out_pruned = (p * ~pruned) @ v
    assert (out_full - out_pruned).abs().max() <= 2 * math.exp(-10) * v.abs().max()


def test_auto_threshold_closed_form():
    """README.md:196-209 of the reference states the same recipe with explicit norms."""
    q, k, _, _, _, _ = make_inputs(2, 3, 17, 29, 32, dtype=torch.float32, seed=12)
    sm = 1 / math.sqrt(32)
    thr = O.auto_threshold(q, k, sm)
    qn = q.double().pow(2).sum(-1).sqrt().amax(-1)
    kn = k.double().pow(2).sum(-1).sqrt().amax(-1)
    expect = -(2 * qn * kn / math.sqrt(32) + math.log(29)) - 10
    assert torch.allclose(thr.double(), expect, atol=1e-4)


# --------------------------------------------------------------------------------------
# committed golden vectors
# --------------------------------------------------------------------------------------
def test_golden_fixture_is_reproduced():
    data = np.load(ROOT / "tests" / "golden" / "c1_b2_t256_h4_d64.npz")
    q, k, v, g = (torch.from_numpy(data[n]) for n in ("q", "k", "v", "log_fgate"))
    out, lse = O.forgetting_attention_ref(q, k, v, g, sm_scale=1 / 8, return_lse=True)
    assert np.allclose(out.numpy(), data["out"], atol=1e-6)
    assert np.allclose(lse.numpy(), data["lse"], atol=1e-5)
    # and against the other restatement, which shares no code with the one that wrote the file
    ref = F.scaled_dot_product_attention
    c = torch.cumsum(g.transpose(1, 2).double(), -1)
    T = q.shape[1]
    bias = (c[..., :, None] - c[..., None, :]).masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float("-inf"))
    o2 = ref(q.transpose(1, 2).double(), k.transpose(1, 2).double(), v.transpose(1, 2).double(), attn_mask=bias, scale=1 / 8)
    assert np.allclose(o2.transpose(1, 2).numpy(), data["out"], atol=1e-5)


# --------------------------------------------------------------------------------------
# token shift
# --------------------------------------------------------------------------------------
def _shift_inputs(B=2, T=7, H=3, D=4, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, T, H, D, generator=g, dtype=dtype)
    curr = torch.rand(B, T, H, generator=g, dtype=dtype)
    prev = torch.rand(B, T, H, generator=g, dtype=dtype)
    return x, prev, curr


def test_token_shift_special_cases():
    x, prev, curr = _shift_inputs()
    one, zero = torch.ones_like(curr), torch.zeros_like(curr)
    assert torch.equal(O.token_shift_ref(x, zero, one), x)                      # identity
    shifted = O.token_shift_ref(x, one, zero)                                    # pure shift by one step
    assert torch.equal(shifted[:, 1:], x[:, :-1]) and shifted[:, 0].abs().max() == 0
    # explicit loop over every element
    out = O.token_shift_ref(x, prev, curr)
    B, T, H, D = x.shape
    for b in range(B):
        for t in range(T):
            for h in range(H):
                want = x[b, t, h] * curr[b, t, h] + (x[b, t - 1, h] * prev[b, t, h] if t > 0 else 0.0)
                assert torch.allclose(out[b, t, h], want, rtol=1e-14, atol=0)
    # linear in x
    x2, _, _ = _shift_inputs(seed=1)
    assert torch.allclose(O.token_shift_ref(2.0 * x - x2, prev, curr), 2.0 * out - O.token_shift_ref(x2, prev, curr), atol=1e-12)


def test_token_shift_gradcheck_and_c_restatement(c_oracle):
    x, prev, curr = _shift_inputs(B=2, T=9, H=2, D=8)
    x, prev, curr = (t.requires_grad_() for t in (x, prev, curr))
    assert torch.autograd.gradcheck(O.token_shift_ref, (x, prev, curr), eps=1e-6, atol=1e-6)
    g = torch.Generator().manual_seed(9)
    dout = torch.randn(x.shape, generator=g, dtype=torch.float64)
    out = O.token_shift_ref(x, prev, curr)
    dx, dprev, dcurr = torch.autograd.grad(out, (x, prev, curr), dout)
    B, T, H, D = x.shape
    xn, pn, cn, gn = (t.detach().numpy().copy() for t in (x, prev, curr, dout))
    out_c, dx_c = np.empty_like(xn), np.empty_like(xn)
    dp_c, dc_c = np.empty_like(pn), np.empty_like(pn)
    c_oracle.fox_oracle_token_shift_fwd(_dptr(xn), _dptr(pn), _dptr(cn), _dptr(out_c), B, T, H, D)
    c_oracle.fox_oracle_token_shift_bwd(_dptr(xn), _dptr(pn), _dptr(cn), _dptr(gn), _dptr(dx_c), _dptr(dp_c), _dptr(dc_c),
                                        B, T, H, D)
    for got, want in ((out_c, out), (dx_c, dx), (dp_c, dprev), (dc_c, dcurr)):
        assert np.allclose(got, want.detach().numpy(), rtol=1e-12, atol=1e-12)


# --------------------------------------------------------------------------------------
# gated per-group RMS norm
# --------------------------------------------------------------------------------------
@pytest.mark.parametrize("activation", ["sigmoid", "swish"])
def test_group_norm_gated_against_library_rms_norm_and_c(c_oracle, activation):
    R, G, D, eps = 11, 3, 8, 1e-5
    gen = torch.Generator().manual_seed(13)
    x = torch.randn(R, G * D, generator=gen, dtype=torch.float64)
    g = torch.randn(R, G * D, generator=gen, dtype=torch.float64)
    w = torch.rand(G * D, generator=gen, dtype=torch.float64) + 0.5
    out = O.group_norm_gated_ref(x, g, w, G, eps, activation)
    # independent pin: the library's rms_norm applied group by group, then the gate
    want = torch.cat([F.rms_norm(x[:, h * D:(h + 1) * D], (D,), w[h * D:(h + 1) * D], eps) for h in range(G)], dim=1)
    want = want * (torch.sigmoid(g) if activation == "sigmoid" else F.silu(g))
    assert torch.allclose(out, want, rtol=1e-12, atol=1e-12)
    # autograd of the restatement: gradcheck, then the C loops for forward and backward
    xr, gr, wr = (t.clone().requires_grad_() for t in (x, g, w))
    assert torch.autograd.gradcheck(lambda a, b, c: O.group_norm_gated_ref(a, b, c, G, eps, activation), (xr, gr, wr),
                                    eps=1e-6, atol=1e-6)
    dy = torch.randn(R, G * D, generator=gen, dtype=torch.float64)
    dx, dg, dw = torch.autograd.grad(O.group_norm_gated_ref(xr, gr, wr, G, eps, activation), (xr, gr, wr), dy)
    xn, gn, wn, dyn = (t.numpy().copy() for t in (x, g, w, dy))
    y_c, dx_c, dg_c, dw_c = np.empty_like(xn), np.empty_like(xn), np.empty_like(xn), np.empty_like(wn)
    swish = int(activation == "swish")
    c_oracle.fox_oracle_norm_gate_fwd(_dptr(xn), _dptr(gn), _dptr(wn), _dptr(y_c), C.c_int64(R), G, D, C.c_double(eps), swish)
    c_oracle.fox_oracle_norm_gate_bwd(_dptr(xn), _dptr(gn), _dptr(wn), _dptr(dyn), _dptr(dx_c), _dptr(dg_c), _dptr(dw_c),
                                      C.c_int64(R), G, D, C.c_double(eps), swish)
    for got, ref in ((y_c, out), (dx_c, dx), (dg_c, dg), (dw_c, dw)):
        assert np.allclose(got, ref.detach().numpy(), rtol=1e-10, atol=1e-12)


def test_group_norm_against_library_rms_norm_and_c(c_oracle):
    """The plain (ungated) per-group RMS norm applied to queries and keys."""
    R, G, D, eps = 9, 4, 8, 1e-5
    gen = torch.Generator().manual_seed(14)
    x = torch.randn(R, G * D, generator=gen, dtype=torch.float64)
    w = torch.rand(G * D, generator=gen, dtype=torch.float64) + 0.5
    out = O.group_norm_ref(x, w, G, eps)
    want = torch.cat([F.rms_norm(x[:, h * D:(h + 1) * D], (D,), w[h * D:(h + 1) * D], eps) for h in range(G)], dim=1)
    assert torch.allclose(out, want, rtol=1e-12, atol=1e-12)
    # one group = the whole row: the textbook RMS norm
    assert torch.allclose(O.group_norm_ref(x, w, 1, eps), F.rms_norm(x, (G * D,), w, eps), rtol=1e-12, atol=1e-12)
    xr, wr = x.clone().requires_grad_(), w.clone().requires_grad_()
    assert torch.autograd.gradcheck(lambda a, b: O.group_norm_ref(a, b, G, eps), (xr, wr), eps=1e-6, atol=1e-6)
    dy = torch.randn(R, G * D, generator=gen, dtype=torch.float64)
    dx, dw = torch.autograd.grad(O.group_norm_ref(xr, wr, G, eps), (xr, wr), dy)
    xn, wn, dyn = (t.numpy().copy() for t in (x, w, dy))
    y_c, dx_c, dw_c = np.empty_like(xn), np.empty_like(xn), np.empty_like(wn)
    c_oracle.fox_oracle_norm_gate_fwd(_dptr(xn), None, _dptr(wn), _dptr(y_c), C.c_int64(R), G, D, C.c_double(eps), 2)
    c_oracle.fox_oracle_norm_gate_bwd(_dptr(xn), None, _dptr(wn), _dptr(dyn), _dptr(dx_c), None, _dptr(dw_c),
                                      C.c_int64(R), G, D, C.c_double(eps), 2)
    for got, ref in ((y_c, out), (dx_c, dx), (dw_c, dw)):
        assert np.allclose(got, ref.detach().numpy(), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("share", [False, True])
def test_qk_norm_threshold_bounds_every_logit(share):
    """The threshold is -(2*bound + log T) + tolerance where `bound` must dominate every |q.k|/sqrt(D) of
    RMS-normalised rows (eps > 0 only shrinks them): brute force over random rows and adversarial ones."""
    H, D, T, tol = 3, 16, 50, -7.5
    gen = torch.Generator().manual_seed(15)
    wq = torch.randn(D if share else H * D, generator=gen, dtype=torch.float64)
    wk = torch.randn(D if share else H * D, generator=gen, dtype=torch.float64)
    thr = O.qk_norm_threshold_ref(wq, wk, H, D, T, tol, share)
    assert thr.shape == (() if share else (H,))
    bound = (-(thr - tol) - math.log(T)) / 2
    x = torch.randn(200, H * D, generator=gen, dtype=torch.float64) * 10
    # adversarial rows: all the mass on the coordinate with the largest |w|
    for h in range(H):
        wqh = wq if share else wq[h * D:(h + 1) * D]
        x[h, h * D:(h + 1) * D] = 0.0
        x[h, h * D + int(wqh.abs().argmax())] = 5.0
    wq_full = wq.repeat(H) if share else wq
    wk_full = wk.repeat(H) if share else wk
    qn = O.group_norm_ref(x, wq_full, H, 0.0).view(-1, H, D)
    kn = O.group_norm_ref(x, wk_full, H, 0.0).view(-1, H, D)
    logits = torch.einsum("ihd,jhd->hij", qn, kn) / math.sqrt(D)
    worst = logits.abs().amax(dim=(1, 2))
    assert (worst <= (bound if not share else bound.expand(H)) * (1 + 1e-12)).all()
    # the closed form itself, head by head
    for h in range(H):
        a = (wq if share else wq[h * D:(h + 1) * D]).abs().max()
        b = (wk if share else wk[h * D:(h + 1) * D]).abs().max()
        want = -(2 * a * b * math.sqrt(D) + math.log(T)) + tol
        assert torch.allclose(thr if share else thr[h], want, rtol=1e-14, atol=0)
