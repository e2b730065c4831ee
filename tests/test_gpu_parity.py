"""GPU parity tests: the HIP kernels, called through the C ABI by the Python
operator, against the oracle on the same seeded inputs.

Tolerance (bf16): max |x - ref| <= 2e-2 * max|ref| for out, dq, dk, dv, dlog_fgate, the bound the benchmark
configurations are judged by ("max-abs error 2e-2 relative to output scale"; the scale is the reference's own
maximum, without a floor, unless the reference is exactly zero everywhere -- a single valid key per row gives
dS = 0 exactly), and row by row for out, dq, dk, dv: |x - ref| <= 2e-2 * max|ref row| + 6e-3 * max|ref|, so
a wrong row of small magnitude cannot hide behind a large one.  dlog_fgate is a reverse running sum whose early
entries dominate its scale, so its steps dc[n] = dlog_fgate[n] - dlog_fgate[n+1] are held to the same tensor-wide
bar as well ("dc_steps").  The measured ratios are printed at the end of the run.  The reference's own grid
(fp16) uses its own bound, atol = 1e-2 (ops/forgetting_attention.py:1416-1425).
"""
import ctypes as C
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import REL_TOL, ROOT, assert_parity, make_inputs, rel_err
from oracle import fox_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from forgetting_transformer import forgetting_attention
    from forgetting_transformer.ops import _lib
    _lib.load()  # fails loudly when the HIP library is missing
    return forgetting_attention


def pruned_reference(q, k, v, g, do, ss, sm_scale, head_first, records, D):
    """(out, dq, dk, dv, dlog_fgate) of the oracle restricted to exactly the entries the kernels report having
    visited: the forward's and the dQ kernel's first key block per query block, the dK/dV kernel's end row per 64
    keys (the records of one forward + backward under record_pruning_bounds).  The oracle never guesses a bound: a
    kernel that visits a block more or a block less than it reports, or reports a bound the scans do not give
    (checked bit for bit in test_backward_pruning_bounds_match_the_scans), fails at the standard bar."""
    from forgetting_transformer.ops import _lib
    bm, bn, _, _ = _lib.tile_config(D)
    fwd = [r for r in records if "fwd_first_block" in r]
    bwd = [r for r in records if "kv_end_row" in r]
    assert len(fwd) == 1 and len(bwd) == 1, "one forward and one backward were recorded"
    assert torch.equal(fwd[0]["fwd_first_block"], bwd[0]["dq_first_block"]), "forward and dQ kernel use the same bound"
    if not head_first:
        q, k, v, do = (x.transpose(1, 2) for x in (q, k, v, do))
        g = g.transpose(1, 2)
    M, N = q.shape[2], k.shape[2]
    row_lo = (fwd[0]["fwd_first_block"].long() * bn).repeat_interleave(bm, dim=-1)[..., :M]
    kv_end = bwd[0]["kv_end_row"].long()
    assert (kv_end >= 0).all() and (kv_end <= M).all(), "every 64-key unit was handled by exactly one dK/dV workgroup"
    col_end = kv_end.repeat_interleave(64, dim=-1)[..., :N]
    outs = []
    for b in range(q.shape[0]):   # batch by batch: the masked oracle keeps several (H, M, N) fp32 matrices alive
        sl = slice(b, b + 1)
        o, _, dq, dk, dv, _, dg = O.manual_backward(q[sl], k[sl], v[sl], g[sl], do[sl], seq_start=None if ss is None else ss[sl],
                                                    sm_scale=sm_scale, compute_dtype=torch.float32, out_round_dtype=q.dtype,
                                                    row_lo=row_lo[sl], col_end=col_end[sl])
        # The gate gradient up to and including seq_start (position 0 without padding) is sum_n dc_n: zero in exact
        # arithmetic (those gates shift every c_j alike), and the operator stores an exact zero there.  Under pruning
        # the row and column sums of dS run over different sets and no longer cancel, so the restated arithmetic (like
        # the reference's reverse cumsum, :390-392) leaves their difference in those positions; the comparison takes
        # the operator's convention.
        dg[..., : (0 if ss is None else int(ss[b])) + 1] = 0
        outs.append((o, dq, dk, dv, dg))
    out, dq, dk, dv, dg = (torch.cat(x, 0) for x in zip(*outs))
    if not head_first:
        out, dq, dk, dv = (x.transpose(1, 2) for x in (out, dq, dk, dv))
        dg = dg.transpose(1, 2)
    return out, dq, dk, dv, dg


def run_case(fa, B, H, M, N, D, *, dtype=torch.bfloat16, head_first=True, thr=None, sm_scale=None, tol=REL_TOL,
             atol=None, masked=None, floor=0.0, context=None, **kw):
    """One forward + backward against the oracle.  Without a threshold the oracle is autograd through the reference's
    materialised-mask attention.  With one, the default (``masked``) is the oracle restricted to the kernels' own
    reported pruning sets, at the same bar: what a threshold prunes changes the result, and the comparison follows it.
    ``masked=False`` compares a pruned run with the unpruned oracle, for thresholds so low that nothing visible is lost."""
    from forgetting_transformer.ops.forgetting_attention import record_pruning_bounds
    q, k, v, g, do, ss = make_inputs(B, H, M, N, D, dtype=dtype, device="cuda", head_first=head_first, **kw)
    masked = thr is not None if masked is None else masked
    q, k, v, g = (x.requires_grad_() for x in (q, k, v, g))
    with record_pruning_bounds() as records:
        out = fa(q, k, v, g, head_first=head_first, seq_start=ss, sm_scale=sm_scale, adaptive_threshold=thr)
        assert out.shape == q.shape and out.dtype == dtype
        out.backward(do)
    if masked:
        ref = pruned_reference(q.detach(), k.detach(), v.detach(), g.detach(), do, ss, sm_scale, head_first, records, D)
    else:
        ref = O.forgetting_attention_ref_grads(q.detach(), k.detach(), v.detach(), g.detach(), do, head_first=head_first,
                                               seq_start=ss, sm_scale=sm_scale, bh_chunk=4)
    got = (out, q.grad, k.grad, v.grad, g.grad)
    for name, x, r in zip(("out", "dq", "dk", "dv", "dlog_fgate"), got, ref):
        assert torch.isfinite(x).all(), name
        if atol is not None:
            err = (x.float() - r.float()).abs().max().item()
            assert err <= atol, f"{name}: abs err {err:.3e} > {atol}"
        else:
            assert_parity(name, x, r, tol=tol, rows=name != "dlog_fgate", floor=floor, context=context)
    if atol is None and tol == REL_TOL and floor == 0.0:
        assert_parity("dc_steps", gate_grad_steps(g.grad, head_first), gate_grad_steps(ref[4], head_first), rows=False)
    return got, ref, ss


def gate_grad_steps(dg, head_first):
    """dc[n] = dg[n] - dg[n+1] (dc[N-1] = dg[N-1]): the gradient with respect to the cumulative sum, position by
    position.  dlog_fgate is its reverse running sum, whose large early entries set the scale of the tensor-wide bound;
    the steps put every position on the scale of its own row and column sums of dS."""
    dg = dg.float()
    axis = -1 if head_first else 1
    last = dg.narrow(axis, dg.shape[axis] - 1, 1)
    return torch.cat([-dg.diff(dim=axis), last], dim=axis)


# --------------------------------------------------------------------------------------
# committed golden vectors
# --------------------------------------------------------------------------------------
def test_golden_forward_backward(fa):
    d = np.load(ROOT / "tests" / "golden" / "bwd_b2_h2_m72_n200_d32.npz")
    t = lambda n, dt=torch.bfloat16: torch.from_numpy(d[n]).to("cuda").to(dt)
    q, k, v, do = t("q"), t("k"), t("v"), t("dout")
    g = t("log_fgate", torch.float32)
    ss = torch.from_numpy(d["seq_start"]).cuda()
    q, k, v, g = (x.requires_grad_() for x in (q, k, v, g))
    out = fa(q, k, v, g, head_first=True, seq_start=ss, sm_scale=0.25)
    out.backward(do)
    for name, x in (("out", out), ("dq", q.grad), ("dk", k.grad), ("dv", v.grad), ("dlog_fgate", g.grad)):
        assert_parity(name, x, torch.from_numpy(d[name]).cuda(), rows=name != "dlog_fgate")
    # batch row 1 starts at key 150 = query 22: queries 0..21 attend to nothing
    assert (out[1, :, :22] == 0).all() and (q.grad[1, :, :22] == 0).all()
    assert (k.grad[1, :, :150] == 0).all() and (v.grad[1, :, :150] == 0).all()
    assert (g.grad[1, :, :151] == 0).all()


def test_golden_c1_shape(fa):
    """Benchmark configuration 1 (B2 T256 H4 D64, sm_scale 1/8): same inputs rounded to bf16."""
    d = np.load(ROOT / "tests" / "golden" / "c1_b2_t256_h4_d64.npz")
    q, k, v = (torch.from_numpy(d[n]).cuda().bfloat16() for n in ("q", "k", "v"))
    g = torch.from_numpy(d["log_fgate"]).cuda()
    out = fa(q, k, v, g, sm_scale=1 / 8)
    ref = O.forgetting_attention_ref(q, k, v, g, sm_scale=1 / 8)
    assert rel_err(out, ref) <= REL_TOL
    # and not far from the fp32-input golden output either (input rounding only)
    assert rel_err(out, torch.from_numpy(d["out"]).cuda()) <= 5e-2


# --------------------------------------------------------------------------------------
# parity grid
# --------------------------------------------------------------------------------------
@pytest.mark.parametrize("D", [16, 32, 64, 128])
def test_config2_library_example(fa, D):
    """Benchmark configuration 2: B4 T512 H12, bf16 fwd+bwd, (batch, time, head, dim) layout."""
    run_case(fa, 4, 12, 512, 512, D, head_first=False, seed=D)


@pytest.mark.parametrize("B,H,M,N,D", [(2, 2, 300, 300, 64), (1, 3, 129, 129, 128), (2, 2, 200, 457, 64), (1, 2, 64, 1000, 32),
                                        (2, 1, 1, 777, 64), (1, 1, 1, 1, 16), (1, 2, 5, 5, 128), (1, 1, 127, 257, 16)])
@pytest.mark.parametrize("seq", [None, "random"])
def test_shapes_tails_and_offsets(fa, B, H, M, N, D, seq):
    run_case(fa, B, H, M, N, D, seq_start=seq, seed=M + N)


@pytest.mark.parametrize("seq", [[0, 0], [299, 5], [150, 299], [1, 128]])
def test_seq_start_edges(fa, seq):
    (out, dq, dk, dv, dg), _, ss = run_case(fa, 2, 2, 200, 300, 64, seq_start=seq, seed=5)
    P = 100
    for b, s in enumerate(seq):
        empty = max(0, s - P)          # queries whose key position is left of seq_start
        assert (out[b, :, :empty] == 0).all() and (dq[b, :, :empty] == 0).all()
        assert (dk[b, :, :s] == 0).all() and (dv[b, :, :s] == 0).all()
        assert (dg[b, :, : s + 1] == 0).all()   # = sum of all dc, zero in exact arithmetic: stored as an exact zero


@pytest.mark.parametrize("thr", [-10.0, "auto", "per_head", "per_bh", "zero_d"])
@pytest.mark.parametrize("gates", [(0.0, 1.0), (-1.0, 2.0)])
def test_adaptive_thresholds(fa, thr, gates):
    """Thresholds low enough that the pruned attention mass is far below bf16 rounding:
    results must match the unpruned oracle.  Covers the broadcast rules of :104-109."""
    B, H = 2, 4
    t = {"per_head": torch.tensor([-1000.0, -100.0, -40.0, -25.0]), "per_bh": torch.linspace(-60, -20, B * H).view(B, H),
         "zero_d": torch.tensor(-30.0)}.get(thr, thr)
    for masked in (False, True):   # against the unpruned oracle, and against the oracle on the kernels' own sets
        run_case(fa, B, H, 700, 1100, 64, thr=t, gate_mean=gates[0], gate_std=gates[1], qkv_std=0.5, seed=11, masked=masked)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("thr", [-3.0, -0.5, 0.0])
def test_aggressive_threshold_prunes_exactly_the_reported_tiles(fa, thr, D):
    """A threshold that changes the result (the reference prunes in all three kernels, :600-613, :1038-1049,
    :1239-1261): out and every gradient must equal the oracle with exactly the entries outside the kernels' reported
    bounds removed, and nothing else, at the standard bar; and the pruning must have mattered."""
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    B, H, M, N = 2, 2, 600, 900
    kw = dict(seed=12, gate_mean=4.0, gate_std=1.0, seq_start=[0, 200])
    (out, dq, dk, dv, dg), ref, ss = run_case(fa, B, H, M, N, D, thr=thr, **kw)
    q, k, v, g, do, _ = make_inputs(B, H, M, N, D, device="cuda", **kw)
    full = O.forgetting_attention_ref_grads(q, k, v, g, do, head_first=True, seq_start=ss)
    for name, r, f in zip(("out", "dq", "dk", "dv"), ref, full):
        assert rel_err(r, f) > 1e-3, name          # the pruning really mattered at this threshold, for every output
    bm, bn, _, _ = _lib.tile_config(D)
    _, _, si = ForgettingAttention.apply(q, k, v, g, ss, True, None, thr, False, True)
    assert (si % bn == 0).all() and (si > 0).any()


@pytest.mark.parametrize("B,H,M,N,D,seq,thr", [(1, 2, 1, 8192, 64, None, None), (2, 2, 128, 4096, 128, [100, 3000], None),
                                                (1, 3, 200, 6000, 64, None, -10.0), (2, 1, 1, 2000, 128, [0, 1999], None),
                                                (1, 1, 64, 9000, 32, [8990], "auto"), (1, 2, 300, 5000, 16, None, None)])
def test_key_split_shapes(fa, B, H, M, N, D, seq, thr):
    """Few query tiles and a long key sequence (decode, chunked prefill): the forward splits the
    key loop over several workgroups and merges the partial results."""
    import ctypes as C_
    from forgetting_transformer.ops import _lib
    need = C_.c_int64(0)
    _lib.check(_lib.load().fox_attn_fwd_workspace_bytes(C_.byref(_lib.Dims(B, H, M, N, D, 0)), C_.byref(need)), "ws")
    assert need.value > 0, "this shape is meant to exercise the split path"
    run_case(fa, B, H, M, N, D, seq_start=seq, thr=thr, seed=N, gate_mean=4.0, gate_std=1.0)


@pytest.mark.parametrize("D", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,head_first,seq,thr", [
    (1, True, None, None), (37, False, None, None), (300, True, [0, 299, 300], None),     # one workgroup per (b, h)
    (5000, False, [17, 4999, 2500], None), (8192, True, None, -8.0), (6001, True, [100, 0, 6000], "auto")])  # key splits
def test_single_query_streaming_kernel(fa, D, dtype, N, head_first, seq, thr):
    """M = 1 (a decode step) runs through the dot-free streaming kernel: every head dim and dtype, both layouts,
    with and without key splits, tails of the 4-wave rounds, left padding up to a fully padded row (o = 0,
    zero gradients), pruning thresholds."""
    B = 3 if seq is not None else 2
    tol = REL_TOL if dtype == torch.bfloat16 else 1e-2
    run_case(fa, B, 2, 1, N, D, dtype=dtype, head_first=head_first, seq_start=seq, thr=thr, tol=tol, seed=N + D,
             gate_mean=3.0, gate_std=1.5, qkv_std=0.8)


def test_single_query_matches_last_row_of_a_full_forward(fa):
    """The decode kernel against the tiled kernel itself: out and lse of the last query row of an M = N call, and the
    first key block the pruning bound keeps (in keys, a multiple of the 64-key block)."""
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    B, H, N, D = 2, 3, 3000, 64
    q, k, v, g, _, _ = make_inputs(B, H, N, N, D, device="cuda", head_first=True, seed=77, gate_mean=1.0, gate_std=2.0)
    for thr in (None, -5.0):
        full, lse_full, start_full = ForgettingAttention.apply(q, k, v, g, None, True, None, thr, True, True)
        one, lse_one, start_one = ForgettingAttention.apply(q[:, :, -1:], k, v, g, None, True, None, thr, True, True)
        assert rel_err(one, full[:, :, -1:]) <= 2.0 ** -7            # both round to bf16 once
        assert torch.allclose(lse_one, lse_full[:, :, -1:], rtol=0, atol=2e-3)
        # the bound of the last 128-row block is taken at its first row, the single row's at itself: never earlier
        assert (start_one[:, :, 0] >= start_full[:, :, -1]).all() and (start_one % 64 == 0).all()
        assert (start_one[:, :, 0] > 0).all() == (thr is not None)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("seq,thr", [(None, None), ([0, 517], -4.0)])
def test_single_query_tile_matches_the_last_tile_of_a_longer_call(fa, D, seq, thr):
    """A (batch, head) with a single query tile and enough keys runs through the forward's streaming instantiation (K and
    V tiles loaded with the non-temporal hint; forced here for a small shape through fox_set_stream_min_kv_bytes); the
    same rows as the second tile of a 256-row call run through the cached one.  Neither call splits its keys (fewer than
    16 key tiles), so both walk the same tiles in the same order: out, the log-normaliser and the reported first key
    block are bit for bit the same."""
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    lib = _lib.load()
    B, H, N = 2, 3, 900
    q, k, v, g, _, _ = make_inputs(B, H, 256, N, D, device="cuda", head_first=True, seed=901 + D, gate_mean=1.0, gate_std=2.0)
    ss = None if seq is None else torch.tensor(seq, device="cuda")
    prev = lib.fox_set_stream_min_kv_bytes(0)
    try:
        full, lse_full, start_full = ForgettingAttention.apply(q, k, v, g, ss, True, None, thr, True, True)
        tail, lse_tail, start_tail = ForgettingAttention.apply(q[:, :, 128:], k, v, g, ss, True, None, thr, True, True)
    finally:
        assert lib.fox_set_stream_min_kv_bytes(prev) == 0
    assert torch.equal(tail, full[:, :, 128:]) and torch.equal(lse_tail, lse_full[:, :, 128:])
    assert torch.equal(start_tail[:, :, 0], start_full[:, :, 1])
    assert torch.isfinite(tail.float()).all() and tail.float().abs().max() > 0.1


@pytest.mark.parametrize("B,H,M,N,D", [(2, 3, 128, 900, 128), (2, 3, 100, 900, 64), (1, 2, 128, 6000, 128), (2, 2, 64, 5000, 64),
                                        (1, 2, 77, 3000, 32), (3, 1, 128, 2100, 16)])
@pytest.mark.parametrize("seq,thr", [(False, None), (True, -6.0)])
def test_streaming_tile_loads_change_no_bit(fa, B, H, M, N, D, seq, thr):
    """The same call with the streaming instantiation forced on and forced off (fox_set_stream_min_kv_bytes 0 and
    INT64_MAX), with and without key splits, every head dim: out, log-normaliser and first key block bit for bit equal,
    and the default limit (512 MiB) is what the setter hands back."""
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    lib = _lib.load()
    q, k, v, g, _, ss = make_inputs(B, H, M, N, D, device="cuda", head_first=True, seed=N + D, gate_mean=2.0, gate_std=1.0,
                                    seq_start="random" if seq else None)
    prev = lib.fox_set_stream_min_kv_bytes(0)
    try:
        streamed = ForgettingAttention.apply(q, k, v, g, ss, True, None, thr, True, True)
        assert lib.fox_set_stream_min_kv_bytes(2 ** 63 - 1) == 0
        cached = ForgettingAttention.apply(q, k, v, g, ss, True, None, thr, True, True)
    finally:
        lib.fox_set_stream_min_kv_bytes(prev)
    assert prev == 512 << 20
    for a_, b_ in zip(streamed, cached):
        assert torch.equal(a_, b_)
    assert streamed[0].float().abs().max() > 0.05


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_row_mass_in_tiny_probabilities(fa, dtype):
    """One key outweighs every other by e^11 while the 32768 others together still hold a third of each row's mass:
    relative to the running maximum their probabilities are 1.7e-5, below the smallest normal fp16 number.  The
    forward's row sum adds the probabilities as rounded for the PV matrix product (a dot-product instruction against
    ones) where the reference adds them in fp32 (tl.sum(p, 1), :650-651): if that instruction dropped subnormal
    inputs that the matrix unit keeps, out and the log-normaliser would be off by that third.  Against the fp64 oracle."""
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    B, H, M, N, D = 1, 2, 256, 32768, 64
    g_ = torch.Generator().manual_seed(123)
    q = torch.randn(B, H, M, D, generator=g_) * 0.05
    k = torch.randn(B, H, N, D, generator=g_) * 0.05
    v = torch.randn(B, H, N, D, generator=g_)
    q[..., 0] = 8.0
    k[..., 0] = 0.0
    k[:, :, 7, 0] = 11.0          # q.k / sqrt(D) = 8 * 11 / 8 = 11 for key 7, about 0 for the others
    v[:, :, 7] = 3.0
    gates = torch.full((B, H, N), -1e-7)
    q, k, v = (x.to(dtype).cuda() for x in (q, k, v))
    gates = gates.cuda()
    out, lse, _ = ForgettingAttention.apply(q, k, v, gates, None, True, None, None, True, False)
    ref, lse_ref = O.forgetting_attention_ref(q, k, v, gates, head_first=True, return_lse=True, compute_dtype=torch.float64)
    share = 1.0 - torch.exp(11.0 - lse_ref).mean().item()     # mass outside the dominant key
    assert 0.2 < share < 0.5
    assert (lse.double() - lse_ref).abs().max().item() <= 2e-3
    assert rel_err(out, ref) <= (REL_TOL if dtype == torch.bfloat16 else 1e-2)


@pytest.mark.parametrize("sm_scale", [None, 0.5, 1.3])
def test_sm_scale(fa, sm_scale):
    run_case(fa, 1, 2, 260, 260, 64, sm_scale=sm_scale, qkv_std=0.5, seed=3)


@pytest.mark.parametrize("sm_scale", [0.0, -0.4, 1e-20])
@pytest.mark.parametrize("M,N", [(400, 400), (130, 700)])
def test_degenerate_sm_scale(fa, sm_scale, M, N):
    """Zero, negative and vanishing scales: the kernels carry the decay terms in the MFMA accumulators
    as term / scale, which must not break down when the scale is not a positive normal number."""
    run_case(fa, 1, 2, M, N, 64, sm_scale=sm_scale, qkv_std=0.5, seed=5, seq_start=[37])


def test_fox_layer_views(fa):
    """The FoX layer passes (B,H,T,D) views of (B,T,H*D) memory and a (B,H,T) view of
    (B,T,H) gates with head_first=True (modeling_forgetting_transformer.py:318-346)."""
    B, T, H, D = 2, 384, 4, 64
    g = torch.Generator().manual_seed(0)
    x = [torch.randn(B, T, H * D, generator=g).bfloat16().cuda() for _ in range(3)]
    q, k, v = (t.view(B, T, H, D).transpose(1, 2).requires_grad_() for t in x)
    gates = F.logsigmoid(torch.randn(B, T, H, generator=g).cuda()).transpose(1, 2).requires_grad_()
    do = torch.randn(B, H, T, D, generator=g).bfloat16().cuda()
    ss = torch.tensor([0, 100]).cuda()
    out = fa(q, k, v, gates, head_first=True, seq_start=ss, sm_scale=1 / math.sqrt(D))
    assert out.stride() == q.stride()                 # the un-permute on return stays free
    out.backward(do)
    ref = O.forgetting_attention_ref_grads(q.detach(), k.detach(), v.detach(), gates.detach(), do, head_first=True, seq_start=ss)
    for name, x_, r in zip(("out", "dq", "dk", "dv", "dlog_fgate"), (out, q.grad, k.grad, v.grad, gates.grad), ref):
        assert_parity(name, x_, r, rows=name != "dlog_fgate")


@pytest.mark.parametrize("Z,H,M,N,D", [(4, 2, 1020, 2098, 64), (4, 2, 1024, 2048, 128)])
@pytest.mark.parametrize("gate_range", [(0, 5), (5, 10)])
@pytest.mark.parametrize("has_seq_start", [True, False])
@pytest.mark.parametrize("thr", [-10.0, None, "tensor"])
def test_reference_grid(fa, Z, H, M, N, D, gate_range, has_seq_start, thr):
    """The parameter grid, input distributions and tolerance of the reference's own test_op (:1360-1425)."""
    t = torch.tensor([-1000.0, -100.0]) if thr == "tensor" else thr
    run_case(fa, Z, H, M, N, D, dtype=torch.float16, qkv_std=0.5, gate_uniform=gate_range, sm_scale=0.5,
             seq_start="random" if has_seq_start else None, thr=t, seed=24, atol=1e-2)


# --------------------------------------------------------------------------------------
# special cases and size-independent properties
# --------------------------------------------------------------------------------------
def test_zero_gates_are_plain_causal_attention(fa):
    q, k, v, _, _, _ = make_inputs(2, 4, 512, 512, 64, device="cuda", seed=8)
    g = torch.zeros(2, 4, 512, device="cuda")
    out = fa(q, k, v, g, head_first=True)
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert rel_err(out, ref) <= REL_TOL


def test_log_normalizer_and_start_index_outputs(fa):
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    q, k, v, g, _, ss = make_inputs(2, 3, 300, 500, 64, device="cuda", seed=9, seq_start=[0, 350], gate_mean=-1, gate_std=2)
    out, L, si = ForgettingAttention.apply(q, k, v, g, ss, True, 0.3, -6.0, True, True)
    _, lse = O.forgetting_attention_ref(q, k, v, g, head_first=True, seq_start=ss, sm_scale=0.3, return_lse=True)
    assert torch.equal(torch.isinf(L), torch.isinf(lse))
    fin = ~torch.isinf(lse)
    assert (L[fin] - lse[fin]).abs().max() < 2e-2
    assert si.dtype == torch.long and si.shape == (2, 3, 3)


@pytest.mark.parametrize("limit", [-1, 0, 64])
@pytest.mark.parametrize("B,H,M,N,seq,thr,gates", [
    (1, 3, 129, 129, None, None, (0.0, 1.0)), (2, 2, 200, 457, [5, 300], None, (0.0, 1.0)), (1, 2, 940, 940, None, -6.0, (0.0, 1.0)),
    (2, 2, 700, 950, None, -10.0, (-1.0, 2.0)), (1, 2, 5, 5, None, None, (0.0, 1.0)), (1, 1, 127, 257, [200], "auto", (1.0, 1.0)),
    (2, 4, 2048, 2048, [0, 1024], -20.0, (2.0, 1.0)), (2, 2, 1000, 3000, None, -20.0, (1.0, 1.0)), (1, 2, 1, 300, None, None, (0.0, 1.0)),
    (2, 3, 515, 515, [0, 77], "fp16", (1.0, 1.5))])
def test_dkdv_kernel_variants(fa, limit, B, H, M, N, seq, thr, gates):
    """The dK/dV pass at head dim 128 has two kernels (long loops; head dim split over two waves for key tiles pruned
    down to a few steps) and a per-tile choice between them.  Every tile through the split variant (-1, with and
    without a threshold), none (0), and a mix decided tile by tile (64 keys): all against the oracle."""
    from forgetting_transformer.ops import _lib
    lib = _lib.load()
    prev = lib.fox_set_acp_light_limit(limit)
    try:
        dtype = torch.bfloat16
        if thr == "fp16":   # the half-precision instantiations of both kernels, pruned by "auto"
            dtype, thr = torch.float16, "auto"
        tol = REL_TOL if dtype == torch.bfloat16 else 1e-2
        run_case(fa, B, H, M, N, 128, dtype=dtype, seq_start=seq, thr=thr, tol=tol, gate_mean=gates[0], gate_std=gates[1], seed=M + N,
                 qkv_std=0.7)
    finally:
        assert lib.fox_set_acp_light_limit(prev) == limit


def test_in_op_timers_fill_the_info_table(fa):
    """The reference's hidden timing flags (:45-70, :176-181, :217-222): same results, and the class-level table
    gets the elapsed milliseconds and call counts under the caller's key."""
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    q, k, v, g, do, _ = make_inputs(2, 2, 512, 512, 64, device="cuda", seed=31, requires_grad=True)
    plain = fa(q, k, v, g, head_first=True, adaptive_threshold=-20.0)
    plain.backward(do)
    want = [t.clone() for t in (plain, q.grad, k.grad, v.grad, g.grad)]
    q.grad = k.grad = v.grad = g.grad = None
    key = "timed-layer"
    ForgettingAttention.info.pop(key, None)
    for _ in range(2):
        out = ForgettingAttention.apply(q, k, v, g, None, True, None, -20.0, False, False, key, True, True)
        out.backward(do)
    info = ForgettingAttention.info[key]
    assert info["fwd_count"] == 2 and info["bwd_count"] == 2 and info["fwd_time"] > 0 and info["bwd_time"] > 0
    assert info["fwd_find_index_count"] == 2 and info["bwd_find_index_kv_count"] == 2 and info["bwd_find_index_q_count"] == 2
    assert torch.equal(out, want[0])
    for got, w in zip((q.grad, k.grad, v.grad, g.grad), want[1:]):
        assert torch.equal(got, 2 * w)       # two backward passes accumulated


def test_pruning_bounds_match_the_scan_bit_exactly(fa):
    """first_block from the kernel's wave-parallel search == the reference's two-pointer scan
    (restated in C) run on the kernel's own cumulative sums."""
    import subprocess
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    so = ROOT / "oracle" / "libfox_oracle.so"
    if not so.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    co = C.CDLL(str(so))
    co.fox_oracle_find_start_index.argtypes = [C.c_void_p, C.c_float] + [C.c_int] * 4 + [C.c_void_p]
    lib = _lib.load()
    B, H, M, N, D = 2, 3, 1500, 4000, 64
    bm, bn, _, _ = _lib.tile_config(D)
    q, k, v, g, _, _ = make_inputs(B, H, M, N, D, device="cuda", seed=13, gate_mean=-1, gate_std=2)
    thr = torch.tensor([[-5.0, -10.0, -40.0], [-1.0, -100.0, -20.0]])
    _, _, si = ForgettingAttention.apply(q, k, v, g, None, True, None, thr, False, True)
    c = torch.empty(B, H, N, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.fox_cumsum_fwd(g.data_ptr(), *g.stride(), None, c.data_ptr(), B, H, N, stream), "cumsum")
    c = c.cpu().numpy()
    for b in range(B):
        for h in range(H):
            row = np.ascontiguousarray(c[b, h])
            exp = np.zeros((M + bm - 1) // bm, np.int64)
            co.fox_oracle_find_start_index(row.ctypes.data_as(C.c_void_p), float(thr[b, h]), M, N, bm, bn,
                                           exp.ctypes.data_as(C.c_void_p))
            assert np.array_equal(si[b, h].cpu().numpy(), exp), (b, h)
    assert (si > 0).any()


def _c_oracle():
    import subprocess
    so = ROOT / "oracle" / "libfox_oracle.so"
    if not so.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    co = C.CDLL(str(so))
    co.fox_oracle_find_start_index.argtypes = [C.c_void_p, C.c_float] + [C.c_int] * 4 + [C.c_void_p]
    co.fox_oracle_find_end_index.argtypes = [C.c_void_p, C.c_float] + [C.c_int] * 5 + [C.c_void_p]
    return co


@pytest.mark.parametrize("D,limit", [(128, 0), (128, -1), (128, 64), (128, 256), (64, 0), (32, 0), (16, 0)])
@pytest.mark.parametrize("M,N,seq", [(1500, 4000, None), (2048, 2048, None), (1111, 1111, [0, 700])])
def test_backward_pruning_bounds_match_the_scans(fa, D, limit, M, N, seq):
    """The bounds the two backward kernels work with, read back through fox_bwd_args.q_first_block / kv_end_row, against
    the reference's scans restated in C (_find_start_index_kernel :695-745, _find_end_index_kernel :747-795 in its
    tight form) run on the kernel's own cumulative sums: bit for bit, for the long-loop dK/dV kernel (128 keys x 128
    rows), the split variant (64 x 64), the per-tile mix of the two, and the head dims that only have the former."""
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import record_pruning_bounds
    co, lib = _c_oracle(), _lib.load()
    B, H = 2, 3
    bm, bn, kv_bn, kv_bm = _lib.tile_config(D)
    q, k, v, g, do, ss = make_inputs(B, H, M, N, D, device="cuda", seed=13 + D, gate_mean=-1, gate_std=2, seq_start=seq,
                                     requires_grad=True)
    thr = torch.tensor([[-5.0, -10.0, -40.0], [-1.0, -100.0, -20.0]])
    prev = lib.fox_set_acp_light_limit(limit)
    try:
        with record_pruning_bounds() as rec:
            fa(q, k, v, g, head_first=True, seq_start=ss, adaptive_threshold=thr).backward(do)
    finally:
        assert lib.fox_set_acp_light_limit(prev) == limit
    q_first, kv_end = rec[1]["dq_first_block"].cpu().numpy(), rec[1]["kv_end_row"].cpu().numpy()
    assert np.array_equal(q_first, rec[0]["fwd_first_block"].cpu().numpy())
    c = torch.empty(B, H, N, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.fox_cumsum_fwd(g.data_ptr(), *g.stride(), None if ss is None else ss.data_ptr(), c.data_ptr(), B, H, N, stream), "cumsum")
    c = c.cpu().numpy()
    P = N - M
    split_ok = D == 128     # the head dim the split variant exists for
    n_light = n_heavy = 0
    for b in range(B):
        s0 = 0 if ss is None else int(ss[b])
        for h in range(H):
            row, t = np.ascontiguousarray(c[b, h]), float(thr[b, h])
            # query side: the scan, then left padding (a walk never starts left of seq_start's block)
            exp_q = np.zeros((M + bm - 1) // bm, np.int64)
            co.fox_oracle_find_start_index(row.ctypes.data_as(C.c_void_p), t, M, N, bm, bn, exp_q.ctypes.data_as(C.c_void_p))
            hi = np.minimum(N, P + np.arange(len(exp_q)) * bm + bm)
            exp_q = np.maximum(exp_q // bn, np.minimum(s0, hi) // bn)
            assert np.array_equal(q_first[b, h], exp_q), (b, h)
            # key side: the tight scan at both granularities; which one applies is decided per 128-key tile
            ends = {}
            for kb, km in ((kv_bn, kv_bm), (64, 64)):
                e = np.zeros((N + kb - 1) // kb, np.int64)
                co.fox_oracle_find_end_index(row.ctypes.data_as(C.c_void_p), t, M, N, km, kb, 1, e.ctypes.data_as(C.c_void_p))
                ends[kb] = e
            for u in range((N + 63) // 64):
                parent = u * 64 // kv_bn
                n_last = min(N - 1, parent * kv_bn + kv_bn - 1)
                light = split_ok and limit != 0 and (limit < 0 or n_last + limit >= N or
                                                     np.float32(row[n_last + limit]) - np.float32(row[n_last]) < np.float32(t))
                kb, km = (64, 64) if light else (kv_bn, kv_bm)
                n0 = u * 64 // kb * kb
                m_lo = max(n0 - P, 0) // km * km            # first query block that reaches the tile
                want = max(int(ends[kb][n0 // kb]), m_lo)   # the kernel's walk starts there: no earlier bound to report
                if n0 + kb <= s0:
                    want = m_lo                             # every key of the tile is left padding: nothing visited
                assert kv_end[b, h, u] == want, (b, h, u, light, int(kv_end[b, h, u]), want)
                n_light += light
                n_heavy += not light
    assert (kv_end < M).any() and (q_first > 0).any()       # bounds that prune
    if limit == 64:
        assert n_light > 0 and n_heavy > 0                  # the mix really is one


def test_delta_stage_alone(fa):
    """fox_attn_bwd_delta (_bwd_preprocess :902-943 as a stage of its own): rowsum(o * do) in fp32, against torch in fp64, and
    the same check on what the dQ stage leaves in its delta buffer (it forms the sums for the rows it holds)."""
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import _view
    lib = _lib.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for D, dtype, M in ((128, torch.bfloat16, 300), (64, torch.float16, 129), (32, torch.bfloat16, 1000), (16, torch.bfloat16, 77)):
        B, H, N = 2, 3, M + 50
        g_ = torch.Generator(device="cuda").manual_seed(D)
        o, do, q = (torch.randn(B, M, H, D, generator=g_, device="cuda").to(dtype).transpose(1, 2) for _ in range(3))
        k, v = (torch.randn(B, N, H, D, generator=g_, device="cuda").to(dtype).transpose(1, 2) for _ in range(2))
        delta = torch.full((B, H, M), float("nan"), device="cuda")
        dims = _lib.Dims(B, H, M, N, D, 0 if dtype == torch.bfloat16 else 1)
        zero = _lib.View()
        args = _lib.BwdArgs(dims, zero, zero, zero, _view(o), _view(do), zero, zero, zero, None, None, None, None, 1.0,
                            delta.data_ptr(), None, None, None, 0, 0, 0, None, None)
        _lib.check(lib.fox_attn_bwd_delta(C.byref(args), stream), "fox_attn_bwd_delta")
        ref = (o.double() * do.double()).sum(-1)
        assert (delta.double() - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()
        # the dQ stage forms the same values for the rows it holds
        c = torch.cumsum(F.logsigmoid(torch.randn(B, H, N, generator=g_, device="cuda")), -1)
        lse = torch.zeros(B, H, M, device="cuda")
        delta2, drow, dc, dg = (torch.empty(B, H, n, device="cuda") for n in (M, M, N, N))
        dq = torch.empty_like(q)
        args2 = _lib.BwdArgs(dims, _view(q), _view(k), _view(v), _view(o), _view(do), _view(dq), zero, zero, c.data_ptr(),
                             lse.data_ptr(), None, None, 0.1, delta2.data_ptr(), drow.data_ptr(), dc.data_ptr(), dg.data_ptr(),
                             0, 0, 0, None, None)
        _lib.check(lib.fox_attn_bwd_dq(C.byref(args2), stream), "fox_attn_bwd_dq")
        assert (delta2.double() - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()


def test_cumsum_kernels(fa):
    from forgetting_transformer.ops import _lib
    lib = _lib.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    B, H, N = 3, 5, 5000
    g = F.logsigmoid(torch.randn(B, N, H, device="cuda") * 2 - 1).transpose(1, 2)   # strided (B,H,N) view
    ss = torch.tensor([0, 1234, 4999], device="cuda")
    c = torch.empty(B, H, N, device="cuda")
    _lib.check(lib.fox_cumsum_fwd(g.data_ptr(), *g.stride(), ss.data_ptr(), c.data_ptr(), B, H, N, stream), "cumsum_fwd")
    ref = O.cumulative_log_decay(g, ss, torch.float64)
    assert (c.double() - ref).abs().max() <= 2e-7 * ref.abs().max()      # correctly rounded fp64 sums: half an ulp
    assert (c[..., 1:] <= c[..., :-1]).all()                              # non-increasing, as the pruning bounds assume
    assert (c[1, :, :1234] == 0).all()
    dc = torch.randn(B, H, N, device="cuda")
    dg = torch.empty_like(dc)
    _lib.check(lib.fox_cumsum_bwd(dc.data_ptr(), dg.data_ptr(), 0, 0, 0, None, B, H, N, stream), "cumsum_bwd")
    ref = torch.flip(torch.cumsum(torch.flip(dc.double(), [-1]), -1), [-1])
    assert (dg.double() - ref)[..., 1:].abs().max() <= 1e-6 * ref.abs().max()
    assert (dg[..., 0] == 0).all()      # the sum of a true dc is zero in exact arithmetic: stored as an exact zero
    # with left padding every position up to and including seq_start is such a sum
    _lib.check(lib.fox_cumsum_bwd(dc.data_ptr(), dg.data_ptr(), 0, 0, 0, ss.data_ptr(), B, H, N, stream), "cumsum_bwd")
    for b_, s_ in enumerate(ss.tolist()):
        assert (dg[b_, :, : s_ + 1] == 0).all()
        assert (dg[b_].double() - ref[b_])[:, s_ + 1:].abs().max() <= 1e-6 * ref.abs().max() if s_ + 1 < N else True
    _lib.check(lib.fox_cumsum_bwd(dc.data_ptr(), dg.data_ptr(), 0, 0, 0, None, B, H, N, stream), "cumsum_bwd")
    # the same into a (B,H,N) view of (B,N,H) memory, the layout of the FoX layer's gates: bit for bit the same values
    dg_t = torch.full((B, N, H), float("nan"), device="cuda").transpose(1, 2)
    _lib.check(lib.fox_cumsum_bwd(dc.data_ptr(), dg_t.data_ptr(), *dg_t.stride(), None, B, H, N, stream), "cumsum_bwd")
    assert torch.equal(dg_t, dg)


def test_mfma_probe_runs(fa):
    """The measuring-stick loop of the power report: launches, returns, leaves its sink alone."""
    from forgetting_transformer.ops import _lib
    lib = _lib.load()
    operands = torch.randn(16 * 64 * 8, device="cuda").to(torch.bfloat16)
    sink = torch.zeros(1, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.fox_probe_mfma(operands.data_ptr(), sink.data_ptr(), 8, 50, stream), "fox_probe_mfma")
    torch.cuda.synchronize()
    assert sink.item() == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_auto_threshold_kernel(fa, dtype):
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import _view
    lib = _lib.load()
    B, H, M, N, D = 2, 3, 700, 1300, 64
    q, k, _, _, _, _ = make_inputs(B, H, M, N, D, dtype=dtype, device="cuda", seed=17)
    thr = torch.empty(B, H, device="cuda")
    scratch = torch.empty(B, H, 3, dtype=torch.int32, device="cuda")
    dims = _lib.Dims(B, H, M, N, D, 0 if dtype == torch.bfloat16 else 1)
    qv, kv = _view(q), _view(k)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.fox_auto_threshold(C.byref(dims), C.byref(qv), C.byref(kv), 0.125, thr.data_ptr(), scratch.data_ptr(), stream), "auto")
    ref = O.auto_threshold(q, k, 0.125)            # the reference's tensor arithmetic, same dtype roundings
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10) * ref.abs().max().item()
    assert (thr - ref).abs().max().item() <= 2 * ulp


def test_bitwise_determinism(fa):
    q, k, v, g, do, _ = make_inputs(2, 4, 1024, 1024, 128, device="cuda", seed=21, requires_grad=True)
    res = []
    for _ in range(2):
        out = fa(q, k, v, g, head_first=True, adaptive_threshold="auto")
        out.backward(do)
        res.append([t.clone() for t in (out, q.grad, k.grad, v.grad, g.grad)])
        q.grad = k.grad = v.grad = g.grad = None
    for a, b in zip(*res):
        assert torch.equal(a, b)          # no atomics anywhere on the path


def test_linearity_in_values_and_upstream_gradient(fa):
    q, k, v, g, do, _ = make_inputs(1, 2, 2048, 2048, 128, device="cuda", seed=22)
    v2 = torch.randn_like(v)
    f = lambda vv: fa(q, k, vv, g, head_first=True).float()
    lhs = f((v.float() + v2.float()).bfloat16())
    rhs = f(v) + f(v2)
    assert rel_err(lhs, rhs) <= REL_TOL


def test_graph_capture_replays_match_eager(fa):
    """Forward + backward captured into a HIP graph (the library allocates nothing, never synchronises and clears its
    scratch with a kernel, not a memset) and replayed on fresh data: every replay must equal the eager result bit for
    bit, with eager work and synchronisations between the replays."""
    B, H, T, D = 2, 2, 1024, 64
    q, k, v, g, do, _ = make_inputs(B, H, T, T, D, device="cuda", head_first=True, seed=90, gate_mean=1.0, gate_std=1.5)
    q, k, v, g = (x.requires_grad_() for x in (q, k, v, g))

    def step():
        out = fa(q, k, v, g, head_first=True, adaptive_threshold="auto")
        out.backward(do)
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # warm-up outside the capture, as autograd under capture requires
        for _ in range(2):
            step()
            q.grad = k.grad = v.grad = g.grad = None
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    captured = (out, q.grad, k.grad, v.grad, g.grad)
    for trial in range(3):
        fresh = make_inputs(B, H, T, T, D, device="cuda", head_first=True, seed=91 + trial, gate_mean=1.0, gate_std=1.5)
        with torch.no_grad():
            for dst, src in zip((q, k, v, g, do), fresh[:5]):
                dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        q2, k2, v2, g2 = (x.detach().clone().requires_grad_() for x in (q, k, v, g))   # eager work between the replays
        out2 = fa(q2, k2, v2, g2, head_first=True, adaptive_threshold="auto")
        out2.backward(do)
        torch.cuda.synchronize()
        for name, a_, b_ in zip(("out", "dq", "dk", "dv", "dlog_fgate"), got, (out2, q2.grad, k2.grad, v2.grad, g2.grad)):
            assert torch.equal(a_, b_), (name, trial)


# --------------------------------------------------------------------------------------
# seeded sweep over random configurations
# --------------------------------------------------------------------------------------
@pytest.mark.parametrize("case", range(48))
def test_random_configurations(fa, case):
    """Shapes, layouts, paddings, thresholds and scales drawn from a fixed seed per case: tails of every
    tile size, M << N, tiny sequences, empty rows, per-head thresholds, both dtypes."""
    rng = np.random.default_rng(1000 + case)
    D = int(rng.choice([16, 32, 64, 128]))
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    N = int(rng.choice([1, 2, 31, 64, 65, 127, 128, 129, 200, 257, 383, 512, 777, 1025]))
    M = int(rng.choice([1, max(1, N // 3), max(1, N - 1), N]))
    dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
    head_first = bool(rng.random() < 0.5)
    seq = None if rng.random() < 0.5 else [int(x) for x in rng.integers(0, N + 1, size=B)]
    thr_kind = rng.choice(["none", "float", "auto", "per_head"])
    thr = {"none": None, "float": float(-rng.uniform(0.5, 30.0)), "auto": "auto",
           "per_head": torch.tensor(-rng.uniform(1.0, 50.0, size=H), dtype=torch.float32, device="cuda")}[str(thr_kind)]
    sm_scale = None if rng.random() < 0.7 else float(rng.uniform(0.05, 1.5))
    gate_mean, gate_std = float(rng.uniform(-2.0, 5.0)), float(rng.uniform(0.3, 2.0))
    # floor: shapes with one or two keys have gradients that vanish by cancellation (inputs are O(1)).  Cases with a
    # threshold are compared with the oracle on the kernels' own pruning sets, at the same bar as the others.
    run_case(fa, B, H, M, N, D, dtype=dtype, head_first=head_first, seq_start=seq, thr=thr, sm_scale=sm_scale,
             tol=REL_TOL if dtype == torch.bfloat16 else 1e-2, floor=0.05, seed=case, gate_mean=gate_mean, gate_std=gate_std,
             qkv_std=0.7, context=(case, dict(B=B, H=H, M=M, N=N, D=D, thr=thr_kind)))


@pytest.mark.parametrize("D", [16, 32, 64])
@pytest.mark.parametrize("M,N,seq,thr", [(4100, 4100, None, None), (3000, 4500, [700], None), (4096, 4096, None, -6.0)])
def test_long_sequences_at_small_head_dims(fa, D, M, N, seq, thr):
    """Dozens of interior steps per key tile (both tile buffers in turn, with tails) on the dK/dV path that head dims
    <= 64 take (two workgroups per CU, plain step for every tile)."""
    run_case(fa, 1, 2, M, N, D, head_first=True, seq_start=seq, thr=thr, seed=40 + D, gate_mean=4.0, gate_std=1.0)


# --------------------------------------------------------------------------------------
# a sequence longer than any benchmark configuration, through properties that need no full-size oracle
# --------------------------------------------------------------------------------------
def test_sequence_of_65536_tokens(fa):
    """T = 65536 (512 query tiles, 1024 key tiles per head).  Causality: the first 8192 rows of the output must equal,
    bit for bit, the output on the first 8192 tokens alone (same tiles in the same order).  Under strong decay
    (gate logits N(-1, 1): a key 200 positions back weighs less than e^-100) the last rows and keys only see the last
    few thousand tokens, so the oracle on that window pins out, dq, dk, dv and the steps of dlog_fgate there (a constant
    shift of the cumulative sums cancels in every c_i - c_j)."""
    B, H, T, D, W = 1, 8, 65536, 64, 4096    # 8 heads: enough query tiles that neither run splits its key loops
    q, k, v, g, do, _ = make_inputs(B, H, T, T, D, dtype=torch.bfloat16, device="cuda", head_first=False, seed=77,
                                    gate_mean=-1.0, gate_std=1.0)
    q, k, v, g = (x.requires_grad_() for x in (q, k, v, g))
    out = fa(q, k, v, g)
    out.backward(do)
    for x in (out, q.grad, k.grad, v.grad, g.grad):
        assert torch.isfinite(x).all()
    assert (g.grad[:, 0] == 0).all()
    with torch.no_grad():
        head = fa(q[:, :8192], k[:, :8192], v[:, :8192], g[:, :8192])
    assert torch.equal(out[:, :8192], head)
    lo = T - W
    ref = O.forgetting_attention_ref_grads(q.detach()[:, lo:], k.detach()[:, lo:], v.detach()[:, lo:], g.detach()[:, lo:], do[:, lo:],
                                           bh_chunk=2)
    half = W // 2   # rows / keys of the window whose whole reach lies inside it
    for name, x, r in zip(("out", "dq", "dk", "dv"), (out, q.grad, k.grad, v.grad), ref):
        assert_parity(name, x[:, lo + half:], r[:, half:], context="last rows of 65536")
    assert_parity("dc_steps", gate_grad_steps(g.grad[:, lo + half:], False), gate_grad_steps(ref[4][:, half:], False), rows=False)


# --------------------------------------------------------------------------------------
# benchmark configurations 3-5 at full size
# --------------------------------------------------------------------------------------
# One (batch, head) pair per XCD: the workgroup -> (batch, head) map of the kernels puts pair bh on XCD bh mod 8,
# and with H = 16 that is h mod 8.
ALL_XCD_PAIRS = [(0, 0), (0, 9), (1, 2), (1, 11), (2, 4), (2, 13), (3, 6), (3, 15)]


def _full_size_check(fa, B, H, T, D, mean, std, thr, pairs, seq_start=None):
    g_ = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = (torch.randn(B, T, H, D, generator=g_, device="cuda").bfloat16().requires_grad_() for _ in range(3))
    gates = F.logsigmoid(torch.randn(B, T, H, generator=g_, device="cuda") * std + mean).requires_grad_()
    do = torch.randn(B, T, H, D, generator=g_, device="cuda").bfloat16()
    ss = None if seq_start is None else torch.tensor(seq_start, device="cuda")
    out = fa(q, k, v, gates, adaptive_threshold=thr, seq_start=ss)
    out.backward(do)
    got = (out, q.grad, k.grad, v.grad)
    for x in got + (gates.grad,):
        assert torch.isfinite(x).all()
    # property: the gate gradient of every position up to seq_start (position 0 without padding) is sum_n dc_n = 0
    for b in range(B):
        upto = 1 if ss is None else int(ss[b]) + 1
        assert (gates.grad[b, :upto] == 0).all(), b
    for b, h in pairs:   # oracle on (batch, head) pairs: one pair needs a 1 GiB score matrix
        sl = lambda x: x.detach()[b:b + 1, :, h:h + 1]
        ref = O.forgetting_attention_ref_grads(sl(q), sl(k), sl(v), gates.detach()[b:b + 1, :, h:h + 1], sl(do),
                                               seq_start=None if ss is None else ss[b:b + 1])
        for name, x, r in zip(("out", "dq", "dk", "dv"), got, ref):
            assert_parity(name, sl(x), r, context=(b, h))
        assert_parity("dlog_fgate", gates.grad[b:b + 1, :, h:h + 1], ref[4], rows=False, context=(b, h))
        assert_parity("dc_steps", gate_grad_steps(gates.grad[b:b + 1, :, h:h + 1], False), gate_grad_steps(ref[4], False),
                      rows=False, context=(b, h))
    return out.detach()


def test_config3_long_context(fa):
    _full_size_check(fa, 4, 16, 16384, 128, 3.0, 1.0, None, ALL_XCD_PAIRS)


@pytest.mark.parametrize("thr", [None, -10.0])
def test_config3_results_do_not_depend_on_where_a_head_sits(fa, thr):
    """Every (batch, head) pair is an independent problem, and the kernels map pair bh to XCD bh mod 8 and to a
    position in the launch order.  Rotating the batch by one and the heads by three moves every pair to another XCD
    and another place in the grid; all five outputs of all 64 pairs must come out bit for bit the same (with the
    oracle on one pair per XCD above, that extends to every pair what those eight pin).  Also under pruning, with
    config 4's gates."""
    B, H, T, D = 4, 16, 16384, 128
    g_ = torch.Generator(device="cuda").manual_seed(5)
    mean, std = (3.0, 1.0) if thr is None else (-1.0, 2.0)
    q, k, v = (torch.randn(B, T, H, D, generator=g_, device="cuda").bfloat16() for _ in range(3))
    gates = F.logsigmoid(torch.randn(B, T, H, generator=g_, device="cuda") * std + mean)
    do = torch.randn(B, T, H, D, generator=g_, device="cuda").bfloat16()
    rot = lambda x: torch.roll(x, shifts=(1, 3), dims=(0, 2)).contiguous()

    def run(q, k, v, gates, do):
        q, k, v, gates = (x.clone().requires_grad_() for x in (q, k, v, gates))
        out = fa(q, k, v, gates, adaptive_threshold=thr)
        out.backward(do)
        return out.detach(), q.grad, k.grad, v.grad, gates.grad

    a = run(q, k, v, gates, do)
    b = run(rot(q), rot(k), rot(v), rot(gates), rot(do))
    for name, x, y in zip(("out", "dq", "dk", "dv", "dlog_fgate"), a, b):
        assert torch.equal(rot(x), y), name


@pytest.mark.parametrize("M", [128, 1])
def test_config5_results_do_not_depend_on_where_a_head_sits(fa, M):
    """The same for the cache shapes (B16 H16 N32768 D128, head-first, left padding): the key-split forward, its
    merge kernel and the single-query streaming kernel, every (batch, head) pair moved to another XCD."""
    B, H, N, D = 16, 16, 32768, 128
    g_ = torch.Generator(device="cuda").manual_seed(6)
    q = torch.randn(B, H, M, D, generator=g_, device="cuda").bfloat16()
    k, v = (torch.randn(B, H, N, D, generator=g_, device="cuda").bfloat16() for _ in range(2))
    gates = F.logsigmoid(torch.randn(B, H, N, generator=g_, device="cuda") + 2.0)
    ss = torch.randint(0, 8192, (B,), generator=g_, device="cuda")
    rot = lambda x: torch.roll(x, shifts=(5, 3), dims=(0, 1)).contiguous()
    with torch.no_grad():
        a = fa(q, k, v, gates, head_first=True, seq_start=ss)
        b = fa(rot(q), rot(k), rot(v), rot(gates), head_first=True, seq_start=torch.roll(ss, 5))
    assert torch.isfinite(a).all()
    assert torch.equal(rot(a), b)


def test_config3_shape_with_left_padding(fa):
    """The long-context shape with left padding, forward and backward: padding inside the first tile, across many
    tiles, ending mid-tile just below the middle, and leaving only the last 300 positions."""
    _full_size_check(fa, 4, 16, 16384, 128, 3.0, 1.0, None, ALL_XCD_PAIRS, seq_start=[5, 3000, 8191, 16084])


def test_config4_pruned(fa):
    base = _full_size_check(fa, 4, 16, 16384, 128, -1.0, 2.0, None, ALL_XCD_PAIRS)
    for thr in ("auto", -10.0):
        out = _full_size_check(fa, 4, 16, 16384, 128, -1.0, 2.0, thr, ALL_XCD_PAIRS)
        assert rel_err(out, base) <= 1e-3     # pruned mass <= e^-10: far below bf16 rounding


def _cache_inputs(B, H, M, N, D, mean, std, seed):
    g_ = torch.Generator(device="cuda").manual_seed(seed)
    q = torch.randn(B, H, M, D, generator=g_, device="cuda").bfloat16()
    k = torch.randn(B, H, N, D, generator=g_, device="cuda").bfloat16()
    v = torch.randn(B, H, N, D, generator=g_, device="cuda").bfloat16()
    gates = F.logsigmoid(torch.randn(B, H, N, generator=g_, device="cuda") * std + mean)
    ss = torch.randint(0, 8192, (B,), generator=g_, device="cuda")
    return q, k, v, gates, ss


@pytest.mark.parametrize("M", [128, 1])
def test_config5_chunked_prefill_and_decode(fa, M):
    B, H, N, D = 16, 16, 32768, 128
    q, k, v, gates, ss = _cache_inputs(B, H, M, N, D, 2.0, 1.0, 5)
    out = fa(q, k, v, gates, head_first=True, seq_start=ss)
    for b in range(B):
        ref = O.forgetting_attention_ref(q[b:b + 1], k[b:b + 1], v[b:b + 1], gates[b:b + 1], head_first=True, seq_start=ss[b:b + 1])
        assert_parity("out", out[b:b + 1], ref, context=b)


@pytest.mark.parametrize("M", [128, 1])
@pytest.mark.parametrize("thr", [None, "auto"])
def test_cache_shapes_under_strong_decay(fa, M, thr):
    """The chunked-prefill (key-split tiled kernel) and decode (streaming kernel) shapes with the strongly decaying
    gates of the pruned configuration, logits ~ N(-1, 2): the cumulative sums reach ~ -7e4 at N = 32768 (fp32 ulp
    2^-7), so a kernel that rounds a score at the magnitude of the cumulative sums instead of forming the difference
    of two nearby sums first loses the result.  out and the log-normaliser, every batch, against the oracle."""
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention
    B, H, N, D = 16, 16, 32768, 128
    q, k, v, gates, ss = _cache_inputs(B, H, M, N, D, -1.0, 2.0, 6)
    ss = (ss * 4 - 1000).clamp_min(0)   # up to 31764: some batches keep only the last few hundred keys
    out, lse, _ = ForgettingAttention.apply(q, k, v, gates, ss, True, None, thr, True, False)
    assert torch.cumsum(gates[0, 0], 0)[-1].item() < -2e4
    for b in range(B):
        # fp64 oracle: its cumulative sums are exact where an fp32 running sum of 32768 terms is not; the operator's
        # own sums are correctly rounded fp32 (half an ulp, 4e-3 at 7e4), which bounds the error of a score and of lse
        ref, lse_ref = O.forgetting_attention_ref(q[b:b + 1], k[b:b + 1], v[b:b + 1], gates[b:b + 1], head_first=True,
                                                  seq_start=ss[b:b + 1], return_lse=True, compute_dtype=torch.float64)
        assert_parity("out", out[b:b + 1], ref, context=b)
        assert torch.isfinite(lse[b]).all() and (lse[b].double() - lse_ref[0]).abs().max().item() <= 2e-2, b
