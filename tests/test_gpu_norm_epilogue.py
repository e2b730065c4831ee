"""GPU parity of the forward with the layer's output norm and gate in its epilogue:
forgetting_attention_norm_gate(q, k, v, log_fgate, gate, w) must equal
group_norm_gated(forgetting_attention(q, k, v, log_fgate), gate, w, is_rms_norm=True, num_groups=heads),
forward and all six gradients.

Checked against the oracle (fp32 attention, its output rounded to the 16-bit dtype as the operator
stores it, then the oracle's per-head RMS norm and gate; autograd through both) with the operator's
tolerance, and against the two separate operators of this library much tighter: they run the same
arithmetic on the same rounded attention output and differ only in the order in which the squares of
a row are added, i.e. by at most a unit in the last place of y.
"""
import ctypes as C

import pytest
import torch

from conftest import REL_TOL, assert_parity, make_inputs, rel_err
from oracle import fox_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from forgetting_transformer import forgetting_attention, forgetting_attention_norm_gate, group_norm, group_norm_gated
    from forgetting_transformer.ops import _lib
    _lib.load()
    return forgetting_attention, forgetting_attention_norm_gate, group_norm_gated, group_norm


def _ulp_close(got, want, dtype, ulps):
    eps = (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10) * ulps
    want = want.float()
    tol = eps * want.abs().clamp_min(1e-3 * want.abs().max().item())
    return bool(((got.float() - want).abs() <= tol).all())


def _gate_and_weight(shape, H, D, dtype, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    gate = (torch.randn(shape, generator=gen, device="cuda") * 2).to(dtype)
    w = torch.rand(H * D, generator=gen, device="cuda") + 0.5
    dy = torch.randn(shape, generator=gen, device="cuda").to(dtype)
    return gate, w, dy


def _run_case(ops, B, H, M, N, D, dtype, activation, head_first, seq, thr=None, seed=0, eps=1e-6):
    fa, fused, gng, gn = ops
    q, k, v, lf, _, ss = make_inputs(B, H, M, N, D, dtype=dtype, device="cuda", head_first=head_first, seq_start=seq,
                                     seed=seed, gate_mean=1.0)
    gate, w, dy = _gate_and_weight(q.shape, H, D, dtype, seed + 100)
    gated = activation is not None
    flat = (lambda t: t.transpose(1, 2).reshape(B, M, H * D)) if head_first else (lambda t: t.reshape(B, M, H * D))

    def leaves():
        ts = [t.detach().clone().requires_grad_() for t in (q, k, v, lf, gate, w)]
        return ts

    # oracle: fp32 attention, rounded to the dtype where the operator stores o, then the norm in fp32
    qr, kr, vr, lr, gr, wr = leaves()
    o_ref = O.forgetting_attention_ref(qr, kr, vr, lr, head_first=head_first, seq_start=ss)
    o_ref = o_ref + (o_ref.detach().to(dtype).float() - o_ref.detach())        # rounded value, straight-through gradient
    y_ref = O.group_norm_gated_ref(flat(o_ref), flat(gr.float()) if gated else None, wr, H, eps, activation or "none")
    y_ref.backward(flat(dy.float()))

    # the two separate operators
    qu, ku, vu, lu, gu, wu = leaves()
    o_u = fa(qu, ku, vu, lu, head_first=head_first, seq_start=ss, adaptive_threshold=thr)
    y_u = gng(flat(o_u), flat(gu), wu, None, activation, is_rms_norm=True, num_groups=H, eps=eps) if gated else \
        gn(flat(o_u), wu, None, is_rms_norm=True, num_groups=H, eps=eps)
    y_u.backward(flat(dy))

    # fused
    qf, kf, vf, lf2, gf, wf = leaves()
    y_f = fused(qf, kf, vf, lf2, gf if gated else None, wf, activation=activation or "sigmoid", eps=eps,
                head_first=head_first, seq_start=ss, adaptive_threshold=thr)
    assert y_f.shape == q.shape and y_f.dtype == dtype
    if not head_first:
        assert y_f.is_contiguous()            # (B, T, H, D): the reshape to (B, T, H*D) is a view
    y_f.backward(dy)

    ctx = (B, H, M, N, D, dtype, activation, head_first, seq, thr)
    assert _ulp_close(flat(y_f), y_u, dtype, 1.01), ("y against the separate operators", ctx)
    assert_parity("y_epilogue", flat(y_f), y_ref, context=ctx)
    names = ["dq", "dk", "dv", "dlog_fgate"] + (["dgate"] if gated else []) + ["dweight"]
    sets = [(qf, qu, qr), (kf, ku, kr), (vf, vu, vr), (lf2, lu, lr)] + ([(gf, gu, gr)] if gated else []) + [(wf, wu, wr)]
    for name, (f, u, r) in zip(names, sets):
        assert f.grad is not None and f.grad.shape == r.grad.shape, name
        rows = name in ("dq", "dk", "dv", "dgate")
        assert_parity(name + "_epi", f.grad, r.grad, rows=rows, context=ctx)
        # the backward runs the same kernels on a bit-identical o; rstd may differ in its last place, which can flip
        # the 16-bit rounding of single elements of do and dgate (at most 2^-8 of the largest element)
        assert rel_err(f.grad, u.grad) <= 5e-3, (name, "against the separate operators", rel_err(f.grad, u.grad), ctx)


@pytest.mark.parametrize("D", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dims_and_dtypes(ops, D, dtype):
    _run_case(ops, 2, 3, 200, 300, D, dtype, "sigmoid", head_first=False, seq=None, seed=D)


@pytest.mark.parametrize("activation", ["sigmoid", "swish", None])
@pytest.mark.parametrize("head_first,seq", [(False, [7, 130]), (True, None)])
def test_activations_layouts_and_left_padding(ops, activation, head_first, seq):
    _run_case(ops, 2, 4, 257, 257, 64, torch.bfloat16, activation, head_first=head_first, seq=seq, seed=3)


def test_with_pruning_threshold(ops):
    _run_case(ops, 1, 2, 1024, 1024, 128, torch.bfloat16, "sigmoid", head_first=False, seq=None, thr=-8.0, seed=5)


@pytest.mark.parametrize("M,N", [(1, 4096), (128, 8192)])
def test_shapes_that_split_the_key_loop_take_two_passes(ops, M, N):
    """Decode and chunked prefill: the library runs the plain forward and the norm kernel behind the same call."""
    _run_case(ops, 2, 4, M, N, 128, torch.bfloat16, "sigmoid", head_first=False, seq=None, seed=M)


def test_with_gate_logits_fused_too(ops):
    """Gate logits in, normalised and gated output out: equal to the operator fed with logsigmoid(logits) and followed
    by the norm, forward and the gradient of the logits."""
    import torch.nn.functional as F
    fa, fused, gng, gn = ops
    B, H, T, D = 2, 4, 300, 64
    q, k, v, _, _, ss = make_inputs(B, H, T, T, D, dtype=torch.bfloat16, device="cuda", head_first=False, seq_start=[0, 90],
                                    seed=13)
    gate, w, dy = _gate_and_weight(q.shape, H, D, torch.bfloat16, 13)
    gen = torch.Generator(device="cuda").manual_seed(2)
    logits = (torch.randn((B, T, H), generator=gen, device="cuda") * 2 + 1).bfloat16()
    xu = logits.clone().requires_grad_()
    o = fa(q, k, v, F.logsigmoid(xu.float()), seq_start=ss)
    y_u = gng(o.reshape(B, T, H * D), gate.reshape(B, T, H * D), w, None, "sigmoid", is_rms_norm=True, num_groups=H)
    y_u.backward(dy.reshape(B, T, H * D))
    xf = logits.clone().requires_grad_()
    y_f, lg = fused(q, k, v, xf, gate, w, seq_start=ss, fgate_is_logit=True)
    y_f.backward(dy)
    assert lg.dtype == torch.float32 and lg.shape == logits.shape and not lg.requires_grad
    assert (lg - F.logsigmoid(logits.float())).abs().max().item() <= 2e-6 * lg.abs().max().item()
    assert rel_err(y_f.reshape(B, T, H * D), y_u) <= 5e-3
    assert xf.grad.dtype == logits.dtype and rel_err(xf.grad, xu.grad) <= REL_TOL


def test_rows_left_of_seq_start_come_out_zero(ops):
    fa, fused, gng, gn = ops
    B, H, T, D = 2, 2, 192, 64
    q, k, v, lf, _, ss = make_inputs(B, H, T, T, D, dtype=torch.bfloat16, device="cuda", head_first=False,
                                     seq_start=[40, 100], seed=9)
    gate, w, _ = _gate_and_weight(q.shape, H, D, torch.bfloat16, 1)
    y = fused(q, k, v, lf, gate, w, seq_start=ss)
    assert torch.isfinite(y).all()
    for b, s in enumerate([40, 100]):
        assert (y[b, :s] == 0).all()


def _c_call(B, H, M, N, D, q, k, v, lf, gate, w, want_o, eps=1e-6, alias=False):
    """fox_attn_fwd_norm_gate straight through the C ABI on (B, H, M, D) views of (B, M, H, D) memory."""
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import _view
    lib = _lib.load()
    dev = q.device
    c = torch.empty((B, H, N), dtype=torch.float32, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.fox_cumsum_fwd(C.c_void_p(lf.data_ptr()), lf.stride(0), lf.stride(1), lf.stride(2), None,
                                  C.c_void_p(c.data_ptr()), B, H, N, stream), "fox_cumsum_fwd")
    L = torch.empty((B, H, M), dtype=torch.float32, device=dev)
    o = torch.zeros((B, M, H, D), dtype=q.dtype, device=dev).transpose(1, 2)
    y = torch.zeros((B, M, H, D), dtype=q.dtype, device=dev).transpose(1, 2)
    rstd = torch.zeros((B, M, H), dtype=torch.float32, device=dev)
    ov = _view(o) if want_o else _lib.View()
    args = _lib.FwdArgs(_lib.Dims(B, H, M, N, D, 0), _view(q), _view(k), _view(v), ov, c.data_ptr(), L.data_ptr(), None, None,
                        D ** -0.5, None, None, 0)
    epi = _lib.FwdEpilogue(_view(gate), _view(o if alias else y), w.data_ptr(), rstd.data_ptr(), eps, _lib.ACT_SIGMOID)
    rc = lib.fox_attn_fwd_norm_gate(C.byref(args), C.byref(epi), stream)
    torch.cuda.synchronize()
    return rc, o, y, rstd, L


def test_c_abi_output_optional_and_rstd_layout(ops):
    B, H, M, N, D = 2, 3, 130, 130, 128
    q, k, v, lf, _, _ = make_inputs(B, H, M, N, D, dtype=torch.bfloat16, device="cuda", head_first=True, seed=2)
    gate, w, _ = _gate_and_weight(q.shape, H, D, torch.bfloat16, 2)
    rc, o, y, rstd, L = _c_call(B, H, M, N, D, q, k, v, lf, gate, w, want_o=True)
    assert rc == 0
    rc2, o2, y2, rstd2, L2 = _c_call(B, H, M, N, D, q, k, v, lf, gate, w, want_o=False)
    assert rc2 == 0
    assert torch.equal(y, y2) and torch.equal(rstd, rstd2) and torch.equal(L, L2)
    assert (o2 == 0).all() and o.abs().max() > 0          # without o nothing is written there
    want = 1.0 / torch.sqrt(o.float().square().mean(dim=-1) + 1e-6)       # (B, H, M)
    assert torch.allclose(rstd, want.transpose(1, 2), rtol=1e-5, atol=0)  # stored as (B, M, H)


def test_c_abi_rejects_bad_arguments(ops):
    from forgetting_transformer.ops import _lib
    B, H, M, N, D = 1, 2, 64, 64, 64
    q, k, v, lf, _, _ = make_inputs(B, H, M, N, D, dtype=torch.bfloat16, device="cuda", head_first=True, seed=2)
    gate, w, _ = _gate_and_weight(q.shape, H, D, torch.bfloat16, 2)
    rc, *_ = _c_call(B, H, M, N, D, q, k, v, lf, gate, w, want_o=True, alias=True)
    assert rc != 0 and b"alias" in _lib.load().fox_last_error()
    # a single-query shape needs o for its two passes
    q1 = q[:, :, :1].contiguous()
    g1 = gate[:, :, :1].contiguous()
    rc, *_ = _c_call(B, H, 1, N, D, q1, k, v, lf, g1, w, want_o=False)
    assert rc != 0 and b"adjacent heads" in _lib.load().fox_last_error()


def test_training_layer_shape_matches_the_separate_operators(ops):
    """B4 T16384 H16 D128, the benchmark's layer shape: every element of y against the two-kernel path."""
    fa, fused, gng, gn = ops
    B, H, T, D = 4, 16, 16384, 128
    q, k, v, lf, _, _ = make_inputs(B, H, T, T, D, dtype=torch.bfloat16, device="cuda", head_first=False, seed=11,
                                    gate_mean=3.0)
    gate, w, _ = _gate_and_weight(q.shape, H, D, torch.bfloat16, 11)
    with torch.no_grad():
        y_f = fused(q, k, v, lf, gate, w)
        o = fa(q, k, v, lf)
        y_u = gng(o.reshape(B, T, H * D), gate.reshape(B, T, H * D), w, None, "sigmoid", is_rms_norm=True, num_groups=H)
    assert _ulp_close(y_f.reshape(B, T, H * D), y_u, torch.bfloat16, 1.01)
