"""GPU parity of the fused gate prologue: forgetting_attention_from_logits(q, k, v, x) must equal
forgetting_attention(q, k, v, logsigmoid(x.float())) -- forward, and all four gradients, where the
gradient of the logits goes through the derivative of logsigmoid.  Checked against the oracle
(autograd through torch's logsigmoid) with the operator's tolerance, and against the unfused
operator much tighter: the two only differ in how logsigmoid is rounded.
"""
import pytest
import torch
import torch.nn.functional as F

from conftest import REL_TOL, make_inputs, rel_err
from oracle import fox_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from forgetting_transformer import forgetting_attention, forgetting_attention_from_logits
    from forgetting_transformer.ops import _lib
    _lib.load()
    return forgetting_attention, forgetting_attention_from_logits


@pytest.mark.parametrize("gate_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("head_first,seq", [(False, None), (True, [5, 170])])
def test_fused_gate_matches_unfused_and_oracle(ops, gate_dtype, head_first, seq):
    fa, fa_logits = ops
    B, H, M, N, D = 2, 3, 200, 300, 64
    q, k, v, _, do, ss = make_inputs(B, H, M, N, D, dtype=torch.bfloat16, device="cuda", head_first=head_first,
                                     seq_start=seq, seed=21)
    g = torch.Generator(device="cuda").manual_seed(4)
    shape = (B, H, N) if head_first else (B, N, H)
    logits = (torch.randn(shape, generator=g, device="cuda") * 2.0 + 1.0).to(gate_dtype)

    # oracle: autograd through torch's logsigmoid of the fp32 cast, as the layer does
    xr = logits.detach().clone().requires_grad_()
    qr, kr, vr = (t.detach().clone().requires_grad_() for t in (q, k, v))
    ref = O.forgetting_attention_ref(qr, kr, vr, F.logsigmoid(xr.float()), head_first=head_first, seq_start=ss)
    ref.backward(do.float())

    # unfused operator
    xu = logits.detach().clone().requires_grad_()
    qu, ku, vu = (t.detach().clone().requires_grad_() for t in (q, k, v))
    out_u = fa(qu, ku, vu, F.logsigmoid(xu.float()), head_first=head_first, seq_start=ss)
    out_u.backward(do)

    # fused
    xf = logits.detach().clone().requires_grad_()
    qf, kf, vf = (t.detach().clone().requires_grad_() for t in (q, k, v))
    out_f, log_fgate = fa_logits(qf, kf, vf, xf, head_first=head_first, seq_start=ss)
    out_f.backward(do)

    assert log_fgate.dtype == torch.float32 and log_fgate.shape == logits.shape and not log_fgate.requires_grad
    want_lg = F.logsigmoid(logits.float())
    assert (log_fgate - want_lg).abs().max().item() <= 2e-6 * max(1.0, want_lg.abs().max().item())
    assert xf.grad.dtype == gate_dtype and xf.grad.shape == logits.shape

    for name, got, unf, r in (("out", out_f, out_u, ref), ("dq", qf.grad, qu.grad, qr.grad), ("dk", kf.grad, ku.grad, kr.grad),
                              ("dv", vf.grad, vu.grad, vr.grad), ("dlogits", xf.grad, xu.grad, xr.grad)):
        assert torch.isfinite(got).all(), name
        assert rel_err(got, r) <= REL_TOL, (name, "oracle", rel_err(got, r))
        # fused vs unfused: same kernels, logsigmoid rounded differently by at most a few fp32 ulps;
        # 16-bit outputs may flip one rounding
        assert rel_err(got, unf) <= 1e-2, (name, "unfused", rel_err(got, unf))


def test_fused_gate_with_pruning_and_extreme_logits(ops):
    """Saturated logits (|x| up to 30) exercise both branches of the stable logsigmoid and its derivative."""
    fa, fa_logits = ops
    B, H, T, D = 1, 2, 513, 128
    q, k, v, _, do, _ = make_inputs(B, H, T, T, D, dtype=torch.bfloat16, device="cuda", head_first=True, seed=8)
    g = torch.Generator(device="cuda").manual_seed(6)
    logits = torch.randn(B, H, T, generator=g, device="cuda") * 12.0
    logits[..., ::7] = 30.0
    logits[..., 3::11] = -30.0
    xf, xu = logits.clone().requires_grad_(), logits.clone().requires_grad_()
    out_f, _ = fa_logits(q, k, v, xf, head_first=True, adaptive_threshold="auto")
    out_u = fa(q, k, v, F.logsigmoid(xu), head_first=True, adaptive_threshold="auto")
    out_f.backward(do)
    out_u.backward(do)
    assert torch.isfinite(xf.grad).all()
    assert rel_err(out_f, out_u) <= 1e-2
    assert rel_err(xf.grad, xu.grad) <= 1e-3


@pytest.mark.parametrize("gate_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_log_gates_are_never_positive_and_sums_never_increase(ops, gate_dtype):
    """Extreme logits (around +-20 and +-80, zeros, the largest finite values of the dtype): logsigmoid from the
    hardware exp / log must stay <= 0, so that the cumulative sums never increase -- the pruning-bound searches rely
    on that order."""
    import ctypes as C
    from forgetting_transformer.ops import _lib
    lib = _lib.load()
    B, H, N = 2, 3, 6000
    g = torch.Generator().manual_seed(5)
    centres = torch.tensor([-80.0, -20.0, -1e-3, 0.0, 1e-3, 20.0, 80.0])
    x = centres[torch.randint(0, 7, (B, H, N), generator=g)] + torch.randn(B, H, N, generator=g) * 0.5
    x[0, 0, :4] = torch.tensor([float(torch.finfo(gate_dtype).max) if gate_dtype != torch.float32 else 3e38, 88.0, 16.7, 17.4])
    x = x.to(gate_dtype).cuda()
    log_fgate = torch.empty(B, H, N, device="cuda")
    c = torch.empty(B, H, N, device="cuda")
    dt = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_FP16, torch.float32: _lib.DTYPE_FP32}[gate_dtype]
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.fox_gate_cumsum_fwd(x.data_ptr(), dt, *x.stride(), None, log_fgate.data_ptr(), c.data_ptr(), B, H, N, stream),
               "fox_gate_cumsum_fwd")
    assert torch.isfinite(log_fgate).all() and (log_fgate <= 0).all()
    assert (c[..., 1:] <= c[..., :-1]).all()
    want = F.logsigmoid(x.double())
    assert (log_fgate.double() - want).abs().max().item() <= 1e-6 * max(1.0, want.abs().max().item())
