"""GPU parity of the plain per-head RMS norm (the FoX layer's QK-norm) through the C ABI against the oracle,
and of the pruning threshold derived from its weights.

Tolerances as for the gated norm: y and dx are fp32 expressions rounded once to the 16-bit dtype -> within
two / three units in the last place of the oracle evaluated in fp32; dweight is an fp32 sum over all rows ->
1e-3 relative to its scale.  The reference has no test of its own for this op.
"""
import math

import pytest
import torch

from conftest import REL_TOL, rel_err
from oracle import fox_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ft():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import forgetting_transformer
    from forgetting_transformer.ops import _lib
    _lib.load()
    return forgetting_transformer


def _close(got, want_fp32, dtype, ulps=2.0):
    eps = (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10) * ulps
    want = want_fp32.float()
    scale = want.abs().max().item()
    tol = eps * want.abs().clamp_min(1e-3 * scale)
    return bool(((got.float() - want).abs() <= tol).all())


def _case(fn, shape, G, dtype, seed=0, eps=1e-5, w_dtype=torch.float32, x=None):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    if x is None:
        x = torch.randn(shape, generator=gen, device="cuda").to(dtype)
    dy = torch.randn(shape, generator=gen, device="cuda").to(dtype)
    w = (torch.rand(shape[-1], generator=gen, device="cuda") + 0.5).to(w_dtype)
    xr, wr = (t.detach().float().clone().requires_grad_() for t in (x, w))
    ref = O.group_norm_ref(xr, wr, G, eps)
    ref.backward(dy.float())
    x1, w1 = x.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    if x.stride() != x1.stride():  # keep the caller's strides
        x1 = torch.empty_strided(x.shape, x.stride(), dtype=dtype, device="cuda").copy_(x).requires_grad_()
    y = fn(x1, w1)
    assert y.shape == x.shape and y.dtype == dtype
    y.backward(dy)
    assert _close(y, ref, dtype), "y"
    assert _close(x1.grad, xr.grad, dtype, ulps=3.0), "dx"
    assert w1.grad.dtype == w_dtype
    assert (w1.grad.float() - wr.grad).abs().max().item() <= (1e-3 if w_dtype == torch.float32 else 1e-2) * wr.grad.abs().max().item()


@pytest.mark.parametrize("D", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_group_norm_head_dims_and_dtypes(ft, D, dtype):
    G = 4
    _case(lambda x, w: ft.group_norm(x, w, None, is_rms_norm=True, num_groups=G), (3, 50, G * D), G, dtype, seed=D)


@pytest.mark.parametrize("shape,G", [((1, 16), 1), ((33, 2048), 16), ((2, 1, 256), 2), ((65, 3 * 64), 3)])
def test_group_norm_shapes(ft, shape, G):
    _case(lambda x, w: ft.group_norm(x, w, None, is_rms_norm=True, num_groups=G), shape, G, torch.bfloat16, seed=shape[0])


def test_shared_weight_rms_norm_on_head_split_tensor(ft):
    """RMSNorm(head_dim) on (B, T, H, D) (modeling_forgetting_transformer.py:261-262, 323-325): one group, the
    last dimension is the head."""
    B, T, H, D = 2, 70, 5, 64
    _case(lambda x, w: ft.rms_norm(x, w), (B, T, H, D), 1, torch.bfloat16, seed=3, w_dtype=torch.bfloat16)


def test_unsupported_options_raise(ft):
    x = torch.randn(4, 64, device="cuda").bfloat16()
    w = torch.ones(64, device="cuda")
    with pytest.raises(NotImplementedError):
        ft.group_norm(x, w, torch.zeros(64, device="cuda"), is_rms_norm=True, num_groups=2)
    with pytest.raises(NotImplementedError):
        ft.group_norm(x, w, None, is_rms_norm=False, num_groups=2)
    with pytest.raises(NotImplementedError):
        ft.group_norm(x, w, None, residual=x, is_rms_norm=True, num_groups=2)
    with pytest.raises(ValueError):
        ft.group_norm(x, w, None, is_rms_norm=True, num_groups=3)


def test_raw_entry_point_ignores_gate_pointers_when_ungated(ft):
    """fox_norm_gate_fwd/bwd with FOX_ACT_NONE and NULL g/dg against the oracle, straight through ctypes."""
    import ctypes as C
    from forgetting_transformer.ops import _lib
    lib = _lib.load()
    R, G, D = 77, 4, 32
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(R, G * D, generator=gen, device="cuda").bfloat16()
    dy = torch.randn(R, G * D, generator=gen, device="cuda").bfloat16()
    w = torch.rand(G * D, generator=gen, device="cuda") + 0.5
    y, dx = torch.empty_like(x), torch.empty_like(x)
    rstd = torch.empty(R, G, device="cuda")
    dw = torch.empty(G * D, device="cuda")
    nbytes = C.c_int64(0)
    assert lib.fox_norm_gate_workspace_bytes(R, G, D, C.byref(nbytes)) == 0
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device="cuda")
    args = _lib.NormGateArgs(R, G, D, _lib.DTYPE_BF16, _lib.ACT_NONE, 1e-5, x.data_ptr(), G * D, None, 0, w.data_ptr(),
                             y.data_ptr(), G * D, rstd.data_ptr(), dy.data_ptr(), G * D, dx.data_ptr(), G * D, None, 0,
                             dw.data_ptr(), ws.data_ptr())
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.fox_norm_gate_fwd(C.byref(args), stream) == 0, lib.fox_last_error()
    assert lib.fox_norm_gate_bwd(C.byref(args), stream) == 0, lib.fox_last_error()
    torch.cuda.synchronize()
    xr, wr = x.float().requires_grad_(), w.clone().requires_grad_()
    ref = O.group_norm_ref(xr, wr, G, 1e-5)
    ref.backward(dy.float())
    assert _close(y, ref, torch.bfloat16) and _close(dx, xr.grad, torch.bfloat16, ulps=3.0)
    want_rstd = 1 / torch.sqrt(x.float().view(R, G, D).square().mean(-1) + 1e-5)
    assert torch.allclose(rstd, want_rstd, rtol=1e-5, atol=0)
    assert (dw - wr.grad).abs().max().item() <= 1e-3 * wr.grad.abs().max().item()
    # a gated activation with a NULL gate is refused on the host
    args.activation = _lib.ACT_SIGMOID
    assert lib.fox_norm_gate_fwd(C.byref(args), stream) != 0


@pytest.mark.parametrize("share", [False, True])
def test_qk_norm_threshold_matches_restatement_and_prunes_safely(ft, share):
    """QK-norm -> threshold from the weights -> attention: the pruned result must agree with the unpruned one
    (the bound guarantees a pruned mass <= exp(tolerance)), and the helper with the restated rule."""
    B, T, H, D = 2, 1024, 4, 64
    gen = torch.Generator(device="cuda").manual_seed(11 + share)
    hidden = torch.randn(B, T, H * D, generator=gen, device="cuda").bfloat16()
    hidden_k = torch.randn(B, T, H * D, generator=gen, device="cuda").bfloat16()
    v = torch.randn(B, T, H, D, generator=gen, device="cuda").bfloat16()
    wq = torch.rand(D if share else H * D, generator=gen, device="cuda") * 0.5 + 0.25
    wk = torch.rand(D if share else H * D, generator=gen, device="cuda") * 0.5 + 0.25
    if share:
        q = ft.rms_norm(hidden.view(B, T, H, D), wq)
        k = ft.rms_norm(hidden_k.view(B, T, H, D), wk)
    else:
        q = ft.group_norm(hidden, wq, None, is_rms_norm=True, num_groups=H).view(B, T, H, D)
        k = ft.group_norm(hidden_k, wk, None, is_rms_norm=True, num_groups=H).view(B, T, H, D)
    tol = -10.0
    thr = ft.qk_norm_threshold(wq, wk, H, D, T, tol, share_param_across_head=share)
    want = O.qk_norm_threshold_ref(wq.cpu(), wk.cpu(), H, D, T, tol, share)
    assert thr.shape == want.shape and torch.allclose(thr.cpu(), want, rtol=1e-6, atol=0)
    # every logit of the normalised rows respects the bound the threshold is built from
    bound = (-(thr - tol) - math.log(T)) / 2
    logits = torch.einsum("bihd,bjhd->bhij", q.float(), k.float()) / math.sqrt(D)
    assert (logits.abs().amax(dim=(0, 2, 3)) <= (bound.expand(H) if share else bound) * 1.01).all()
    log_fgate = torch.nn.functional.logsigmoid(torch.randn(B, T, H, generator=gen, device="cuda") * 2 - 1)
    full = ft.forgetting_attention(q, k, v, log_fgate, sm_scale=1 / math.sqrt(D))
    pruned = ft.forgetting_attention(q, k, v, log_fgate, sm_scale=1 / math.sqrt(D), adaptive_threshold=thr)
    ref = O.forgetting_attention_ref(q.float(), k.float(), v.float(), log_fgate, sm_scale=1 / math.sqrt(D))
    assert rel_err(pruned, ref) <= 2e-2 and rel_err(full, ref) <= 2e-2
    assert (pruned.float() - full.float()).abs().max().item() <= 2 * math.exp(tol) * v.float().abs().max().item() + 2 ** -8 * full.float().abs().max().item()
