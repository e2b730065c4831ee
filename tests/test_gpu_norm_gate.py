"""GPU parity of the gated per-head RMS norm kernels (through the C ABI) against the oracle.

Tolerances: y, dx, dg are fp32 expressions rounded once to the 16-bit dtype -> within two units in the
last place of the oracle evaluated in fp32 (the kernels use the fast exponential and reassociate the
products); dweight is an fp32 sum over all rows -> 1e-3 relative to its scale.  The reference's test
of this op (fuse_norm_gate.py has none for the group variant) gives no bar of its own.
"""
import pytest
import torch

from oracle import fox_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gng():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from forgetting_transformer import group_norm_gated
    from forgetting_transformer.ops import _lib
    _lib.load()
    return group_norm_gated


def _close(got, want_fp32, dtype, ulps=2.0):
    eps = (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10) * ulps
    want = want_fp32.float()
    scale = want.abs().max().item()
    tol = eps * want.abs().clamp_min(1e-3 * scale)
    return bool(((got.float() - want).abs() <= tol).all())


def _case(gng, shape, G, dtype, activation, seed=0, eps=1e-6, w_dtype=torch.float32):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(shape, generator=gen, device="cuda").to(dtype)
    g = (torch.randn(shape, generator=gen, device="cuda") * 2).to(dtype)
    dy = torch.randn(shape, generator=gen, device="cuda").to(dtype)
    w = (torch.rand(shape[-1], generator=gen, device="cuda") + 0.5).to(w_dtype)
    xr, gr, wr = (t.detach().float().clone().requires_grad_() for t in (x, g, w))
    ref = O.group_norm_gated_ref(xr, gr, wr, G, eps, activation)
    ref.backward(dy.float())
    x1, g1, w1 = (t.detach().clone().requires_grad_() for t in (x, g, w))
    y = gng(x1, g1, w1, None, activation, is_rms_norm=True, num_groups=G, eps=eps)
    assert y.shape == x.shape and y.dtype == dtype
    y.backward(dy)
    assert _close(y, ref, dtype), "y"
    assert _close(x1.grad, xr.grad, dtype, ulps=3.0), "dx"
    assert _close(g1.grad, gr.grad, dtype, ulps=3.0), "dg"
    assert w1.grad.dtype == w_dtype
    assert (w1.grad.float() - wr.grad).abs().max().item() <= (1e-3 if w_dtype == torch.float32 else 1e-2) * wr.grad.abs().max().item()


@pytest.mark.parametrize("D", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("activation", ["sigmoid", "swish"])
def test_head_dims_dtypes_activations(gng, D, dtype, activation):
    _case(gng, (3, 50, 4 * D), 4, dtype, activation, seed=D)


@pytest.mark.parametrize("shape,G", [((1, 16), 1), ((33, 2048), 16), ((2, 1, 256), 2), ((65, 3 * 64), 3)])
def test_shapes(gng, shape, G):
    _case(gng, shape, G, torch.bfloat16, "sigmoid", seed=shape[0])


def test_layer_configuration_and_weight_dtype(gng):
    """The FoX layer's call: (B, T, hidden) bf16, groups = heads, eps 1e-6 (modeling_forgetting_transformer.py:243)."""
    _case(gng, (2, 300, 16 * 128), 16, torch.bfloat16, "sigmoid", seed=2, eps=1e-6, w_dtype=torch.bfloat16)


def test_weight_gradient_is_reproducible(gng):
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(4096, 1024, generator=gen, device="cuda").bfloat16()
    g = torch.randn(4096, 1024, generator=gen, device="cuda").bfloat16()
    dy = torch.randn(4096, 1024, generator=gen, device="cuda").bfloat16()
    w = torch.rand(1024, generator=gen, device="cuda")
    grads = []
    for _ in range(3):
        w1 = w.clone().requires_grad_()
        gng(x, g, w1, None, "sigmoid", is_rms_norm=True, num_groups=8).backward(dy)
        grads.append(w1.grad.clone())
    assert torch.equal(grads[0], grads[1]) and torch.equal(grads[0], grads[2])


def test_full_size_properties(gng):
    """Training-layer shape (B4 T16384, 16 heads of 128): oracle on a slice of rows; scale invariance:
    RMS norm ignores a per-(row, head) rescaling of x by a power of two exactly."""
    B, T, G, D = 4, 16384, 16, 128
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(B, T, G * D, generator=gen, device="cuda").bfloat16()
    g = torch.randn(B, T, G * D, generator=gen, device="cuda").bfloat16()
    w = torch.rand(G * D, generator=gen, device="cuda") + 0.5
    y = gng(x, g, w, None, "sigmoid", is_rms_norm=True, num_groups=G, eps=0.0)
    ref = O.group_norm_gated_ref(x[2, 100:612].float(), g[2, 100:612].float(), w, G, 0.0, "sigmoid")
    assert _close(y[2, 100:612], ref, torch.bfloat16)
    y4 = gng(x * 4.0, g, w, None, "sigmoid", is_rms_norm=True, num_groups=G, eps=0.0)
    assert torch.equal(y, y4)


def test_unsupported_options_raise(gng):
    x = torch.randn(4, 64, device="cuda").bfloat16()
    w = torch.ones(64, device="cuda")
    with pytest.raises(NotImplementedError):
        gng(x, x, w, torch.zeros(64, device="cuda"), "sigmoid", is_rms_norm=True, num_groups=1)
    with pytest.raises(NotImplementedError):
        gng(x, x, w, None, "sigmoid", is_rms_norm=False, num_groups=1)
    with pytest.raises(ValueError):
        gng(x, x, w, None, "relu", is_rms_norm=True, num_groups=1)
