"""The chain the FoX (Pro) attention layer runs around the operator, end to end on the GPU against the
oracle chain: token shift of the key and value projections, per-head RMS norm of queries and keys, the
pruning threshold from the norm weights, attention fed with the gate logits, gated per-head RMS norm of
the output (reference: model/forgetting_transformer/modeling_forgetting_transformer.py:68-95, 303-325,
343-346, 366-423).  The projections themselves are plain matmuls and stay in torch on both sides.

Forward and every gradient that flows back through the chain are compared with the operator's bar,
max|x - ref| <= 2e-2 * max|ref|; the oracle chain runs in fp32 from the same 16-bit inputs.
"""
import math

import pytest
import torch
import torch.nn.functional as F

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


def _leaves(B, T, H, D, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    rnd = lambda *shape, scale=1.0: torch.randn(*shape, generator=gen, device="cuda") * scale
    leaves = dict(
        q_proj=rnd(B, T, H * D).bfloat16(), k_proj=rnd(B, T, H * D).bfloat16(), v_proj=rnd(B, T, H * D).bfloat16(),
        k_alpha_logit=rnd(B, T, H), v_alpha_logit=rnd(B, T, H),          # shift weights: sigmoid of a projection (:84-93)
        fgate_logit=(rnd(B, T, H, scale=2.0) + 2.0).bfloat16(), ogate=rnd(B, T, H * D).bfloat16(),
        q_norm_w=(torch.rand(H * D, generator=gen, device="cuda") * 0.5 + 0.75),
        k_norm_w=(torch.rand(H * D, generator=gen, device="cuda") * 0.5 + 0.75),
        out_norm_w=(torch.rand(H * D, generator=gen, device="cuda") + 0.5),
    )
    dout = rnd(B, T, H * D).bfloat16()
    return leaves, dout


def _chain_device(ft, L, B, T, H, D, seq_start, tolerance):
    alpha_k, alpha_v = torch.sigmoid(L["k_alpha_logit"]), torch.sigmoid(L["v_alpha_logit"])
    k = ft.token_shift(L["k_proj"].view(B, T, H, D), alpha_k, 1.0 - alpha_k).reshape(B, T, H * D)
    v = ft.token_shift(L["v_proj"].view(B, T, H, D), alpha_v, 1.0 - alpha_v)
    q = ft.group_norm(L["q_proj"], L["q_norm_w"], None, is_rms_norm=True, num_groups=H).view(B, T, H, D)
    k = ft.group_norm(k, L["k_norm_w"], None, is_rms_norm=True, num_groups=H).view(B, T, H, D)
    thr = ft.qk_norm_threshold(L["q_norm_w"], L["k_norm_w"], H, D, T, tolerance) if tolerance is not None else None
    # the layer hands the operator head-first *views* of (B, T, H*D) memory (:353-359)
    o, log_fgate = ft.forgetting_attention_from_logits(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                                       L["fgate_logit"].transpose(1, 2), head_first=True,
                                                       seq_start=seq_start, sm_scale=1 / math.sqrt(D), adaptive_threshold=thr)
    o = o.transpose(1, 2).reshape(B, T, H * D)
    y = ft.group_norm_gated(o, L["ogate"], L["out_norm_w"], None, "sigmoid", is_rms_norm=True, num_groups=H, eps=1e-6)
    return y, log_fgate


def _chain_oracle(L, B, T, H, D, seq_start):
    f = {n: t.float() for n, t in L.items()}
    alpha_k, alpha_v = torch.sigmoid(f["k_alpha_logit"]), torch.sigmoid(f["v_alpha_logit"])
    # the device chain rounds to bf16 between its stages; the oracle chain does the same so that only the
    # arithmetic inside each stage differs
    r16 = lambda t: t.bfloat16().float()
    k = r16(O.token_shift_ref(f["k_proj"].view(B, T, H, D), alpha_k, 1.0 - alpha_k)).reshape(B, T, H * D)
    v = r16(O.token_shift_ref(f["v_proj"].view(B, T, H, D), alpha_v, 1.0 - alpha_v))
    q = r16(O.group_norm_ref(f["q_proj"], f["q_norm_w"], H, 1e-5)).view(B, T, H, D)
    k = r16(O.group_norm_ref(k, f["k_norm_w"], H, 1e-5)).view(B, T, H, D)
    log_fgate = F.logsigmoid(f["fgate_logit"])
    o = O.forgetting_attention_ref(q, k, v, log_fgate, head_first=False, seq_start=seq_start, sm_scale=1 / math.sqrt(D))
    o = r16(o).reshape(B, T, H * D)
    return O.group_norm_gated_ref(o, f["ogate"], f["out_norm_w"], H, 1e-6, "sigmoid"), log_fgate


@pytest.mark.parametrize("B,T,H,D,seq,tolerance", [(2, 640, 3, 64, None, None), (2, 900, 2, 128, [0, 333], -10.0),
                                                    (1, 2048, 12, 64, None, -10.0)])
def test_layer_chain_forward_and_gradients(ft, B, T, H, D, seq, tolerance):
    leaves, dout = _leaves(B, T, H, D, seed=T + D)
    seq_start = None if seq is None else torch.tensor(seq, dtype=torch.long, device="cuda")

    dev = {n: t.detach().clone().requires_grad_() for n, t in leaves.items()}
    y, log_fgate = _chain_device(ft, dev, B, T, H, D, seq_start, tolerance)
    y.backward(dout)

    ref = {n: t.detach().clone().requires_grad_() for n, t in leaves.items()}
    y_ref, log_fgate_ref = _chain_oracle(ref, B, T, H, D, seq_start)
    y_ref.backward(dout.float())

    assert y.dtype == torch.bfloat16 and y.shape == (B, T, H * D)
    assert rel_err(y, y_ref) <= REL_TOL, ("y", rel_err(y, y_ref))
    assert torch.allclose(log_fgate.transpose(1, 2), log_fgate_ref, rtol=1e-5, atol=1e-6)   # the by-product the decode cache keeps
    for name in leaves:
        got, want = dev[name].grad, ref[name].grad
        assert got is not None and torch.isfinite(got).all(), name
        assert rel_err(got, want) <= REL_TOL, (name, rel_err(got, want))
