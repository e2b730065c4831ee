"""The entry point that allocates nothing, fox_attn_fwd_noalloc, against fox_attn_fwd.

Both are called straight through the C ABI on the same inputs.  fox_attn_fwd gets a caller-allocated
workspace for the key-split partials, fox_attn_fwd_noalloc uses the array inside the library; the
kernels are the same, so o and lse must agree bit for bit.  Two calls in a row share the library's
array, the second with a smaller input (its partials cover only the start of what the first call
left behind), then a single-query call and a shape that is not split at all.
"""
import ctypes as C

import pytest
import torch

from conftest import make_inputs

pytestmark = pytest.mark.gpu


def _fwd_pair(lib, _lib, _view, B, H, M, N, D, seed, seq_start=None, thr=None):
    q, k, v, g, _, ss = make_inputs(B, H, M, N, D, device="cuda", seed=seed, gate_mean=2.0, seq_start=seq_start)
    dims = _lib.Dims(B, H, M, N, D, _lib.DTYPE_BF16)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    c = torch.empty(B, H, N, device="cuda")
    _lib.check(lib.fox_cumsum_fwd(g.data_ptr(), *g.stride(), None if ss is None else ss.data_ptr(), c.data_ptr(),
                                  B, H, N, stream), "fox_cumsum_fwd")
    thr_t = None if thr is None else torch.full((B, H), thr, device="cuda")
    need = C.c_int64(0)
    _lib.check(lib.fox_attn_fwd_workspace_bytes(C.byref(dims), C.byref(need)), "fox_attn_fwd_workspace_bytes")
    ws = torch.empty(max(need.value, 16), dtype=torch.uint8, device="cuda")
    res = []
    for name in ("fox_attn_fwd", "fox_attn_fwd_noalloc"):
        o = torch.full_like(q, float("nan"))
        lse = torch.full((B, H, M), float("nan"), device="cuda")
        own_ws = name == "fox_attn_fwd" and need.value > 0
        args = _lib.FwdArgs(dims, _view(q), _view(k), _view(v), _view(o), c.data_ptr(), lse.data_ptr(),
                            None if ss is None else ss.data_ptr(), None if thr_t is None else thr_t.data_ptr(),
                            1.0 / D ** 0.5, None, ws.data_ptr() if own_ws else None, need.value if own_ws else 0)
        _lib.check(getattr(lib, name)(C.byref(args), stream), name)
        res.append((o, lse))
    torch.cuda.synchronize()
    return res, need.value, (q, k, v, g, ss)


def test_noalloc_forward_matches_the_workspace_forward():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import _view
    from oracle import fox_oracle as O
    lib = _lib.load()

    cases = [
        # first call: a chunked-prefill shape, 16 key splits per query tile (17 MB of partials)
        dict(B=4, H=4, M=128, N=8192, D=128, seed=1, seq_start=[0, 100, 4000, 8100]),
        # second call, smaller: overwrites only the start of what the first one left in the array
        dict(B=2, H=2, M=64, N=2048, D=64, seed=2, thr=-10.0),
        # one query row against the cache (streaming kernel, 8 splits)
        dict(B=2, H=2, M=1, N=4096, D=64, seed=3, seq_start=[7, 1000]),
        # not split: the library's array is not touched
        dict(B=2, H=4, M=256, N=256, D=32, seed=4),
    ]
    expect_split = [True, True, True, False]
    for case, split in zip(cases, expect_split):
        (ref, got), need, (q, k, v, g, ss) = _fwd_pair(lib, _lib, _view, **case)
        assert (need > 0) == split, (case, need)
        assert torch.isfinite(got[0]).all(), case
        assert torch.equal(ref[0], got[0]), case                                   # o, bit for bit
        assert torch.equal(ref[1].view(torch.int32), got[1].view(torch.int32)), case   # lse, bit for bit (-inf included)
        if case.get("thr") is None:   # and both are the operator's result: the oracle on the same inputs
            out_ref, lse_ref = O.forgetting_attention_ref(q, k, v, g, head_first=True, seq_start=ss, return_lse=True)
            assert (got[0].float() - out_ref.float()).abs().max().item() <= 2e-2 * out_ref.abs().max().item(), case
            fin = torch.isfinite(lse_ref)
            assert torch.equal(fin, torch.isfinite(got[1])), case
            assert (got[1][fin] - lse_ref[fin]).abs().max().item() <= 2e-2, case
