"""Decoding on the cache that grows in place: prefill, single-token steps and a chunk of several tokens, each
attention call fed with the cache's views (whose (batch, head) slices are `capacity` rows apart).  Every call
must equal, bit for bit, the same call on contiguous concatenated copies (the reference's cache hands out those,
fgate_cache.py:107-116), and match the oracle on the whole prefix at the operator's bar."""
import pytest
import torch

from conftest import assert_parity, make_inputs
from oracle import fox_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("D,max_length", [(64, None), (128, 512)])
def test_decode_loop_on_the_growing_cache(D, max_length):
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from forgetting_transformer import FgateDynamicCache, forgetting_attention
    B, H, T0, T = 2, 4, 300, 300 + 40 + 17
    q, k, v, g, _, ss = make_inputs(B, H, T, T, D, dtype=torch.bfloat16, device="cuda", head_first=True, seq_start=[0, 37],
                                    seed=31, gate_mean=1.0)
    cache = FgateDynamicCache(max_length=max_length, min_capacity=64)
    moved = 0
    stages = [(0, T0)] + [(t, t + 1) for t in range(T0, T0 + 40)] + [(T0 + 40, T)]
    for lo, hi in stages:
        ptr = cache._key_buf[0].data_ptr() if len(cache) else None
        kk, vv, gg = cache.update(k[:, :, lo:hi], v[:, :, lo:hi], g[:, :, lo:hi], 0)
        moved += ptr is not None and cache._key_buf[0].data_ptr() != ptr
        assert kk.shape == (B, H, hi, D) and gg.shape == (B, H, hi)
        assert kk.is_contiguous() == (hi == cache.capacity())          # otherwise the slices are `capacity` rows apart
        with torch.no_grad():
            out = forgetting_attention(q[:, :, lo:hi], kk, vv, gg, head_first=True, seq_start=ss)
            same = forgetting_attention(q[:, :, lo:hi], k[:, :, :hi].contiguous(), v[:, :, :hi].contiguous(),
                                        g[:, :, :hi].contiguous(), head_first=True, seq_start=ss)
        assert torch.equal(out, same), (lo, hi)
        ref = O.forgetting_attention_ref(q[:, :, lo:hi], k[:, :, :hi], v[:, :, :hi], g[:, :, :hi], head_first=True, seq_start=ss)
        assert_parity("out", out, ref, context=(lo, hi))
    assert moved <= (0 if max_length else 3)     # 64 -> 320 at the prefill, then at most doubling: a few moves in 42 calls
