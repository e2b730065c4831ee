"""The decode cache that grows in place (forgetting_transformer.FgateDynamicCache) against the reference's
append-by-concatenation semantics (fgate_cache.py:78-118): same tensors out of every call, whatever the capacity
policy, plus the bookkeeping methods the generation utilities call.  CPU only; the attention on top of it is
covered by the GPU tests."""
import pytest
import torch

from forgetting_transformer import FgateDynamicCache


def _tokens(B, H, T, D, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, H, T, D, generator=g).bfloat16(), torch.randn(B, H, T, D, generator=g).bfloat16(),
            -torch.rand(B, H, T, generator=g))


@pytest.mark.parametrize("max_length,min_capacity", [(None, 256), (None, 64), (400, 256)])
def test_update_equals_concatenation(max_length, min_capacity):
    B, H, D, layers = 2, 3, 16, 2
    cache = FgateDynamicCache(max_length=max_length, min_capacity=min_capacity)
    want = [None] * layers
    steps = [70, 1, 1, 5, 1, 130, 1, 1, 60]
    for s, t in enumerate(steps):
        for layer in range(layers):
            k, v, g = _tokens(B, H, t, D, 100 * s + layer)
            want[layer] = (k, v, g) if want[layer] is None else tuple(
                torch.cat([a, b], dim=2 if a.ndim == 4 else -1) for a, b in zip(want[layer], (k, v, g)))
            ptr = cache._key_buf[layer].data_ptr() if layer < len(cache) else None
            cap = cache.capacity(layer)
            got = cache.update(k, v, g, layer)
            for a, b in zip(got, want[layer]):
                assert a.shape == b.shape and torch.equal(a, b)
            if ptr is not None and want[layer][0].shape[2] <= cap:
                assert cache._key_buf[layer].data_ptr() == ptr        # nothing moved: only the new tokens were copied
            assert got[0].stride(-1) == 1 and got[0].stride(2) == D     # rows of a (batch, head) slice stay adjacent
        assert cache.get_seq_length() == cache.get_seq_length(1) == sum(steps[:s + 1])
        assert cache._seen_tokens == sum(steps[:s + 1])
    assert len(cache) == layers and cache.get_seq_length(5) == 0
    assert cache.get_max_length() == max_length
    if max_length is None:
        assert cache.capacity() >= sum(steps) and cache.capacity() % 64 == 0
    else:
        assert cache.capacity() == max_length
        with pytest.raises(ValueError, match="built for 400"):
            cache.update(*_tokens(B, H, 200, D, 1), 0)
    k0, v0, g0 = cache[0]
    assert torch.equal(k0, want[0][0]) and torch.equal(g0, want[0][2])
    assert [torch.equal(a[0], w[0]) for a, w in zip(cache, want)] == [True, True]
    assert all(torch.equal(a, b) for a, b in zip(cache.to_legacy_cache()[1], want[1]))
    with pytest.raises(KeyError):
        cache[2]


def test_growth_is_geometric_and_reserve_prevents_it():
    cache = FgateDynamicCache(min_capacity=64)
    caps = set()
    for s in range(700):
        cache.update(*_tokens(1, 1, 1, 8, s), 0)
        caps.add(cache.capacity())
    assert sorted(caps) == [64, 128, 256, 512, 1024]          # 5 reallocations for 700 single-token steps
    cache.reserve(5000)
    ptr = cache._key_buf[0].data_ptr()
    for s in range(300):
        cache.update(*_tokens(1, 1, 1, 8, s), 0)
    assert cache._key_buf[0].data_ptr() == ptr and cache.get_seq_length() == 1000


def test_crop_and_continue():
    B, H, D = 2, 2, 8
    cache = FgateDynamicCache()
    k, v, g = _tokens(B, H, 50, D, 0)
    cache.update(k, v, g, 0)
    cache.crop(-10)
    assert cache.get_seq_length() == 40 and cache._seen_tokens == 40
    cache.crop(100)                                            # longer than the cache: nothing happens
    assert cache.get_seq_length() == 40
    k2, v2, g2 = _tokens(B, H, 3, D, 1)
    kk, vv, gg = cache.update(k2, v2, g2, 0)
    assert torch.equal(kk, torch.cat([k[:, :, :40], k2], dim=2)) and torch.equal(gg, torch.cat([g[..., :40], g2], dim=-1))


def test_batch_operations():
    B, H, D = 4, 2, 8
    cache = FgateDynamicCache()
    for layer in range(2):
        cache.update(*_tokens(B, H, 20, D, layer), layer)
    ref = [tuple(t.clone() for t in cache[layer]) for layer in range(2)]
    parts = cache.batch_split(B, 2)
    assert len(parts) == 2 and torch.equal(parts[1][0][0], ref[0][0][2:4]) and parts[0].get_seq_length() == 20
    joined = FgateDynamicCache.from_batch_splits(parts)
    assert all(torch.equal(a, b) for layer in range(2) for a, b in zip(joined[layer], ref[layer]))
    idx = torch.tensor([3, 1])
    cache.batch_select_indices(idx)
    assert all(torch.equal(a, b[idx]) for a, b in zip(cache[1], ref[1]))
    cache.batch_repeat_interleave(2)
    assert cache[0][0].shape[0] == 4 and torch.equal(cache[0][0][1], ref[0][0][3]) and torch.equal(cache[0][2][2], ref[0][2][1])
    cache.update(*_tokens(4, H, 1, D, 9), 0)                   # still usable afterwards
    assert cache.get_seq_length(0) == 21 and cache.get_seq_length(1) == 20


def test_splits_and_parent_grow_independently():
    """The reference builds a new tensor on every update (torch.cat, fgate_cache.py:107-116), so a split and its
    parent never see each other's later tokens; the in-place cache must behave the same although a split starts
    out as views of the parent's buffers."""
    B, H, D = 4, 2, 8
    cache = FgateDynamicCache(min_capacity=64)         # spare capacity in the parent's buffers
    cache.update(*_tokens(B, H, 10, D, 0), 0)
    before = [t.clone() for t in cache[0]]
    parts = cache.batch_split(B, 2)
    k1, v1, g1 = _tokens(2, H, 3, D, 5)
    k2, v2, g2 = _tokens(B, H, 3, D, 6)
    got_part = [t.clone() for t in parts[0].update(k1, v1, g1, 0)]     # the split grows first ...
    got_full = [t.clone() for t in cache.update(k2, v2, g2, 0)]        # ... then the parent, over the same positions
    for got, old, new, sl in ((got_part, before, (k1, v1, g1), slice(0, 2)), (got_full, before, (k2, v2, g2), slice(None))):
        for x, o, n in zip(got, old, new):
            assert torch.equal(x, torch.cat([o[sl], n], dim=2))
    for x, o, n in zip(parts[0][0], before, (k1, v1, g1)):            # and the split still holds its own tokens
        assert torch.equal(x, torch.cat([o[:2], n], dim=2))
    for x, o in zip(parts[1][0], before):                              # the untouched split is unchanged
        assert torch.equal(x, o[2:4])


def test_shift_states_and_errors():
    cache = FgateDynamicCache()
    ks, vs = torch.zeros(2, 16), torch.ones(2, 16)
    cache.update_shift_cache(ks, vs, 0)
    assert cache.key_shift_cache[0] is ks and cache.value_shift_cache[0] is vs
    with pytest.raises(AssertionError):
        cache.update_shift_cache(ks, vs, 2)                    # layers in order
    with pytest.raises(AssertionError, match="log_fgate must be"):
        cache.update(torch.zeros(1, 1, 2, 8), torch.zeros(1, 1, 2, 8), torch.zeros(1, 2), 0)
    with pytest.raises(NotImplementedError):
        FgateDynamicCache.from_legacy_cache(())
