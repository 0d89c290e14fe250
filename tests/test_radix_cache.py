"""The native radix prefix cache (C ABI of include/msgl_radix_cache.h behind the reference's
class names) against the reference's own scenarios and, operation by operation, against the
pure-Python oracle on random workloads.  Host code only: runs without a GPU."""
import random

import pytest
import torch

from _radix_util import (NativeHybrid, NativePlain, OracleHybrid, OraclePlain, SCENARIOS,
                         run_scenario)


@pytest.mark.parametrize("name", sorted(SCENARIOS))
def test_reference_scenarios_on_the_native_tree(name):
    run_scenario(name, NativeHybrid if SCENARIOS[name][1] else NativePlain)


def test_fast_compare_key_matches_the_reference_contract():
    from mini_sglang_amd_kernel import fast_compare_key as f
    from oracle.radix_oracle import fast_compare_key as want

    rng = random.Random(3)
    for dtype in (torch.int32, torch.int64):
        t = lambda v: torch.tensor(v, dtype=dtype)
        assert f(t([]), t([])) == 0 and f(t([1]), t([])) == 0
        assert f(t([1, 2, 3]), t([1, 2, 3])) == 3
        assert f(t([1, 2, 3]), t([1, 2, 4, 5])) == 2
        for _ in range(200):
            n, m = rng.randrange(0, 70), rng.randrange(0, 70)
            a = [rng.randrange(3) for _ in range(n)]
            b = a[: rng.randrange(0, n + 1)] + [rng.randrange(3) for _ in range(m)]
            assert f(t(a), t(b)) == want(a, b)
        big = torch.arange(1 << 20, dtype=dtype)
        other = big.clone()
        other[-7] = -1
        assert f(big, other) == (1 << 20) - 7
    hi = torch.tensor([1 << 40, 5], dtype=torch.int64)  # differs only above bit 31
    assert f(hi, torch.tensor([1 << 41, 5], dtype=torch.int64)) == 0
    with pytest.raises(RuntimeError, match="fast_compare_key: Both arrays must be 1D."):
        f(torch.zeros((2, 2), dtype=torch.int32), torch.zeros(2, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="Both arrays must be contiguous."):
        f(torch.zeros(8, dtype=torch.int32)[::2], torch.zeros(2, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="Both arrays must have the same dtype."):
        f(torch.zeros(2, dtype=torch.int32), torch.zeros(2, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="Arrays must be int32 or int64."):
        f(torch.zeros(2, dtype=torch.int16), torch.zeros(2, dtype=torch.int16))


def _random_tokens(rng, vocab, max_len):
    return [rng.randrange(vocab) for _ in range(rng.randrange(0, max_len + 1))]


@pytest.mark.parametrize("hybrid,seed,vocab", [(False, 1, 2), (False, 2, 4), (True, 3, 2),
                                               (True, 4, 3), (True, 5, 50)])
def test_random_operations_agree_with_the_oracle(hybrid, seed, vocab):
    """Inserts, matches, locks, unlocks and both kinds of eviction in random order on a small
    vocabulary (deep shared prefixes, many splits); after every operation the two trees must
    return the same values and hold the same nodes, counts, snapshots and timestamps."""
    rng = random.Random(seed)
    a = (OracleHybrid if hybrid else OraclePlain)(num_pages=400, num_slots=12)
    b = (NativeHybrid if hybrid else NativePlain)(num_pages=400, num_slots=12)
    locked = []  # (token path, oracle node, native node)
    for step in range(600):
        op = rng.random()
        if op < 0.40:
            toks = _random_tokens(rng, vocab, 24)
            slot = None
            if hybrid and toks and rng.random() < 0.6 and a.pool.available_size:
                slot = a.pool.alloc()
                assert b.pool.alloc() == slot
            if len(toks) > a.available_size:
                continue
            pa, pb = a.cache_prefix(toks, slot), b.cache_prefix(toks, slot)
            assert pa == pb, step
        elif op < 0.65:
            toks = _random_tokens(rng, vocab, 28)
            ra, rb = a.match_prefix(toks), b.match_prefix(toks)
            assert (ra[0], ra[2]) == (rb[0], rb[2]), step
            if ra[0] and rng.random() < 0.5:
                a.lock(ra[1])
                b.lock(rb[1])
                locked.append((ra[1], rb[1]))
        elif op < 0.80 and locked:
            na, nb = locked.pop(rng.randrange(len(locked)))
            a.unlock(na)
            b.unlock(nb)
        elif op < 0.92:
            size = rng.randrange(0, a.sizes()[0] + 1)
            ea, eb = a.evict(size), b.evict(size)
            assert ea == eb, step
            a.free(ea)
            b.free(eb)
        elif hybrid:
            count = rng.randrange(0, 4)
            assert a.evict_for_mamba(count) == b.evict_for_mamba(count), step
        assert a.sizes() == b.sizes(), step
        assert a.free_pages == b.free_pages, step
        assert a.dump() == b.dump(), step
        if hybrid:
            assert sorted(a.collect_mamba_slots()) == sorted(b.collect_mamba_slots())
            assert sorted(a.pool._free_slots) == sorted(b.pool._free_slots)
            ca, cb = a.coldest_snapshot_node(), b.coldest_snapshot_node()
            assert (ca is None) == (cb is None)
            if ca is not None:
                assert ca.mamba_slot == cb.mamba_slot
        a.page_balance()
        b.page_balance()
    for na, nb in locked:
        a.unlock(na)
        b.unlock(nb)
    assert a.sizes() == b.sizes() and a.sizes()[1] == 0
    everything = a.sizes()[0]
    assert a.evict(everything) == b.evict(everything)
    assert b.dump() == [] and b.root_is_leaf()


def test_locked_prefixes_survive_eviction_and_unlock_errors_are_reported():
    m = NativePlain(num_pages=64)
    m.cache_prefix([1, 2, 3, 4])
    m.cache_prefix([1, 2, 7, 8])
    m.cache_prefix([5, 6])
    _, node, indices = m.match_prefix([1, 2, 3, 4])
    m.lock(node)
    assert m.sizes() == (4, 4)  # [1,2] and [3,4] protected; [7,8] and [5,6] evictable
    m.free(m.evict(4))
    assert m.match_prefix([1, 2, 3, 4])[2] == indices  # untouched
    assert m.match_prefix([1, 2, 7, 8])[0] == 2 and m.match_prefix([5, 6])[0] == 0
    with pytest.raises(AssertionError, match="Cannot evict"):
        m.evict(1)
    m.unlock(node)
    with pytest.raises(AssertionError, match="not locked"):
        m.unlock(node)
    assert m.sizes() == (4, 0)
    m.page_balance()


def test_node_views_follow_the_tree():
    from mini_sglang_amd.kvcache import RadixCacheManager

    mgr = RadixCacheManager()
    t = lambda *v: torch.tensor(v, dtype=torch.int32)
    assert mgr.insert_prefix(t(1, 2, 3, 4), t(10, 11, 12, 13)) == 0
    assert mgr.insert_prefix(t(1, 2, 9), t(10, 11, 20)) == 2
    root = mgr.root_node
    assert root.is_root() and not root.is_leaf() and list(root.children) == [1]
    upper = root.children[1]
    assert upper._key.tolist() == [1, 2] and upper.value.tolist() == [10, 11]
    assert sorted(upper.children.keys()) == [3, 9] and 3 in upper.children and 4 not in upper.children
    lower = upper.children[3]
    assert lower.parent is upper and upper.parent is root and lower.is_leaf()
    assert lower.get_match_len(t(3, 4, 5)) == 2
    assert root.children[1] is upper  # one view per node
    handle, indices = mgr.match_prefix(t(1, 2, 3, 4, 5))
    assert handle.cached_len == 4 and handle.node is lower and indices.tolist() == [10, 11, 12, 13]
    mgr.evict(3)  # both leaves (2 + 1 values), least recently used first
    with pytest.raises(KeyError):
        lower.length
    assert upper.is_leaf()
    with pytest.raises(NotImplementedError):
        mgr.reset()
    with pytest.raises(TypeError, match="int32"):
        mgr.match_prefix(torch.tensor([1, 2], dtype=torch.int64))
