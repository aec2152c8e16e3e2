"""Pins of the integer oracle (oracle/routing.py) by what the mathematics fixes: brute-force loops,
permutation/sortedness/stability properties, offsets identities, and stock torch ops."""

import numpy as np
import pytest
import torch

from oracle import routing as oracle
from tests.utils import get_1d_tensor_sizes, zipf_ids


def _brute_count(ids, bins):
    out = [0] * bins
    for v in ids:
        out[int(v)] += 1
    return out


def _insertion_sort_perm(ids):
    """textbook stable sort: insertion sort of (key, original position)"""
    order = []
    for i, v in enumerate(ids):
        j = len(order)
        while j > 0 and ids[order[j - 1]] > v:
            j -= 1
        order.insert(j, i)
    return order


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_continuous_count_brute_force(dtype):
    rng = np.random.default_rng(0)
    for n in [0, 1, 2, 63, 64, 65, 1000]:
        for bins in [2, 3, 8, 72]:
            ids = rng.integers(0, bins, n).astype(dtype)
            got = oracle.continuous_count(ids, bins)
            assert got.dtype == np.uint32 and got.shape == (bins,)
            assert got.tolist() == _brute_count(ids, bins)
            assert int(got.sum()) == n


def test_continuous_count_special_cases():
    assert oracle.continuous_count(np.array([5, 7, 9], np.int64), 1).tolist() == [3]  # bins == 1 never looks at the values
    assert oracle.continuous_count(np.zeros(0, np.int32), 4).tolist() == [0, 0, 0, 0]
    assert oracle.continuous_count(np.full(100, 2, np.int32), 4).tolist() == [0, 0, 100, 0]
    with pytest.raises(ValueError):
        oracle.continuous_count(np.array([-1], np.int64), 4)


def test_continuous_count_matches_torch_bincount_on_reference_grid():
    # the reference test's grid: bins = 72, n over the 1-D size grid, seed 42 (continuous_count_test.py:22-41)
    for n in get_1d_tensor_sizes()[::7]:
        torch.manual_seed(42)
        x = torch.randint(0, 72, (n,))
        want = x.bincount(minlength=72).to(torch.uint32)
        assert oracle.continuous_count(x.numpy(), 72).tolist() == want.view(torch.int32).tolist()


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_route_brute_force_stable(dtype):
    rng = np.random.default_rng(1)
    for n in [1, 2, 20, 64, 200]:
        for E in [1, 2, 5, 8]:
            ids = rng.integers(0, E, n).astype(dtype)
            r = oracle.route(ids, E)
            assert r["sorted_scattered_idxs"].tolist() == _insertion_sort_perm(ids.tolist())
            assert r["sorted_expert_idxs"].tolist() == sorted(ids.tolist())
            assert r["counts"].tolist() == _brute_count(ids, E)


def test_route_properties_large():
    for ids in [torch.randint(0, 64, (200000,), generator=torch.Generator().manual_seed(0), dtype=torch.int32),
                zipf_ids(200000, 64, 1.1, 0)]:
        a = ids.numpy()
        r = oracle.route(a, 64)
        perm = r["sorted_scattered_idxs"]
        assert np.array_equal(np.sort(perm), np.arange(a.size))  # a permutation
        s = a[perm]
        assert np.array_equal(s, r["sorted_expert_idxs"]) and np.all(np.diff(s) >= 0)  # sorted
        assert np.all(np.diff(perm)[np.diff(s) == 0] > 0)  # stable
        incl, excl, c = r["offsets_inclusive"], r["offsets_exclusive"], r["counts"].astype(np.int64)
        assert incl[-1] == a.size and excl[0] == 0
        assert np.array_equal(incl - excl, c) and np.array_equal(excl[1:], incl[:-1])
        for e in (0, 17, 63):  # rows [excl, incl) of expert e really hold expert e
            assert np.all(s[excl[e]:incl[e]] == e)
        # the same answer as torch's stable sort and cumsum (what the layer would compute, moe/__init__.py:210-217)
        ts, ti = torch.from_numpy(a).sort(stable=True)
        assert np.array_equal(ti.numpy(), perm) and np.array_equal(ts.numpy(), s)
        assert np.array_equal(torch.from_numpy(a).long().bincount(minlength=64).cumsum(-1).numpy(), incl)
