"""GPU parity of continuous_count and route against the integer oracle: bit-exact
(reference test: tests/functional/continuous_count_test.py:22-41, exact equality
with bincount for bins = 72 over the 1-D size grid, int32 and int64)."""

import numpy as np
import pytest
import torch

from oracle import routing as oracle
from tests.utils import get_1d_tensor_sizes, np_of, zipf_ids

pytestmark = pytest.mark.gpu

_MAX_EXPERTS = 72
_SEED = 42


def _kb():
    from xma import KernelBackend

    return KernelBackend.rocm


@pytest.mark.parametrize("dtype", [torch.long, torch.int])
def test_continuous_count_size_grid(dtype):
    from xma import set_seed
    from xma.functional import continuous_count

    for n in get_1d_tensor_sizes():
        set_seed(_SEED)
        x = torch.randint(0, _MAX_EXPERTS, (n,), device="cuda", dtype=dtype)
        got = continuous_count(x=x, bins=_MAX_EXPERTS, kernel_backend=_kb())
        assert got.dtype == torch.uint32 and got.shape == (_MAX_EXPERTS,)
        want = oracle.continuous_count(x.cpu().numpy(), _MAX_EXPERTS)
        assert np.array_equal(np_of(got), want), f"n={n}"


def test_continuous_count_edge_cases():
    from xma.functional import continuous_count

    # bins == 1 shortcut, empty input, single hot bin, misaligned view, many bins, out-of-range ids ignored
    x = torch.randint(0, 5, (1000,), device="cuda")
    assert continuous_count(x, 1, kernel_backend=_kb()).tolist() == [1000]
    assert continuous_count(x[:0], 8, kernel_backend=_kb()).tolist() == [0] * 8
    hot = torch.full((100003,), 3, device="cuda", dtype=torch.int32)
    assert continuous_count(hot, 8, kernel_backend=_kb()).tolist() == [0, 0, 0, 100003, 0, 0, 0, 0]
    base = torch.randint(0, 64, (70001,), device="cuda", dtype=torch.int32)
    for off in (1, 2, 3):
        v = base[off:]
        assert np.array_equal(np_of(continuous_count(v, 64, kernel_backend=_kb())), oracle.continuous_count(v.cpu().numpy(), 64))
    for bins in (2, 3, 255, 1024, 5000, 20000):
        y = torch.randint(0, bins, (50000,), device="cuda")
        assert np.array_equal(np_of(continuous_count(y, bins, kernel_backend=_kb())), oracle.continuous_count(y.cpu().numpy(), bins))
    z = torch.tensor([0, 1, 9, -1, 3, 3, 100], device="cuda", dtype=torch.int64)
    assert continuous_count(z, 4, kernel_backend=_kb()).tolist() == [1, 1, 0, 2]


def test_continuous_count_overwrites_or_accumulates():
    """The two histogram ops behind the functional: continuous_count_set writes the counts whatever the output held
    (one workgroup for up to 4096 ids, per-unit histograms plus a storing reduction beyond), continuous_count adds to
    what the caller put there, as the reference's kernel does (cuda_implementation.py:139-145)."""
    from xma.rocm import ops

    for n in (0, 1, 4096, 4097, 70000, 300000):
        ids = torch.randint(0, 72, (n,), device="cuda", dtype=torch.int32)
        want = oracle.continuous_count(ids.cpu().numpy(), 72)
        y = torch.full((72,), -559038737, dtype=torch.int32, device="cuda").view(torch.uint32)
        ops.continuous_count_set_rocm(ids, y)
        assert np.array_equal(np_of(y), want), n
        acc = torch.zeros(72, dtype=torch.uint32, device="cuda")
        ops.continuous_count_rocm(ids, acc, None)
        ops.continuous_count_rocm(ids, acc, None)
        assert np.array_equal(np_of(acc), 2 * want), n


@pytest.mark.parametrize("dist", ["uniform", "zipf", "sorted"])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_continuous_count_4m(dist, dtype):
    """The routing benchmark configuration: 4 Mi ids over E = 64, uniform and Zipf(s = 1.1); also the sorted input the MoE feeds."""
    from xma.functional import continuous_count

    n, E = 4 * 1024 * 1024, 64
    g = torch.Generator().manual_seed(0)
    ids = zipf_ids(n, E, 1.1, 0, dtype) if dist == "zipf" else torch.randint(0, E, (n,), generator=g, dtype=dtype)
    if dist == "sorted":
        ids = ids.sort().values
    got = continuous_count(ids.cuda(), E, kernel_backend=_kb())
    assert np.array_equal(np_of(got), oracle.continuous_count(ids.numpy(), E))
    assert int(np_of(got).astype(np.int64).sum()) == n


def _check_route(ids_cpu: torch.Tensor, E: int):
    from xma.layers.moe import rocm_implementation as R

    counts, incl, excl, sorted_e, sorted_s = R.route(ids_cpu.cuda(), E)
    want = oracle.route(ids_cpu.numpy(), E)
    assert np.array_equal(np_of(counts), want["counts"])
    assert np.array_equal(np_of(incl), want["offsets_inclusive"])
    assert np.array_equal(np_of(excl), want["offsets_exclusive"])
    assert np.array_equal(np_of(sorted_s), want["sorted_scattered_idxs"])
    assert np.array_equal(np_of(sorted_e), want["sorted_expert_idxs"])


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_route_small_and_ragged(dtype):
    g = torch.Generator().manual_seed(1)
    for n in [1, 2, 63, 64, 65, 127, 2047, 2048, 2049, 4097, 8191, 8192, 8193, 50000]:
        for E in [1, 2, 3, 8, 64, 72, 128, 1000]:
            _check_route(torch.randint(0, E, (n,), generator=g, dtype=dtype), E)
    # empty experts, a single expert taking everything, already sorted, reverse sorted
    _check_route(torch.full((5000,), 5, dtype=dtype), 8)
    _check_route(torch.randint(0, 3, (9000,), generator=g, dtype=dtype) * 3, 8)
    s = torch.randint(0, 64, (30000,), generator=g, dtype=dtype).sort().values
    _check_route(s, 64)
    _check_route(s.flip(0).contiguous(), 64)
    _check_route(torch.zeros(0, dtype=dtype), 4)


@pytest.mark.parametrize("dist", ["uniform", "zipf"])
def test_route_4m(dist):
    """The routing benchmark configuration at full size: bit-exact against the oracle plus the size-independent properties
    (permutation, sortedness, stability, offsets identities)."""
    from xma.layers.moe import rocm_implementation as R

    n, E = 4 * 1024 * 1024, 64
    g = torch.Generator().manual_seed(0)
    ids = zipf_ids(n, E, 1.1, 0) if dist == "zipf" else torch.randint(0, E, (n,), generator=g, dtype=torch.int32)
    _check_route(ids, E)
    counts, incl, excl, sorted_e, sorted_s = R.route(ids.cuda(), E)
    perm = sorted_s.cpu().numpy()
    assert np.array_equal(np.sort(perm), np.arange(n))
    se = ids.numpy()[perm]
    assert np.all(np.diff(se) >= 0)
    same = np.diff(se) == 0
    assert np.all(np.diff(perm)[same] > 0)  # stable: original order inside an expert
    assert int(incl[-1]) == n and int(excl[0]) == 0


def test_route_moe_shapes():
    """routing of the three MoE configurations (top-k of random logits, skewed for the fine-grained one)"""
    g = torch.Generator().manual_seed(0)
    for T, E, k, bias in [(8192, 8, 2, 0.0), (16384, 64, 6, 1.5), (32768, 128, 8, 0.0)]:
        logits = torch.randn(T, E, generator=g) + bias * torch.randn(E, generator=g)
        sel = logits.topk(k, dim=-1).indices
        _check_route(sel.flatten(), E)


def test_route_rank_methods_agree():
    """The scatter kernel has two ways to rank an id among the equal ids of its wave: the value returned by an LDS atomic
    add (relies on gfx950 applying the lanes of one instruction in lane order) and wave ballots (relies on nothing).
    Both must give the oracle's stable permutation, bit for bit, on uniform, skewed, sorted and single-expert ids."""
    from xma.rocm import get_library

    lib = get_library()
    g = torch.Generator().manual_seed(9)
    cases = [
        (torch.randint(0, 64, (1 << 20,), generator=g, dtype=torch.int32), 64),
        (zipf_ids(300001, 64, 1.1, 3), 64),
        (torch.randint(0, 128, (70000,), generator=g, dtype=torch.int64).sort().values, 128),
        (torch.full((20000,), 2, dtype=torch.int32), 3),
        (torch.randint(0, 1000, (50000,), generator=g, dtype=torch.int64), 1000),
    ]
    try:
        for method in (1, 0):
            assert lib.xma_rocm_route_set_rank_method(method) == 0
            for ids, E in cases:
                print(f"rank method {method}: n={ids.numel()} E={E}", flush=True)
                _check_route(ids, E)
        assert lib.xma_rocm_route_set_rank_method(2) == -1
    finally:
        lib.xma_rocm_route_set_rank_method(0)
