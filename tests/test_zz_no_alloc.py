"""xma_rocm_route_static, the entry point that allocates nothing (its scratch is a device array inside the library),
against xma_rocm_route with a caller's workspace: bit-exact on counts, offsets and the stable permutation, on two calls
in a row of which the second is smaller (the scratch keeps the first call's contents), then on a larger one again, and
the size limit is rejected before anything is launched.  Both entry points are called through the C ABI."""

import numpy as np
import pytest
import torch

from tests.utils import np_of, zipf_ids

pytestmark = pytest.mark.gpu


def _route(lib, ids, E, static):
    from xma.rocm.loader import check

    n, dev = ids.numel(), ids.device
    out = dict(
        counts=torch.full((E,), 0x7FFFFFFF, dtype=torch.int32, device=dev),
        incl=torch.full((E,), -7, dtype=torch.int64, device=dev),
        excl=torch.full((E,), -7, dtype=torch.int64, device=dev),
        sorted_e=torch.full((n,), -7, dtype=ids.dtype, device=dev),
        sorted_s=torch.full((n,), -7, dtype=torch.int64, device=dev),
    )
    stream = torch.cuda.current_stream().cuda_stream
    head = (ids.data_ptr(), int(ids.dtype == torch.int64), n, E, out["counts"].data_ptr(), out["incl"].data_ptr(),
            out["excl"].data_ptr(), out["sorted_e"].data_ptr(), out["sorted_s"].data_ptr())
    if static:
        check(lib.xma_rocm_route_static(*head, stream), "xma_rocm_route_static")
    else:
        ws = torch.empty(max(lib.xma_rocm_route_workspace_bytes(n, E) // 4, 1), dtype=torch.int32, device=dev)
        check(lib.xma_rocm_route(*head, ws.data_ptr(), ws.numel() * 4, stream), "xma_rocm_route")
    torch.cuda.synchronize()
    return {k: np_of(v) for k, v in out.items()}


def test_route_static_matches_route_with_workspace():
    from oracle import routing as oracle
    from xma.rocm import get_library

    lib = get_library()
    g = torch.Generator().manual_seed(3)
    cases = [  # (n, E, dtype): a large call, then smaller ones on the same scratch, then a larger one again
        (1 << 20, 64, torch.int32),
        (50001, 64, torch.int32),
        (777, 8, torch.int64),
        (262144, 128, torch.int64),
        (0, 4, torch.int32),
        (4 * 1024 * 1024, 64, torch.int32),
    ]
    for n, E, dtype in cases:
        print(f"route_static case n={n} E={E} {dtype}", flush=True)
        ids_cpu = zipf_ids(n, E, 1.1, 5, dtype) if n == 50001 else torch.randint(0, E, (n,), generator=g, dtype=dtype)
        ids = ids_cpu.cuda()
        got = _route(lib, ids, E, static=True)
        want = _route(lib, ids, E, static=False)
        for key in want:
            assert np.array_equal(got[key], want[key]), (n, E, key)
        ref = oracle.route(ids_cpu.numpy(), E)
        assert np.array_equal(got["sorted_s"], ref["sorted_scattered_idxs"])
        assert np.array_equal(got["counts"].view(np.uint32), ref["counts"])


def test_route_static_rejects_sizes_beyond_its_scratch():
    from xma.rocm import get_library

    lib = get_library()
    limit = lib.xma_rocm_route_static_max_units_times_experts()
    assert limit == 1 << 18
    E = 2048
    n = (limit // E + 1) * 4096  # one unit too many
    ids = torch.zeros(n, dtype=torch.int32, device="cuda")
    counts = torch.zeros(E, dtype=torch.int32, device="cuda")
    incl = torch.zeros(E, dtype=torch.int64, device="cuda")
    pos = torch.zeros(n, dtype=torch.int64, device="cuda")
    rc = lib.xma_rocm_route_static(ids.data_ptr(), 0, n, E, counts.data_ptr(), incl.data_ptr(), None, None, pos.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream)
    assert rc == -3  # XMA_ROCM_EWORKSPACE
    assert b"static scratch" in lib.xma_rocm_last_error()
    torch.cuda.synchronize()
    assert int(pos.abs().sum()) == 0  # nothing ran


def test_route_static_captured_in_a_graph_after_a_warm_up_call():
    """The use the entry point exists for: one ordinary call per device first (it resolves the scratch's address and raises
    the scatter kernel's LDS limit, neither of which is a stream operation), then the call is captured in a HIP graph and
    replayed on new ids written into the same input buffer; every replay against xma_rocm_route, with eager work and
    synchronisations between the replays."""
    from xma.rocm import get_library
    from xma.rocm.loader import check

    lib = get_library()
    n, E = 300000, 64
    g = torch.Generator().manual_seed(9)
    ids = torch.randint(0, E, (n,), generator=g, dtype=torch.int32).cuda()
    _route(lib, ids, E, static=True)  # warm-up, outside any capture
    counts = torch.zeros(E, dtype=torch.int32, device="cuda")
    incl = torch.zeros(E, dtype=torch.int64, device="cuda")
    excl = torch.zeros(E, dtype=torch.int64, device="cuda")
    sorted_e = torch.zeros(n, dtype=torch.int32, device="cuda")
    sorted_s = torch.zeros(n, dtype=torch.int64, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        check(lib.xma_rocm_route_static(ids.data_ptr(), 0, n, E, counts.data_ptr(), incl.data_ptr(), excl.data_ptr(),
                                        sorted_e.data_ptr(), sorted_s.data_ptr(), torch.cuda.current_stream().cuda_stream),
              "xma_rocm_route_static")
    for rep in range(3):
        ids.copy_(torch.randint(0, E, (n,), generator=g, dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        want = _route(lib, ids, E, static=False)  # eager work between the replays
        assert np.array_equal(np_of(counts), want["counts"]) and np.array_equal(np_of(incl), want["incl"]), rep
        assert np.array_equal(np_of(excl), want["excl"]) and np.array_equal(np_of(sorted_e), want["sorted_e"]), rep
        assert np.array_equal(np_of(sorted_s), want["sorted_s"]), rep
