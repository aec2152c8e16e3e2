"""The rocm path under torch.compile(fullgraph=True) and under HIP graph capture.

The reference runs every op eager and compiled (tests/layers/moe_test.py:104-105 wraps the module in
torch.compile(fullgraph=True)); its ops are traceable because they are registered custom ops that mutate
caller-allocated outputs (xma/custom_op.py:72-108).  The same must hold here, and since the tile schedule is
derived on the device from the offsets, a whole step must also be capturable in a graph and replayable."""

import pytest
import torch

from tests.utils import nerr

pytestmark = pytest.mark.gpu


def _make(T=300, E=8, k=2, H=256, I=512, dtype=torch.bfloat16, seed=0):
    from xma import set_seed
    from xma.functional import swiglu_packed
    from xma.layers import MoE

    set_seed(seed)
    moe = MoE(E, k, H, I, swiglu_packed, True, add_bias=False, std=0.02).to(dtype).cuda()
    x = torch.randn(T, H, device="cuda").to(dtype)
    return moe, x


@pytest.mark.parametrize("T", [300, 7])  # 7 tokens: the grouped GEMMs take the kernels of the few-token regime
@pytest.mark.parametrize("k", [2, 4])  # 4: the backward that takes dW2 from the scaled activations of the dX2 epilogue
@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_module_matches_eager(backend, k, T):
    """torch.compile(fullgraph=True) of the module, with the tracing-only backend and with the default one the
    reference's test uses (tests/layers/moe_test.py:104-105 passes no backend, i.e. inductor): the custom ops mutate
    caller-allocated outputs, so functionalisation has to carry them through unchanged."""
    from xma import KernelBackend

    torch._dynamo.reset()
    moe, x = _make(T=T, k=k)
    print("compile: eager run", flush=True)
    xe = x.clone().requires_grad_()
    ye, _ = moe(xe, kernel_backend=KernelBackend.rocm)
    ye.sum().backward()
    want = {"y": ye.detach().clone(), "dx": xe.grad.clone(), "dw_fc": moe.c_fc.weight.grad.clone(),
            "dw_proj": moe.c_proj.weight.grad.clone(), "dgate": moe.gate.weight.grad.clone()}
    for p in moe.parameters():
        p.grad = None
    print("compile: compiled run (fullgraph)", flush=True)
    cmoe = torch.compile(moe, fullgraph=True, backend=backend)
    xc = x.clone().requires_grad_()
    try:
        yc, _ = cmoe(xc, kernel_backend=KernelBackend.rocm)
        yc.sum().backward()
    except torch._dynamo.exc.BackendCompilerFailed as err:  # the code generator's own toolchain, not the ops under test
        if backend == "inductor":
            pytest.skip(f"inductor cannot generate code on this machine: {str(err)[:300]}")
        raise
    torch.cuda.synchronize()
    got = {"y": yc, "dx": xc.grad, "dw_fc": moe.c_fc.weight.grad, "dw_proj": moe.c_proj.weight.grad,
           "dgate": moe.gate.weight.grad}
    for name in want:
        # same kernels on the same inputs: bit-identical.  The code generator may fold the sum of the two contributions
        # to dx (experts and gate) and the gate's stock GEMMs into other kernels than eager mode runs: one rounding apart.
        if backend == "inductor" and name in ("dx", "dgate"):
            assert nerr(got[name], want[name]) <= 2.0**-7, name  # a unit in the last place of bf16
        else:
            assert torch.equal(got[name], want[name]), name


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_functionals_match_eager(backend):
    """The functionals under torch.compile(fullgraph=True), as the reference's tests run them
    (tests/functional/continuous_count_test.py:25, tests/functional/swiglu_test.py: eager and compiled function side by
    side): continuous_count over sizes of the reference's 1-D rule in both id types against the oracle, swiglu and
    swiglu_packed forward and backward bit-identical to their eager runs."""
    from oracle import routing as oracle_routing
    from tests.utils import get_1d_tensor_sizes, np_of
    from xma import KernelBackend
    from xma.functional import continuous_count, swiglu, swiglu_packed

    torch._dynamo.reset()
    g = torch.Generator().manual_seed(3)
    bins = 72
    try:
        cc = torch.compile(continuous_count, fullgraph=True, backend=backend)
        sizes = get_1d_tensor_sizes()
        for n in sizes[:: max(1, len(sizes) // 10)] + [70000]:  # 70000: the two-pass path, its scratch allocated in the op
            for dtype in (torch.int32, torch.int64):
                ids = torch.randint(0, bins, (n,), generator=g, dtype=dtype)
                got = cc(ids.cuda(), bins, kernel_backend=KernelBackend.rocm)
                assert got.dtype == torch.uint32 and got.shape == (bins,)
                assert np_of(got).tolist() == oracle_routing.continuous_count(ids.numpy(), bins).tolist(), (n, dtype)
        assert np_of(cc(torch.zeros(5, dtype=torch.int32, device="cuda"), 1, kernel_backend=KernelBackend.rocm)).tolist() == [5]

        csw = torch.compile(swiglu, fullgraph=True, backend=backend)
        cswp = torch.compile(swiglu_packed, fullgraph=True, backend=backend)
        for dtype in (torch.bfloat16, torch.float32):
            for rows, cols in [(7, 9), (64, 64), (300, 1408), (1025, 513)]:
                gate = torch.randn(rows, cols, generator=g).to(dtype).cuda()
                up = torch.randn(rows, cols, generator=g).to(dtype).cuda()
                dy = torch.randn(rows, cols, generator=g).to(dtype).cuda()
                res = []
                for fn in (swiglu, csw):
                    gd, ud = gate.clone().requires_grad_(), up.clone().requires_grad_()
                    y = fn(gd, ud, kernel_backend=KernelBackend.rocm)
                    y.backward(dy)
                    res.append((y.detach(), gd.grad, ud.grad))
                assert all(torch.equal(a, b) for a, b in zip(*res)), (rows, cols, dtype)
                xp = torch.randn(rows, 2 * cols, generator=g).to(dtype).cuda()
                res = []
                for fn in (swiglu_packed, cswp):
                    xd = xp.clone().requires_grad_()
                    y = fn(xd, kernel_backend=KernelBackend.rocm)
                    y.backward(dy)
                    res.append((y.detach(), xd.grad))
                assert all(torch.equal(a, b) for a, b in zip(*res)), (rows, cols, dtype)
    except torch._dynamo.exc.BackendCompilerFailed as err:  # the code generator's own toolchain, not the ops under test
        if backend == "inductor":
            pytest.skip(f"inductor cannot generate code on this machine: {str(err)[:300]}")
        raise


@pytest.mark.parametrize("T", [300, 7])  # 7 tokens: the kernels of the few-token regime, whose passes depend on the routing
@pytest.mark.parametrize("k", [2, 4])
def test_graph_capture_and_replay(k, T):
    """fwd + bwd of the router (behind the gate) and of the expert computation captured once and replayed on new
    inputs (new routing included); every replay is checked against an eager run, with eager work and synchronisations
    in between."""
    from xma import KernelBackend

    E = 8
    moe, x = _make(T=T, E=E, k=k)
    T, H = x.shape
    g = torch.Generator(device="cuda").manual_seed(1)

    def inputs():
        logits = torch.randn(T, E, device="cuda", generator=g).to(x.dtype)
        xx = torch.randn(T, H, device="cuda", generator=g).to(x.dtype)
        gy = torch.randn(T, H, device="cuda", generator=g).to(x.dtype)
        return xx, logits, gy

    def step(xx, logits, gy):
        from xma.layers.moe import rocm_implementation as R

        xx = xx.detach().requires_grad_()
        logits = logits.detach().requires_grad_()
        for p in (moe.c_fc.weight, moe.c_proj.weight):
            p.grad = None
        rw, sel = R.router_topk(logits, k)  # top-k + softmax + ids: part of the captured sequence
        y = moe._compute_experts(xx, rw, sel, kernel_backend=KernelBackend.rocm)
        y.backward(gy)
        return y.detach(), xx.grad, logits.grad, moe.c_fc.weight.grad, moe.c_proj.weight.grad

    sx, slg, sgy = inputs()
    print("graph: warm-up on a side stream", flush=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(sx, slg, sgy)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    print("graph: capture", flush=True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(sx, slg, sgy)
    for it in range(3):
        nx, nlg, ngy = inputs()
        print(f"graph: replay {it}", flush=True)
        sx.copy_(nx), slg.copy_(nlg), sgy.copy_(ngy)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = step(nx, nlg, ngy)  # eager, same kernels
        torch.cuda.synchronize()
        for a, b, name in zip(got, want, ("y", "dx", "d_router_logits", "dw_fc", "dw_proj")):
            assert torch.equal(a, b), f"replay {it}: {name} differs, nerr {nerr(a, b):.2e}"
