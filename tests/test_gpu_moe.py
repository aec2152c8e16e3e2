"""GPU parity of the MoE layer (KernelBackend.rocm) against the CPU oracle, forward and backward.

Modelled on the reference's tests/layers/moe_test.py:26-157 (dtype x experts x top-k x GLU grid, 7
tokens, y / x.grad / expert weight grads compared), widened with what it leaves out: SwiGLU, more
tokens than one tile, skewed routing with empty experts, a random upstream gradient and the router
weight gradient.  Operands are bit-identical on both sides; the oracle runs in fp32.
Tolerance: max-abs-normalised error <= 1e-2 (bf16/fp16 results, fp32 accumulation)."""

import pytest
import torch
import torch.nn as nn

from oracle import moe as oracle
from tests.utils import nerr

pytestmark = pytest.mark.gpu

TOL = 1e-2
TOL_F32 = 5e-5  # fp32 kernels against the fp32 oracle: summation order and exp/rcp approximations only


def _act(name):
    from xma.functional import swiglu_packed

    return {"swiglu_packed": swiglu_packed, "glu": nn.GLU(), "gelu": nn.GELU(approximate="tanh")}[name]


def _oracle_act(name):
    return {"swiglu_packed": oracle.swiglu_packed, "glu": nn.GLU(), "gelu": nn.GELU(approximate="tanh")}[name]


def _run_case(dtype, T, E, k, H, I, act_name, skew=0.0, empty=(), seed=42, add_bias=False, save_activations=True):
    from xma import KernelBackend, set_seed
    from xma.layers import MoE

    print(f"case {dtype} T={T} E={E} k={k} H={H} I={I} act={act_name} skew={skew} empty={empty}", flush=True)
    set_seed(seed)
    is_glu = act_name != "gelu"
    moe = MoE(E, k, H, I, _act(act_name), is_glu, add_bias=add_bias, std=0.02).to(dtype)
    moe.save_activations = save_activations
    b_fc = b_proj = None
    if add_bias:  # the module zero-fills its biases; the test wants values that matter
        with torch.no_grad():
            moe.c_fc.bias.copy_((torch.randn(moe.c_fc.bias.shape) * 0.5).to(dtype))
            moe.c_proj.bias.copy_((torch.randn(moe.c_proj.bias.shape) * 0.5).to(dtype))
        b_fc, b_proj = moe.c_fc.bias.data, moe.c_proj.bias.data
    x = torch.randn(T, H).to(dtype)
    logits = torch.randn(T, E) + skew * torch.randn(E)
    for e in empty:
        logits[:, e] = -1e9
    rw, sel = oracle.routing_weights(logits, k, dtype)
    grad = torch.randn(T, H).to(dtype)

    want = oracle.experts_forward_backward(
        x, rw, sel, moe.c_fc.weight.data, moe.c_proj.weight.data, _oracle_act(act_name), grad, compute_dtype=torch.float32,
        b_fc=b_fc, b_proj=b_proj,
    )

    moe = moe.cuda()
    xd = x.cuda().requires_grad_()
    rwd = rw.cuda().requires_grad_()
    y = moe._compute_experts(xd, rwd, sel.cuda(), kernel_backend=KernelBackend.rocm)
    y.backward(grad.cuda())
    torch.cuda.synchronize()

    got = {"y": y, "dx": xd.grad, "d_router_weights": rwd.grad, "dw_fc": moe.c_fc.weight.grad, "dw_proj": moe.c_proj.weight.grad}
    if add_bias:
        got["db_fc"], got["db_proj"] = moe.c_fc.bias.grad, moe.c_proj.bias.grad
    for name, w in want.items():
        g = got[name]
        assert g is not None and g.dtype == dtype and g.shape == w.shape, name
        assert torch.isfinite(g).all(), name
        e = nerr(g, w)
        print(f"   {name}: nerr={e:.2e}", flush=True)
        assert e <= (TOL_F32 if dtype == torch.float32 else TOL), f"{name}: {e}"
    # experts without tokens: zero weight gradient slices
    for e in empty:
        assert (moe.c_fc.weight.grad[e] == 0).all() and (moe.c_proj.weight.grad[e] == 0).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("E", [2, 4, 6, 8])
@pytest.mark.parametrize("k", [2, 4])
@pytest.mark.parametrize("act_name", ["swiglu_packed", "glu", "gelu"])
def test_moe_reference_grid_7_tokens(dtype, E, k, act_name):
    if k > E:
        pytest.skip("more experts per token than experts")
    _run_case(dtype, 7, E, k, 512, 1024, act_name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("act_name", ["swiglu_packed", "glu"])
def test_moe_reference_sizes(dtype, act_name):
    # the two size points of the reference grid (moe_test.py:31-32 and :43-46) in its three dtypes
    _run_case(dtype, 7, 8, 2, 2048, 8192, act_name)
    _run_case(dtype, 7, 128, 8, 576, 256, act_name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act_name", ["swiglu_packed", "gelu"])
def test_moe_many_tokens_ragged(dtype, act_name):
    _run_case(dtype, 1500, 8, 2, 256, 384, act_name, skew=1.5, empty=(2,))
    _run_case(dtype, 777, 16, 4, 264, 136, act_name, skew=2.0, empty=(0, 15))
    _run_case(dtype, 2048, 4, 1, 128, 256, act_name)


@pytest.mark.parametrize("act_name", ["swiglu_packed", "gelu"])
def test_moe_tiles_split_along_k(act_name):
    """Few tiles and a long K: the tiles of the only (partial) round are cut into K slices that a second kernel adds
    up, in all three epilogues (up-projection K = H, dX2 K = H, down-projection K = I, dX1 K = 2 I)."""
    _run_case(torch.bfloat16, 64, 2, 1, 1024, 1536, act_name)
    _run_case(torch.float16, 300, 3, 2, 2048, 512, act_name, skew=1.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("act_name", ["swiglu_packed", "glu", "gelu"])
def test_moe_with_expert_biases(dtype, act_name):
    """add_bias=True: Experts.bias (E, out) on both projections, as the reference's torch path applies it
    (F.linear(x[e], weight[e], bias[e]), moe/__init__.py:96-100), forward and all gradients including the two biases'
    against the fp32 oracle: the reference's 7-token shape, ragged routing with empty experts (their bias gradient is
    zero), top-4 (dW2 and the down-projection's bias gradient from unscaled dy through the index) and tiles split along K."""
    _run_case(dtype, 7, 8, 2, 512, 1024, act_name, add_bias=True)
    _run_case(dtype, 777, 16, 4, 264, 136, act_name, skew=2.0, empty=(0, 15), add_bias=True)
    _run_case(dtype, 1500, 8, 2, 256, 384, act_name, skew=1.5, empty=(2,), add_bias=True)
    _run_case(dtype, 300, 3, 2, 2048, 512, act_name, skew=1.0, add_bias=True)


@pytest.mark.parametrize("k", [2, 4])
def test_moe_recomputed_activations(k):
    """save_activations = False: the backward recomputes h and the expert outputs from the kept pre-activations; the
    results are those of the default path bit for bit (same kernels on the same operands), and within tolerance of the
    oracle, with and without biases."""
    from xma import KernelBackend, set_seed
    from xma.layers import MoE

    _run_case(torch.bfloat16, 777, 16, k, 264, 136, "swiglu_packed", skew=2.0, empty=(0, 15), save_activations=False)
    _run_case(torch.bfloat16, 300, 8, k, 512, 256, "swiglu_packed", add_bias=True, save_activations=False)
    set_seed(5)
    T, E, H, I = 900, 8, 256, 384
    moe = MoE(E, k, H, I, _act("swiglu_packed"), True, add_bias=False, std=0.02).to(torch.bfloat16).cuda()
    x = torch.randn(T, H, device="cuda").to(torch.bfloat16)
    rw, sel = oracle.routing_weights(torch.randn(T, E, device="cuda"), k, torch.bfloat16)
    grad = torch.randn(T, H, device="cuda").to(torch.bfloat16)
    res = []
    for keep in (True, False):
        moe.save_activations = keep
        for p in moe.parameters():
            p.grad = None
        xd, rwd = x.clone().requires_grad_(), rw.clone().requires_grad_()
        y = moe._compute_experts(xd, rwd, sel, kernel_backend=KernelBackend.rocm)
        y.backward(grad)
        torch.cuda.synchronize()
        res.append([t.clone() for t in (y.detach(), xd.grad, rwd.grad, moe.c_fc.weight.grad, moe.c_proj.weight.grad)])
    for a, b, name in zip(res[0], res[1], ("y", "dx", "d_router_weights", "dw_fc", "dw_proj")):
        assert torch.equal(a, b), name


def test_moe_plumbing_config_shape():
    """The small plumbing configuration (T=512, H=256, I=512, E=8, top-2, SwiGLU, weights N(0, 0.02)) in fp32 and in bf16."""
    _run_case(torch.float32, 512, 8, 2, 256, 512, "swiglu_packed", seed=0)
    _run_case(torch.bfloat16, 512, 8, 2, 256, 512, "swiglu_packed", seed=0)


@pytest.mark.parametrize("act_name", ["swiglu_packed", "gelu"])
def test_moe_fp32_ragged(act_name):
    _run_case(torch.float32, 777, 16, 4, 264, 136, act_name, skew=2.0, empty=(0, 15))
    _run_case(torch.float32, 300, 3, 2, 1024, 512, act_name, skew=1.0)


def test_moe_forward_module_and_state_dict():
    """full forward incl. the gate on the device: selection taken from the device run, experts from the oracle"""
    from xma import KernelBackend, set_seed
    from xma.layers import MoE

    set_seed(0)
    moe = MoE(8, 2, 256, 512, _act("swiglu_packed"), True, add_bias=False, std=0.02).to(torch.bfloat16).cuda()
    assert set(moe.state_dict()) == {"gate.weight", "c_fc.weight", "c_fc.N_array", "c_fc.K_array", "c_proj.weight",
                                     "c_proj.N_array", "c_proj.K_array"}
    x = torch.randn(4, 33, 256, device="cuda", dtype=torch.bfloat16)
    y, logits = moe(x)  # default backend on a ROCm GPU is rocm
    assert y.shape == x.shape and logits.shape == (4 * 33, 8)
    rw, sel = oracle.routing_topk(logits.float().cpu(), 2, torch.bfloat16)  # the rocm router's order among equal logits
    want = oracle.experts_forward(x.view(-1, 256).float().cpu(), rw.float(), sel, moe.c_fc.weight.float().cpu(),
                                  moe.c_proj.weight.float().cpu(), oracle.swiglu_packed)
    assert nerr(y.view(-1, 256), want) <= TOL
    y2, _ = moe(x, kernel_backend=KernelBackend.torch)
    assert nerr(y2.view(-1, 256), want) <= 2e-2  # the torch path accumulates the k terms in bf16


def test_moe_results_are_bitwise_reproducible():
    """no float atomics anywhere: every output of two runs on the same inputs is identical, also where tiles are split
    along K (the slices are added in a fixed order) and under skewed routing"""
    from xma import KernelBackend, set_seed
    from xma.layers import MoE

    set_seed(11)
    T, E, k, H, I = 1500, 8, 2, 1096, 320
    moe = MoE(E, k, H, I, _act("swiglu_packed"), True, add_bias=False, std=0.02).to(torch.bfloat16).cuda()
    x = torch.randn(T, H, device="cuda").to(torch.bfloat16)
    logits = torch.randn(T, E, device="cuda") + 1.5 * torch.randn(E, device="cuda")
    rw, sel = oracle.routing_weights(logits, k, torch.bfloat16)
    grad = torch.randn(T, H, device="cuda").to(torch.bfloat16)

    def run():
        for p in moe.parameters():
            p.grad = None
        xd, rwd = x.clone().requires_grad_(), rw.clone().requires_grad_()
        y = moe._compute_experts(xd, rwd, sel, kernel_backend=KernelBackend.rocm)
        y.backward(grad)
        torch.cuda.synchronize()
        return [t.clone() for t in (y.detach(), xd.grad, rwd.grad, moe.c_fc.weight.grad, moe.c_proj.weight.grad)]

    first = run()
    for _ in range(3):
        for a, b, name in zip(first, run(), ("y", "dx", "d_router_weights", "dw_fc", "dw_proj")):
            assert torch.equal(a, b), name
