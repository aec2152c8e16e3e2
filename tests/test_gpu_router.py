"""GPU parity of the fused router (top-k + fp32 softmax + expert ids behind the gate, and its backward)
against the CPU oracle's restatement of xma/layers/moe/__init__.py:186-193, 256-262.

Expert ids: bit-exact, also among equal logits (16-bit logits tie often; the rule is "lower expert index first",
oracle.routing_topk).  Router weights and the logits' gradient: fp32 softmax on both sides, so the difference is the
exp/division rounding before the cast: at most one unit in the last place of the result dtype."""

import pytest
import torch

from oracle import moe as oracle

pytestmark = pytest.mark.gpu

ULP = {torch.float32: 2.0**-22, torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}  # weights are <= 1

CASES = [  # T, E, k
    (7, 8, 2),
    (1000, 8, 2),
    (513, 64, 6),
    (300, 128, 8),
    (33, 1, 1),
    (50, 5, 5),
    (64, 100, 1),
    (257, 3, 2),
    (40, 200, 7),
    (19, 2048, 64),
    (8192, 8, 2),
    (130, 65, 33),
]


def _logits(T, E, dtype, seed=0, coarse=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, E, generator=g)
    if coarse:  # few distinct values: every row has equal logits
        x = (x * 2).round() / 2
    return x.to(dtype)


def _run_fwd(logits, k, id_dtype=torch.int64):
    from xma.rocm import ops

    d = logits.cuda()
    w = torch.empty(d.size(0), k, dtype=d.dtype, device="cuda")
    ids = torch.empty(d.size(0), k, dtype=id_dtype, device="cuda")
    ops.router_topk_rocm(d, w, ids)
    torch.cuda.synchronize()
    return w.cpu(), ids.cpu()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,E,k", CASES)
@pytest.mark.parametrize("coarse", [False, True])
def test_router_topk_forward(dtype, T, E, k, coarse):
    print(f"router fwd {dtype} T={T} E={E} k={k} coarse={coarse}", flush=True)
    logits = _logits(T, E, dtype, seed=T + E + k, coarse=coarse)
    want_w, want_ids = oracle.routing_topk(logits, k, dtype)
    w, ids = _run_fwd(logits, k)
    assert torch.equal(ids, want_ids)
    assert (w.float() - want_w.float()).abs().max().item() <= ULP[dtype]
    if not coarse and dtype == torch.float32:  # no equal values: the library routine gives the same selection
        lib_w, lib_ids = oracle.routing_weights(logits, k, dtype)
        assert torch.equal(ids, lib_ids)


def test_router_topk_int32_ids_strided_rows_and_special_values():
    logits = _logits(200, 16, torch.float32, seed=5)
    logits[3, 4] = float("nan")
    logits[4, :] = float("-inf")
    logits[4, 9] = 1.0
    logits[5, 2] = float("inf")
    logits[6, 1], logits[6, 7] = 0.0, -0.0
    logits[6, [0, 2, 3, 4, 5, 6]] = -1.0
    want_w, want_ids = oracle.routing_topk(logits, 3, torch.float32)
    w, ids = _run_fwd(logits, 3, torch.int32)
    assert ids.dtype == torch.int32 and torch.equal(ids.long(), want_ids)
    torch.testing.assert_close(w, want_w, rtol=0, atol=ULP[torch.float32], equal_nan=True)
    # rows of a wider buffer (row stride 24)
    wide = torch.zeros(200, 24)
    wide[:, :16] = logits
    from xma.rocm import ops

    d = wide.cuda()[:, :16]
    w2 = torch.empty(200, 3, device="cuda")
    ids2 = torch.empty(200, 3, dtype=torch.int64, device="cuda")
    ops.router_topk_rocm(d, w2, ids2)
    assert torch.equal(ids2.cpu(), want_ids)
    torch.testing.assert_close(w2.cpu(), want_w, rtol=0, atol=ULP[torch.float32], equal_nan=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,E,k", CASES)
def test_router_topk_backward(dtype, T, E, k):
    from xma.layers.moe import rocm_implementation as R

    print(f"router bwd {dtype} T={T} E={E} k={k}", flush=True)
    logits = _logits(T, E, dtype, seed=3 * T + E)
    dw = torch.randn(T, k, generator=torch.Generator().manual_seed(1)).to(dtype)
    lg = logits.clone().requires_grad_()
    w, _ = oracle.routing_topk(lg, k, dtype)
    w.backward(dw)
    d = logits.cuda().requires_grad_()
    wd, ids = R.router_topk(d, k)
    assert not ids.requires_grad
    wd.backward(dw.cuda())
    got = d.grad.cpu()
    assert got.dtype == dtype and got.shape == (T, E)
    mask = torch.zeros(T, E, dtype=torch.bool).scatter_(1, ids.cpu(), True)
    assert (got[~mask] == 0).all()  # exact zeros outside the selection
    scale = max(dw.float().abs().max().item(), 1.0)
    assert (got.float() - lg.grad.float()).abs().max().item() <= 2 * ULP[dtype] * scale


def test_router_in_the_layer_forward_and_gate_gradient():
    """MoE.forward on the rocm backend routes through the fused router: logits, selection (taken from the device
    logits) and the gate's gradient against the oracle"""
    from xma import KernelBackend, set_seed
    from xma.functional import swiglu_packed
    from xma.layers import MoE
    from tests.utils import nerr

    set_seed(3)
    T, H, I, E, k = 192, 256, 128, 16, 4
    moe = MoE(E, k, H, I, swiglu_packed, True, add_bias=False, std=0.02).to(torch.bfloat16).cuda()
    x = torch.randn(T, H, device="cuda", dtype=torch.bfloat16)
    grad = torch.randn(T, H, device="cuda", dtype=torch.bfloat16)
    y, logits = moe(x, kernel_backend=KernelBackend.rocm)
    y.backward(grad)
    # oracle: the gate in fp32; selection and softmax from the device's bf16 logits
    xc = x.float().cpu()
    wg = moe.gate.weight.detach().float().cpu().requires_grad_()
    dev_logits = logits.detach().float().cpu()
    lg = xc @ wg.t()
    assert (lg.detach() - dev_logits).abs().max().item() <= 2.0**-8 * max(1.0, dev_logits.abs().max().item())
    lg = lg + (dev_logits - lg).detach()  # the device's values, the fp32 chain's gradient
    _, sel = oracle.routing_topk(dev_logits, k, torch.float32)
    rw = torch.softmax(lg.gather(-1, sel), -1)
    want = oracle.experts_forward(xc, rw, sel, moe.c_fc.weight.detach().float().cpu(),
                                  moe.c_proj.weight.detach().float().cpu(), oracle.swiglu_packed)
    want.backward(grad.float().cpu())
    assert nerr(y, want.detach()) <= 1e-2
    assert nerr(moe.gate.weight.grad, wg.grad) <= 2e-2  # bf16 router weights and a bf16 gate GEMM in the chain


GATE_CASES = [  # T, H, E, k
    (7, 64, 8, 2),
    (1000, 4096, 8, 2),
    (513, 2048, 64, 6),
    (300, 2048, 128, 8),
    (33, 72, 1, 1),
    (257, 136, 3, 2),
    (100, 200, 100, 32),
    (65, 8, 33, 5),
    (8192, 4096, 8, 2),
    (4133, 1032, 96, 4),
    (2085, 2048, 128, 8),
    (98333, 136, 40, 3),  # enough tokens for the variant without a K split
    (8192, 256, 64, 4),  # the gate's weight gradient as a batched GEMM over slices of the tokens
    (98305, 64, 128, 8),
    (16384, 2048, 64, 6),  # the two benchmark layers with more than 32 experts, at their exact shapes: two pairs of waves
    (32768, 2048, 128, 8),  # per workgroup with a K split (below 98304 tokens); 16 K steps per pair through the LDS ring
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,k", GATE_CASES)
def test_router_gate_topk_fused(dtype, T, H, E, k):
    """Gate projection fused with the router (xma/layers/moe/__init__.py:182-195, 256-262).  Logits against the fp32
    product (one rounding to the 16-bit dtype plus the summation order); expert ids bit-exact and router weights within a
    unit in the last place against the oracle's top-k and softmax applied to the logits the device produced; int32 ids;
    d_x and d_Wg against the fp32 chain's gradient (2e-2: 16-bit router weights and 16-bit d_logits in the chain)."""
    from tests.utils import nerr
    from xma.layers.moe import rocm_implementation as R

    print(f"router gate {dtype} T={T} H={H} E={E} k={k}", flush=True)
    g = torch.Generator().manual_seed(T + H + E + k)
    x = torch.randn(T, H, generator=g).to(dtype)
    wg = (torch.randn(E, H, generator=g) * (H**-0.5)).to(dtype)
    dw = torch.randn(T, k, generator=g).to(dtype)
    xd, wd = x.cuda().requires_grad_(), wg.cuda().requires_grad_()
    assert R.router_gate_topk_supported(xd, wd, k)
    logits, w, ids = R.router_gate_topk(xd, wd, k)
    assert ids.dtype == torch.int32 and not ids.requires_grad and logits.shape == (T, E) and logits.dtype == dtype
    dev_logits = logits.detach().cpu()
    xf, wf = x.float().requires_grad_(), wg.float().requires_grad_()
    lg = xf @ wf.t()
    ulp = ULP[dtype] * 2  # values up to 2^k have ulps of 2^(k - mantissa bits)
    assert (lg.detach() - dev_logits.float()).abs().max().item() <= ulp * max(1.0, lg.detach().abs().max().item())
    want_w, want_ids = oracle.routing_topk(dev_logits, k, dtype)
    assert torch.equal(ids.cpu().long(), want_ids)
    assert (w.detach().cpu().float() - want_w.float()).abs().max().item() <= ULP[dtype]
    # gradients: the device's logit values, the fp32 chain's derivative
    lg = lg + (dev_logits.float() - lg).detach()
    rw = torch.softmax(lg.gather(-1, want_ids), -1)
    rw.backward(dw.float())
    w.backward(dw.cuda())
    assert nerr(xd.grad, xf.grad) <= 2e-2 and nerr(wd.grad, wf.grad) <= 2e-2


def test_router_gate_topk_strided_rows_and_fallback():
    """x as a column slice of a wider tensor (row pitch > H); shapes the fused kernel does not cover are reported as such
    and the layer falls back to the linear layer + router_topk"""
    from xma.layers.moe import rocm_implementation as R
    from xma.rocm import ops

    g = torch.Generator().manual_seed(2)
    wide = torch.randn(300, 512 + 64, generator=g).to(torch.bfloat16).cuda()
    x = wide[:, 64:]
    wg = (torch.randn(16, 512, generator=g) * 0.05).to(torch.bfloat16).cuda()
    assert R.router_gate_topk_supported(x, wg, 4)
    logits, w, ids = R.router_gate_topk(x, wg, 4)
    l2, w2, ids2 = R.router_gate_topk(x.contiguous(), wg, 4)
    assert torch.equal(logits, l2) and torch.equal(w, w2) and torch.equal(ids, ids2)
    assert not ops.router_gate_topk_supported(512, 129, 2, torch.bfloat16)
    assert not ops.router_gate_topk_supported(512, 64, 33, torch.bfloat16)
    assert not ops.router_gate_topk_supported(516, 64, 2, torch.bfloat16)
    assert not ops.router_gate_topk_supported(512, 64, 2, torch.float32)
    # a gate weight of another dtype is not taken by the fused kernel although the shape is covered: the layer then runs
    # gate(x) + router_topk; rows that start off a 16-byte boundary are copied inside the op
    assert not R.router_gate_topk_supported(x, wg.float(), 4)
    xs = wide[:, 4 : 4 + 512]
    assert R.router_gate_topk_supported(xs, wg, 4)
    l3, w3, ids3 = R.router_gate_topk(xs, wg, 4)
    l4, w4, ids4 = R.router_gate_topk(xs.contiguous(), wg, 4)
    assert torch.equal(l3, l4) and torch.equal(w3, w4) and torch.equal(ids3, ids4)


def test_router_gate_backward_with_a_loss_on_the_logits():
    """The gate's gradients with and without a loss on the returned router logits (an auxiliary loss adds its gradient to
    the router's d_logits; without one that output's gradient arrives as None), against the fp32 chain."""
    from tests.utils import nerr
    from xma.layers.moe import rocm_implementation as R

    g = torch.Generator().manual_seed(5)
    T, H, E, k = 257, 512, 16, 4
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    wg = (torch.randn(E, H, generator=g) * H**-0.5).to(torch.bfloat16)
    dw = torch.randn(T, k, generator=g).to(torch.bfloat16)
    dl = torch.randn(T, E, generator=g).to(torch.bfloat16)
    for with_logits in (False, True):
        xd, wd = x.cuda().requires_grad_(), wg.cuda().requires_grad_()
        logits, w, ids = R.router_gate_topk(xd, wd, k)
        loss = (w * dw.cuda()).sum()
        if with_logits:
            loss = loss + (logits * dl.cuda()).sum()
        loss.backward()
        xf, wf = x.float().requires_grad_(), wg.float().requires_grad_()
        lg = xf @ wf.t()
        lg = lg + (logits.detach().cpu().float() - lg).detach()  # the device's logit values, the fp32 chain's derivative
        rw = torch.softmax(lg.gather(-1, ids.cpu().long()), -1)
        ref = (rw * dw.float()).sum()
        if with_logits:
            ref = ref + (lg * dl.float()).sum()
        ref.backward()
        assert nerr(xd.grad, xf.grad) <= 2e-2 and nerr(wd.grad, wf.grad) <= 2e-2, with_logits
