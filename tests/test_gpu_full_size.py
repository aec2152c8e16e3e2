"""The MoE path at the full sizes of the benchmark configurations, where the CPU oracle cannot run a whole step in
seconds: (1) tokens are independent, so the oracle is run in fp32 on a sample of tokens (first and last rows of every
expert's group, rows next to tile boundaries, random ones) and compared with those rows of the full-size device
result (y, dx, d_router_weights); (2) with one weight matrix shared by all experts the layer is a dense MLP scaled by
the sum of the router weights whatever the routing, so the full result - the weight gradients summed over the experts
included - is compared with the dense computation by the stock GEMM.  Two further shapes put byte offsets past 2^32
inside one tensor and 2^20 rows into the grouped order.
Tolerance: max-abs-normalised error <= 1e-2 (bf16 results, fp32 accumulation), as for the small cases."""

import pytest
import torch

from oracle import moe as oracle
from tests.utils import nerr

pytestmark = pytest.mark.gpu

TOL = 1e-2

CONFIGS = {  # T, H, I, E, k, bias of the router logits (skew)
    "c3": (8192, 4096, 14336, 8, 2, 0.0),
    "c4": (16384, 2048, 1408, 64, 6, 1.5),
    "c5": (32768, 2048, 768, 128, 8, 0.0),
    # not a benchmark configuration: 2^18 grouped rows whose pre-activations (and their gradient) take 4.3 GB each, so
    # that byte offsets inside one tensor pass 2^32; and 2^20 grouped rows of small matrices
    "over_4_gib": (65536, 512, 4096, 8, 4, 0.0),
    "many_rows": (262144, 256, 128, 16, 4, 1.0),
}


def _inputs(name, shared_weights=False, empty_expert=None):
    from xma import set_seed
    from xma.functional import swiglu_packed
    from xma.layers import MoE

    T, H, I, E, k, bias = CONFIGS[name]
    set_seed(7)
    g = torch.Generator(device="cuda").manual_seed(7)
    with torch.device("meta"):
        moe = MoE(E, k, H, I, swiglu_packed, True, add_bias=False, std=0.02)
    moe = moe.to_empty(device="cuda").to(torch.bfloat16)
    with torch.no_grad():
        for p in (moe.c_fc.weight, moe.c_proj.weight):
            if shared_weights:
                p.copy_((torch.randn(p.shape[1:], generator=g, device="cuda") * 0.02).to(p.dtype).expand_as(p))
            else:
                p.copy_((torch.randn(p.shape, generator=g, device="cuda") * 0.02).to(p.dtype))
    x = torch.randn(T, H, generator=g, device="cuda").to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g, device="cuda")
    if bias:
        logits = logits + bias * torch.randn(E, generator=g, device="cuda")
    if empty_expert is not None:
        logits[:, empty_expert] = -1e9  # never selected
    rw, sel = oracle.routing_weights(logits, k, torch.bfloat16)
    grad = torch.randn(T, H, generator=g, device="cuda").to(torch.bfloat16)
    return moe, x, rw, sel, grad


def _run(moe, x, rw, sel, grad):
    from xma import KernelBackend

    xd = x.clone().requires_grad_()
    rwd = rw.clone().requires_grad_()
    y = moe._compute_experts(xd, rwd, sel, kernel_backend=KernelBackend.rocm)
    y.backward(grad)
    torch.cuda.synchronize()
    return y.detach(), xd.grad, rwd.grad


@pytest.mark.parametrize("name", ["c3", "c4", "c5", "over_4_gib", "many_rows"])
def test_full_size_sampled_tokens_against_oracle(name):
    from xma.layers.moe import rocm_implementation as R

    print(f"full size {name}: sampled tokens", flush=True)
    T, H, I, E, k, _ = CONFIGS[name]
    moe, x, rw, sel, grad = _inputs(name)
    y, dx, d_rw = _run(moe, x, rw, sel, grad)
    assert torch.isfinite(y).all() and torch.isfinite(dx).all() and torch.isfinite(d_rw).all()

    # sample: per expert the first and last row of its group and the rows around every 256-row tile boundary of the
    # first two tiles, plus random tokens
    counts, incl, excl, _, ss = R.route(sel, E)
    incl, excl, ss = incl.cpu(), excl.cpu(), ss.cpu()
    rows = []
    for e in range(E):
        lo, hi = int(excl[e]), int(incl[e])
        for r in (lo, lo + 255, lo + 256, lo + 511, lo + 512, hi - 1):
            if lo <= r < hi:
                rows.append(r)
    rows = rows[:: max(1, len(rows) // 96)]  # about a hundred rows
    tokens = set((ss[rows] // k).tolist())
    gen = torch.Generator().manual_seed(0)
    tokens |= set(torch.randint(0, T, (32,), generator=gen).tolist())
    tok = torch.tensor(sorted(tokens))
    print(f"   {len(tok)} tokens", flush=True)

    xs = x[tok.cuda()].float().cpu().requires_grad_()
    rws = rw[tok.cuda()].float().cpu().requires_grad_()
    want = oracle.experts_forward(xs, rws, sel[tok.cuda()].cpu(), moe.c_fc.weight.detach().float().cpu(),
                                  moe.c_proj.weight.detach().float().cpu(), oracle.swiglu_packed)
    want.backward(grad[tok.cuda()].float().cpu())
    for label, got, ref in (("y", y, want.detach()), ("dx", dx, xs.grad), ("d_router_weights", d_rw, rws.grad)):
        e = nerr(got[tok.cuda()], ref)
        print(f"   {label}: nerr={e:.2e}", flush=True)
        assert e <= TOL, f"{name} {label}: {e}"


@pytest.mark.parametrize("name", ["c3", "c4", "c5"])
def test_full_size_weight_gradients_per_expert(name):
    """dW of single experts at full size.  An expert's weight gradients depend only on its own tokens, so the fp32 oracle
    is run on exactly those tokens as a one-expert layer (k = 1, router weight = the weight of the slot that chose the
    expert) and compared with that expert's slices of the device's dw_fc and dw_proj, each normalised by its own
    maximum: the smallest non-empty expert, the largest and one in the middle.  A wrong expert -> slice mapping or a bad
    ragged K tail shows here even if it cancels in the sum over experts.  One expert is left without tokens: its
    slices must be exact zeros."""
    from xma.layers.moe import rocm_implementation as R

    print(f"full size {name}: per-expert weight gradients", flush=True)
    T, H, I, E, k, _ = CONFIGS[name]
    empty = E // 2
    moe, x, rw, sel, grad = _inputs(name, empty_expert=empty)
    _run(moe, x, rw, sel, grad)
    dw_fc, dw_proj = moe.c_fc.weight.grad, moe.c_proj.weight.grad
    assert torch.isfinite(dw_fc).all() and torch.isfinite(dw_proj).all()
    counts, incl, excl, _, ss = R.route(sel, E)
    counts = counts.cpu().view(torch.int32).tolist()
    assert counts[empty] == 0
    assert float(dw_fc[empty].abs().max()) == 0.0 and float(dw_proj[empty].abs().max()) == 0.0
    order = sorted((c, e) for e, c in enumerate(counts) if c > 0)
    picks = {order[0][1], order[len(order) // 2][1], order[-1][1]}
    for e in sorted(picks):
        idx = ss[int(excl[e]) : int(incl[e])]
        tok, flat_w = idx // k, rw.flatten()[idx]
        n = idx.numel()
        want = oracle.experts_forward_backward(
            x[tok].cpu(), flat_w.view(n, 1).cpu(), torch.zeros(n, 1, dtype=torch.int64),
            moe.c_fc.weight.detach()[e : e + 1].cpu(), moe.c_proj.weight.detach()[e : e + 1].cpu(), oracle.swiglu_packed,
            grad[tok].cpu(), compute_dtype=torch.float32,
        )
        e1, e2 = nerr(dw_fc[e], want["dw_fc"][0]), nerr(dw_proj[e], want["dw_proj"][0])
        print(f"   expert {e} ({n} rows): dw_fc nerr={e1:.2e} dw_proj nerr={e2:.2e}", flush=True)
        assert e1 <= TOL and e2 <= TOL, (name, e, e1, e2)
    moe.c_fc.weight.grad = None
    moe.c_proj.weight.grad = None


def test_full_size_shared_weights_equal_dense_mlp():
    """Mixtral-shaped configuration with one weight pair shared by all experts"""
    print("full size c3: shared weights against the dense MLP", flush=True)
    T, H, I, E, k, _ = CONFIGS["c3"]
    moe, x, rw, sel, grad = _inputs("c3", shared_weights=True)
    y, dx, d_rw = _run(moe, x, rw, sel, grad)
    dw_fc = moe.c_fc.weight.grad.float().sum(0)
    dw_proj = moe.c_proj.weight.grad.float().sum(0)
    moe.c_fc.weight.grad = None
    moe.c_proj.weight.grad = None

    s = rw.float().sum(-1, keepdim=True)
    xr = x.clone().requires_grad_()
    w1 = moe.c_fc.weight[0].detach().clone().requires_grad_()
    w2 = moe.c_proj.weight[0].detach().clone().requires_grad_()
    o = oracle.swiglu_packed(xr @ w1.t()) @ w2.t()  # the stock GEMM, bf16 with fp32 accumulation
    want = (s * o.float()).to(torch.bfloat16)
    want.backward(grad)
    want_d_rw = (o.detach().float() * grad.float()).sum(-1, keepdim=True).expand(T, k)
    for label, got, ref in (("y", y, want.detach()), ("dx", dx, xr.grad), ("d_router_weights", d_rw, want_d_rw),
                            ("sum of dw_fc", dw_fc, w1.grad), ("sum of dw_proj", dw_proj, w2.grad)):
        e = nerr(got, ref)
        print(f"   {label}: nerr={e:.2e}", flush=True)
        assert e <= TOL, f"{label}: {e}"


def test_full_size_layer_forward_with_fused_gate():
    """MoE.forward on the Mixtral-shaped configuration: the gate projection runs inside the router kernel, and its int32
    expert ids go straight into the routing kernels.  Router logits of sampled tokens against the fp32 product (one
    rounding to bf16 plus the summation order); the layer's output rows of those tokens against the oracle run on the
    experts and router weights that the oracle's top-k / softmax derive from the device's own logits (a 16-bit logit
    that differs in its last place may legitimately pick another expert)."""
    from xma import KernelBackend

    print("full size c3: MoE.forward with the fused gate", flush=True)
    T, H, I, E, k, _ = CONFIGS["c3"]
    moe, x, _, _, _ = _inputs("c3")
    g = torch.Generator(device="cuda").manual_seed(11)
    with torch.no_grad():
        moe.gate.weight.copy_((torch.randn(E, H, generator=g, device="cuda") * H**-0.5).to(torch.bfloat16))
        y, logits = moe(x, kernel_backend=KernelBackend.rocm)
    torch.cuda.synchronize()
    assert y.shape == (T, H) and logits.shape == (T, E) and logits.dtype == torch.bfloat16
    assert torch.isfinite(y).all() and torch.isfinite(logits).all()
    gen = torch.Generator().manual_seed(1)
    tok = torch.cat([torch.tensor([0, 1, 31, 32, 63, 64, T - 1]), torch.randint(0, T, (57,), generator=gen)]).unique()
    xs = x[tok.cuda()].float().cpu()
    dev_logits = logits[tok.cuda()].cpu()
    lg = xs @ moe.gate.weight.detach().float().cpu().t()
    assert (lg - dev_logits.float()).abs().max().item() <= 2.0**-7 * max(1.0, lg.abs().max().item())  # 2 ulp of bf16
    rw, sel = oracle.routing_topk(dev_logits, k, torch.bfloat16)
    want = oracle.experts_forward(xs, rw.float(), sel, moe.c_fc.weight.detach().float().cpu(),
                                  moe.c_proj.weight.detach().float().cpu(), oracle.swiglu_packed)
    e = nerr(y[tok.cuda()], want)
    print(f"   {len(tok)} tokens: y nerr={e:.2e}", flush=True)
    assert e <= TOL
