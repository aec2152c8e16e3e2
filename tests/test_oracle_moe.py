"""Pins of the floating-point oracle (oracle/moe.py): closed forms evaluated scalar-by-scalar, reductions to a
dense MLP, a per-token fp64 brute force, gradcheck (finite differences) of the fp64 restatement, and the
op-level restatements against each other.  A dropped term, a wrong sign, a transposed weight or a wrong
gather/scatter index fails at least one of these."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import moe as oracle


def _dense_mlp(x, w1, w2, act):
    return F.linear(act(F.linear(x, w1)), w2)


def test_swiglu_scalar_closed_form():
    g = torch.tensor([-3.0, -0.5, 0.0, 0.7, 4.0], dtype=torch.float64)
    u = torch.tensor([1.5, -2.0, 3.0, 0.25, -1.0], dtype=torch.float64)
    want = [uu * gg / (1.0 + math.exp(-gg)) for gg, uu in zip(g.tolist(), u.tolist())]
    assert torch.allclose(oracle.swiglu(g, u), torch.tensor(want, dtype=torch.float64), rtol=1e-12, atol=0)
    packed = torch.stack([g, u], -1).flatten()  # gate on even, up on odd positions
    assert torch.allclose(oracle.swiglu_packed(packed), torch.tensor(want, dtype=torch.float64), rtol=1e-12, atol=0)
    # swapping the two roles must change the answer (pins which half is the gate)
    assert not torch.allclose(oracle.swiglu(u, g), oracle.swiglu(g, u))
    # low precision inputs: fp32 math, one rounding
    gb, ub = g.bfloat16(), u.bfloat16()
    assert torch.equal(oracle.swiglu(gb, ub), (ub.float() * gb.float() * torch.sigmoid(gb.float())).bfloat16())


def test_swiglu_backward_matches_autograd_and_finite_differences():
    torch.manual_seed(0)
    g = torch.randn(4, 6, dtype=torch.float64, requires_grad=True)
    u = torch.randn(4, 6, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(4, 6, dtype=torch.float64)
    assert torch.autograd.gradcheck(oracle.swiglu, (g, u))
    oracle.swiglu(g, u).backward(dy)
    dg, du = oracle.swiglu_backward(g.detach(), u.detach(), dy)
    assert torch.allclose(dg, g.grad, rtol=1e-10, atol=1e-12) and torch.allclose(du, u.grad, rtol=1e-10, atol=1e-12)


def test_routing_weights_brute_force():
    torch.manual_seed(1)
    logits = torch.randn(9, 6)
    for k in (1, 2, 4):
        w, idx = oracle.routing_weights(logits, k, torch.float32)
        for t in range(9):
            order = sorted(range(6), key=lambda e: -logits[t, e].item())[:k]
            assert idx[t].tolist() == order
            ex = [math.exp(logits[t, e].item()) for e in order]
            assert torch.allclose(w[t], torch.tensor([v / sum(ex) for v in ex]), rtol=1e-5, atol=1e-7)
        assert torch.allclose(w.sum(-1), torch.ones(9), atol=1e-6)


def test_routing_topk_tie_rule_and_agreement_with_topk():
    """the restatement with the spelled-out tie rule: equals torch.topk on rows without equal values, picks the
    lowest expert indices among equal values (brute force), NaN first, k = E gives the full softmax, and its
    gradient is the softmax Jacobian scattered to the selected columns"""
    torch.manual_seed(2)
    logits = torch.randn(64, 10)
    for k in (1, 3, 10):
        w0, i0 = oracle.routing_weights(logits, k, torch.float32)
        w1, i1 = oracle.routing_topk(logits, k, torch.float32)
        assert torch.equal(i0, i1) and torch.equal(w0, w1)
    # heavy ties: values from a set of 3
    tied = torch.randint(0, 3, (50, 7)).float()
    tied[0, :] = 1.0
    tied[1, 3] = float("nan")
    tied[2, 2], tied[2, 5] = 0.0, -0.0
    for k in (1, 2, 5, 7):
        w, idx = oracle.routing_topk(tied, k, torch.float32)
        for t in range(50):
            row = tied[t].tolist()
            key = lambda e: (0 if math.isnan(row[e]) else 1, -row[e] if not math.isnan(row[e]) else 0.0, e)
            assert idx[t].tolist() == sorted(range(7), key=key)[:k], (t, k)
        ok = ~torch.isnan(w).any(-1)
        assert torch.allclose(w[ok].sum(-1), torch.ones(int(ok.sum())), atol=1e-6)
    w, idx = oracle.routing_topk(logits, 10, torch.float32)
    full = torch.softmax(logits, -1)
    assert torch.allclose(w, full.gather(-1, idx), rtol=1e-6, atol=1e-7)
    # gradient: d_logits[t, idx_j] = w_j (dw_j - sum_i w_i dw_i), zero elsewhere
    lg = logits.clone().requires_grad_()
    w, idx = oracle.routing_topk(lg, 3, torch.float32)
    dw = torch.randn(64, 3)
    w.backward(dw)
    wd = w.detach()
    want = torch.zeros(64, 10).scatter_(1, idx, wd * (dw - (wd * dw).sum(-1, keepdim=True)))
    assert torch.allclose(lg.grad, want, rtol=1e-5, atol=1e-7)


def _random_case(T, E, k, H, I, dtype=torch.float64, seed=0, glu=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g, dtype=dtype)
    w1 = torch.randn(E, 2 * I if glu else I, H, generator=g, dtype=dtype) * 0.3
    w2 = torch.randn(E, H, I, generator=g, dtype=dtype) * 0.3
    logits = torch.randn(T, E, generator=g)
    rw, sel = oracle.routing_weights(logits, k, dtype)
    return x, rw, sel, w1, w2


def test_single_expert_reduces_to_dense_mlp():
    x, rw, sel, w1, w2 = _random_case(11, 1, 1, 8, 12)
    y = oracle.experts_forward(x, rw, sel, w1, w2, oracle.swiglu_packed)
    assert torch.allclose(y, _dense_mlp(x, w1[0], w2[0], oracle.swiglu_packed), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("k", [1, 2, 3])
def test_shared_weights_reduce_to_dense_mlp_for_any_routing(k):
    # router weights of a token sum to one, so if every expert holds the same weights the layer is the dense MLP
    x, rw, sel, w1, w2 = _random_case(13, 5, k, 8, 6, seed=k)
    w1 = w1[:1].expand(5, -1, -1).contiguous()
    w2 = w2[:1].expand(5, -1, -1).contiguous()
    y = oracle.experts_forward(x, rw, sel, w1, w2, oracle.swiglu_packed)
    # the weights come from an fp32 softmax, so they sum to one only to fp32 precision
    assert torch.allclose(y, _dense_mlp(x, w1[0], w2[0], oracle.swiglu_packed), rtol=1e-5, atol=1e-6)


def test_per_token_brute_force():
    x, rw, sel, w1, w2 = _random_case(10, 4, 2, 6, 5, seed=3)
    y = oracle.experts_forward(x, rw, sel, w1, w2, oracle.swiglu_packed)
    want = torch.zeros_like(x)
    for t in range(10):
        for j in range(2):
            e = int(sel[t, j])
            z = w1[e] @ x[t]
            h = torch.stack([z[2 * c + 1] * z[2 * c] / (1 + torch.exp(-z[2 * c])) for c in range(5)])
            want[t] += rw[t, j] * (w2[e] @ h)
    assert torch.allclose(y, want, rtol=1e-10, atol=1e-12)


def test_biases_per_token_brute_force_and_their_gradients():
    """Experts.bias as the torch path applies it (moe/__init__.py:96-100): z = W1[e] x + b1[e], out = W2[e] h + b2[e].
    Forward against a per-token loop; the bias gradients against their closed forms - db2[e] = sum over the (token, slot)
    pairs routed to e of w * dy[token], db1[e] = sum of dz over the expert's rows (by finite differences) - and zero for
    an expert that no token selects."""
    x, rw, sel, w1, w2 = _random_case(10, 4, 2, 6, 5, seed=4)
    sel = sel.clamp(max=2)  # expert 3 never selected
    g = torch.Generator().manual_seed(9)
    b1 = torch.randn(4, 10, generator=g, dtype=torch.float64)
    b2 = torch.randn(4, 6, generator=g, dtype=torch.float64)
    y = oracle.experts_forward(x, rw, sel, w1, w2, oracle.swiglu_packed, b1, b2)
    want = torch.zeros_like(x)
    for t in range(10):
        for j in range(2):
            e = int(sel[t, j])
            z = w1[e] @ x[t] + b1[e]
            h = torch.stack([z[2 * c + 1] * z[2 * c] / (1 + torch.exp(-z[2 * c])) for c in range(5)])
            want[t] += rw[t, j] * (w2[e] @ h + b2[e])
    assert torch.allclose(y, want, rtol=1e-10, atol=1e-12)
    dy = torch.randn(10, 6, generator=g, dtype=torch.float64)
    out = oracle.experts_forward_backward(x, rw, sel, w1, w2, oracle.swiglu_packed, dy, b_fc=b1, b_proj=b2)
    want_db2 = torch.zeros(4, 6, dtype=torch.float64)
    for t in range(10):
        for j in range(2):
            want_db2[int(sel[t, j])] += rw[t, j] * dy[t]
    assert torch.allclose(out["db_proj"], want_db2, rtol=1e-10, atol=1e-12)
    assert (out["db_fc"][3] == 0).all() and (out["db_proj"][3] == 0).all() and out["db_fc"][:3].abs().sum() > 0
    eps = 1e-6
    for e, c in ((0, 0), (1, 3), (2, 9)):
        bp, bm = b1.clone(), b1.clone()
        bp[e, c] += eps
        bm[e, c] -= eps
        fd = ((oracle.experts_forward(x, rw, sel, w1, w2, oracle.swiglu_packed, bp, b2) -
               oracle.experts_forward(x, rw, sel, w1, w2, oracle.swiglu_packed, bm, b2)) * dy).sum() / (2 * eps)
        assert abs(float(fd) - float(out["db_fc"][e, c])) <= 1e-6 * max(1.0, abs(float(fd)))


def test_backward_gradcheck_and_empty_expert():
    x, rw, sel, w1, w2 = _random_case(6, 4, 2, 4, 3, seed=5)
    sel = sel.clamp(max=2)  # expert 3 never selected; duplicates inside a token are allowed by the math
    f = lambda a, b, c, d: oracle.experts_forward(a, b, sel, c, d, oracle.swiglu_packed)
    args = [t.clone().requires_grad_() for t in (x, rw, w1, w2)]
    assert torch.autograd.gradcheck(f, args, eps=1e-6, atol=1e-6)
    out = oracle.experts_forward_backward(x, rw, sel, w1, w2, oracle.swiglu_packed, torch.randn(6, 4, dtype=torch.float64))
    assert (out["dw_fc"][3] == 0).all() and (out["dw_proj"][3] == 0).all()
    assert out["dw_fc"][:3].abs().sum() > 0


def test_low_precision_path_close_to_wide_path():
    x, rw, sel, w1, w2 = _random_case(64, 8, 2, 32, 48, dtype=torch.float32, seed=7)
    xb, rwb, w1b, w2b = (t.bfloat16() for t in (x, rw, w1 * 0.2, w2 * 0.2))
    g = torch.randn(64, 32).bfloat16()
    lo = oracle.experts_forward_backward(xb, rwb, sel, w1b, w2b, oracle.swiglu_packed, g)
    hi = oracle.experts_forward_backward(xb, rwb, sel, w1b, w2b, oracle.swiglu_packed, g, compute_dtype=torch.float32)
    for name in hi:
        assert lo[name].dtype == torch.bfloat16 and hi[name].dtype == torch.float32
        assert oracle.normalised_max_error(lo[name].float(), hi[name]) < 3e-2, name


def test_op_level_restatements_compose_to_the_layer():
    """scatter2scatter (up, grouped) -> act -> scatter2scatter (down, scattered) -> combine == experts_forward, and
    group_bwd_W / combine_bwd agree with autograd: pins gather/scatter index conventions and inclusive offsets."""
    T, E, k, H, I = 12, 4, 2, 6, 5
    x, rw, sel, w1, w2 = _random_case(T, E, k, H, I, seed=9)
    se, ss = sel.flatten().sort(stable=True)
    offs = torch.bincount(se, minlength=E).cumsum(0)
    f64 = torch.float64
    z = oracle.scatter2scatter(x, w1.permute(0, 2, 1), se, ss, k, False, True, compute_dtype=f64)
    h = oracle.swiglu_packed(z)
    eo = oracle.scatter2scatter(h, w2.permute(0, 2, 1), se, ss, 1, True, False, compute_dtype=f64)
    y = oracle.combine(eo, rw, k, f64)
    ref = oracle.experts_forward_backward(x, rw, sel, w1, w2, oracle.swiglu_packed, torch.ones(T, H, dtype=f64))
    assert torch.allclose(y, ref["y"], rtol=1e-10, atol=1e-12)
    dy = torch.ones(T, H, dtype=f64)
    assert torch.allclose(oracle.combine_bwd(eo, dy, k, f64), ref["d_router_weights"], rtol=1e-10, atol=1e-12)
    gdy = oracle.group(dy, ss, rw.flatten(), k)
    dw2 = oracle.group_bwd_W(gdy, h, offs, E, f64)  # (E, I, H) logical = permuted parameter gradient
    assert torch.allclose(dw2.permute(0, 2, 1), ref["dw_proj"], rtol=1e-10, atol=1e-12)
    # row_scale folded into the GEMM equals scaling the gathered rows first
    a = oracle.scatter2scatter(dy, w2, se, ss, k, False, True, row_scale=rw.flatten(), compute_dtype=f64)
    b = oracle.scatter2scatter(gdy, w2, se, ss, 1, True, True, compute_dtype=f64)
    assert torch.allclose(a, b, rtol=1e-10, atol=1e-12)
