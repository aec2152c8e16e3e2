"""Floating-point oracle for the MoE expert computation (CPU torch).

Test infrastructure only.  Restates the reference's torch path

* router weights           xma/layers/moe/__init__.py:182-195, 256-262
* expert computation       xma/layers/moe/__init__.py:235-250
* per-expert linear loop   xma/layers/moe/__init__.py:89-105
* SwiGLU definitions       xma/functional/swiglu/torch_implementation.py:9-30
* SwiGLU closed-form grads xma/functional/swiglu/triton_implementation/backward.py:14-23

All tensors are CPU tensors.  ``experts_forward`` works in whatever dtype it
is given: bf16 reproduces the reference's rounding points (gate multiply and
the k-term accumulation happen in the activation dtype), fp32/fp64 inputs give
the high-precision value of the same mathematical function.
"""

from __future__ import annotations

from typing import Callable

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- activations
def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """up * gate * sigmoid(gate), computed in fp32 then cast back
    (swiglu/torch_implementation.py:9-18)."""
    dtype = gate.dtype
    wide = torch.float64 if dtype == torch.float64 else torch.float32
    g = gate.to(wide)
    return (up.to(wide) * (g * torch.sigmoid(g))).to(dtype)


def swiglu_packed(x: torch.Tensor) -> torch.Tensor:
    """Interleaved layout: gate = even columns, up = odd columns
    (swiglu/torch_implementation.py:21-30)."""
    return swiglu(x[..., 0::2], x[..., 1::2])


def swiglu_backward(gate: torch.Tensor, up: torch.Tensor, dy: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """dg = dy*u*(s + g*s*(1-s)), du = dy*g*s with s = sigmoid(g)
    (swiglu/triton_implementation/backward.py:14-23)."""
    dtype = gate.dtype
    wide = torch.float64 if dtype == torch.float64 else torch.float32
    g, u, d = gate.to(wide), up.to(wide), dy.to(wide)
    s = torch.sigmoid(g)
    silu = g * s
    return (d * u * (s + silu * (1 - s))).to(dtype), (d * silu).to(dtype)


# --------------------------------------------------------------------------- router
def routing_weights(router_logits: torch.Tensor, top_k: int, out_dtype: torch.dtype):
    """Top-k selection and fp32 softmax over the k selected logits
    (moe/__init__.py:186-193 and :256-262).  Returns (weights (T,k) in
    out_dtype, selected experts int64 (T,k))."""
    if top_k == 1:
        vals, idx = router_logits.max(dim=-1, keepdim=True)
    else:
        vals, idx = router_logits.topk(top_k, dim=-1)
    w = F.softmax(vals.float(), dim=-1).to(out_dtype)
    return w, idx


def routing_topk(router_logits: torch.Tensor, top_k: int, out_dtype: torch.dtype):
    """routing_weights with the order among equal logits spelled out, which torch.topk leaves open: the k largest
    values in descending order, the lower expert index first among equals (a stable descending sort; NaN counts as
    the largest value, -0 equals +0).  On rows without equal values it is routing_weights.  Differentiable in the
    logits (moe/__init__.py:186-193, 256-262)."""
    idx = torch.sort(router_logits.detach().float(), dim=-1, descending=True, stable=True).indices[:, :top_k].contiguous()
    vals = router_logits.gather(-1, idx)
    w = F.softmax(vals.float(), dim=-1).to(out_dtype)
    return w, idx


# --------------------------------------------------------------------------- experts
def experts_forward(
    x: torch.Tensor,  # (T, H)
    router_weights: torch.Tensor,  # (T, k) same dtype as x
    selected_experts: torch.Tensor,  # (T, k) integer
    w_fc: torch.Tensor,  # (E, F, H)   F = 2I for a GLU activation, else I
    w_proj: torch.Tensor,  # (E, H, I)
    act: Callable[[torch.Tensor], torch.Tensor],
    b_fc: torch.Tensor | None = None,  # (E, F)
    b_proj: torch.Tensor | None = None,  # (E, H)
) -> torch.Tensor:
    """The torch branch of ``MoE._compute_experts`` (moe/__init__.py:210-211,
    235-250) with ``Experts.torch_forward`` (:89-105) inlined.  The sort is
    taken stable (ties in original order); the result does not depend on the
    order inside an expert except through floating-point summation order of
    ``index_add``."""
    T, H = x.shape
    E = w_fc.shape[0]
    k = selected_experts.shape[1]

    flat = selected_experts.flatten()
    sorted_expert_idxs, sorted_scattered_idxs = flat.sort(stable=True)
    counts = torch.bincount(sorted_expert_idxs, minlength=E).tolist()

    fan_in_index = sorted_scattered_idxs // k
    batch_gates = router_weights.flatten()[sorted_scattered_idxs]

    grouped = x[fan_in_index].split(counts, dim=0)
    outs = []
    for e in range(E):
        h = F.linear(grouped[e], w_fc[e], None if b_fc is None else b_fc[e])
        h = act(h)
        outs.append(F.linear(h, w_proj[e], None if b_proj is None else b_proj[e]))
    out = torch.cat(outs, dim=0)

    out = out * batch_gates.unsqueeze(-1)
    zeros = torch.zeros((T, H), dtype=out.dtype)
    return zeros.index_add(0, fan_in_index, out)


def experts_forward_backward(
    x: torch.Tensor,
    router_weights: torch.Tensor,
    selected_experts: torch.Tensor,
    w_fc: torch.Tensor,
    w_proj: torch.Tensor,
    act: Callable[[torch.Tensor], torch.Tensor],
    grad_out: torch.Tensor,
    compute_dtype: torch.dtype | None = None,
    b_fc: torch.Tensor | None = None,
    b_proj: torch.Tensor | None = None,
) -> dict[str, torch.Tensor]:
    """Forward and stock-autograd backward of ``experts_forward`` for an
    upstream gradient ``grad_out`` (the reference test uses ones,
    tests/layers/moe_test.py:125; a general gradient pins more).  With
    ``compute_dtype`` the (bit-identical) inputs are first widened, which
    gives the fp32/fp64 value of the same function."""
    cd = compute_dtype or x.dtype
    leaves = [t.detach().to(cd).clone().requires_grad_() for t in (x, router_weights, w_fc, w_proj)]
    xx, rw, w1, w2 = leaves
    b1 = None if b_fc is None else b_fc.detach().to(cd).clone().requires_grad_()
    b2 = None if b_proj is None else b_proj.detach().to(cd).clone().requires_grad_()
    y = experts_forward(xx, rw, selected_experts, w1, w2, act, b1, b2)
    y.backward(grad_out.to(cd))
    out = {"y": y.detach(), "dx": xx.grad, "d_router_weights": rw.grad, "dw_fc": w1.grad, "dw_proj": w2.grad}
    if b1 is not None:  # an expert without rows never enters the graph: its bias gradient is zero
        out["db_fc"] = b1.grad if b1.grad is not None else torch.zeros_like(b1)
    if b2 is not None:
        out["db_proj"] = b2.grad if b2.grad is not None else torch.zeros_like(b2)
    return out


def normalised_max_error(got: torch.Tensor, want: torch.Tensor) -> float:
    """max|got - want| / max|want| in fp64: the error measure the parity bar
    (1e-2 for bf16 outputs and gradients) is stated on."""
    want = want.double()
    denom = want.abs().max().item()
    err = (got.double() - want).abs().max().item() if want.numel() else 0.0
    return err / denom if denom > 0 else err


# --------------------------------------------------------------------------- op-level restatements
# Semantics of the reference's three MoE kernels, written as dense loops over experts in fp32/fp64.
def scatter2scatter(
    X: torch.Tensor,  # (rows, K)
    W: torch.Tensor,  # (E, K, N) logical
    sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    fan_out: int,
    x_grouped: bool,
    y_grouped: bool,
    row_scale: torch.Tensor | None = None,
    compute_dtype: torch.dtype = torch.float32,
    bias: torch.Tensor | None = None,  # (E, N)
) -> torch.Tensor:
    """out[dst(n)] = X[src(n)] @ W[e(n)] with src(n) = n or idx[n] // fan_out and dst(n) = n or idx[n]
    (xma/layers/moe/triton_implementation/scatter_kernel.py:58-134: row selection :105-108, store :128-134); with
    `bias`, the expert's bias row is added to the product as F.linear adds it (xma/layers/moe/__init__.py:96-100)."""
    M = sorted_scattered_idxs.numel()
    N = W.shape[-1]
    out = torch.zeros(M, N, dtype=compute_dtype)
    Xc, Wc = X.to(compute_dtype), W.to(compute_dtype)
    for n in range(M):
        e = int(sorted_expert_idxs[n])
        s = int(sorted_scattered_idxs[n])
        src = n if x_grouped else s // fan_out
        dst = n if y_grouped else s
        v = Xc[src] @ Wc[e]
        if bias is not None:
            v = v + bias[e].to(compute_dtype)
        if row_scale is not None:
            v = v * row_scale[s].to(compute_dtype)
        out[dst] = v
    return out


def group(A: torch.Tensor, idx: torch.Tensor, coeff: torch.Tensor | None, fan_out: int) -> torch.Tensor:
    """out[n] = A[idx[n] // fan_out] * coeff[idx[n]], multiply in the input dtype
    (xma/layers/moe/triton_implementation/group_kernel.py:12-66)."""
    out = A[idx // fan_out]
    if coeff is not None:
        out = out * coeff[idx].unsqueeze(-1)
    return out


def group_bwd_W(
    DY: torch.Tensor, X: torch.Tensor, expert_offsets: torch.Tensor, E: int, compute_dtype: torch.dtype = torch.float32
) -> torch.Tensor:
    """DW[e] (K, N) = X_e^T @ DY_e over the expert's contiguous row range given by INCLUSIVE offsets; experts
    without rows stay zero (xma/layers/moe/triton_implementation/group_backward_kernel.py:21-99)."""
    K, N = X.shape[1], DY.shape[1]
    DW = torch.zeros(E, K, N, dtype=compute_dtype)
    lo = 0
    for e in range(E):
        hi = int(expert_offsets[e])
        if hi > lo:
            DW[e] = X[lo:hi].to(compute_dtype).T @ DY[lo:hi].to(compute_dtype)
        lo = hi
    return DW


def combine(expert_out: torch.Tensor, w: torch.Tensor | None, k: int, compute_dtype: torch.dtype = torch.float32):
    """y[t] = sum_j w[t, j] * expert_out[t*k + j] (the bmm of triton_implementation/__init__.py:100-101; w None
    is the plain `.sum(-2)` of :70)."""
    T = expert_out.shape[0] // k
    o = expert_out.to(compute_dtype).view(T, k, -1)
    if w is None:
        return o.sum(1)
    return (w.to(compute_dtype).unsqueeze(-1) * o).sum(1)


def combine_bwd(expert_out: torch.Tensor, dy: torch.Tensor, k: int, compute_dtype: torch.dtype = torch.float32):
    """d_w[t, j] = <expert_out[t*k + j], dy[t]> (the bmm of triton_implementation/__init__.py:130-131)."""
    T = dy.shape[0]
    return (expert_out.to(compute_dtype).view(T, k, -1) * dy.to(compute_dtype).unsqueeze(1)).sum(-1)
