"""KernelBackend.rocm implementation of the MoE expert computation.

Mirrors the op-level interface of the reference's Triton implementation
(xma/layers/moe/triton_implementation/__init__.py): ``scatter2scatter``,
``group``, ``group_bwd_W`` and the two autograd Functions behind
``up_projection_experts`` / ``down_projection_experts``; adds ``route`` (one op
for sort + histogram + offsets), ``router_topk`` (top-k + softmax behind the gate) and ``fused_swiglu_experts`` (the whole expert
computation with SwiGLU folded into the GEMM epilogues).

Differences from the reference's data flow, all of which remove HBM passes:
  * dW reads its gathered operand through the index instead of a materialised
    ``grouped_x`` / ``grouped_grad_out`` copy, and writes every element of dW
    (no zeros_like fill);
  * the router-weight scaling of dy is applied in the dX2 epilogue; dW2 reads one scaled grouped copy of dy, or, from
    four experts per token on in the fused SwiGLU path, dy through the index and activations that the dX2 epilogue
    wrote already scaled (then h is not kept for the backward either);
  * backward reuses the un-weighted expert outputs saved by forward instead of
    recomputing them with another GEMM (triton_implementation/__init__.py:117-128);
  * combine and its backward are dedicated coalesced kernels, not bmm.
"""

from __future__ import annotations

import torch

from ...rocm import ops


# ----------------------------------------------------------------------------------------- routing
@torch.no_grad()
def route(selected_experts: torch.Tensor, num_experts: int):
    """(counts uint32 (E,), inclusive offsets int64 (E,), exclusive offsets int64 (E,),
    sorted_expert_idxs, sorted_scattered_idxs int64) of the flattened (T, k) selection; stable order."""
    ids = selected_experts.flatten().contiguous()
    n, dev = ids.numel(), ids.device
    counts = torch.empty(num_experts, dtype=torch.uint32, device=dev)
    incl = torch.empty(num_experts, dtype=torch.int64, device=dev)
    excl = torch.empty(num_experts, dtype=torch.int64, device=dev)
    sorted_expert_idxs = torch.empty_like(ids)
    sorted_scattered_idxs = torch.empty(n, dtype=torch.int64, device=dev)
    ops.route_rocm(ids, counts, incl, excl, sorted_expert_idxs, sorted_scattered_idxs, None)
    return counts, incl, excl, sorted_expert_idxs, sorted_scattered_idxs


class _RouterTopK(torch.autograd.Function):
    """top-k + fp32 softmax over the selected logits + cast, and the gradient of the logits
    (xma/layers/moe/__init__.py:186-193, 256-262)"""

    @staticmethod
    def forward(ctx, router_logits: torch.Tensor, top_k: int, ids_dtype: torch.dtype):
        T = router_logits.size(0)
        weights = torch.empty(T, top_k, dtype=router_logits.dtype, device=router_logits.device)
        ids = torch.empty(T, top_k, dtype=ids_dtype, device=router_logits.device)
        ops.router_topk_rocm(router_logits, weights, ids)
        ctx.save_for_backward(router_logits, ids)
        ctx.mark_non_differentiable(ids)
        ctx.set_materialize_grads(False)  # no zero fill for the gradient of the ids, which nothing reads
        return weights, ids

    @staticmethod
    def backward(ctx, d_weights: torch.Tensor | None, _d_ids):
        if d_weights is None:  # nothing downstream depends on the router weights
            return None, None, None
        router_logits, ids = ctx.saved_tensors
        d_logits = torch.empty_like(router_logits, memory_format=torch.contiguous_format)
        ops.router_topk_bwd_rocm(router_logits, ids, d_weights.contiguous(), d_logits)
        return d_logits, None, None


class _RouterGateTopK(torch.autograd.Function):
    """gate projection + top-k + fp32 softmax + cast + int32 expert ids in one kernel; backward: the router's
    d_logits kernel, then the two skinny GEMMs of the linear layer (d_x = d_logits @ Wg, d_Wg = d_logits^T @ x) on the
    stock GEMM.  (d_x as k gathered rows of Wg per token, which is all a row of d_logits selects when no loss hangs on the
    logits themselves, measured slower than the dense product: 70 against 51 us at T = 32768, E = 128, H = 2048.)  Counterpart of gate(x) and xma/layers/moe/__init__.py:186-193, 256-262."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, gate_weight: torch.Tensor, top_k: int):
        T, E = x.size(0), gate_weight.size(0)
        logits = torch.empty(T, E, dtype=x.dtype, device=x.device)
        weights = torch.empty(T, top_k, dtype=x.dtype, device=x.device)
        ids = torch.empty(T, top_k, dtype=torch.int32, device=x.device)
        ops.router_gate_topk_rocm(x, gate_weight, logits, weights, ids)
        ctx.save_for_backward(x, gate_weight, logits, ids)
        ctx.mark_non_differentiable(ids)
        ctx.set_materialize_grads(False)  # an output nothing depends on arrives as None in backward, not as zeros
        return logits, weights, ids

    @staticmethod
    def backward(ctx, d_logits_out, d_weights, _d_ids):
        x, gate_weight, logits, ids = ctx.saved_tensors
        if d_weights is None and d_logits_out is None:
            return None, None, None
        if d_weights is None:
            d_logits = d_logits_out
        else:
            d_logits = torch.empty_like(logits)
            ops.router_topk_bwd_rocm(logits, ids, d_weights.contiguous(), d_logits)
            if d_logits_out is not None:  # the caller also used the returned router logits (an auxiliary loss)
                d_logits = d_logits + d_logits_out
        d_x = d_logits @ gate_weight if ctx.needs_input_grad[0] else None
        d_w = _gate_weight_grad(d_logits, x) if ctx.needs_input_grad[1] else None
        return d_x, d_w, None


def _gate_weight_grad(d_logits: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """d_Wg = d_logits^T @ x, (E, T) x (T, H): an output of E x H elements with a reduction over all tokens, for which the
    stock GEMM launches few workgroups.  From 32 experts and 8192 tokens on the tokens are cut into 32 slices whose
    products run as one batched GEMM and are added in fp32 (measured 158 -> 51 us at T = 32768, E = 128, H = 2048;
    104 -> 38 us at T = 16384, E = 64; with 8 experts the single GEMM is faster)."""
    T, E = d_logits.shape
    slices = 32
    if E >= 32 and T >= 8192 and T % slices == 0 and x.is_contiguous() and d_logits.is_contiguous():
        partial = torch.bmm(d_logits.view(slices, T // slices, E).transpose(1, 2), x.view(slices, T // slices, x.size(1)))
        return partial.sum(0, dtype=torch.float32).to(x.dtype)
    return d_logits.t() @ x


def router_gate_topk(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int):
    """(router logits (T, E), router weights (T, k), selected experts int32 (T, k)) from the activations and the gate's
    weight (E, H); differentiable in both."""
    return _RouterGateTopK.apply(x, gate_weight, top_k)


def router_gate_topk_supported(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int) -> bool:
    """Whether the fused kernel takes these tensors; anything else (mixed dtypes, tensors on different devices, a row
    pitch that is no multiple of 16 bytes, a shape outside the kernel's range) goes through gate(x) + router_topk.  Only
    properties a traced caller can evaluate are looked at; a tensor that starts off a 16-byte boundary is copied inside
    the op.  Note that the fused path returns int32 expert ids, the fallback int64 like torch.topk: `route` reads either."""
    return x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and gate_weight.is_contiguous() and \
        gate_weight.dtype == x.dtype and gate_weight.device == x.device and gate_weight.dim() == 2 and \
        ops.router_gate_topk_supported(x.size(1), gate_weight.size(0), top_k, x.dtype)


def router_topk(router_logits: torch.Tensor, top_k: int, ids_dtype: torch.dtype = torch.int64):
    """(router weights (T, k) in the logits' dtype, selected experts (T, k), int64 as torch.topk gives them or int32 for
    the routing kernel); differentiable in the logits."""
    return _RouterTopK.apply(router_logits, top_k, ids_dtype)


# ----------------------------------------------------------------------------------------- op mirrors
def scatter2scatter(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    out: torch.Tensor,
    FAN_OUT: int,
    x_grouped: bool = False,
    y_grouped: bool = False,
    expert_offsets: torch.Tensor | None = None,
    row_scale: torch.Tensor | None = None,
) -> None:
    """Signature of the reference op (scatter_kernel.py:137-147) plus the inclusive ``expert_offsets`` the
    expert-major tile schedule is derived from (computed from ``sorted_expert_idxs`` when not given)."""
    assert sorted_scattered_idxs.size(0) == sorted_expert_idxs.size(0)
    assert sorted_scattered_idxs.size(0) == X.size(0) * (1 if x_grouped else FAN_OUT)
    assert out.size(0) == sorted_expert_idxs.size(0) and out.size(1) == W.size(-1)
    if expert_offsets is None:
        expert_offsets = torch.bincount(sorted_expert_idxs, minlength=W.size(0)).cumsum(-1)
    ops.scatter2scatter_rocm(X, W, sorted_scattered_idxs, expert_offsets, out, row_scale, FAN_OUT, x_grouped, y_grouped)


def group(
    A: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    out: torch.Tensor,
    coeff: torch.Tensor | None = None,
    fan_out: int = 1,
) -> None:
    """Signature of the reference op (group_kernel.py:69-76)."""
    ops.group_rocm(A, sorted_expert_idxs, out, coeff, fan_out)


def group_bwd_W(DY: torch.Tensor, X: torch.Tensor, expert_offsets: torch.Tensor, DW: torch.Tensor, E: int) -> None:
    """Signature of the reference op (group_backward_kernel.py:102-103): both operands already grouped."""
    assert DW.size(0) == E
    idx = torch.empty(0, dtype=torch.int64, device=DY.device)
    ops.group_bwd_W_rocm(DY, X, idx, expert_offsets, DW, None, 0, 0)


def _empty_dw_like(expert_weights: torch.Tensor) -> torch.Tensor:
    """Uninitialised gradient with the shape and strides of ``expert_weights`` ((E, in, out) view of
    (E, out, in) storage); the dW kernel writes every element, so no zero fill is needed."""
    return torch.empty_like(expert_weights)


def _scaled_grouped_dy(grad_out: torch.Tensor, sorted_scattered_idxs: torch.Tensor, flat_w: torch.Tensor, top_k: int):
    """grouped_dy[n] = dy[idx[n] // k] * w[idx[n]] (the reference's grouped_grad_out, triton_implementation/__init__.py:134-140).
    The scale sits on the reduction index of dW2, so it has to be on an operand; one HBM-bound pass over (T*k, H) is
    cheaper than rescaling fragments inside the MFMA loop.  dX2 does not read this copy: it gathers dy through the index
    and scales in its epilogue."""
    out = torch.empty(sorted_scattered_idxs.numel(), grad_out.size(1), dtype=grad_out.dtype, device=grad_out.device)
    ops.group_rocm(grad_out, sorted_scattered_idxs, out, flat_w, top_k)
    return out


def _scale_activations_for_dw2(top_k: int, grad_out: torch.Tensor) -> bool:
    """Whether the fused SwiGLU backward scales h (in the dX2 epilogue) rather than dy (with `group`) for dW2.  The scaled
    grouped copy of dy is top_k times the size of dy and goes through HBM twice; from four experts per token on that
    costs more than the extra output of the epilogue (measured on the whole forward + backward step, two boxes: -2.4 / -3.1 % at
    top-8 with H = 2048, I = 768; -1.0 / -1.4 % at top-6 with I = 1408; +0.7 / +1.0 % at top-2 with H = 4096, I = 14336).  h then is not kept for
    the backward.  16-bit only: the fp32 kernels have no such epilogue."""
    return top_k >= 4 and grad_out.dtype in (torch.bfloat16, torch.float16)


# ----------------------------------------------------------------------------------------- autograd
def _bias_grad(A, sorted_scattered_idxs, expert_offsets, bias, row_scale=None, fan_out=1):
    """d_bias (E, out) = per-expert column sums of the grouped (or gathered and scaled) gradient rows"""
    d_bias = torch.empty_like(bias, memory_format=torch.contiguous_format)
    ops.expert_column_sums_rocm(A, sorted_scattered_idxs, expert_offsets, d_bias, row_scale, fan_out)
    return d_bias


class _UpProjectionExperts(torch.autograd.Function):
    """x (T, H) -> grouped (T*k, out); counterpart of triton_implementation/__init__.py:12-72, plus the experts' bias
    that the reference has on its torch path only (moe/__init__.py:96-100)."""

    @staticmethod
    def forward(ctx, x, expert_weights, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, bias=None):
        output = torch.empty(sorted_expert_idxs.size(0), expert_weights.size(-1), device=x.device, dtype=x.dtype)
        ops.scatter2scatter_rocm(x, expert_weights, sorted_scattered_idxs, expert_offsets, output, None, k, False, True, bias)
        ctx.save_for_backward(x, expert_weights, sorted_scattered_idxs, expert_offsets, bias)
        ctx.k = k
        return output

    @staticmethod
    def backward(ctx, grad_out):
        x, expert_weights, sorted_scattered_idxs, expert_offsets, bias = ctx.saved_tensors
        k = ctx.k
        grad_out = grad_out.contiguous()

        d_weights = _empty_dw_like(expert_weights)
        ops.group_bwd_W_rocm(grad_out, x, sorted_scattered_idxs, expert_offsets, d_weights, None, 0, k)
        d_bias = None if bias is None else _bias_grad(grad_out, None, expert_offsets, bias)

        scattered = torch.empty(sorted_scattered_idxs.size(0), x.size(1), dtype=x.dtype, device=x.device)
        ops.scatter2scatter_rocm(
            grad_out, expert_weights.permute(0, 2, 1), sorted_scattered_idxs, expert_offsets, scattered, None, 1, True, False
        )
        d_input = torch.empty_like(x)
        ops.combine_rocm(scattered, None, d_input, k)
        return d_input, d_weights, None, None, None, None, d_bias


class _DownProjectionExperts(torch.autograd.Function):
    """grouped h (T*k, I) -> y (T, H) = sum_j w[t, j] * expert_out[t*k + j]; counterpart of
    triton_implementation/__init__.py:75-162 (there called with k = 1 and router_weights (T, top_k))."""

    @staticmethod
    def forward(ctx, x, expert_weights, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, router_weights, bias=None):
        assert k == 1
        T, top_k = router_weights.shape
        expert_out = torch.empty(sorted_expert_idxs.size(0), expert_weights.size(-1), device=x.device, dtype=x.dtype)
        ops.scatter2scatter_rocm(x, expert_weights, sorted_scattered_idxs, expert_offsets, expert_out, None, 1, True, False, bias)
        router_weights = router_weights.contiguous()
        y = torch.empty(T, expert_out.size(1), device=x.device, dtype=x.dtype)
        ops.combine_rocm(expert_out, router_weights, y, top_k)
        ctx.save_for_backward(x, expert_weights, sorted_scattered_idxs, expert_offsets, router_weights, expert_out, bias)
        return y

    @staticmethod
    def backward(ctx, grad_out):
        x, expert_weights, sorted_scattered_idxs, expert_offsets, router_weights, expert_out, bias = ctx.saved_tensors
        top_k = router_weights.size(1)
        grad_out = grad_out.contiguous()

        d_router_weights = torch.empty_like(router_weights)
        ops.combine_bwd_rocm(expert_out, grad_out, d_router_weights)

        flat_w = router_weights.view(-1)
        d_weights = _empty_dw_like(expert_weights)
        grouped_dy = _scaled_grouped_dy(grad_out, sorted_scattered_idxs, flat_w, top_k)
        ops.group_bwd_W_rocm(grouped_dy, x, sorted_scattered_idxs, expert_offsets, d_weights, None, 0, 0)
        d_bias = None if bias is None else _bias_grad(grouped_dy, None, expert_offsets, bias)

        d_input = torch.empty_like(x)
        ops.scatter2scatter_rocm(
            grad_out, expert_weights.permute(0, 2, 1), sorted_scattered_idxs, expert_offsets, d_input, flat_w, top_k, False, True
        )
        return d_input, d_weights, None, None, None, None, d_router_weights, d_bias


class _FusedSwiGLUExperts(torch.autograd.Function):
    """Whole expert computation with packed SwiGLU in the GEMM epilogues:
    forward  up-projection (+ bias, SwiGLU) -> down-projection (+ bias, scattered) -> combine
    backward combine' -> dX2 (+ SwiGLU') -> dW2, dW1 (and the bias gradients) -> dX1 (scattered) -> k-way sum.
    save_activations = False keeps x and the pre-activations z only: the backward then recomputes h = swiglu_packed(z)
    and the expert outputs (one more down-projection GEMM), as the reference's backward recomputes its expert outputs
    (triton_implementation/__init__.py:117-128)."""

    @staticmethod
    def forward(ctx, x, w_fc, w_proj, router_weights, sorted_scattered_idxs, expert_offsets, b_fc=None, b_proj=None,
                save_activations=True):
        # w_fc: (E, H, 2I) view, w_proj: (E, I, H) view (both permuted views of the parameters)
        T, top_k = router_weights.shape
        M = sorted_scattered_idxs.numel()
        z = torch.empty(M, w_fc.size(-1), device=x.device, dtype=x.dtype)
        h = torch.empty(M, w_fc.size(-1) // 2, device=x.device, dtype=x.dtype)
        ops.up_projection_swiglu_rocm(x, w_fc, sorted_scattered_idxs, expert_offsets, z, h, top_k, b_fc)
        expert_out = torch.empty(M, w_proj.size(-1), device=x.device, dtype=x.dtype)
        ops.scatter2scatter_rocm(h, w_proj, sorted_scattered_idxs, expert_offsets, expert_out, None, 1, True, False, b_proj)
        router_weights = router_weights.contiguous()
        y = torch.empty(T, expert_out.size(1), device=x.device, dtype=x.dtype)
        ops.combine_rocm(expert_out, router_weights, y, top_k)
        # h is an operand of dW2 only where dW2 takes the scaled grouped copy of dy; otherwise the backward rebuilds it,
        # scaled, from z in the dX2 epilogue and h lives until the end of this forward only
        kept_h = h if save_activations and not _scale_activations_for_dw2(top_k, x) else h.new_empty(0)
        kept_out = expert_out if save_activations else expert_out.new_empty(0)
        ctx.save_for_backward(x, w_fc, w_proj, router_weights, sorted_scattered_idxs, expert_offsets, z, kept_h, kept_out,
                              b_fc, b_proj)
        return y

    @staticmethod
    def backward(ctx, grad_out):
        (x, w_fc, w_proj, router_weights, sorted_scattered_idxs, expert_offsets, z, h, expert_out, b_fc,
         b_proj) = ctx.saved_tensors
        top_k = router_weights.size(1)
        grad_out = grad_out.contiguous()
        flat_w = router_weights.view(-1)
        scaled_act_path = _scale_activations_for_dw2(top_k, grad_out)

        if expert_out.numel() == 0 and z.numel() != 0:  # not kept: recomputed from z
            if h.numel() == 0:
                h = torch.empty(z.size(0), z.size(1) // 2, dtype=z.dtype, device=z.device)
                ops.swiglu_packed_forward_rocm(z, h)
            expert_out = torch.empty(z.size(0), w_proj.size(-1), device=z.device, dtype=z.dtype)
            ops.scatter2scatter_rocm(h, w_proj, sorted_scattered_idxs, expert_offsets, expert_out, None, 1, True, False, b_proj)
        d_router_weights = torch.empty_like(router_weights)
        ops.combine_bwd_rocm(expert_out, grad_out, d_router_weights)

        dz = torch.empty_like(z)
        d_w_proj = _empty_dw_like(w_proj)
        d_b_proj = None
        if scaled_act_path and z.numel() != 0:
            # dW2 = sum_n (w_n dy_n)^T h_n = sum_n dy_n^T (w_n h_n): the dX2 epilogue, which has z and w_n at hand, writes
            # w_n h_n (T*k, I), and dW2 takes dy unscaled through the index - instead of a scaled, grouped copy of dy
            # (T*k, H) written by `group` and read back by the GEMM
            scaled_h = torch.empty(z.size(0), z.size(1) // 2, dtype=z.dtype, device=z.device)
            ops.down_projection_dx_swiglu_scaled_act_rocm(
                grad_out, w_proj.permute(0, 2, 1), sorted_scattered_idxs, expert_offsets, z, dz, scaled_h, flat_w, top_k
            )
            ops.group_bwd_W_rocm(grad_out, scaled_h, sorted_scattered_idxs, expert_offsets, d_w_proj, None, top_k, 0)
            if b_proj is not None:
                d_b_proj = _bias_grad(grad_out, sorted_scattered_idxs, expert_offsets, b_proj, flat_w, top_k)
        else:
            ops.down_projection_dx_swiglu_rocm(
                grad_out, w_proj.permute(0, 2, 1), sorted_scattered_idxs, expert_offsets, z, dz, flat_w, top_k
            )
            if b_proj is None and ops._few_rows(z.size(0), w_proj.size(0), z.dtype, "dW"):
                # a handful of rows per expert: the weight gradient's loader gathers and scales the rows of dy itself (and
                # rounds them like the copy would), one launch less
                ops.group_bwd_W_rocm(grad_out, h, sorted_scattered_idxs, expert_offsets, d_w_proj, flat_w, top_k, 0)
            else:
                grouped_dy = _scaled_grouped_dy(grad_out, sorted_scattered_idxs, flat_w, top_k)
                ops.group_bwd_W_rocm(grouped_dy, h, sorted_scattered_idxs, expert_offsets, d_w_proj, None, 0, 0)
                if b_proj is not None:
                    d_b_proj = _bias_grad(grouped_dy, None, expert_offsets, b_proj)
        d_w_fc = _empty_dw_like(w_fc)
        ops.group_bwd_W_rocm(dz, x, sorted_scattered_idxs, expert_offsets, d_w_fc, None, 0, top_k)
        d_b_fc = None if b_fc is None else _bias_grad(dz, None, expert_offsets, b_fc)

        scattered = torch.empty(z.size(0), x.size(1), dtype=x.dtype, device=x.device)
        ops.scatter2scatter_rocm(dz, w_fc.permute(0, 2, 1), sorted_scattered_idxs, expert_offsets, scattered, None, 1, True, False)
        d_x = torch.empty_like(x)
        ops.combine_rocm(scattered, None, d_x, top_k)
        return d_x, d_w_fc, d_w_proj, d_router_weights, None, None, d_b_fc, d_b_proj, None


def up_projection_experts(x, expert_weights, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, bias=None):
    return _UpProjectionExperts.apply(x, expert_weights, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, bias)


def down_projection_experts(x, expert_weights, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, router_weights,
                            bias=None):
    return _DownProjectionExperts.apply(
        x, expert_weights, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, router_weights, bias
    )


def fused_swiglu_experts(x, w_fc, w_proj, router_weights, sorted_scattered_idxs, expert_offsets, b_fc=None, b_proj=None,
                         save_activations=True):
    """save_activations = False: the backward recomputes h and the expert outputs instead of keeping them, which frees
    T k (H + I) elements per layer between forward and backward (Mixtral-shaped layer: 604 MB of 1.5 GB) for one more
    down-projection GEMM."""
    return _FusedSwiGLUExperts.apply(x, w_fc, w_proj, router_weights, sorted_scattered_idxs, expert_offsets, b_fc, b_proj,
                                     save_activations)
