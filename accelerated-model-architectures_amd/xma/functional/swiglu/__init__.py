"""swiglu / swiglu_packed with the reference's signatures
(xma/functional/swiglu/__init__.py:39-87).  The torch branch restates
xma/functional/swiglu/torch_implementation.py:9-30; the rocm branch runs the
stand-alone HIP kernels (any 2-D size, bf16 / fp16 / fp32, forward and
backward).  ``swiglu_packed`` is also the activation the MoE layer recognises
and fuses into its grouped GEMMs."""

from __future__ import annotations

import torch
import torch.nn.functional as F

from ...accelerator import Accelerator, KernelBackend


def _resolve(kernel_backend: KernelBackend | None, x: torch.Tensor) -> KernelBackend:
    if kernel_backend is None:
        kernel_backend = Accelerator.get_kernel_backend() if x.is_cuda else KernelBackend.torch
    else:
        assert kernel_backend.verify_accelerator()
    return kernel_backend


def _swiglu_torch(g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    dtype = g.dtype
    return (u.float() * F.silu(g.float())).to(dtype)


def _swiglu_packed_torch(x: torch.Tensor) -> torch.Tensor:
    return _swiglu_torch(x[..., ::2], x[..., 1::2])


class _SwigluPackedROCm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: torch.Tensor) -> torch.Tensor:
        from ...rocm.ops import swiglu_packed_forward_rocm

        x = x.contiguous()
        y = torch.empty(x.size(0), x.size(1) // 2, dtype=x.dtype, device=x.device)
        swiglu_packed_forward_rocm(x=x, y=y)
        ctx.save_for_backward(x)
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor) -> torch.Tensor:
        from ...rocm.ops import swiglu_packed_backward_rocm

        (x,) = ctx.saved_tensors
        dx = torch.empty_like(x)
        swiglu_packed_backward_rocm(x=x, dy=dy.contiguous(), dx=dx)
        return dx


def _row_major_2d(t: torch.Tensor) -> torch.Tensor:
    """2-D view with contiguous rows that do not overlap (any row pitch >= the row length is fine for the kernels).
    Anything else is copied: transposed views, and the broadcast views autograd hands to a backward - the gradient of
    ``y.sum(0)`` has strides (0, 1) - or a caller passes as an expanded operand."""
    t = t.reshape(-1, t.size(-1)) if t.dim() != 2 else t
    rows_ok = t.stride(1) == 1 or t.size(1) == 1
    pitch_ok = t.size(0) <= 1 or t.stride(0) >= t.size(1)
    return t if rows_ok and pitch_ok else t.contiguous()


class _SwigluROCm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
        from ...rocm.ops import swiglu_forward_rocm

        g, u = _row_major_2d(g), _row_major_2d(u)
        y = torch.empty(g.shape, dtype=g.dtype, device=g.device)
        swiglu_forward_rocm(g=g, u=u, y=y)
        ctx.save_for_backward(g, u)
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        from ...rocm.ops import swiglu_backward_rocm

        g, u = ctx.saved_tensors
        dg = torch.empty(g.shape, dtype=g.dtype, device=g.device)
        du = torch.empty(u.shape, dtype=u.dtype, device=u.device)
        swiglu_backward_rocm(g=g, u=u, dy=_row_major_2d(dy), dg=dg, du=du)
        return dg, du


def _check_rocm_dtype(x: torch.Tensor, what: str) -> None:
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError(f"{what} on KernelBackend.rocm covers bf16/fp16/fp32 (got {x.dtype})")


def swiglu(gate: torch.Tensor, up: torch.Tensor, *, kernel_backend: KernelBackend | None = None) -> torch.Tensor:
    """computes swiglu activation as `up * gate * sigmoid(gate)`"""
    assert gate.size() == up.size(), "tensors gate and up should have same shape"
    assert gate.type() == up.type(), "tensors gate and up should have same dtype"

    kernel_backend = _resolve(kernel_backend, gate)
    if kernel_backend == KernelBackend.rocm:
        _check_rocm_dtype(gate, "swiglu")
        original_shape = gate.size()
        if gate.numel() == 0:
            return torch.empty_like(gate)
        return _SwigluROCm.apply(gate.reshape(-1, original_shape[-1]), up.reshape(-1, original_shape[-1])).view(original_shape)
    if kernel_backend == KernelBackend.torch:
        return _swiglu_torch(gate, up)
    raise ValueError(f"unexpected kernel_backend ({kernel_backend})")


def swiglu_packed(x: torch.Tensor, *, kernel_backend: KernelBackend | None = None) -> torch.Tensor:
    """swiglu of a tensor whose last dimension interleaves gate, up, gate, up, ..."""
    original_shape = x.size()
    assert original_shape[-1] % 2 == 0
    H = original_shape[-1] // 2

    kernel_backend = _resolve(kernel_backend, x)
    if kernel_backend == KernelBackend.rocm:
        _check_rocm_dtype(x, "swiglu_packed")
        y = _SwigluPackedROCm.apply(x.flatten(0, -2))
    elif kernel_backend == KernelBackend.torch:
        y = _swiglu_packed_torch(x.flatten(0, -2))
    else:
        raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

    return y.view(*original_shape[:-1], H)


# marker the MoE layer looks for when deciding to fuse the activation into its GEMM epilogues
swiglu_packed._xma_fused_activation = "swiglu_packed"
