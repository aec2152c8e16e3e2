"""swiglu / swiglu_packed with the reference's signatures
(xma/functional/swiglu/__init__.py:39-87).  The torch branch restates
xma/functional/swiglu/torch_implementation.py:9-30; the rocm branch of the
packed form runs the stand-alone HIP kernels.  ``swiglu_packed`` is also the
activation the MoE layer recognises and fuses into its grouped GEMMs."""

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


def swiglu(gate: torch.Tensor, up: torch.Tensor, *, kernel_backend: KernelBackend | None = None) -> torch.Tensor:
    """computes swiglu activation as `up * gate * sigmoid(gate)`"""
    assert gate.size() == up.size(), "tensors gate and up should have same shape"
    assert gate.type() == up.type(), "tensors gate and up should have same dtype"

    kernel_backend = _resolve(kernel_backend, gate)
    if kernel_backend == KernelBackend.rocm:
        # the separate-operand form has no dedicated kernel: interleave and use the packed one
        packed = torch.stack([gate, up], dim=-1).flatten(-2)
        return swiglu_packed(packed, kernel_backend=kernel_backend)
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
        if x.dtype not in (torch.bfloat16, torch.float16, torch.float32) or H % 8 != 0:
            raise NotImplementedError(
                f"swiglu_packed on KernelBackend.rocm covers bf16/fp16/fp32 with an output width that is a multiple of "
                f"8 (got {x.dtype}, {H})"
            )
        y = _SwigluPackedROCm.apply(x.flatten(0, -2))
    elif kernel_backend == KernelBackend.torch:
        y = _swiglu_packed_torch(x.flatten(0, -2))
    else:
        raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

    return y.view(*original_shape[:-1], H)


# marker the MoE layer looks for when deciding to fuse the activation into its GEMM epilogues
swiglu_packed._xma_fused_activation = "swiglu_packed"
