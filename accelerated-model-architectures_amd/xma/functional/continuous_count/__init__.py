"""continuous_count with the signature of the reference
(xma/functional/continuous_count/__init__.py:15-51) and a ``rocm`` branch."""

from __future__ import annotations

import torch

from ...accelerator import Accelerator, KernelBackend


@torch.no_grad()
def continuous_count(x: torch.Tensor, bins: int, *, kernel_backend: KernelBackend | None = None) -> torch.Tensor:
    """Counts the occurrences of the values [0, bins) in ``x``; values outside
    that range are the caller's responsibility (the rocm kernel ignores them,
    ``bincount`` on the torch path does not).

    :param x: 1-D int32 or int64 tensor
    :param bins: number of bins
    :param kernel_backend: KernelBackend.rocm | KernelBackend.torch | None (platform default)
    :return: uint32 tensor of shape (bins,)
    """
    if bins == 1:
        return torch.tensor([x.numel()], dtype=torch.uint32, device=x.device)

    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in [torch.int32, torch.long]

    if kernel_backend is None:
        kernel_backend = Accelerator.get_kernel_backend()
    else:
        assert kernel_backend.verify_accelerator()

    if kernel_backend == KernelBackend.rocm:
        from ...rocm.ops import CONTINUOUS_COUNT_SET_MAX_BINS, continuous_count_rocm, continuous_count_set_rocm

        if bins <= CONTINUOUS_COUNT_SET_MAX_BINS:  # the kernels write the counts: no zero fill
            y = torch.empty(bins, dtype=torch.uint32, device=x.device)
            continuous_count_set_rocm(x=x.contiguous(), y=y)
        else:
            y = torch.zeros(bins, dtype=torch.uint32, device=x.device)
            continuous_count_rocm(x=x.contiguous(), y=y, workspace=None)
    elif kernel_backend == KernelBackend.torch:
        y = x.bincount(minlength=bins).to(torch.uint32)
    else:
        raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

    return y
