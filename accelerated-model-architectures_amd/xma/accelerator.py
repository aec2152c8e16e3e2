"""Backend selector for the path (reference: xma/accelerator.py:22-53, 123-139).

Only what the MoE layer and continuous_count consult is restated: the two
enums, accelerator detection, ``verify_accelerator`` and the default backend.
One deliberate difference: on a ROCm GPU the default backend is ``rocm`` (the
reference falls through to ``triton`` there, xma/accelerator.py:128-137) and
on a host without a GPU it is ``torch``.
"""

from __future__ import annotations

from enum import Enum
from functools import lru_cache

import torch


class KernelBackend(Enum):
    # the full set of names is kept so that call sites and configs interchange
    cuda = "cuda"
    jax = "jax"
    mps = "mps"
    nki = "nki"
    pallas = "pallas"
    rocm = "rocm"
    torch = "torch"
    triton = "triton"

    def get_compatible_accelerator(self) -> "Accelerator | None":
        found = Accelerator.get_accelerator()
        if self is KernelBackend.torch:
            return found
        if self is KernelBackend.triton and found in (Accelerator.cuda, Accelerator.rocm):
            return found
        return {
            KernelBackend.cuda: Accelerator.cuda,
            KernelBackend.mps: Accelerator.mps,
            KernelBackend.nki: Accelerator.trainium,
            KernelBackend.pallas: Accelerator.tpu,
            KernelBackend.rocm: Accelerator.rocm,
        }.get(self)

    def verify_accelerator(self) -> bool:
        return self.get_compatible_accelerator() == Accelerator.get_accelerator()


class Accelerator(Enum):
    cpu = "cpu"
    cuda = "cuda"
    mps = "mps"
    rocm = "rocm"
    tpu = "tpu"
    trainium = "trainium"

    @staticmethod
    @lru_cache
    def get_accelerator() -> "Accelerator":
        if torch.cuda.is_available():
            return Accelerator.rocm if torch.version.hip is not None else Accelerator.cuda
        return Accelerator.cpu

    @staticmethod
    def get_current_device() -> int | str:
        if Accelerator.get_accelerator() in (Accelerator.cuda, Accelerator.rocm):
            return torch.cuda.current_device()
        return "cpu"

    @staticmethod
    def device_count() -> int:
        if Accelerator.get_accelerator() in (Accelerator.cuda, Accelerator.rocm):
            return torch.cuda.device_count()
        return 1

    @staticmethod
    @lru_cache
    def get_kernel_backend() -> KernelBackend:
        found = Accelerator.get_accelerator()
        if found is Accelerator.rocm:
            return KernelBackend.rocm
        if found is Accelerator.cuda:
            return KernelBackend.cuda
        return KernelBackend.torch

    @staticmethod
    def synchronize() -> None:
        if Accelerator.get_accelerator() in (Accelerator.cuda, Accelerator.rocm):
            torch.cuda.synchronize()

    @staticmethod
    def get_core_count() -> int:
        if Accelerator.get_accelerator() in (Accelerator.cuda, Accelerator.rocm):
            return torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
        raise ValueError(f"unexpected accelerator ({Accelerator.get_accelerator()})")
