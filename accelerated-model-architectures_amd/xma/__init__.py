"""MI355X-native host side of XMA's MoE hot path.

Same import surface as the reference for this path: ``Accelerator``,
``KernelBackend``, ``set_seed``, ``xma.functional.continuous_count``,
``xma.functional.swiglu``/``swiglu_packed`` and ``xma.layers.MoE``.  The
``KernelBackend.rocm`` branches call hand-written gfx950 kernels through the
C ABI of ``xma/rocm/libxma_rocm.so``.
"""

from .accelerator import Accelerator, KernelBackend
from .utils import ceil_divide, set_seed
