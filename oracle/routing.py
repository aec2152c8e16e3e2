"""Integer routing oracle (numpy).  Test infrastructure only.

Restates, on the CPU, what the reference computes with stock torch ops:

* histogram of expert ids      xma/functional/continuous_count/__init__.py:32-47
* sort of the flattened top-k  xma/layers/moe/__init__.py:210
* inclusive expert offsets     xma/layers/moe/__init__.py:217
"""

from __future__ import annotations

import numpy as np


def continuous_count(ids: np.ndarray, bins: int) -> np.ndarray:
    """Occurrences of each value in [0, bins) as uint32 of shape (bins,).

    Follows xma/functional/continuous_count/__init__.py:32-33 (bins == 1
    returns the element count without looking at the values) and :46-47
    (``bincount(minlength=bins)`` cast to uint32).  The contract is
    ids in [0, bins); like ``bincount`` this raises on negative ids.
    """
    ids = np.asarray(ids)
    if bins == 1:
        return np.array([ids.size], dtype=np.uint32)
    assert ids.ndim == 1, "x should be 1-dimensional"
    assert ids.dtype in (np.int32, np.int64)
    if ids.size and int(ids.min()) < 0:
        raise ValueError("negative id")
    return np.bincount(ids, minlength=bins).astype(np.uint32)


def route(ids: np.ndarray, num_experts: int) -> dict[str, np.ndarray]:
    """counts, offsets and the stable expert-major permutation of ``ids``.

    ``ids`` is the flattened (T*k,) top-k selection
    (xma/layers/moe/__init__.py:210: ``selected_experts.flatten().sort()``).
    The reference's sort is not guaranteed stable; the contract pinned here is
    the stable one (ties keep their original order), which is what
    ``torch.sort(stable=True)`` and ``numpy.argsort(kind="stable")`` give.

    Returns
      counts                 uint32 (E,)   continuous_count of the ids
      offsets_inclusive      int64  (E,)   cumsum(counts), as moe/__init__.py:217
      offsets_exclusive      int64  (E,)   inclusive - counts
      sorted_expert_idxs     ids.dtype (N,) ids in non-decreasing order
      sorted_scattered_idxs  int64  (N,)   position in the flattened (T,k) array
    """
    ids = np.asarray(ids)
    assert ids.ndim == 1 and ids.dtype in (np.int32, np.int64)
    perm = np.argsort(ids, kind="stable").astype(np.int64)
    counts = continuous_count(ids, num_experts) if num_experts > 1 else np.array([ids.size], np.uint32)
    incl = np.cumsum(counts.astype(np.int64))
    return {
        "counts": counts,
        "offsets_inclusive": incl,
        "offsets_exclusive": incl - counts.astype(np.int64),
        "sorted_expert_idxs": ids[perm],
        "sorted_scattered_idxs": perm,
    }
