"""Writes the small golden fixtures next to this script.

The reference holds no stored vectors for this path (its tests are differential and need an NVIDIA GPU), so these
are produced by this repository's own oracle (plain numpy / CPU torch restatement, seed 0) AFTER it passed the
pins in tests/test_oracle_*.py.  They guard the oracle and the host code against regressions and travel to the GPU
box as data; the reference itself was neither imported nor run.

    python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import moe, routing  # noqa: E402


def main():
    # routing: 257 ids over 8 experts (one left empty), int64
    rng = np.random.default_rng(0)
    ids = rng.integers(0, 7, 257).astype(np.int64)
    r = routing.route(ids, 8)
    np.savez(os.path.join(HERE, "routing_257x8.npz"), ids=ids, **r)

    # expert computation, fp32: T=24, H=16, I=24, E=4, top-2, packed SwiGLU, W ~ N(0, 0.02)-like scaled up for signal
    g = torch.Generator().manual_seed(0)
    T, H, I, E, k = 24, 16, 24, 4, 2
    x = torch.randn(T, H, generator=g)
    w1 = torch.randn(E, 2 * I, H, generator=g) * 0.2
    w2 = torch.randn(E, H, I, generator=g) * 0.2
    logits = torch.randn(T, E, generator=g)
    grad = torch.randn(T, H, generator=g)
    rw, sel = moe.routing_weights(logits, k, torch.float32)
    out = moe.experts_forward_backward(x, rw, sel, w1, w2, moe.swiglu_packed, grad)
    np.savez(
        os.path.join(HERE, "moe_swiglu_24x16x24_e4k2.npz"),
        x=x.numpy(), w_fc=w1.numpy(), w_proj=w2.numpy(), logits=logits.numpy(), grad_out=grad.numpy(),
        router_weights=rw.numpy(), selected_experts=sel.numpy(),
        **{name: t.numpy() for name, t in out.items()},
    )
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
