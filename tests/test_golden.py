"""The oracle and the host-side torch backend against the committed golden fixtures (tests/golden/*.npz).

The fixtures were written by this oracle (tests/golden/make_golden.py; the reference holds no vectors for this path), so
they pin regressions of the oracle and of the torch backend, not parity: what pins the oracle itself is
tests/test_oracle_routing.py and tests/test_oracle_moe.py."""

import os

import numpy as np
import torch

from oracle import moe as oracle_moe
from oracle import routing as oracle_routing

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_routing_fixture():
    f = np.load(os.path.join(GOLDEN, "routing_257x8.npz"))
    r = oracle_routing.route(f["ids"], 8)
    for name, v in r.items():
        assert np.array_equal(v, f[name]) and v.dtype == f[name].dtype, name
    assert f["counts"][7] == 0 and f["offsets_inclusive"][-1] == 257


def test_moe_fixture_oracle_and_torch_backend():
    from xma import KernelBackend
    from xma.functional import swiglu_packed
    from xma.layers import MoE

    f = np.load(os.path.join(GOLDEN, "moe_swiglu_24x16x24_e4k2.npz"))
    t = {k: torch.from_numpy(f[k]) for k in f.files}
    rw, sel = oracle_moe.routing_weights(t["logits"], 2, torch.float32)
    assert torch.equal(sel, t["selected_experts"]) and torch.allclose(rw, t["router_weights"], rtol=1e-6, atol=1e-7)
    out = oracle_moe.experts_forward_backward(t["x"], rw, sel, t["w_fc"], t["w_proj"], oracle_moe.swiglu_packed, t["grad_out"])
    for name, v in out.items():
        assert torch.allclose(v, t[name], rtol=1e-5, atol=1e-6), name

    # the package's KernelBackend.torch branch is the same function
    moe = MoE(4, 2, 16, 24, swiglu_packed, True, add_bias=False, std=0.02)
    with torch.no_grad():
        moe.c_fc.weight.copy_(t["w_fc"])
        moe.c_proj.weight.copy_(t["w_proj"])
    x = t["x"].clone().requires_grad_()
    r = rw.clone().requires_grad_()
    y = moe._compute_experts(x, r, sel, kernel_backend=KernelBackend.torch)
    y.backward(t["grad_out"])
    got = {"y": y, "dx": x.grad, "d_router_weights": r.grad, "dw_fc": moe.c_fc.weight.grad, "dw_proj": moe.c_proj.weight.grad}
    for name, v in got.items():
        assert torch.allclose(v, t[name], rtol=1e-5, atol=1e-6), name
