"""Host logic that needs no GPU: the C-ABI library loads and exports every symbol include/xma_rocm.h declares,
backend selection and error behaviour mirror the reference, module layout matches its state-dict."""

import ctypes
import os
import re

import pytest
import torch
import torch.nn as nn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "xma_rocm.h")).read()
    return sorted(set(re.findall(r"\b(xma_rocm_[a-zA-Z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from xma.rocm import LIBRARY_PATH, get_library
    from xma.rocm.loader import SIGNATURES

    assert os.path.isfile(LIBRARY_PATH), "build the library first: python __graft_entry__.py"
    lib = ctypes.CDLL(LIBRARY_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 13
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/xma_rocm.h but not exported"
    assert sorted(SIGNATURES) == declared  # the ctypes table covers exactly the header
    lib = get_library()
    assert lib.xma_rocm_abi_version() == 1
    # host-only entry points (no GPU work)
    assert lib.xma_rocm_route_workspace_bytes(4 * 1024 * 1024, 64) == (4 * 1024 * 1024 // 4096) * 64 * 4
    assert lib.xma_rocm_continuous_count_workspace_bytes(4 * 1024 * 1024, 64) == 1024 * 64 * 4
    assert lib.xma_rocm_continuous_count_workspace_bytes(1000, 64) == 0
    assert lib.xma_rocm_route_workspace_bytes(0, 8) == 8 * 4
    assert lib.xma_rocm_route_workspace_bytes(-1, 8) == 0


def test_argument_errors_are_reported_before_any_launch():
    from xma.rocm import get_library

    lib = get_library()
    # bins < 1, E out of range, unsupported dtype, misaligned sizes: all rejected on the host
    assert lib.xma_rocm_continuous_count(None, 0, 10, None, 0, None, 0, None) == -1
    assert b"continuous_count" in lib.xma_rocm_last_error()
    assert lib.xma_rocm_route(None, 0, 10, 100000, None, None, None, None, None, None, 0, None) == -1
    # the entry point with static scratch refuses what does not fit its array, before touching the device
    assert lib.xma_rocm_route_static_max_units_times_experts() == 1 << 18
    big = ctypes.c_void_p(256)
    assert lib.xma_rocm_route_static(big, 0, 4096 * 129, 2048, big, big, None, None, big, None) == -3
    assert b"static scratch" in lib.xma_rocm_last_error()
    assert lib.xma_rocm_route_static(None, 0, 10, 100000, None, None, None, None, None, None) == -1
    assert lib.xma_rocm_combine(None, 8, None, None, 8, 4, 2, 12, 0, None) == -1  # H % 8 != 0
    assert lib.xma_rocm_combine(None, 8, None, None, 8, 4, 2, 16, 7, None) == -2  # dtype
    rc = lib.xma_rocm_scatter2scatter(None, 64, None, 64 * 64, 64, 0, None, None, None, 64, None, 0, None, 16, 60, 64, 2, 1, 1, 1,
                                      0, 0, None, 0, None)
    assert rc == -2 and b"multiples of 8" in lib.xma_rocm_last_error()
    # router: k > E, E and k beyond what a wave holds, row stride shorter than a row, dtype
    assert lib.xma_rocm_router_topk(None, 8, 4, 8, 9, 0, None, None, 1, None) == -1 and b"k <= E" in lib.xma_rocm_last_error()
    assert lib.xma_rocm_router_topk(None, 4096, 4, 4096, 2, 0, None, None, 1, None) == -2
    assert lib.xma_rocm_router_topk(None, 128, 4, 128, 65, 0, None, None, 1, None) == -2
    assert lib.xma_rocm_router_topk(None, 4, 4, 8, 2, 0, None, None, 1, None) == -1
    assert lib.xma_rocm_router_topk(None, 8, 4, 8, 2, 5, None, None, 1, None) == -2
    assert lib.xma_rocm_router_topk(None, 8, 4, 8, 2, 0, None, None, 1, None) == -1  # null pointers with T > 0
    assert lib.xma_rocm_router_topk_bwd(None, 8, 4, 8, 2, 0, None, 1, None, None, 4, None) == -1  # ldd < E
    assert lib.xma_rocm_router_topk(None, 8, 0, 8, 2, 0, None, None, 1, None) == 0
    # the few-token entry points: dtype (no fp32), M beyond the epilogue's grid, a missing workspace where sums go through
    # one (few column blocks and a long K: the launch is cut along K), none needed for W as (N, K) with a plain store (fails later, on the null operands), dW shapes
    p = ctypes.c_void_p(256)
    few = lib.xma_rocm_scatter2scatter_few_rows
    assert few(p, 64, p, 64 * 64, 64, 0, p, p, p, 64, None, 0, None, 0, None, None, 0, 4, 64, 64, 2, 1, 1, 1, 0, 2, None, 0, None) == -2
    assert few(p, 64, p, 64 * 64, 64, 0, p, p, p, 64, None, 0, None, 0, None, None, 0, 70000, 64, 64, 2, 1, 1, 1, 0, 0, None, 0, None) == -1
    assert few(p, 16384, p, 16384 * 64, 64, 1, p, p, p, 64, None, 0, None, 0, None, None, 0, 4, 64, 16384, 2, 1, 1, 1, 0, 0, None, 0, None) == -3
    assert b"workspace" in lib.xma_rocm_last_error()
    assert few(None, 64, None, 64 * 64, 64, 0, p, p, p, 64, None, 0, None, 0, None, None, 0, 4, 64, 64, 2, 1, 1, 1, 0, 0, None, 0, None) == -1
    assert b"null or misaligned" in lib.xma_rocm_last_error()
    # W as (N, K) is addressed with 32-bit byte offsets inside an expert
    assert few(p, 64, p, 64 << 26, 1 << 26, 0, p, p, p, 64, None, 0, None, 0, None, None, 0, 4, 64, 64, 2, 1, 1, 1, 0, 0, None, 0, None) == -2
    assert b"N * ldw" in lib.xma_rocm_last_error()
    ws = lib.xma_rocm_scatter2scatter_few_rows_workspace_bytes  # (M, N, K, E, w_is_kn, epilogue)
    assert ws(4, 64, 2048, 2, 0, 0) == 0 and ws(4, 64, 2048, 2, 0, 1) == 0  # the vector kernel finishes the job itself (2 rows per expert)
    assert ws(4, 64, 2048, 2, 0, 2) == 4 * 64 * 4  # SwiGLU backward: through the epilogue kernel
    assert ws(4, 64, 64, 2, 0, 2) == 0  # short rows of W: the small tile, one K range, epilogue in the kernel
    assert ws(4, 64, 16384, 2, 1, 0) == 32 * 4 * 64 * 4  # W as (K, N): the small tile at any number of rows, 32 ranges of K
    assert ws(64, 2048, 16384, 8, 1, 0) == 4 * 64 * 2048 * 4 and ws(64, 8192, 2048, 8, 1, 2) == 0  # small tile: 4 ranges of K; none
    assert ws(64, 16384, 2048, 8, 0, 1) == 0  # small MFMA tile, enough workgroups from N alone
    assert ws(64, 2048, 8192, 8, 0, 0) == 4 * 64 * 2048 * 4  # small MFMA tile cut into 4 ranges of K
    assert ws(0, 64, 64, 2, 1, 0) == 0
    dw = lib.xma_rocm_group_bwd_W_few_rows
    assert dw(p, 64, 1, 1, None, p, 64, 1, 1, p, p, p, 64 * 64, 64, 64, 64, 2, 4, 2, None) == -2  # fp32
    assert dw(p, 64, 1, 1, None, p, 60, 1, 1, p, p, p, 64 * 64, 64, 64, 64, 2, 4, 0, None) == -2  # ldx % 8
    assert dw(p, 60, 1, 1, None, p, 64, 1, 1, p, p, p, 64 * 64, 64, 64, 64, 2, 4, 0, None) == -2  # lddy % 8
    assert dw(None, 64, 1, 1, None, p, 64, 1, 1, p, p, p, 64 * 64, 64, 64, 64, 2, 4, 0, None) == -1
    # empty problems are accepted without touching a pointer
    assert few(None, 64, None, 64 * 64, 64, 0, None, None, None, 64, None, 0, None, 0, None, None, 0, 0, 64, 64, 2, 1, 1, 1, 0, 0, None, 0, None) == 0
    assert lib.xma_rocm_combine(None, 8, None, None, 8, 0, 2, 16, 0, None) == 0
    assert lib.xma_rocm_continuous_count(None, 0, 0, ctypes.c_void_p(16), 4, None, 0, None) == 0


def test_few_token_dispatch_rule():
    """which grouped GEMM forms take the kernels of the few-token regime: by rows per expert on average, per form, with a
    cap on the rows in all; fp32 never"""
    from xma.rocm import ops

    bf = torch.bfloat16
    assert ops._few_rows(14, 8, bf, "x @ W^T") and ops._few_rows(768, 8, bf, "x @ W^T") and not ops._few_rows(769, 8, bf, "x @ W^T")
    assert ops._few_rows(3072, 128, bf, "dy @ W") and not ops._few_rows(16385, 1024, bf, "x @ W^T")  # the cap on the rows
    assert ops._few_rows(768, 8, bf, "dy @ W") and not ops._few_rows(769, 8, bf, "dy @ W")
    assert ops._few_rows(1024, 8, bf, "dW") and not ops._few_rows(1025, 8, bf, "dW")
    assert ops._few_rows(16384, 128, bf, "dW") and not ops._few_rows(16385, 128, bf, "dW")
    assert not ops._few_rows(0, 8, bf, "dW") and not ops._few_rows(14, 8, torch.float32, "dW")
    assert ops._few_rows(14, 8, torch.float16, "dy @ W")


def test_fused_router_shape_rule_matches_the_library():
    """the Python restatement of the fused gate + router kernel's coverage (evaluated under torch.compile, where a ctypes
    call cannot be traced) against the library's own answer"""
    from xma.rocm import get_library
    from xma.rocm.ops import router_gate_topk_supported

    lib = get_library()
    codes = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
    for dtype, code in codes.items():
        for H in (0, 4, 8, 12, 64, 4096):
            for E in (0, 1, 8, 32, 33, 128, 129, 2048):
                for k in (0, 1, 2, 8, 32, 33, 128):
                    assert router_gate_topk_supported(H, E, k, dtype) == bool(
                        lib.xma_rocm_router_gate_topk_supported(H, E, k, code)), (dtype, H, E, k)


def test_backend_selection_and_errors():
    from xma import Accelerator, KernelBackend
    from xma.functional import continuous_count, swiglu_packed
    from xma.layers import MoE

    assert KernelBackend.torch.verify_accelerator()
    if not torch.cuda.is_available():
        assert Accelerator.get_accelerator() == Accelerator.cpu
        assert Accelerator.get_kernel_backend() == KernelBackend.torch
        assert not KernelBackend.rocm.verify_accelerator()
        with pytest.raises(AssertionError):  # explicit backend on the wrong accelerator (moe/__init__.py:205-208)
            continuous_count(torch.zeros(4, dtype=torch.int32), 4, kernel_backend=KernelBackend.rocm)
    x = torch.randint(0, 5, (100,))
    assert continuous_count(x, 1).tolist() == [100]
    assert continuous_count(x, 5, kernel_backend=KernelBackend.torch).dtype == torch.uint32
    with pytest.raises(AssertionError):
        continuous_count(x.view(10, 10), 5, kernel_backend=KernelBackend.torch)
    with pytest.raises(AssertionError):
        continuous_count(x.float(), 5, kernel_backend=KernelBackend.torch)
    moe = MoE(4, 2, 16, 24, swiglu_packed, True, add_bias=False, std=0.02)
    with pytest.raises((ValueError, AssertionError)):  # a backend this build does not have (moe/__init__.py:251-252)
        moe(torch.randn(3, 16), kernel_backend=KernelBackend.triton)


def test_module_layout_matches_reference_state_dict():
    from xma.layers import MoE
    from xma.layers.moe import Experts

    moe = MoE(6, 2, 32, 48, nn.GLU(), True, add_bias=True, std=0.02)
    sd = moe.state_dict()
    assert {k: tuple(v.shape) for k, v in sd.items()} == {
        "gate.weight": (6, 32),
        "c_fc.weight": (6, 96, 32), "c_fc.bias": (6, 96), "c_fc.N_array": (6,), "c_fc.K_array": (6,),
        "c_proj.weight": (6, 32, 48), "c_proj.bias": (6, 32), "c_proj.N_array": (6,), "c_proj.K_array": (6,),
    }
    assert sd["c_fc.N_array"].dtype == torch.uint32 and sd["c_fc.N_array"].view(torch.int32).tolist() == [96] * 6
    assert sd["c_proj.K_array"].view(torch.int32).tolist() == [48] * 6
    assert (sd["c_fc.bias"] == 0).all()
    y, logits = moe(torch.randn(2, 5, 32))
    assert y.shape == (2, 5, 32) and logits.shape == (10, 6)
    e = Experts(3, 4, 5, add_bias=False, std=0.1)
    assert e.bias is None and "in_features=4" in e.extra_repr()
    moe1 = MoE(4, 1, 16, 8, nn.GELU(approximate="tanh"), False, add_bias=False, std=0.02)  # top-1 uses max
    assert moe1(torch.randn(7, 16))[0].shape == (7, 16)


def test_torch_backend_matches_oracle_in_bf16():
    from oracle import moe as oracle
    from xma import KernelBackend, set_seed
    from xma.functional import swiglu_packed
    from xma.layers import MoE

    set_seed(3)
    moe = MoE(8, 2, 64, 96, swiglu_packed, True, add_bias=False, std=0.02).to(torch.bfloat16)
    x = torch.randn(50, 64).bfloat16()
    rw, sel = oracle.routing_weights(torch.randn(50, 8), 2, torch.bfloat16)
    y = moe._compute_experts(x, rw, sel, kernel_backend=KernelBackend.torch)
    want = oracle.experts_forward(x, rw, sel, moe.c_fc.weight.data, moe.c_proj.weight.data, oracle.swiglu_packed)
    assert torch.equal(y, want)


def test_rocm_ops_fail_loudly_without_the_library(monkeypatch):
    from xma.rocm import loader

    monkeypatch.setattr(loader, "_lib", None)
    monkeypatch.setattr(loader, "LIBRARY_PATH", "/nonexistent/libxma_rocm.so")
    with pytest.raises(loader.RocmLibraryError):
        loader.get_library()
