"""torch.library custom ops over the C ABI of libxma_rocm.so.

Same shape as the reference's op boundary (xma/custom_op.py:72-108): every op
is a ``torch.library.custom_op`` that mutates caller-allocated outputs and
returns nothing, so autograd Functions and ``torch.compile`` see ordinary ops.
The Python side validates shapes/dtypes/contiguity and raises like the
reference (asserts), then hands raw device pointers, sizes, strides and the
current HIP stream to the library.  The stream is looked up per call because
backward runs on autograd's thread.
"""

from __future__ import annotations

import torch

from .loader import check, get_library


_DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

EPI_STORE, EPI_SWIGLU, EPI_SWIGLU_BWD = 0, 1, 2


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _code(t: torch.Tensor) -> int:
    if t.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"KernelBackend.rocm covers bfloat16, float16 and float32, got {t.dtype}")
    return _DTYPE_CODE[t.dtype]


def _rows(t: torch.Tensor, name: str) -> int:
    """leading dimension of a 2-D row-major tensor"""
    assert t.dim() == 2 and t.is_cuda, f"{name} should be a 2-D device tensor"
    assert t.stride(1) == 1 or t.size(1) == 1, f"{name} should have contiguous rows"
    return t.stride(0) if t.size(0) > 1 else max(t.size(1), t.stride(0))


def _weight_layout(W: torch.Tensor) -> tuple[int, int, int]:
    """W is logically (E, K, N) as in the reference's scatter2scatter.  Returns
    (w_is_kn, expert stride, leading dimension) of its storage."""
    assert W.dim() == 3 and W.is_cuda
    E, K, N = W.shape
    if W.stride(1) == 1 and (W.stride(2) >= K or N == 1):  # permuted view of (E, N, K): x @ W[e]^T form
        return 0, W.stride(0), W.stride(2)
    assert W.stride(2) == 1, "expert weights should be contiguous along K or along N"
    return 1, W.stride(0), W.stride(1)


# --------------------------------------------------------------------------- a1
def continuous_count_workspace_elements(n: int, bins: int) -> int:
    return (get_library().xma_rocm_continuous_count_workspace_bytes(n, bins) + 3) // 4


@torch.library.custom_op("xma_rocm::continuous_count", mutates_args={"y", "workspace"})
def continuous_count_rocm(x: torch.Tensor, y: torch.Tensor, workspace: torch.Tensor | None) -> None:
    """y (uint32, zero-filled by the caller) += histogram of x
    (reference op: _continuous_count_cuda, continuous_count/cuda_implementation.py:171-197).  `workspace` (int32, from
    continuous_count_workspace_elements; None: taken from torch's allocator inside the op) lets large inputs take the
    two-pass path."""
    assert x.is_cuda and y.is_cuda and x.dim() == 1 and x.is_contiguous() and y.is_contiguous()
    assert x.dtype in (torch.int32, torch.int64) and y.dtype == torch.uint32
    lib = get_library()
    if workspace is None:  # allocated here, inside the op, so that a traced caller never sees the size query
        ws = continuous_count_workspace_elements(x.numel(), y.numel())
        workspace = torch.empty(ws, dtype=torch.int32, device=x.device) if ws else None
    else:
        assert workspace.dtype == torch.int32 and workspace.is_contiguous() and workspace.is_cuda
    check(
        lib.xma_rocm_continuous_count(
            _ptr(x), int(x.dtype == torch.int64), x.numel(), _ptr(y), y.numel(), _ptr(workspace),
            0 if workspace is None else workspace.numel() * 4, _stream(x),
        ),
        "xma_rocm_continuous_count",
    )


CONTINUOUS_COUNT_SET_MAX_BINS = 8192
# The grouped GEMMs take the entry points written for the few-token regime, which stream the weights instead of tiling
# them 256 x 256 for the matrix pipes, up to FEW_ROWS_PER_EXPERT rows per expert on average.  The limits are measured
# cross-overs (8 experts of H = 2048, I = 8192; 64 of H = 2048, I = 1408; 128 of H = 576, I = 256): the forward-type GEMMs
# walk an expert's rows 32 or 128 at a time (small MFMA tile; vector FMAs up to 2 rows per expert and 64 rows in all, the
# library decides), each pass streaming the weights again, so they lead while most experts need one pass (at 128 rows
# per expert on average uneven routing gives enough experts a second pass); the weight gradient holds a 128 x 128 tile of
# dW in registers while it walks the rows, so it leads as long as its stores outweigh its loads.
FEW_ROWS_PER_EXPERT = {"x @ W^T": 96, "dy @ W": 96, "dW": 128}
FEW_ROWS_MAX = 16384  # rows in all, every form (beyond the measured range; 0 switches the few-token entry points off)
FEW_ROWS_MAX_WORKSPACE = 256 << 20  # bytes of fp32 partial sums a forward-type launch may ask for


@torch.library.custom_op("xma_rocm::continuous_count_set", mutates_args={"y"})
def continuous_count_set_rocm(x: torch.Tensor, y: torch.Tensor) -> None:
    """y (uint32, any contents) = histogram of x: the counts are written, not added to, so the caller allocates y with
    torch.empty and no zero fill is launched (reference op: _continuous_count_cuda, which accumulates into torch.zeros,
    continuous_count/__init__.py:41-45).  The scratch of large inputs is taken from torch's allocator inside the op."""
    assert x.is_cuda and y.is_cuda and x.dim() == 1 and x.is_contiguous() and y.is_contiguous()
    assert x.dtype in (torch.int32, torch.int64) and y.dtype == torch.uint32 and y.numel() <= CONTINUOUS_COUNT_SET_MAX_BINS
    lib = get_library()
    ws_bytes = lib.xma_rocm_continuous_count_set_workspace_bytes(x.numel(), y.numel())
    workspace = torch.empty(ws_bytes // 4, dtype=torch.int32, device=x.device) if ws_bytes else None
    check(
        lib.xma_rocm_continuous_count_set(_ptr(x), int(x.dtype == torch.int64), x.numel(), _ptr(y), y.numel(), _ptr(workspace),
                                          ws_bytes, _stream(x)),
        "xma_rocm_continuous_count_set",
    )


# --------------------------------------------------------------------------- a2
def route_workspace_elements(n: int, num_experts: int) -> int:
    return (get_library().xma_rocm_route_workspace_bytes(n, num_experts) + 3) // 4


@torch.library.custom_op(
    "xma_rocm::route",
    mutates_args={"counts", "offsets_inclusive", "offsets_exclusive", "sorted_expert_idxs", "sorted_scattered_idxs", "workspace"},
)
def route_rocm(
    ids: torch.Tensor,
    counts: torch.Tensor,
    offsets_inclusive: torch.Tensor,
    offsets_exclusive: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    workspace: torch.Tensor | None,
) -> None:
    """counts / offsets / stable expert-major permutation of ``ids`` in one op
    (replaces sort + continuous_count + cumsum, moe/__init__.py:210-217)."""
    E = counts.numel()
    assert ids.is_cuda and ids.dim() == 1 and ids.is_contiguous() and ids.dtype in (torch.int32, torch.int64)
    assert counts.dtype == torch.uint32 and offsets_inclusive.dtype == torch.int64 and offsets_exclusive.dtype == torch.int64
    assert offsets_inclusive.numel() == E and offsets_exclusive.numel() == E
    assert sorted_expert_idxs.dtype == ids.dtype and sorted_expert_idxs.numel() == ids.numel()
    assert sorted_scattered_idxs.dtype == torch.int64 and sorted_scattered_idxs.numel() == ids.numel()
    lib = get_library()
    if workspace is None:  # allocated here, inside the op, so that a traced caller never sees the size query
        workspace = torch.empty(route_workspace_elements(ids.numel(), E), dtype=torch.int32, device=ids.device)
    assert workspace.dtype == torch.int32 and workspace.is_contiguous()
    check(
        lib.xma_rocm_route(
            _ptr(ids), int(ids.dtype == torch.int64), ids.numel(), E, _ptr(counts), _ptr(offsets_inclusive),
            _ptr(offsets_exclusive), _ptr(sorted_expert_idxs), _ptr(sorted_scattered_idxs), _ptr(workspace),
            workspace.numel() * 4, _stream(ids),
        ),
        "xma_rocm_route",
    )


# --------------------------------------------------------------------------- a5 a7 a8 a10
_S2S_WORKSPACE_BYTES: dict[tuple[int, int, int, int, int], int] = {}


def scatter2scatter_workspace_bytes(M: int, N: int, K: int, E: int, device_index: int) -> int:
    """scratch of one grouped GEMM launch (0 for launches of many rounds of tiles); the library's answer depends on the
    shape and the device only, so it is asked once per shape"""
    key = (M, N, K, E, device_index)
    if key not in _S2S_WORKSPACE_BYTES:
        with torch.cuda.device(device_index):
            _S2S_WORKSPACE_BYTES[key] = get_library().xma_rocm_scatter2scatter_workspace_bytes(M, N, K, E)
    return _S2S_WORKSPACE_BYTES[key]


FEW_ROWS_NT_MAX_ELEMENTS = (1 << 31) - 128  # limit of the few-token entry point for W as (N, K): N * ldw


def _few_rows(M: int, E: int, dtype: torch.dtype, form: str) -> bool:
    """whether a grouped GEMM of M rows over E experts takes an entry point written for the few-token regime"""
    return 0 < M <= min(FEW_ROWS_MAX, FEW_ROWS_PER_EXPERT[form] * E) and dtype in (torch.bfloat16, torch.float16)


def _few_rows_fwd(lib, M: int, N: int, K: int, E: int, w_is_kn: int, ldw: int, dtype: torch.dtype, epilogue: int) -> bool:
    """the same for a forward-type GEMM, whose few-token entry point has limits of its own"""
    if not _few_rows(M, E, dtype, "dy @ W" if w_is_kn else "x @ W^T"):
        return False
    if not w_is_kn and N * ldw >= FEW_ROWS_NT_MAX_ELEMENTS:  # it addresses the rows of W[e] with 32-bit byte offsets
        return False
    return lib.xma_rocm_scatter2scatter_few_rows_workspace_bytes(M, N, K, E, w_is_kn, epilogue) <= FEW_ROWS_MAX_WORKSPACE


def _scatter2scatter_few_rows(lib, X, W, w_is_kn, w_es, ldw, idx, offs, out, aux, aux2, scale, bias, fan_out, x_grouped,
                              y_grouped, epilogue, M, N, K):
    # whatever does not finish in one kernel sums through a workspace (0 bytes: none needed)
    ws_bytes = lib.xma_rocm_scatter2scatter_few_rows_workspace_bytes(M, N, K, W.size(0), w_is_kn, epilogue)
    workspace = torch.empty(ws_bytes // 4, dtype=torch.float32, device=X.device) if ws_bytes else None
    check(
        lib.xma_rocm_scatter2scatter_few_rows(
            _ptr(X), _rows(X, "X"), _ptr(W), w_es, ldw, w_is_kn, _ptr(idx), _ptr(offs),
            _ptr(out), 0 if out is None else _rows(out, "out"), _ptr(aux), 0 if aux is None else _rows(aux, "aux"),
            _ptr(aux2), 0 if aux2 is None else _rows(aux2, "aux2"), _ptr(scale), _ptr(bias),
            0 if bias is None else bias.stride(0), M, N, K, W.size(0), fan_out, int(x_grouped), int(y_grouped), epilogue,
            _code(X), _ptr(workspace), ws_bytes, _stream(X),
        ),
        "xma_rocm_scatter2scatter_few_rows",
    )


def _scatter2scatter(X, W, idx, offs, out, aux, scale, fan_out, x_grouped, y_grouped, epilogue, M, N, K, bias=None):
    w_is_kn, w_es, ldw = _weight_layout(W)
    if bias is not None:  # (E, N): the experts' bias, the first term of every fp32 sum
        assert bias.dtype == X.dtype and bias.shape == (W.size(0), N) and bias.is_cuda
        assert bias.stride(1) == 1 and bias.stride(0) % 8 == 0 and bias.data_ptr() % 16 == 0, \
            "bias rows should be contiguous, 16-byte aligned and a multiple of 8 elements apart"
    assert W.dtype == X.dtype
    assert idx.dtype == torch.int64 and idx.is_contiguous() and offs.dtype == torch.int64 and offs.is_contiguous()
    assert offs.numel() == W.size(0)
    if scale is not None:
        assert scale.dtype == X.dtype and scale.is_contiguous()
    lib = get_library()
    if _few_rows_fwd(lib, M, N, K, W.size(0), w_is_kn, ldw, X.dtype, epilogue):
        _scatter2scatter_few_rows(lib, X, W, w_is_kn, w_es, ldw, idx, offs, out, aux, None, scale, bias, fan_out, x_grouped,
                                  y_grouped, epilogue, M, N, K)
        return
    # scratch for the K slices of the tiles of a last, partial round (0 bytes for launches of many rounds); it comes from
    # torch's caching allocator like every other buffer of the op
    ws_bytes = scatter2scatter_workspace_bytes(M, N, K, W.size(0), X.device.index or 0)
    workspace = torch.empty(ws_bytes // 4, dtype=torch.float32, device=X.device) if ws_bytes else None
    check(
        lib.xma_rocm_scatter2scatter_bias(
            _ptr(X), _rows(X, "X"), _ptr(W), w_es, ldw, w_is_kn, _ptr(idx), _ptr(offs),
            _ptr(out), 0 if out is None else _rows(out, "out"), _ptr(aux), 0 if aux is None else _rows(aux, "aux"),
            _ptr(scale), _ptr(bias), 0 if bias is None else bias.stride(0), M, N, K, W.size(0), fan_out, int(x_grouped),
            int(y_grouped), epilogue, _code(X), _ptr(workspace), ws_bytes, _stream(X),
        ),
        "xma_rocm_scatter2scatter_bias",
    )


@torch.library.custom_op("xma_rocm::scatter2scatter", mutates_args={"out"})
def scatter2scatter_rocm(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    out: torch.Tensor,
    row_scale: torch.Tensor | None,
    FAN_OUT: int,
    x_grouped: bool,
    y_grouped: bool,
    bias: torch.Tensor | None = None,
) -> None:
    """out[dst(n)] = (bias[e(n)] + X[src(n)] @ W[e(n)]) (* row_scale[idx[n]]), W logically (E, K, N), bias (E, N) or None."""
    M = sorted_scattered_idxs.numel()
    E, K, N = W.shape
    assert X.size(1) == K and out.size(1) == N and out.size(0) == M
    assert X.size(0) * (1 if x_grouped else FAN_OUT) == M
    _scatter2scatter(X, W, sorted_scattered_idxs, expert_offsets, out, None, row_scale, FAN_OUT, x_grouped, y_grouped,
                     EPI_STORE, M, N, K, bias)


@torch.library.custom_op("xma_rocm::up_projection_swiglu", mutates_args={"z", "h"})
def up_projection_swiglu_rocm(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    z: torch.Tensor,
    h: torch.Tensor,
    FAN_OUT: int,
    bias: torch.Tensor | None = None,
) -> None:
    """z (grouped pre-activations, (Tk, 2I), bias (E, 2I) included) and h = swiglu_packed(z) (Tk, I) in one GEMM."""
    M = sorted_scattered_idxs.numel()
    E, K, N = W.shape
    assert X.size(1) == K and X.size(0) * FAN_OUT == M
    assert z.shape == (M, N) and h.shape == (M, N // 2) and N % 2 == 0
    _scatter2scatter(X, W, sorted_scattered_idxs, expert_offsets, z, h, None, FAN_OUT, False, True, EPI_SWIGLU, M, N, K, bias)


@torch.library.custom_op("xma_rocm::down_projection_dx_swiglu", mutates_args={"dz"})
def down_projection_dx_swiglu_rocm(
    dY: torch.Tensor,
    W: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    z: torch.Tensor,
    dz: torch.Tensor,
    row_scale: torch.Tensor,
    FAN_OUT: int,
) -> None:
    """dz = swiglu_packed'(z) * ((dY[idx // k] * w[idx]) @ W[e]); W logically (E, H, I), dY is (T, H)."""
    M = sorted_scattered_idxs.numel()
    E, K, N = W.shape
    assert dY.size(1) == K and dY.size(0) * FAN_OUT == M
    assert z.shape == (M, 2 * N) and dz.shape == (M, 2 * N)
    _scatter2scatter(dY, W, sorted_scattered_idxs, expert_offsets, dz, z, row_scale, FAN_OUT, False, True,
                     EPI_SWIGLU_BWD, M, N, K)


@torch.library.custom_op("xma_rocm::down_projection_dx_swiglu_scaled_act", mutates_args={"dz", "scaled_act"})
def down_projection_dx_swiglu_scaled_act_rocm(
    dY: torch.Tensor,
    W: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    z: torch.Tensor,
    dz: torch.Tensor,
    scaled_act: torch.Tensor,
    row_scale: torch.Tensor,
    FAN_OUT: int,
) -> None:
    """down_projection_dx_swiglu with a second output, scaled_act[n] = swiglu_packed(z[n]) * row_scale[idx[n]] (M, N) in
    grouped order: the X operand of dW2 = sum_n dY[idx[n] // k]^T scaled_act[n], which then needs no scaled grouped copy
    of dY."""
    M = sorted_scattered_idxs.numel()
    E, K, N = W.shape
    assert dY.size(1) == K and dY.size(0) * FAN_OUT == M
    assert z.shape == (M, 2 * N) and dz.shape == (M, 2 * N) and scaled_act.shape == (M, N)
    assert W.dtype == dY.dtype == z.dtype == dz.dtype == scaled_act.dtype == row_scale.dtype and row_scale.is_contiguous()
    assert sorted_scattered_idxs.dtype == torch.int64 and sorted_scattered_idxs.is_contiguous()
    assert expert_offsets.dtype == torch.int64 and expert_offsets.is_contiguous() and expert_offsets.numel() == E
    w_is_kn, w_es, ldw = _weight_layout(W)
    assert w_is_kn == 1, "W should be the down-projection parameter as stored, (E, H, I) with I contiguous"
    lib = get_library()
    if _few_rows_fwd(lib, M, N, K, E, 1, ldw, dY.dtype, EPI_SWIGLU_BWD):
        _scatter2scatter_few_rows(lib, dY, W, 1, w_es, ldw, sorted_scattered_idxs, expert_offsets, dz, z, scaled_act,
                                  row_scale, None, FAN_OUT, False, True, EPI_SWIGLU_BWD, M, N, K)
        return
    ws_bytes = scatter2scatter_workspace_bytes(M, N, K, E, dY.device.index or 0)
    workspace = torch.empty(ws_bytes // 4, dtype=torch.float32, device=dY.device) if ws_bytes else None
    check(
        lib.xma_rocm_down_projection_dx_swiglu(
            _ptr(dY), _rows(dY, "dY"), _ptr(W), w_es, ldw, _ptr(sorted_scattered_idxs), _ptr(expert_offsets),
            _ptr(z), _rows(z, "z"), _ptr(dz), _rows(dz, "dz"), _ptr(scaled_act), _rows(scaled_act, "scaled_act"),
            _ptr(row_scale), M, N, K, E, FAN_OUT, _code(dY), _ptr(workspace), ws_bytes, _stream(dY),
        ),
        "xma_rocm_down_projection_dx_swiglu",
    )


@torch.library.custom_op("xma_rocm::group_bwd_W", mutates_args={"DW"})
def group_bwd_W_rocm(
    DY: torch.Tensor,
    X: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    DW: torch.Tensor,
    dy_scale: torch.Tensor | None,
    dy_fan_out: int,
    x_fan_out: int,
) -> None:
    """DW[e] = sum_n DY[dsrc(n)]^T X[xsrc(n)].  DW is logically (E, K_in, N_out) with the storage of the
    parameter (E, N_out, K_in), as the reference's zeros_like(weight.permute(0, 2, 1)).  A fan_out of 0
    marks an operand that is already in grouped order."""
    E, K_in, N_out = DW.shape
    assert DW.stride(1) == 1 and DW.is_cuda, "DW should be a permuted view of (E, N_out, K_in) storage"
    assert DY.size(1) == N_out and X.size(1) == K_in and DY.dtype == X.dtype == DW.dtype
    assert expert_offsets.numel() == E and expert_offsets.dtype == torch.int64
    assert sorted_scattered_idxs.dtype == torch.int64 and sorted_scattered_idxs.is_contiguous()
    if dy_scale is not None:
        assert dy_scale.dtype == DY.dtype and dy_scale.is_contiguous()
    lib = get_library()
    # a handful of rows per expert (the index has one entry per row): the launch is a stream of stores, not arithmetic
    M = sorted_scattered_idxs.numel()
    few = _few_rows(M, E, DW.dtype, "dW")
    name = "xma_rocm_group_bwd_W_few_rows" if few else "xma_rocm_group_bwd_W"
    operands = (
        _ptr(DY), _rows(DY, "DY"), int(dy_fan_out == 0), max(dy_fan_out, 1), _ptr(dy_scale),
        _ptr(X), _rows(X, "X"), int(x_fan_out == 0), max(x_fan_out, 1),
        _ptr(sorted_scattered_idxs), _ptr(expert_offsets), _ptr(DW), DW.stride(0), DW.stride(2), N_out, K_in, E,
    )
    # the few-token entry point also takes the number of rows: it picks the shape of a workgroup's tile of dW by it
    check(getattr(lib, name)(*operands, *((M,) if few else ()), _code(X), _stream(X)), name)


@torch.library.custom_op("xma_rocm::expert_column_sums", mutates_args={"out"})
def expert_column_sums_rocm(
    A: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor | None,
    expert_offsets: torch.Tensor,
    out: torch.Tensor,
    row_scale: torch.Tensor | None,
    fan_out: int,
) -> None:
    """out[e] = sum over the grouped rows n of expert e of A[src(n)] * row_scale[idx[n]], src(n) = n when no index is given,
    else idx[n] // fan_out: the gradient of the experts' bias (autograd of F.linear's bias, moe/__init__.py:96-100)."""
    E, N = out.shape
    assert A.size(1) == N and A.dtype == out.dtype and expert_offsets.numel() == E and expert_offsets.dtype == torch.int64
    assert out.stride(1) == 1 and expert_offsets.is_contiguous()
    if sorted_scattered_idxs is not None:
        assert sorted_scattered_idxs.dtype == torch.int64 and sorted_scattered_idxs.is_contiguous()
    if row_scale is not None:
        assert row_scale.dtype == A.dtype and row_scale.is_contiguous() and sorted_scattered_idxs is not None
    lib = get_library()
    check(
        lib.xma_rocm_expert_column_sums(_ptr(A), _rows(A, "A"), _ptr(sorted_scattered_idxs), max(fan_out, 1), _ptr(row_scale),
                                        _ptr(expert_offsets), _ptr(out), _rows(out, "out"), N, E, _code(A), _stream(A)),
        "xma_rocm_expert_column_sums",
    )


@torch.library.custom_op("xma_rocm::group", mutates_args={"out"})
def group_rocm(A: torch.Tensor, sorted_expert_idxs: torch.Tensor, out: torch.Tensor, coeff: torch.Tensor | None, fan_out: int) -> None:
    """out[n] = A[idx[n] // fan_out] * coeff[idx[n]] (reference: group_kernel.py:69-100; the index argument
    keeps the reference's name although it receives sorted_scattered_idxs)."""
    M, K = out.shape
    assert A.size(1) == K and sorted_expert_idxs.numel() == M and sorted_expert_idxs.dtype == torch.int64
    if coeff is not None:
        assert coeff.dtype == A.dtype and coeff.is_contiguous()
    lib = get_library()
    check(
        lib.xma_rocm_group(_ptr(A), _rows(A, "A"), _ptr(sorted_expert_idxs), _ptr(out), _rows(out, "out"), _ptr(coeff),
                           M, K, fan_out, _code(A), _stream(A)),
        "xma_rocm_group",
    )


# --------------------------------------------------------------------------- combine
@torch.library.custom_op("xma_rocm::combine", mutates_args={"y"})
def combine_rocm(expert_out: torch.Tensor, w: torch.Tensor | None, y: torch.Tensor, k: int) -> None:
    """y[t] = sum_j w[t, j] * expert_out[t * k + j]  (w None: plain sum over the k slots)."""
    T, H = y.shape
    assert expert_out.shape == (T * k, H) and expert_out.dtype == y.dtype
    if w is not None:
        assert w.shape == (T, k) and w.is_contiguous() and w.dtype == y.dtype
    lib = get_library()
    check(
        lib.xma_rocm_combine(_ptr(expert_out), _rows(expert_out, "expert_out"), _ptr(w), _ptr(y), _rows(y, "y"), T, k, H,
                             _code(y), _stream(y)),
        "xma_rocm_combine",
    )


@torch.library.custom_op("xma_rocm::combine_bwd", mutates_args={"d_w"})
def combine_bwd_rocm(expert_out: torch.Tensor, dy: torch.Tensor, d_w: torch.Tensor) -> None:
    """d_w[t, j] = <expert_out[t * k + j], dy[t]>."""
    T, k = d_w.shape
    H = dy.size(1)
    assert expert_out.shape == (T * k, H) and dy.shape == (T, H) and d_w.is_contiguous()
    assert expert_out.dtype == dy.dtype == d_w.dtype
    lib = get_library()
    check(
        lib.xma_rocm_combine_bwd(_ptr(expert_out), _rows(expert_out, "expert_out"), _ptr(dy), _rows(dy, "dy"), _ptr(d_w),
                                 T, k, H, _code(dy), _stream(dy)),
        "xma_rocm_combine_bwd",
    )


# --------------------------------------------------------------------------- stand-alone packed SwiGLU
@torch.library.custom_op("xma_rocm::swiglu_packed_forward", mutates_args={"y"})
def swiglu_packed_forward_rocm(x: torch.Tensor, y: torch.Tensor) -> None:
    rows, cols = y.shape
    assert x.shape == (rows, 2 * cols) and x.dtype == y.dtype
    lib = get_library()
    check(
        lib.xma_rocm_swiglu_packed_forward(_ptr(x), _rows(x, "x"), _ptr(y), _rows(y, "y"), rows, cols, _code(x), _stream(x)),
        "xma_rocm_swiglu_packed_forward",
    )


@torch.library.custom_op("xma_rocm::swiglu_packed_backward", mutates_args={"dx"})
def swiglu_packed_backward_rocm(x: torch.Tensor, dy: torch.Tensor, dx: torch.Tensor) -> None:
    rows, cols = dy.shape
    assert x.shape == (rows, 2 * cols) and dx.shape == x.shape and x.dtype == dy.dtype == dx.dtype
    lib = get_library()
    check(
        lib.xma_rocm_swiglu_packed_backward(_ptr(x), _rows(x, "x"), _ptr(dy), _rows(dy, "dy"), _ptr(dx), _rows(dx, "dx"),
                                            rows, cols, _code(x), _stream(x)),
        "xma_rocm_swiglu_packed_backward",
    )


# --------------------------------------------------------------------------- stand-alone SwiGLU, separate operands
@torch.library.custom_op("xma_rocm::swiglu_forward", mutates_args={"y"})
def swiglu_forward_rocm(g: torch.Tensor, u: torch.Tensor, y: torch.Tensor) -> None:
    """y = u * g * sigmoid(g) over 2-D tensors of any size (reference op: _Swiglu, swiglu/__init__.py:15, 39-63)."""
    rows, cols = y.shape
    assert g.shape == u.shape == y.shape and g.dtype == u.dtype == y.dtype
    lib = get_library()
    check(
        lib.xma_rocm_swiglu_forward(_ptr(g), _rows(g, "g"), _ptr(u), _rows(u, "u"), _ptr(y), _rows(y, "y"), rows, cols,
                                    _code(g), _stream(g)),
        "xma_rocm_swiglu_forward",
    )


@torch.library.custom_op("xma_rocm::swiglu_backward", mutates_args={"dg", "du"})
def swiglu_backward_rocm(g: torch.Tensor, u: torch.Tensor, dy: torch.Tensor, dg: torch.Tensor, du: torch.Tensor) -> None:
    """(dg, du) of swiglu_forward_rocm (closed form of swiglu/triton_implementation/backward.py:14-23)."""
    rows, cols = dy.shape
    assert g.shape == u.shape == dy.shape == dg.shape == du.shape
    assert g.dtype == u.dtype == dy.dtype == dg.dtype == du.dtype
    lib = get_library()
    check(
        lib.xma_rocm_swiglu_backward(_ptr(g), _rows(g, "g"), _ptr(u), _rows(u, "u"), _ptr(dy), _rows(dy, "dy"), _ptr(dg),
                                     _rows(dg, "dg"), _ptr(du), _rows(du, "du"), rows, cols, _code(g), _stream(g)),
        "xma_rocm_swiglu_backward",
    )


# --------------------------------------------------------------------------- router behind the gate GEMM
@torch.library.custom_op("xma_rocm::router_topk", mutates_args={"weights", "ids"})
def router_topk_rocm(logits: torch.Tensor, weights: torch.Tensor, ids: torch.Tensor) -> None:
    """weights[t], ids[t] = softmax over / indices of the k largest logits of row t, k = weights.size(1)
    (xma/layers/moe/__init__.py:186-193, 256-262)."""
    T, E = logits.shape
    k = weights.size(1)
    assert weights.shape == (T, k) and ids.shape == (T, k) and weights.is_contiguous() and ids.is_contiguous()
    assert weights.dtype == logits.dtype and ids.dtype in (torch.int32, torch.int64)
    lib = get_library()
    check(
        lib.xma_rocm_router_topk(_ptr(logits), _rows(logits, "logits"), T, E, k, _code(logits), _ptr(weights), _ptr(ids),
                                 int(ids.dtype == torch.int64), _stream(logits)),
        "xma_rocm_router_topk",
    )


ROUTER_GATE_MAX_E, ROUTER_GATE_MAX_K = 128, 32


def router_gate_topk_supported(H: int, E: int, k: int, dtype: torch.dtype) -> bool:
    """whether the fused gate projection + router kernel covers the shape (otherwise: linear layer + router_topk_rocm).
    Plain Python, so that a traced caller (torch.compile) can evaluate it; it restates
    xma_rocm_router_gate_topk_supported, and a test holds the two together."""
    return (dtype in (torch.bfloat16, torch.float16) and H >= 8 and H % 8 == 0 and 1 <= E <= ROUTER_GATE_MAX_E
            and 1 <= k <= min(E, ROUTER_GATE_MAX_K))


@torch.library.custom_op("xma_rocm::router_gate_topk", mutates_args={"logits", "weights", "ids"})
def router_gate_topk_rocm(x: torch.Tensor, gate_weight: torch.Tensor, logits: torch.Tensor, weights: torch.Tensor,
                          ids: torch.Tensor) -> None:
    """logits = x @ gate_weight^T (rounded to x's dtype), then weights / ids as router_topk_rocm, in one kernel
    (xma/layers/moe/__init__.py:182-195, 256-262)."""
    T, H = x.shape
    E = gate_weight.size(0)
    k = weights.size(1)
    assert gate_weight.shape == (E, H) and logits.shape == (T, E) and weights.shape == (T, k) and ids.shape == (T, k)
    assert x.dtype == gate_weight.dtype == logits.dtype == weights.dtype and ids.dtype in (torch.int32, torch.int64)
    assert weights.is_contiguous() and ids.is_contiguous()
    lib = get_library()
    # the kernel reads 16-byte pieces: a view that starts off such a boundary (a column slice at an odd offset) is copied
    if x.data_ptr() % 16:
        x = x.contiguous()
    if gate_weight.data_ptr() % 16:
        gate_weight = gate_weight.clone()
    check(
        lib.xma_rocm_router_gate_topk(_ptr(x), _rows(x, "x"), _ptr(gate_weight), _rows(gate_weight, "gate_weight"), T, H, E, k,
                                      _code(x), _ptr(logits), _rows(logits, "logits"), _ptr(weights), _ptr(ids),
                                      int(ids.dtype == torch.int64), _stream(x)),
        "xma_rocm_router_gate_topk",
    )


@torch.library.custom_op("xma_rocm::router_topk_bwd", mutates_args={"d_logits"})
def router_topk_bwd_rocm(logits: torch.Tensor, ids: torch.Tensor, d_weights: torch.Tensor, d_logits: torch.Tensor) -> None:
    """d_logits = gradient of the logits through top-k and softmax, every element written."""
    T, E = logits.shape
    k = ids.size(1)
    assert ids.shape == (T, k) and d_weights.shape == (T, k) and d_logits.shape == (T, E)
    assert ids.is_contiguous() and d_weights.is_contiguous() and ids.dtype in (torch.int32, torch.int64)
    assert d_weights.dtype == logits.dtype == d_logits.dtype
    lib = get_library()
    check(
        lib.xma_rocm_router_topk_bwd(_ptr(logits), _rows(logits, "logits"), T, E, k, _code(logits), _ptr(ids),
                                     int(ids.dtype == torch.int64), _ptr(d_weights), _ptr(d_logits),
                                     _rows(d_logits, "d_logits"), _stream(logits)),
        "xma_rocm_router_topk_bwd",
    )


# ------------------------------------------------------------------------------------------------ eager fast path
def _eager_fast_path(op):
    """The registered op when a compiler is tracing (the graph gets its node), its Python body directly otherwise: the
    dispatcher's way to the same body costs 7 us per call on the host (measured: 14.5 against 7.2 us for `combine`), which
    is most of an eager step of a handful of tokens.  The ops return nothing and write tensors that their callers have
    just allocated, so nothing that autograd does for a registered op (version counters of mutated arguments) is missed."""
    body = op._init_fn

    def call(*args, **kwargs):
        if torch.compiler.is_compiling():
            return op(*args, **kwargs)
        return body(*args, **kwargs)

    call.__name__, call.__doc__, call.registered_op = body.__name__, body.__doc__, op
    return call


for _name, _obj in list(globals().items()):
    if isinstance(_obj, torch._library.custom_ops.CustomOpDef):
        globals()[_name] = _eager_fast_path(_obj)
del _name, _obj
