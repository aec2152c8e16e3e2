"""GPU parity of the MoE ops (grouped GEMMs, dW, group, combine) through the C ABI against the
op-level oracle.  Tolerance: max-abs-normalised error <= 1e-2 for bf16/fp16 results with fp32
accumulation (the bar of the north star), <= 2e-5 for the fp32 kernels; operands are bit-identical on both sides."""

import pytest
import torch

from oracle import moe as oracle
from tests.utils import nerr

pytestmark = pytest.mark.gpu

TOL = 1e-2
TOL_F32 = 2e-5  # fp32 kernels: fp32 operands and accumulators, only the summation order differs from the oracle's


def _tol(dtype):
    return TOL_F32 if dtype == torch.float32 else TOL


def _routing(T, E, k, seed, skew=0.0, empty=()):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g) + skew * torch.randn(E, generator=g)
    for e in empty:
        logits[:, e] = -1e9
    sel = logits.topk(k, dim=-1).indices
    se, ss = sel.flatten().sort(stable=True)
    offs = torch.bincount(se, minlength=E).cumsum(0)
    return sel, se, ss, offs


class _few_rows_limit:
    """the number of rows up to which the ops take the few-token entry points, whatever the number of experts, set for the
    length of a with block (0: never)"""

    def __init__(self, limit):
        self.limit = limit

    def __enter__(self):
        from xma.rocm import ops

        self.saved = (ops.FEW_ROWS_MAX, ops.FEW_ROWS_PER_EXPERT)
        ops.FEW_ROWS_MAX, ops.FEW_ROWS_PER_EXPERT = self.limit, dict.fromkeys(ops.FEW_ROWS_PER_EXPERT, 1 << 30)

    def __exit__(self, *exc):
        from xma.rocm import ops

        ops.FEW_ROWS_MAX, ops.FEW_ROWS_PER_EXPERT = self.saved


def _limits(rows):
    """both code paths where the number of rows would pick the few-token one, else the only one there is"""
    from xma.rocm import ops

    return (0, ops.FEW_ROWS_MAX) if rows <= ops.FEW_ROWS_MAX else (ops.FEW_ROWS_MAX,)


CASES = [
    # T, E, k, K, N, skew, empty experts
    (7, 4, 2, 64, 64, 0.0, ()),
    (7, 8, 4, 128, 72, 0.0, ()),
    (300, 3, 2, 192, 320, 0.0, ()),
    (700, 8, 2, 256, 512, 1.5, (3,)),
    (1024, 2, 1, 64, 264, 0.0, ()),
    (513, 6, 4, 72, 40, 2.0, (0, 5)),
    (100, 2, 1, 96, 136, 0.0, ()),  # about 50 rows per expert: two of a wave's four row blocks are computed
    (300, 3, 2, 1096, 320, 0.0, ()),  # few tiles, long K (with a tail): tiles are split into K slices
    (400, 100, 3, 128, 264, 1.0, (7, 99)),  # more experts than lanes of a wave: the schedule is scanned through LDS
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("w_kn", [False, True])
@pytest.mark.parametrize("x_grouped,y_grouped", [(False, True), (True, False), (True, True), (False, False)])
def test_scatter2scatter(dtype, case, w_kn, x_grouped, y_grouped):
    from xma.layers.moe import rocm_implementation as R

    T, E, k, K, N, skew, empty = case
    print(f"case T={T} E={E} k={k} K={K} N={N} w_kn={w_kn} xg={x_grouped} yg={y_grouped} {dtype}", flush=True)
    sel, se, ss, offs = _routing(T, E, k, 0, skew, empty)
    g = torch.Generator().manual_seed(1)
    M = T * k
    X = torch.randn(M if x_grouped else T, K, generator=g).to(dtype)
    if w_kn:
        W = (torch.randn(E, K, N, generator=g) * 0.1).to(dtype)  # contiguous (E, K, N)
    else:
        W = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype).permute(0, 2, 1)  # view of (E, N, K)
    scale = torch.rand(M, generator=g).to(dtype)
    for rs in (None, scale):
        want = oracle.scatter2scatter(X, W, se, ss, k, x_grouped, y_grouped, rs)
        Wd = W.cuda() if w_kn else W.permute(0, 2, 1).contiguous().cuda().permute(0, 2, 1)
        for limit in _limits(M):
            out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
            with _few_rows_limit(limit):
                R.scatter2scatter(X.cuda(), Wd, se.cuda(), ss.cuda(), out, k, x_grouped, y_grouped, offs.cuda(),
                                  None if rs is None else rs.cuda())
            torch.cuda.synchronize()
            assert torch.isfinite(out).all()
            assert nerr(out, want) <= _tol(dtype), limit


def test_scatter2scatter_launches_outside_the_persistent_kernel():
    """Three launches that the layer itself never makes and that take the one-workgroup-per-tile kernel instead of the
    persistent one: more experts than its schedule tables hold (E = 1100, most of them empty), a row scale that starts
    off a 4-byte boundary (the persistent kernel fetches the aligned dword around a 16-bit scale), and dy @ W (W as
    (K, N)) with the SwiGLU forward epilogue, reachable through the C ABI only."""
    from xma.layers.moe import rocm_implementation as R
    from xma.rocm.loader import get_library

    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(31)
    # (1) E = 1100
    T, E, k, K, N = 700, 1100, 2, 136, 264
    sel, se, ss, offs = _routing(T, E, k, 5, skew=2.0)
    M = T * k
    X = torch.randn(T, K, generator=g).to(dtype)
    W = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)
    want = oracle.scatter2scatter(X, W.permute(0, 2, 1), se, ss, k, False, True, None)
    out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    R.scatter2scatter(X.cuda(), W.cuda().permute(0, 2, 1), se.cuda(), ss.cuda(), out, k, False, True, offs.cuda(), None)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and nerr(out, want) <= TOL
    # (2) a row scale at an odd element offset, grouped rows in, scattered rows out
    T, E, k, K, N = 300, 3, 2, 192, 320
    sel, se, ss, offs = _routing(T, E, k, 6)
    M = T * k
    X = torch.randn(M, K, generator=g).to(dtype)
    W = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)
    scale_buf = torch.rand(M + 1, generator=g).to(dtype)
    want = oracle.scatter2scatter(X, W.permute(0, 2, 1), se, ss, k, True, False, scale_buf[1:])
    sd = scale_buf.cuda()[1:]
    assert sd.data_ptr() % 4 == 2
    out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    R.scatter2scatter(X.cuda(), W.cuda().permute(0, 2, 1), se.cuda(), ss.cuda(), out, k, True, False, offs.cuda(), sd)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and nerr(out, want) <= TOL
    # (3) W[e] as (K, N) with the SwiGLU forward epilogue: z and h = swiglu_packed(z), straight through the C ABI
    lib = get_library()
    K, N = 200, 272
    X = torch.randn(T, K, generator=g).to(dtype)
    Wkn = (torch.randn(E, K, N, generator=g) * 0.1).to(dtype)
    want_z = oracle.scatter2scatter(X, Wkn, se, ss, k, False, True, None)
    want_h = oracle.swiglu_packed(want_z.float())
    Xd, Wd, ssd, offsd = X.cuda(), Wkn.cuda(), ss.cuda(), offs.cuda()
    z = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    h = torch.full((M, N // 2), float("nan"), dtype=dtype, device="cuda")
    rc = lib.xma_rocm_scatter2scatter(Xd.data_ptr(), K, Wd.data_ptr(), K * N, N, 1, ssd.data_ptr(), offsd.data_ptr(),
                                      z.data_ptr(), N, h.data_ptr(), N // 2, None, M, N, K, E, k, 0, 1, 1, 0, None, 0,
                                      torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0, lib.xma_rocm_last_error()
    assert torch.isfinite(z).all() and torch.isfinite(h).all()
    assert nerr(z, want_z) <= TOL and nerr(h, want_h) <= TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_scatter2scatter_bias_and_expert_column_sums(dtype):
    """The experts' bias as the first term of the grouped GEMM's sums (plain store and SwiGLU epilogues, both weight
    layouts, with and without a row scale, a tile split along K), and its gradient, the per-expert column sums of grouped
    rows or of gathered and scaled rows; experts without rows give zero sums."""
    from xma.rocm import ops

    for T, E, k, K, N, skew, empty in [(300, 3, 2, 192, 320, 0.0, ()), (513, 6, 4, 72, 40, 2.0, (0, 5)), (300, 3, 2, 1096, 320, 0.0, ())]:
        print(f"bias case T={T} E={E} k={k} K={K} N={N} {dtype}", flush=True)
        sel, se, ss, offs = _routing(T, E, k, 3, skew, empty)
        g = torch.Generator().manual_seed(4)
        M = T * k
        X = torch.randn(T, K, generator=g).to(dtype)
        bias = torch.randn(E, N, generator=g).to(dtype)
        scale = torch.rand(M, generator=g).to(dtype)
        for w_kn in (False, True):
            W = (torch.randn(E, K, N, generator=g) * 0.1).to(dtype)
            Wd = W.cuda() if w_kn else W.permute(0, 2, 1).contiguous().cuda().permute(0, 2, 1)
            for rs in (None, scale):
                want = oracle.scatter2scatter(X, W, se, ss, k, False, True, rs, bias=bias)
                out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
                ops.scatter2scatter_rocm(X.cuda(), Wd, ss.cuda(), offs.cuda(), out, None if rs is None else rs.cuda(), k, False,
                                         True, bias.cuda())
                torch.cuda.synchronize()
                assert torch.isfinite(out).all() and nerr(out, want) <= _tol(dtype), (w_kn, rs is None)
            if not w_kn and N % 16 == 0:
                want_z = oracle.scatter2scatter(X, W, se, ss, k, False, True, None, bias=bias)
                z = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
                h = torch.full((M, N // 2), float("nan"), dtype=dtype, device="cuda")
                ops.up_projection_swiglu_rocm(X.cuda(), Wd, ss.cuda(), offs.cuda(), z, h, k, bias.cuda())
                torch.cuda.synchronize()
                assert nerr(z, want_z) <= _tol(dtype) and nerr(h, oracle.swiglu_packed(want_z)) <= _tol(dtype)
        # column sums: grouped rows; gathered rows times a scale
        A = torch.randn(M, N, generator=g).to(dtype)
        counts = torch.bincount(se, minlength=E).tolist()
        want = torch.stack([a.float().sum(0) for a in A.split(counts)])
        got = torch.full((E, N), float("nan"), dtype=dtype, device="cuda")
        ops.expert_column_sums_rocm(A.cuda(), None, offs.cuda(), got, None, 1)
        B = torch.randn(T, N, generator=g).to(dtype)
        rows = B.float()[ss // k] * scale.float()[ss][:, None]
        want2 = torch.stack([a.sum(0) for a in rows.split(counts)])
        got2 = torch.full((E, N), float("nan"), dtype=dtype, device="cuda")
        ops.expert_column_sums_rocm(B.cuda(), ss.cuda(), offs.cuda(), got2, scale.cuda(), k)
        torch.cuda.synchronize()
        assert nerr(got, want) <= _tol(dtype) and nerr(got2, want2) <= _tol(dtype)
        for e in empty:
            assert torch.count_nonzero(got[e]) == 0 and torch.count_nonzero(got2[e]) == 0


def _routing_with_counts(counts, k, seed):
    """a routing whose experts own exactly `counts` rows (sum divisible by k): the slots are dealt out at random"""
    g = torch.Generator().manual_seed(seed)
    E, M = len(counts), sum(counts)
    assert M % k == 0
    flat = torch.repeat_interleave(torch.arange(E), torch.tensor(counts))[torch.randperm(M, generator=g)]
    sel = flat.view(M // k, k)
    se, ss = flat.sort(stable=True)
    offs = torch.bincount(se, minlength=E).cumsum(0)
    assert torch.bincount(se, minlength=E).tolist() == list(counts)
    return sel, se, ss, offs


# rows per expert around the 32-row blocks and 256-row tiles of the kernels (an empty expert, single rows, one row more or
# less than a block, a tile and two tiles), with K = 4 or 6 steps of 64 (complete and with a tail) and one odd step count:
# tiles of more than 192 rows and an even number of at least four K steps fetch the next tile's operands inside their
# last K step, all others behind it
ROW_COUNT_CASES = [
    # counts, k, K, N
    ((1, 31, 33, 65, 129, 257, 0, 512), 2, 256, 264),
    ((257, 1, 193, 192, 511, 513, 224, 3), 2, 232, 520),
    ((300, 260, 1, 255), 1, 384, 72),
    ((256, 200, 700, 4), 4, 328, 512),
    ((193, 250, 256, 257), 1, 320, 264),  # five K steps: odd
    ((3333, 259, 4000), 2, 256, 520),  # 14 and 16 row tiles: the tiles of such an expert are walked in bands of row tiles
    ((3100, 7), 1, 64, 776),  # 13 row tiles in bands of 5, 5 and 3
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", ROW_COUNT_CASES)
@pytest.mark.parametrize("w_kn", [False, True])
def test_scatter2scatter_expert_row_counts(dtype, case, w_kn):
    from xma.layers.moe import rocm_implementation as R

    counts, k, K, N = case
    print(f"case counts={counts} k={k} K={K} N={N} w_kn={w_kn} {dtype}", flush=True)
    sel, se, ss, offs = _routing_with_counts(counts, k, 11)
    E, M = len(counts), sum(counts)
    T = M // k
    g = torch.Generator().manual_seed(12)
    scale = torch.rand(M, generator=g).to(dtype)
    if w_kn:
        W = (torch.randn(E, K, N, generator=g) * 0.1).to(dtype)
        Wd = W.cuda()
    else:
        W = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype).permute(0, 2, 1)
        Wd = W.permute(0, 2, 1).contiguous().cuda().permute(0, 2, 1)
    for x_grouped, y_grouped, rs in [(False, True, None), (True, False, scale), (True, True, None), (False, False, scale)]:
        X = torch.randn(M if x_grouped else T, K, generator=g).to(dtype)
        want = oracle.scatter2scatter(X, W, se, ss, k, x_grouped, y_grouped, rs)
        out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
        R.scatter2scatter(X.cuda(), Wd, se.cuda(), ss.cuda(), out, k, x_grouped, y_grouped, offs.cuda(),
                          None if rs is None else rs.cuda())
        torch.cuda.synchronize()
        assert torch.isfinite(out).all()
        assert nerr(out, want) <= _tol(dtype)
        # every row against its own magnitude: a wrong row of a small expert does not hide behind the large ones
        row_err = (out.cpu().float() - want.float()).abs().amax(dim=1) / want.float().abs().amax(dim=1).clamp_min(1e-6)
        assert row_err.max() <= 4 * _tol(dtype), int(row_err.argmax())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", ROW_COUNT_CASES)
def test_group_bwd_W_expert_row_counts(dtype, case):
    from xma.rocm import ops

    counts, k, K, N = case
    print(f"case counts={counts} k={k} K={K} N={N} {dtype}", flush=True)
    sel, se, ss, offs = _routing_with_counts(counts, k, 13)
    E, M = len(counts), sum(counts)
    T = M // k
    g = torch.Generator().manual_seed(14)
    x_tok = torch.randn(T, K, generator=g).to(dtype)
    dy_grp = torch.randn(M, N, generator=g).to(dtype)
    x_grp = torch.randn(M, K, generator=g).to(dtype)
    for X, x_fan, want in [(x_grp, 0, oracle.group_bwd_W(dy_grp, x_grp, offs, E)),
                           (x_tok, k, oracle.group_bwd_W(dy_grp, oracle.group(x_tok, ss, None, k), offs, E))]:
        for limit in _limits(M):
            DW = torch.full((E, N, K), float("nan"), dtype=dtype, device="cuda").permute(0, 2, 1)
            with _few_rows_limit(limit):
                ops.group_bwd_W_rocm(dy_grp.cuda(), X.cuda(), ss.cuda(), offs.cuda(), DW, None, 0, x_fan)
            torch.cuda.synchronize()
            assert torch.isfinite(DW).all()
            for e in range(E):  # every expert's slice against its own magnitude
                if counts[e] == 0:
                    assert (DW[e] == 0).all()
                else:
                    assert nerr(DW[e], want[e]) <= _tol(dtype), (e, limit)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", CASES)
def test_group_bwd_W(dtype, case):
    from xma.rocm import ops

    T, E, k, K, N, skew, empty = case
    print(f"case T={T} E={E} k={k} K={K} N={N} {dtype}", flush=True)
    sel, se, ss, offs = _routing(T, E, k, 2, skew, empty)
    g = torch.Generator().manual_seed(3)
    M = T * k
    x_tok = torch.randn(T, K, generator=g).to(dtype)
    dy_tok = torch.randn(T, N, generator=g).to(dtype)
    dy_grp = torch.randn(M, N, generator=g).to(dtype)
    x_grp = torch.randn(M, K, generator=g).to(dtype)
    scale = torch.rand(M, generator=g).to(dtype)

    def run(DY, X, dy_scale, dy_fan, x_fan):
        DW = torch.full((E, N, K), float("nan"), dtype=dtype, device="cuda").permute(0, 2, 1)
        ops.group_bwd_W_rocm(DY.cuda(), X.cuda(), ss.cuda(), offs.cuda(), DW, None if dy_scale is None else dy_scale.cuda(),
                             dy_fan, x_fan)
        torch.cuda.synchronize()
        assert torch.isfinite(DW).all()
        return DW

    for limit in _limits(M):
        with _few_rows_limit(limit):
            # both grouped (the reference op), x gathered (dW1), dy gathered and scaled (dW2)
            want = oracle.group_bwd_W(dy_grp, x_grp, offs, E)
            assert nerr(run(dy_grp, x_grp, None, 0, 0), want) <= _tol(dtype)
            want = oracle.group_bwd_W(dy_grp, oracle.group(x_tok, ss, None, k), offs, E)
            assert nerr(run(dy_grp, x_tok, None, 0, k), want) <= _tol(dtype)
            want = oracle.group_bwd_W(oracle.group(dy_tok, ss, scale, k), x_grp, offs, E)
            assert nerr(run(dy_tok, x_grp, scale, k, 0), want) <= _tol(dtype)
            # experts without rows get an all-zero slice
            got = run(dy_grp, x_grp, None, 0, 0)
            for e in empty:
                assert (got[e] == 0).all()


FEW_ROWS_CASES = [
    # T, E, k, H, I, empty experts
    (7, 8, 2, 264, 136, ()),
    (3, 128, 8, 576, 256, ()),  # more experts than rows
    (16, 4, 4, 2048, 72, (2,)),  # about twenty rows per expert: several passes of 4 or 8 rows over the weights
    (1, 8, 1, 64, 8, ()),
    (9, 5, 3, 4104, 24, (0, 4)),  # a row of W as (N, K) is 513 pieces of 16 bytes: two passes of a wave and one lane more
    (7, 8, 2, 512, 8192, ()),  # long K for the down-projection and dX1: both cut into ranges of K
    (5, 2, 2, 64, 3200, ()),  # down-projection: 25 K steps in 6 ranges of 5, of which only 5 hold a step
    (5, 8, 2, 2056, 40, (3,)),  # one or two rows per expert and rows of W longer than 4 KB: the vector kernel for the up-projection
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", FEW_ROWS_CASES)
def test_forward_type_gemms_few_rows(dtype, case):
    """The six operand forms of the layer's forward-type GEMMs through the kernels written for a handful of rows (weights
    streamed once per 32 rows of an expert; vector FMAs or a small MFMA tile, sums through a workspace and one small
    epilogue kernel where K is cut), each against the oracle and against the 256 x 256 kernels on the same operands: up-projection + SwiGLU with a bias (z and h), up-projection with a plain store,
    down-projection with a bias, a row scale and scattered rows, dX1 (dz @ W1, scattered), dX2 + SwiGLU backward with and
    without the scaled activations."""
    from xma.rocm import ops

    T, E, k, H, I, empty = case
    print(f"case T={T} E={E} k={k} H={H} I={I} {dtype}", flush=True)
    sel, se, ss, offs = _routing(T, E, k, 41, 0.0, empty)
    M = T * k
    assert M <= ops.FEW_ROWS_MAX
    g = torch.Generator().manual_seed(42)
    x = torch.randn(T, H, generator=g).to(dtype)
    W1 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).to(dtype)  # c_fc.weight (E, out, in)
    W2 = (torch.randn(E, H, I, generator=g) * 0.05).to(dtype)  # c_proj.weight
    b1 = torch.randn(E, 2 * I, generator=g).to(dtype)
    b2 = torch.randn(E, H, generator=g).to(dtype)
    w = torch.rand(M, generator=g).to(dtype)
    dy = torch.randn(T, H, generator=g).to(dtype)
    dzg = torch.randn(M, 2 * I, generator=g).to(dtype)
    xd, W1d, W2d, b1d, b2d, wd, dyd, dzd, ssd, offsd = (t.cuda() for t in (x, W1, W2, b1, b2, w, dy, dzg, ss, offs))
    tol = _tol(dtype)

    def both(fn):
        """fn() -> tuple of device outputs; run with the MFMA kernels and with the few-row kernels"""
        res = {}
        for limit in (0, ops.FEW_ROWS_MAX):
            with _few_rows_limit(limit):
                res[limit] = fn()
            torch.cuda.synchronize()
        return res[ops.FEW_ROWS_MAX], res[0]

    def new(*shape):
        return torch.full(shape, float("nan"), dtype=dtype, device="cuda")

    # up-projection + SwiGLU, bias
    def up():
        z, h = new(M, 2 * I), new(M, I)
        ops.up_projection_swiglu_rocm(xd, W1d.permute(0, 2, 1), ssd, offsd, z, h, k, b1d)
        return z, h

    want_z = oracle.scatter2scatter(x, W1.permute(0, 2, 1), se, ss, k, False, True, None, bias=b1)
    (z_f, h_f), (z_m, h_m) = both(up)
    assert torch.isfinite(z_f).all() and torch.isfinite(h_f).all()
    assert nerr(z_f, want_z) <= tol and nerr(z_f, z_m) <= tol
    assert nerr(h_f, oracle.swiglu_packed(want_z)) <= tol and nerr(h_f, h_m) <= tol

    # up-projection, plain store, no bias
    def up_store():
        z = new(M, 2 * I)
        ops.scatter2scatter_rocm(xd, W1d.permute(0, 2, 1), ssd, offsd, z, None, k, False, True)
        return (z,)

    (z_f,), (z_m,) = both(up_store)
    assert nerr(z_f, oracle.scatter2scatter(x, W1.permute(0, 2, 1), se, ss, k, False, True, None)) <= tol and nerr(z_f, z_m) <= tol

    # down-projection: grouped rows in, scattered rows out, bias and row scale
    hg = torch.randn(M, I, generator=g).to(dtype)
    hgd = hg.cuda()

    def down():
        out = new(M, H)
        ops.scatter2scatter_rocm(hgd, W2d.permute(0, 2, 1), ssd, offsd, out, wd, 1, True, False, b2d)
        return (out,)

    (o_f,), (o_m,) = both(down)
    want = oracle.scatter2scatter(hg, W2.permute(0, 2, 1), se, ss, 1, True, False, w, bias=b2)
    assert torch.isfinite(o_f).all() and nerr(o_f, want) <= tol and nerr(o_f, o_m) <= tol

    # dX1: dz @ W1 (W as (K, N) = the parameter as stored), scattered rows out
    def dx1():
        out = new(M, H)
        ops.scatter2scatter_rocm(dzd, W1d, ssd, offsd, out, None, 1, True, False)
        return (out,)

    (o_f,), (o_m,) = both(dx1)
    want = oracle.scatter2scatter(dzg, W1, se, ss, 1, True, False, None)
    assert torch.isfinite(o_f).all() and nerr(o_f, want) <= tol and nerr(o_f, o_m) <= tol

    # dX2 + SwiGLU backward, without and with the scaled activations
    zg = torch.randn(M, 2 * I, generator=g).to(dtype)
    zgd = zg.cuda()

    def dx2():
        dz = new(M, 2 * I)
        ops.down_projection_dx_swiglu_rocm(dyd, W2d, ssd, offsd, zgd, dz, wd, k)
        return (dz,)

    def dx2_act():
        dz, act = new(M, 2 * I), new(M, I)
        ops.down_projection_dx_swiglu_scaled_act_rocm(dyd, W2d, ssd, offsd, zgd, dz, act, wd, k)
        return dz, act

    z32 = zg.float().requires_grad_()
    h32 = oracle.swiglu_packed(z32)
    dh = torch.stack([(dy.float()[ss[n] // k] * w.float()[ss[n]]) @ W2.float()[se[n]] for n in range(M)])
    h32.backward(dh)
    (dz_f,), (dz_m,) = both(dx2)
    assert torch.isfinite(dz_f).all() and nerr(dz_f, z32.grad) <= tol and nerr(dz_f, dz_m) <= tol
    (dz_a, act_f), (_, act_m) = both(dx2_act)
    assert torch.equal(dz_a, dz_f)
    assert nerr(act_f, h32.detach() * w.float()[ss][:, None]) <= tol and nerr(act_f, act_m) <= tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", [(7, 8, 2, 264, 136, ()), (3, 128, 8, 576, 512, ()), (16, 4, 4, 2048, 72, (2,)), (1, 8, 1, 64, 8, ()),
                                  (9, 5, 3, 4104, 24, (0, 4)), (100, 3, 2, 200, 328, ())])
def test_group_bwd_W_few_rows(dtype, case):
    """The weight gradient written for a handful of rows (a 128 x 128 tile of dW per workgroup, the expert's rows as the K
    dimension of the MFMAs, 32 at a time, streamed stores) against the oracle and against the 256 x 256 kernel on the same
    operands: every operand form of the layer, tiles partly outside dW in both directions, experts without rows (zeros),
    more experts than rows, about 67 rows per expert (two full passes and a partial one)."""
    from xma.rocm import ops

    T, E, k, K, N, empty = case
    print(f"case T={T} E={E} k={k} K={K} N={N} {dtype}", flush=True)
    sel, se, ss, offs = _routing(T, E, k, 21, 0.0, empty)
    M = T * k
    assert M <= ops.FEW_ROWS_MAX
    g = torch.Generator().manual_seed(22)
    x_tok = torch.randn(T, K, generator=g).to(dtype)
    dy_tok = torch.randn(T, N, generator=g).to(dtype)
    dy_grp = torch.randn(M, N, generator=g).to(dtype)
    x_grp = torch.randn(M, K, generator=g).to(dtype)
    scale = torch.rand(M, generator=g).to(dtype)
    forms = [(dy_grp, x_grp, None, 0, 0, oracle.group_bwd_W(dy_grp, x_grp, offs, E)),
             (dy_grp, x_tok, None, 0, k, oracle.group_bwd_W(dy_grp, oracle.group(x_tok, ss, None, k), offs, E)),
             (dy_tok, x_grp, scale, k, 0, oracle.group_bwd_W(oracle.group(dy_tok, ss, scale, k), x_grp, offs, E)),
             (dy_tok, x_grp, None, k, 0, oracle.group_bwd_W(oracle.group(dy_tok, ss, None, k), x_grp, offs, E))]
    counts = torch.bincount(se, minlength=E)
    for DY, X, sc, dy_fan, x_fan, want in forms:
        got = {}
        for limit in (0, ops.FEW_ROWS_MAX):
            DW = torch.full((E, N, K), float("nan"), dtype=dtype, device="cuda").permute(0, 2, 1)
            with _few_rows_limit(limit):
                ops.group_bwd_W_rocm(DY.cuda(), X.cuda(), ss.cuda(), offs.cuda(), DW, None if sc is None else sc.cuda(), dy_fan, x_fan)
            torch.cuda.synchronize()
            assert torch.isfinite(DW).all()
            got[limit] = DW
        few, mfma = got[ops.FEW_ROWS_MAX], got[0]
        assert nerr(few, want) <= _tol(dtype)
        assert nerr(few, mfma) <= _tol(dtype)
        for e in range(E):
            if counts[e] == 0:
                assert (few[e] == 0).all()
            else:
                assert nerr(few[e], want[e]) <= _tol(dtype), e


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_group_and_combine(dtype):
    from xma.layers.moe import rocm_implementation as R
    from xma.rocm import ops

    g = torch.Generator().manual_seed(5)
    for T, k, H in [(7, 2, 64), (33, 4, 136), (1000, 8, 2048), (513, 1, 72)]:
        E = 8
        sel, se, ss, offs = _routing(T, E, k, 6)
        A = torch.randn(T, H, generator=g).to(dtype)
        coeff = torch.rand(T * k, generator=g).to(dtype)
        for c in (None, coeff):
            out = torch.empty(T * k, H, dtype=dtype, device="cuda")
            R.group(A.cuda(), ss.cuda(), out, None if c is None else c.cuda(), k)
            assert torch.equal(out.cpu(), oracle.group(A, ss, c, k))  # one rounding of an fp32 product: exact match
        eo = torch.randn(T * k, H, generator=g).to(dtype)
        w = torch.rand(T, k, generator=g).to(dtype)
        dy = torch.randn(T, H, generator=g).to(dtype)
        for ww in (None, w):
            y = torch.empty(T, H, dtype=dtype, device="cuda")
            ops.combine_rocm(eo.cuda(), None if ww is None else ww.cuda(), y, k)
            assert nerr(y, oracle.combine(eo, ww, k)) <= _tol(dtype)
        d_w = torch.empty(T, k, dtype=dtype, device="cuda")
        ops.combine_bwd_rocm(eo.cuda(), dy.cuda(), d_w)
        assert nerr(d_w, oracle.combine_bwd(eo, dy, k)) <= _tol(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_swiglu_packed_standalone(dtype):
    from xma import KernelBackend
    from xma.functional import swiglu_packed

    g = torch.Generator().manual_seed(7)
    for rows, cols in [(1, 8), (7, 64), (300, 1408), (65, 4096)]:
        x = (torch.randn(rows, 2 * cols, generator=g) * 2).to(dtype)
        dy = torch.randn(rows, cols, generator=g).to(dtype)
        xd = x.cuda().requires_grad_()
        y = swiglu_packed(xd, kernel_backend=KernelBackend.rocm)
        y.backward(dy.cuda())
        assert nerr(y, oracle.swiglu_packed(x.float())) <= _tol(dtype)
        dg, du = oracle.swiglu_backward(x[..., 0::2].float(), x[..., 1::2].float(), dy.float())
        want = torch.stack([dg, du], dim=-1).flatten(-2)
        assert nerr(xd.grad, want) <= _tol(dtype)


def _2d_sizes():
    """the reference's 2-D size rule (tests/utils.py:31-42: squares 2^i + j, and ragged sizes around 3000), thinned so
    that the CPU oracle stays within seconds"""
    import random

    rng = random.Random(0)
    sizes = [(2**i + j, 2**i + j) for i in range(11) for j in (0, 1, 3, 7, 9)]
    ragged = [(3000 + rng.randint(-1000, 1000), 3000 + rng.randint(-1000, 1000)) for _ in range(50)]
    return sizes + ragged[:8]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_swiglu_two_operands(dtype):
    """swiglu(gate, up) on separate operands, forward and backward, over the reference's 2-D size grid
    (tests/functional/swiglu_test.py:62-95: integer-valued inputs in [-8, 8), fp32 atol 7e-5 / 4.6e-5) - odd widths,
    widths below one 16-byte access, rows that are not 16-byte aligned - against the oracle's closed forms."""
    from xma import KernelBackend
    from xma.functional import swiglu

    g = torch.Generator().manual_seed(11)
    for rows, cols in _2d_sizes():
        print(f"swiglu case {rows}x{cols} {dtype}", flush=True)
        gate = torch.randint(-8, 8, (rows, cols), generator=g).to(dtype)
        up = torch.randint(-8, 8, (rows, cols), generator=g).to(dtype)
        dy = torch.randn(rows, cols, generator=g).to(dtype)
        gd, ud = gate.cuda().requires_grad_(), up.cuda().requires_grad_()
        y = swiglu(gd, ud, kernel_backend=KernelBackend.rocm)
        y.backward(dy.cuda())
        want = oracle.swiglu(gate.float(), up.float())
        dg, du = oracle.swiglu_backward(gate.float(), up.float(), dy.float())
        assert y.dtype == dtype and y.shape == (rows, cols)
        assert nerr(y, want) <= _tol(dtype), (rows, cols)
        assert nerr(gd.grad, dg) <= _tol(dtype) and nerr(ud.grad, du) <= _tol(dtype), (rows, cols)
        if dtype == torch.float32:
            assert (y.cpu() - want).abs().max() <= 7e-5
            assert (gd.grad.cpu() - dg).abs().max() <= 4.6e-5 * dy.abs().max() * 4


def test_swiglu_views_and_shapes():
    """3-D inputs, operands that are column slices of one wider tensor (row pitch larger than the width, starts not
    16-byte aligned), empty input; and the packed form at widths that are not multiples of 8."""
    from xma import KernelBackend
    from xma.functional import swiglu, swiglu_packed

    g = torch.Generator().manual_seed(12)
    for dtype in (torch.bfloat16, torch.float32):
        x = (torch.randn(3, 37, 2 * 203, generator=g) * 2).to(dtype)
        xd = x.cuda()
        for lo in (0, 1, 8):  # chunk-style halves of one tensor; lo shifts the alignment of the row starts
            gate, up = x[..., lo:203], x[..., 203 + lo :]
            y = swiglu(xd[..., lo:203], xd[..., 203 + lo :], kernel_backend=KernelBackend.rocm)
            assert y.shape == gate.shape
            assert nerr(y, oracle.swiglu(gate.float(), up.float())) <= _tol(dtype)
        for cols in (1, 3, 12, 203, 1001):
            xp = (torch.randn(5, 29, 2 * cols, generator=g) * 2).to(dtype)
            dy = torch.randn(5, 29, cols, generator=g).to(dtype)
            xpd = xp.cuda().requires_grad_()
            y = swiglu_packed(xpd, kernel_backend=KernelBackend.rocm)
            y.backward(dy.cuda())
            assert nerr(y, oracle.swiglu_packed(xp.float())) <= _tol(dtype), cols
            dg, du = oracle.swiglu_backward(xp[..., 0::2].float(), xp[..., 1::2].float(), dy.float())
            assert nerr(xpd.grad, torch.stack([dg, du], dim=-1).flatten(-2)) <= _tol(dtype), cols
        empty = torch.empty(0, 16, dtype=dtype, device="cuda")
        assert swiglu(empty, empty, kernel_backend=KernelBackend.rocm).shape == (0, 16)


def test_swiglu_broadcast_operands_and_gradients():
    """Operands and upstream gradients whose rows overlap in memory: the gradient autograd hands back for ``y.sum(0)``
    has strides (0, 1), an ``expand``-ed operand too.  The rocm path copies them (the kernels want rows that do not
    overlap); results against the oracle's closed forms."""
    from xma import KernelBackend
    from xma.functional import swiglu, swiglu_packed

    g = torch.Generator().manual_seed(13)
    for dtype in (torch.bfloat16, torch.float32):
        rows, cols = 37, 203
        gate = (torch.randn(rows, cols, generator=g) * 2).to(dtype)
        up = (torch.randn(rows, cols, generator=g) * 2).to(dtype)
        v = torch.randn(cols, generator=g).to(dtype)
        gd, ud, vd = gate.cuda().requires_grad_(), up.cuda().requires_grad_(), v.cuda()
        (swiglu(gd, ud, kernel_backend=KernelBackend.rocm).sum(0) * vd).sum().backward()
        dy = v.float().expand(rows, cols)  # what the sum over the rows hands back, up to the rounding of y.sum(0)
        dg, du = oracle.swiglu_backward(gate.float(), up.float(), dy)
        assert nerr(gd.grad, dg) <= _tol(dtype) and nerr(ud.grad, du) <= _tol(dtype)
        # one row of `up` for all rows of `gate`, forward and backward
        u1 = (torch.randn(1, cols, generator=g) * 2).to(dtype)
        gd, u1d = gate.cuda().requires_grad_(), u1.cuda().requires_grad_()
        y = swiglu(gd, u1d.expand(rows, cols), kernel_backend=KernelBackend.rocm)
        y.backward(torch.ones_like(y))
        assert nerr(y, oracle.swiglu(gate.float(), u1.float().expand(rows, cols))) <= _tol(dtype)
        dg, du = oracle.swiglu_backward(gate.float(), u1.float().expand(rows, cols), torch.ones(rows, cols))
        assert nerr(gd.grad, dg) <= _tol(dtype) and nerr(u1d.grad, du.sum(0, keepdim=True)) <= 2 * _tol(dtype)
        # the packed form with the same kind of gradient
        xp = (torch.randn(rows, 2 * cols, generator=g) * 2).to(dtype)
        xpd = xp.cuda().requires_grad_()
        (swiglu_packed(xpd, kernel_backend=KernelBackend.rocm).sum(0) * vd).sum().backward()
        dg, du = oracle.swiglu_backward(xp[..., 0::2].float(), xp[..., 1::2].float(), dy)
        assert nerr(xpd.grad, torch.stack([dg, du], dim=-1).flatten(-2)) <= _tol(dtype)


SCALED_ACT_CASES = [
    # counts, k, H (= K of dX2), I (= N)
    ((1, 31, 33, 65, 129, 257, 0, 512), 2, 256, 264),
    ((256, 200, 700, 4), 4, 328, 512),
    ((300, 260, 1, 255), 1, 1096, 72),  # few tiles and a long K with a tail: the tiles are split into K slices
    ((3333, 259, 4000), 2, 64, 136),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", SCALED_ACT_CASES)
def test_down_projection_dx_swiglu_scaled_act(dtype, case):
    """dX2 + SwiGLU backward with the second output of its epilogue (xma_rocm_down_projection_dx_swiglu): dz bit-identical
    to the launch without it; scaled_act[n] = swiglu_packed(z[n]) * w[idx[n]] against the oracle's activation in fp32
    (one rounding); and dW2 from it, sum_n dy[idx[n] // k]^T scaled_act[n], against the oracle's weight gradient of the
    scaled grouped dy, sum_n (w dy)[n]^T h[n], per expert."""
    from xma.rocm import ops

    counts, k, H, I = case
    print(f"case counts={counts} k={k} H={H} I={I} {dtype}", flush=True)
    sel, se, ss, offs = _routing_with_counts(counts, k, 21)
    E, M = len(counts), sum(counts)
    T = M // k
    g = torch.Generator().manual_seed(22)
    dy = torch.randn(T, H, generator=g).to(dtype)
    W2 = (torch.randn(E, H, I, generator=g) * 0.1).to(dtype)  # c_proj.weight: (E, out = H, in = I)
    z = torch.randn(M, 2 * I, generator=g).to(dtype)
    w = torch.rand(M, generator=g).to(dtype)
    dyd, W2d, zd, wd, ssd, offsd = dy.cuda(), W2.cuda(), z.cuda(), w.cuda(), ss.cuda(), offs.cuda()
    dz0 = torch.full((M, 2 * I), float("nan"), dtype=dtype, device="cuda")
    ops.down_projection_dx_swiglu_rocm(dyd, W2d, ssd, offsd, zd, dz0, wd, k)  # W logically (E, K = H, N = I)
    dz1 = torch.full_like(dz0, float("nan"))
    hs = torch.full((M, I), float("nan"), dtype=dtype, device="cuda")
    ops.down_projection_dx_swiglu_scaled_act_rocm(dyd, W2d, ssd, offsd, zd, dz1, hs, wd, k)
    torch.cuda.synchronize()
    assert torch.equal(dz0, dz1) and torch.isfinite(dz1).all()
    h32 = oracle.swiglu_packed(z.float())
    want_hs = h32 * w.float()[ss][:, None]
    assert torch.isfinite(hs).all()
    assert nerr(hs, want_hs) <= _tol(dtype)
    row_err = (hs.cpu().float() - want_hs).abs().amax(dim=1) / want_hs.abs().amax(dim=1).clamp_min(1e-6)
    assert row_err.max() <= 4 * _tol(dtype), int(row_err.argmax())
    # dW2 both ways against the oracle (grouped scaled dy, unscaled h)
    gdy = (dy.float()[ss // k] * w.float()[ss][:, None]).to(dtype)
    want_dw = oracle.group_bwd_W(gdy, h32.to(dtype), offs, E)  # (E, I, H)
    dw = torch.full((E, H, I), float("nan"), dtype=dtype, device="cuda").permute(0, 2, 1)
    ops.group_bwd_W_rocm(dyd, hs, ssd, offsd, dw, None, k, 0)
    torch.cuda.synchronize()
    assert torch.isfinite(dw).all()
    for e in range(E):
        if counts[e] == 0:
            assert torch.count_nonzero(dw[e]) == 0
        else:
            assert nerr(dw[e], want_dw[e]) <= 2 * _tol(dtype), e  # two roundings (w h, then the sum) against (w dy, h)


def test_scatter2scatter_with_and_without_workspace():
    """The same launch through the C ABI with the scratch for splitting the last round of tiles along K and without
    it (every tile by one workgroup): both within tolerance of the oracle; the workspace query and its error code."""
    from xma.rocm.loader import get_library

    lib = get_library()
    T, E, k, K, N = 300, 3, 2, 2048, 320
    dtype = torch.bfloat16
    sel, se, ss, offs = _routing(T, E, k, 0)
    g = torch.Generator().manual_seed(3)
    M = T * k
    X = torch.randn(M, K, generator=g).to(dtype)
    W = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)
    want = oracle.scatter2scatter(X, W.permute(0, 2, 1), se, ss, k, True, True, None)
    Xd, Wd, ssd, offsd = X.cuda(), W.cuda(), ss.cuda(), offs.cuda()
    st = torch.cuda.current_stream().cuda_stream
    need = lib.xma_rocm_scatter2scatter_workspace_bytes(M, N, K, E)
    assert need > 0  # a handful of tiles: a last (and only) round that can be split
    ws = torch.empty(need // 4, dtype=torch.float32, device="cuda")

    def run(wptr, wbytes):
        out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
        rc = lib.xma_rocm_scatter2scatter(Xd.data_ptr(), K, Wd.data_ptr(), N * K, K, 0, ssd.data_ptr(), offsd.data_ptr(),
                                          out.data_ptr(), N, None, 0, None, M, N, K, E, k, 1, 1, 0, 0, wptr, wbytes, st)
        torch.cuda.synchronize()
        return rc, out

    rc, split = run(ws.data_ptr(), need)
    assert rc == 0 and nerr(split, want) <= TOL
    rc, whole = run(None, 0)
    assert rc == 0 and nerr(whole, want) <= TOL
    assert nerr(split, whole) <= 2e-3  # the two differ only in the order of the fp32 summation over K
    rc, _ = run(ws.data_ptr(), need - 16)
    assert rc == -3 and b"workspace" in lib.xma_rocm_last_error()
    # launches of many rounds of tiles never split: no scratch asked for
    assert lib.xma_rocm_scatter2scatter_workspace_bytes(16384, 28672, 4096, 8) == 0
