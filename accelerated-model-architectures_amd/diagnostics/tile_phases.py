"""Where a tile of the persistent grouped GEMM kernel spends its time, in shader cycles and microseconds.

    python accelerated-model-architectures_amd/build.py --timing       (here, no GPU needed)
    python accelerated-model-architectures_amd/diagnostics/tile_phases.py [c3] [c4] [c5]    (on the GPU box)

The timing build of the library (xma/rocm/libxma_rocm_timing.so, grouped_gemm.hip compiled with -DXMA_PST_TIMING) makes
thread 0 of every workgroup read the 100 MHz real-time counter and the shader clock counter at six points of each of its
first 48 tiles, and the shader clock counter behind every K step of its fourth tile.  Per workload and forward-type GEMM
this prints

  phases   mean duration of the phases of a tile (first and last tile of every workgroup left out):
           wait (top of the tile: its first K step has landed, all waves have met), setup (up to the main loop), loop,
           issue (behind the loop: the next tile's first K step, for tiles that do not overlap it with their last step),
           epi (the epilogue)
  loop     shader cycles per K step (2048 = the 64 MFMAs of a step back to back) and the clock the loop ran at
  steps    median cycles of the single K steps of one tile: the first step (which also looks up the next tile and
           fetches its row indices; its figure starts at the stamp in front of the loop and includes that stamp's read
           of the 100 MHz counter, 600 to 3300 cycles depending on how many workgroups stamp at the same moment), the following ones (loads of a fresh operand panel), the steady state, the last two
           (the last one sets up and issues the next tile's first K step)
  ends     when the workgroups finish (the launch ends with the slowest)

and for the two weight-gradient GEMMs (one workgroup per tile, thread 0 stamps the shader clock at four points) the median
cycles of a tile's prologue, main loop (per K step) and epilogue.
"""

from __future__ import annotations

import ctypes
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

from xma.rocm.loader import SIGNATURES  # noqa: E402

WORKLOADS = {"c3": (8192, 4096, 14336, 8, 2, 0.0), "c4": (16384, 2048, 1408, 64, 6, 1.5), "c5": (32768, 2048, 768, 128, 8, 0.0)}
TILES, STAMPS, MAX_STEPS, STEP_TILE, DW_TILES = 48, 8, 240, 3, 8192


def load(path=None):
    path = path or os.path.join(os.path.dirname(HERE), "xma", "rocm", "libxma_rocm_timing.so")
    if not os.path.isfile(path):
        sys.exit(f"{path} is missing: build it with `python accelerated-model-architectures_amd/build.py --timing`")
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        if hasattr(lib, name):
            f = getattr(lib, name)
            f.restype, f.argtypes = res, args
    for name in ("xma_rocm_debug_pst_times", "xma_rocm_debug_pst_cycles", "xma_rocm_debug_pst_steps", "xma_rocm_debug_dw_cycles"):
        getattr(lib, name).argtypes = [ctypes.c_void_p]
    return lib


def make_ops(lib, name, split_last_round=False, zero_operands=False):
    """the four forward-type GEMMs of a workload as closures, with their K step counts, and the two weight-gradient GEMMs;
    split_last_round passes the workspace that lets a launch cut the tiles of its last, partial round into K slices (what
    the layer does), otherwise every tile is computed by one workgroup (what the stamps of this script describe);
    zero_operands clears every matrix operand (same instruction stream, same addresses, nothing toggles in the matrix pipes)"""
    T, H, I, E, k, bias = WORKLOADS[name]
    dev, bf = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    Tk = T * k
    x = torch.randn(T, H, device=dev, generator=g).to(bf)
    w1 = (torch.randn(E, 2 * I, H, device=dev, generator=g) * 0.02).to(bf)
    w2 = (torch.randn(E, H, I, device=dev, generator=g) * 0.02).to(bf)
    logits = torch.randn(T, E, device=dev, generator=g) + bias * torch.randn(E, device=dev, generator=g)
    se, ss = logits.topk(k, dim=-1).indices.flatten().sort(stable=True)
    offs = torch.bincount(se, minlength=E).cumsum(0)
    z = torch.empty(Tk, 2 * I, device=dev, dtype=bf)
    h = torch.randn(Tk, I, device=dev, generator=g).to(bf)
    dz = torch.randn(Tk, 2 * I, device=dev, generator=g).to(bf)
    dy = torch.randn(T, H, device=dev, generator=g).to(bf)
    rw = torch.rand(Tk, device=dev, generator=g).to(bf)
    eo = torch.empty(Tk, H, device=dev, dtype=bf)
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()  # noqa: E731
    gdy = torch.randn(Tk, H, device=dev, generator=g).to(bf)
    dw1 = torch.empty(E, 2 * I, H, device=dev, dtype=bf)
    dw2 = torch.empty(E, H, I, device=dev, dtype=bf)
    keep = (x, w1, w2, ss, offs, z, h, dz, dy, rw, eo, gdy, dw1, dw2)
    if zero_operands:
        for t in (x, w1, w2, h, dz, dy, gdy, z):
            t.zero_()

    ws = {}

    def s2s(*a):
        M, N, K = a[13], a[14], a[15]
        nbytes = lib.xma_rocm_scatter2scatter_workspace_bytes(M, N, K, E) if split_last_round else 0
        if nbytes and (N, K) not in ws:
            ws[(N, K)] = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        rc = lib.xma_rocm_scatter2scatter(*a, ws[(N, K)].data_ptr() if nbytes else None, nbytes, st)
        assert rc == 0, lib.xma_rocm_last_error()

    return {
        "up-projection + SwiGLU": (lambda: s2s(P(x), H, P(w1), 2 * I * H, H, 0, P(ss), P(offs), P(z), 2 * I, P(h), I, None, Tk, 2 * I, H, E, k, 0, 1, 1, 0), H // 64),
        "down-projection": (lambda: s2s(P(h), I, P(w2), H * I, I, 0, P(ss), P(offs), P(eo), H, None, 0, None, Tk, H, I, E, 1, 1, 0, 0, 0), I // 64),
        "dX2 + SwiGLU backward": (lambda: s2s(P(dy), H, P(w2), H * I, I, 1, P(ss), P(offs), P(dz), 2 * I, P(z), 2 * I, P(rw), Tk, I, H, E, k, 0, 1, 2, 0), H // 64),
        "dX1": (lambda: s2s(P(dz), 2 * I, P(w1), 2 * I * H, H, 1, P(ss), P(offs), P(eo), H, None, 0, None, Tk, H, 2 * I, E, 1, 1, 0, 0, 0), 2 * I // 64),
    }, {
        "dW2": lambda: lib.xma_rocm_group_bwd_W(P(gdy), H, 1, 1, None, P(h), I, 1, 1, P(ss), P(offs), P(dw2), H * I, I, H, I, E, 0, st),
        "dW1": lambda: lib.xma_rocm_group_bwd_W(P(dz), 2 * I, 1, 1, None, P(x), H, 0, k, P(ss), P(offs), P(dw1), 2 * I * H, H, 2 * I, H, E, 0, st),
    }, keep


def measure_dw(lib, op):
    """one launch of a weight-gradient GEMM -> median cycles of the parts of its tiles that have at least 8 K steps"""
    for _ in range(2):
        assert op() == 0, lib.xma_rocm_last_error()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    assert op() == 0
    e.record()
    torch.cuda.synchronize()
    buf = np.zeros((DW_TILES, 6), dtype=np.uint64)
    assert lib.xma_rocm_debug_dw_cycles(buf.ctypes.data) == 0
    c = buf.astype(np.int64)
    c = c[(c[:, 3] > 0) & (c[:, 4] >= 8)]
    kt = c[:, 4]
    return {"launch_us": s.elapsed_time(e) * 1e3, "tiles": len(c), "steps": float(kt.mean()), "prologue": float(np.median(c[:, 1] - c[:, 0])),
            "per_step": float(np.median((c[:, 2] - c[:, 1]) / kt)), "epilogue": float(np.median(c[:, 3] - c[:, 2])), "tile": float(np.median(c[:, 3] - c[:, 0]))}


def measure(lib, op, KT):
    """one launch with cleared stamps -> dict of the figures this script prints"""
    for _ in range(2):
        op()
    torch.cuda.synchronize()
    assert lib.xma_rocm_debug_pst_reset() == 0
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    op()
    e.record()
    torch.cuda.synchronize()
    tb = np.zeros((256, TILES, STAMPS), dtype=np.uint64)
    cb = np.zeros_like(tb)
    sb = np.zeros((256, MAX_STEPS), dtype=np.uint64)
    assert lib.xma_rocm_debug_pst_times(tb.ctypes.data) == 0 and lib.xma_rocm_debug_pst_cycles(cb.ctypes.data) == 0
    assert lib.xma_rocm_debug_pst_steps(sb.ctypes.data) == 0
    t, c, st = tb.astype(np.int64), cb.astype(np.int64), sb.astype(np.int64)
    n_tiles = (t[:, :, 5] > 0).sum(1)
    sel = [(b, i) for b in range(256) for i in range(1, min(n_tiles[b], TILES - 1) - 1)]
    ph = np.array([[t[b, i, j + 1] - t[b, i, j] for j in range(5)] + [t[b, i + 1, 0] - t[b, i, 0]] for b, i in sel]) * 0.01
    lc = np.array([c[b, i, 3] - c[b, i, 2] for b, i in sel], dtype=np.float64)
    lt = ph[:, 2]
    out = {"launch_us": s.elapsed_time(e) * 1e3, "tiles": (int(n_tiles.min()), int(n_tiles.max())), "phases_us": ph.mean(0),
           "cycles_per_step": lc.mean() / KT, "clock_ghz": lc.sum() / lt.sum() / 1e3,
           "behind_loop_cycles": float(np.mean([c[b, i, 5] - c[b, i, 3] for b, i in sel]))}
    ok = n_tiles > 0
    ends = np.array([t[b, min(n_tiles[b], TILES) - 1, 5] for b in range(256) if ok[b]]) - t[ok, 0, 0].min()
    out["ends_us"] = (ends.min() * 0.01, np.median(ends) * 0.01, ends.max() * 0.01) if (n_tiles[ok] <= TILES).all() else None
    n = min(KT, MAX_STEPS)
    have = (st[:, n - 1] > 0) & (c[:, STEP_TILE, 5] > 0)
    if have.any():
        sv, cv = st[have], c[have]
        d = np.median(np.diff(sv[:, :n], axis=1), axis=0)
        out["steps"] = {"first": float(np.median(sv[:, 0] - cv[:, STEP_TILE, 2])), "next": d[:6], "steady": float(np.median(d[6:max(7, n - 4)])),
                        "last": d[-2:], "top_to_loop": float(np.median(cv[:, STEP_TILE, 2] - cv[:, STEP_TILE, 0]))}
    return out


def run(lib, name):
    ops, dw_ops, _keep = make_ops(lib, name)
    for what, (op, KT) in ops.items():
        r = measure(lib, op, KT)
        m = r["phases_us"]
        print(f"{name} {what}: launch {r['launch_us']:.0f} us, {r['tiles'][0]}-{r['tiles'][1]} tiles per workgroup", flush=True)
        print(f"   phases (us): wait {m[0]:.2f} setup {m[1]:.2f} loop {m[2]:.2f} issue {m[3]:.2f} epi {m[4]:.2f} total {m[5]:.2f}")
        print(f"   loop: {r['cycles_per_step']:.0f} shader cycles per K step at {r['clock_ghz']:.3f} GHz; behind the loop {r['behind_loop_cycles']:.0f} cycles")
        if "steps" in r:
            s = r["steps"]
            print(f"   steps (cycles, {KT} per tile): top of tile to loop {s['top_to_loop']:.0f}; first {s['first']:.0f}; then "
                  f"{' '.join(f'{v:.0f}' for v in s['next'])}; steady {s['steady']:.0f}; last two {' '.join(f'{v:.0f}' for v in s['last'])}")
        if r["ends_us"]:
            print(f"   workgroups end at (us from the first start): min {r['ends_us'][0]:.0f} median {r['ends_us'][1]:.0f} max {r['ends_us'][2]:.0f}")
    for what, op in dw_ops.items():
        r = measure_dw(lib, op)
        print(f"{name} {what}: launch {r['launch_us']:.0f} us; {r['tiles']} tiles of {r['steps']:.1f} K steps (mean); cycles: prologue {r['prologue']:.0f}, "
              f"loop {r['per_step']:.0f} per K step, epilogue {r['epilogue']:.0f}, whole tile {r['tile']:.0f}", flush=True)


if __name__ == "__main__":
    library = load()
    for w in (sys.argv[1:] or ["c3", "c4", "c5"]):
        run(library, w)
