"""Where a tile of the persistent grouped GEMM kernel spends its time.

    python accelerated-model-architectures_amd/build.py --timing       (here, no GPU needed)
    python accelerated-model-architectures_amd/diagnostics/tile_phases.py [c3] [c4] [c5]    (on the GPU box)

The timing build of the library (xma/rocm/libxma_rocm_timing.so, grouped_gemm.hip compiled with -DXMA_PST_TIMING) makes
thread 0 of every workgroup write the 100 MHz real-time counter at six points of each of its first 48 tiles;
xma_rocm_debug_pst_times copies the stamps out.  Per workload and forward-type GEMM this prints the mean duration of
the phases of a tile, first and last tile of every workgroup left out:

    wait   top of the tile: its first K step and the rows of its epilogue have landed, all waves have met
    setup  what precedes the main loop (second K step's first loads; for tiles that do not overlap: the next tile's
           schedule entry and row indices)
    loop   the K loop (for tiles that overlap it contains the next tile's set-up and the issue of its first K step)
    issue  behind the loop: operand addresses and first K step of the next tile (tiles that do not overlap)
    epi    the epilogue
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
TILES, STAMPS = 48, 8


def load():
    path = os.path.join(os.path.dirname(HERE), "xma", "rocm", "libxma_rocm_timing.so")
    if not os.path.isfile(path):
        sys.exit(f"{path} is missing: build it with `python accelerated-model-architectures_amd/build.py --timing`")
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        f = getattr(lib, name)
        f.restype, f.argtypes = res, args
    lib.xma_rocm_debug_pst_times.argtypes = [ctypes.c_void_p]
    return lib


def run(lib, name):
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

    def s2s(*a):
        rc = lib.xma_rocm_scatter2scatter(*a, None, 0, st)
        assert rc == 0, lib.xma_rocm_last_error()

    ops = {
        "up-projection + SwiGLU": lambda: s2s(P(x), H, P(w1), 2 * I * H, H, 0, P(ss), P(offs), P(z), 2 * I, P(h), I, None, Tk, 2 * I, H, E, k, 0, 1, 1, 0),
        "down-projection": lambda: s2s(P(h), I, P(w2), H * I, I, 0, P(ss), P(offs), P(eo), H, None, 0, None, Tk, H, I, E, 1, 1, 0, 0, 0),
        "dX2 + SwiGLU backward": lambda: s2s(P(dy), H, P(w2), H * I, I, 1, P(ss), P(offs), P(dz), 2 * I, P(z), 2 * I, P(rw), Tk, I, H, E, k, 0, 1, 2, 0),
        "dX1": lambda: s2s(P(dz), 2 * I, P(w1), 2 * I * H, H, 1, P(ss), P(offs), P(eo), H, None, 0, None, Tk, H, 2 * I, E, 1, 1, 0, 0, 0),
    }
    for what, op in ops.items():
        for _ in range(3):
            op()
        torch.cuda.synchronize()
        assert lib.xma_rocm_debug_pst_reset() == 0
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        op()
        e.record()
        torch.cuda.synchronize()
        buf = np.zeros((256, TILES, STAMPS), dtype=np.uint64)
        assert lib.xma_rocm_debug_pst_times(buf.ctypes.data) == 0
        t = buf.astype(np.int64)
        n_tiles = (t[:, :, 5] > 0).sum(1)
        rows = []
        for b in range(256):
            for i in range(1, min(n_tiles[b], TILES - 1) - 1):
                rows.append([t[b, i, j + 1] - t[b, i, j] for j in range(5)] + [t[b, i + 1, 0] - t[b, i, 0]])
        r = np.array(rows) * 0.01  # 100 MHz ticks -> microseconds
        m = r.mean(0)
        print(f"{name} {what}: launch {s.elapsed_time(e) * 1e3:.0f} us, {n_tiles.min()}-{n_tiles.max()} tiles per workgroup; per tile "
              f"wait {m[0]:.2f} setup {m[1]:.2f} loop {m[2]:.2f} issue {m[3]:.2f} epi {m[4]:.2f} total {m[5]:.2f} us", flush=True)


if __name__ == "__main__":
    library = load()
    for w in (sys.argv[1:] or ["c3", "c4", "c5"]):
        run(library, w)
