"""Board power while a kernel runs in a loop: the MFMA-only stream, the grouped GEMMs of the Mixtral-shaped layer and the
stock dense GEMM of the same sizes.

    python accelerated-model-architectures_amd/diagnostics/power_clock.py        (on the GPU box)

Each kernel is launched back to back for a few seconds while a thread samples the board's power sensor
(/sys/class/drm/card*/device/hwmon/hwmon*/power1_input, microwatts) every 20 ms; the first third of the samples is
dropped.  Printed per kernel: milliseconds per call, mean watts, joules per call, and the energy per FLOP.  A kernel
that sits at the board's power limit runs as fast as its energy per FLOP allows, whatever its instruction stream does.
The lines marked `zeros:` repeat a launch with every matrix operand cleared: the same instructions and the same memory
traffic, but nothing toggles in the matrix pipes, so the launch shows how fast its instruction stream runs when power
does not hold the clock down.
"""

from __future__ import annotations

import glob
import os
import sys
import threading
import time

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

from xma.rocm import get_library  # noqa: E402
from xma.rocm.loader import check  # noqa: E402


def sensors():
    return [p for h in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*") for p in (os.path.join(h, "power1_input"), os.path.join(h, "power1_average")) if os.path.exists(p)]


def read_watts(paths):
    for p in paths:
        try:
            return int(open(p).read().strip()) * 1e-6
        except (OSError, ValueError):
            pass
    return float("nan")


def measure(name, fn, flops, paths, secs=2.5):
    fn()
    torch.cuda.synchronize()
    samples, stop = [], [False]

    def sampler():
        while not stop[0]:
            samples.append(read_watts(paths))
            time.sleep(0.02)

    th = threading.Thread(target=sampler)
    th.start()
    n, t0 = 0, time.perf_counter()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    while time.perf_counter() - t0 < secs:
        for _ in range(10):
            fn()
        n += 10
        torch.cuda.synchronize()
    e.record()
    torch.cuda.synchronize()
    stop[0] = True
    th.join()
    ms = s.elapsed_time(e) / max(n, 1)
    kept = samples[len(samples) // 3:]
    watts = sum(kept) / max(len(kept), 1)
    line = f"{name:44s} {ms:8.3f} ms/call  {watts:7.0f} W  {watts * ms * 1e-3:6.3f} J/call"
    if flops:
        line += f"  {flops / ms / 1e9:7.0f} TFLOP/s  {watts * ms * 1e-3 / flops * 1e12:5.2f} pJ/FLOP"
    print(line, flush=True)


def main():
    import tile_phases

    lib = get_library()
    paths = sensors()
    print("power sensor:", paths[0] if paths else "none found (the watt columns are nan)", flush=True)
    for cap in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap"):
        try:
            print(f"board power limit ({cap}): {int(open(cap).read().strip()) * 1e-6:.0f} W", flush=True)
        except (OSError, ValueError):
            pass
    measure("idle (no kernel)", lambda: None, 0, paths, secs=1.0)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    st = torch.cuda.current_stream().cuda_stream
    out = torch.empty(cus * 256, dtype=torch.float32, device="cuda")
    iters = 4000
    stream_flops = 2.0 * 32 * 32 * 16 * 64 * 4 * cus * iters
    rnd = (torch.rand(16 * 256 * 8, device="cuda") * 4 - 2).to(torch.bfloat16)
    for label, opnd in (("MFMA stream, random operands", rnd), ("MFMA stream, zero operands", torch.zeros_like(rnd))):
        measure(label, lambda: check(lib.xma_rocm_diag_mfma_stream(opnd.data_ptr(), iters, out.data_ptr(), cus, st), "diag"), stream_flops, paths)
    ops, dw_ops, keep = tile_phases.make_ops(lib, "c3", split_last_round=True)
    T, H, I, E, k, _ = tile_phases.WORKLOADS["c3"]
    f = 2.0 * T * k * H * I
    for (what, (op, _kt)), fl in zip(ops.items(), (2 * f, f, f, 2 * f)):
        measure("grouped " + what, op, fl, paths)
    for (what, op), fl in zip(dw_ops.items(), (f, 2 * f)):
        measure("grouped " + what, op, fl, paths)
    del ops, dw_ops, keep
    # the same launches on all-zero operands: same instructions, same memory traffic, but the matrix pipes toggle nothing
    ops, dw_ops, keep = tile_phases.make_ops(lib, "c3", split_last_round=True, zero_operands=True)
    for (what, (op, _kt)), fl in zip(ops.items(), (2 * f, f, f, 2 * f)):
        measure("zeros: grouped " + what, op, fl, paths)
    for (what, op), fl in zip(dw_ops.items(), (f, 2 * f)):
        measure("zeros: grouped " + what, op, fl, paths)
    g = torch.Generator(device="cuda").manual_seed(0)
    Tk = T * k
    xg = torch.randn(Tk, H, device="cuda", generator=g).to(torch.bfloat16)
    w1 = (torch.randn(2 * I, H, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
    measure("stock x @ W^T, up-projection size", lambda: torch.nn.functional.linear(xg, w1), 2 * f, paths)
    hh = torch.randn(Tk, I, device="cuda", generator=g).to(torch.bfloat16)
    w2 = (torch.randn(H, I, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
    measure("stock x @ W^T, down-projection size", lambda: torch.nn.functional.linear(hh, w2), f, paths)
    dz = torch.randn(Tk, 2 * I, device="cuda", generator=g).to(torch.bfloat16)
    measure("stock dy @ W, dX1 size", lambda: dz @ w1, 2 * f, paths)
    measure("stock dy^T @ x, dW1 size", lambda: dz.t() @ xg, 2 * f, paths)
    xg.zero_()
    w1.zero_()
    measure("zeros: stock x @ W^T, up-projection size", lambda: torch.nn.functional.linear(xg, w1), 2 * f, paths)
    del keep


if __name__ == "__main__":
    main()
