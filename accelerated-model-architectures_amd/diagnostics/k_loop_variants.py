"""What the K loop of the persistent grouped GEMM kernel pays for: shader cycles per K step with one ingredient removed.

    python accelerated-model-architectures_amd/build.py                                     (the normal build, once)
    python accelerated-model-architectures_amd/diagnostics/k_loop_variants.py build         (here, no GPU needed)
    python accelerated-model-architectures_amd/diagnostics/k_loop_variants.py run [c3] [c5] (on the GPU box)

`build` writes patched copies of csrc/grouped_gemm.hip to diagnostics/variants/, compiles each with -DXMA_PST_TIMING (bf16,
forward-type kernels only) and links it with the other objects of the normal build.  The patches touch the steady K steps
only (complete steps in the middle of a tile; the first and last steps of a tile keep every wait), and all variants but
`base` compute WRONG RESULTS on purpose - they exist to be timed, nothing else loads them:

  base     the kernel as it is
  novm     the barrier of a step no longer waits for the loads of the next step (s_waitcnt vmcnt)
  nowait   no barrier and no wait at all in a steady step: what the instruction stream alone costs
  nodma    steady steps issue no loads (the first two steps' operands are multiplied over and over)
  noreads  steady steps read no fragments from LDS
  lead2    the weight tile of a step is requested two steps ahead instead of one (into a stage that is still being read)

`run` prints, per variant and GEMM, the mean shader cycles per K step (2048 = 64 MFMAs back to back), the clock of the
loop and the loop's duration.  Cycles isolate the instruction stream from the clock, which the board's power limit sets.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(HERE, "variants")  # generated sources and libraries: not tracked, but they travel to the GPU box
VARIANTS = ["base", "novm", "nowait", "nodma", "noreads", "lead2"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
OTHER_OBJECTS = ["api", "routing", "elementwise", "grouped_gemm_staged", "fp32", "router", "swiglu", "bias", "few_rows", "diagnostics"]


def _sub(s: str, old: str, new: str) -> str:
    assert s.count(old) == 1, f"k_loop_variants.py is out of step with csrc/grouped_gemm.hip: {old[:70]!r} found {s.count(old)} times"
    return s.replace(old, new)


def _k_step_body(s: str):
    a = s.index("            auto k_step = [&](int kt, auto FULL, auto MODE) {")
    b = s.index("            int kt = 0, kt_end = KT;")
    return a, b


def make_source(tag: str) -> str:
    s = open(os.path.join(PKG, "csrc", "grouped_gemm.hip")).read()
    # bf16, three forward-type instantiations: a third of the compile time
    s = _sub(s, "    return dispatch_fwd<_Float16>(a, w_is_kn ? 1 : 0, epilogue, st);", "    return XMA_ROCM_EUNSUPPORTED;")
    s = _sub(s, "    if (dtype == XMA_ROCM_BF16) return dispatch_dw<__bf16>(a, (int)grid, st);\n    return dispatch_dw<_Float16>(a, (int)grid, st);",
             "    return XMA_ROCM_EUNSUPPORTED;")
    a, b = s.index("template <typename T> int dispatch_fwd("), s.index("// Compute units of the current device")
    s = s[:a] + """template <typename T> int dispatch_fwd(const FwdArgs &a, int wt, int epi, hipStream_t st) {
    if (wt == 0 && epi == XMA_ROCM_EPI_STORE) return launch_fwd<T, 0, XMA_ROCM_EPI_STORE>(a, st);
    if (wt == 0 && epi == XMA_ROCM_EPI_SWIGLU) return launch_fwd<T, 0, XMA_ROCM_EPI_SWIGLU>(a, st);
    if (wt == 1 && epi == XMA_ROCM_EPI_STORE) return launch_fwd<T, 1, XMA_ROCM_EPI_STORE>(a, st);
    return XMA_ROCM_EUNSUPPORTED;
}

""" + s[b:]
    steady = "mode == 0 && FULL.value == 1"
    wait = {"novm": 's_waitcnt lgkmcnt(0)\\n\\ts_barrier', "nowait": "s_nop 0", "lead2": 's_waitcnt vmcnt(8) lgkmcnt(0)\\n\\ts_barrier'}.get(tag)
    if wait:
        s = _sub(s, """                if constexpr (mode == 0)
                    XMA_WAIT_LOADS_AND_BARRIER(); // step kt + 1 has landed; nobody reads this stage any more
""", f"""                if constexpr ({steady})
                    asm volatile("{wait}" ::: "memory");
                else if constexpr (mode == 0)
                    XMA_WAIT_LOADS_AND_BARRIER();
""")
    if tag in ("nowait", "noreads"):
        s = _sub(s, "template <typename T, int PTR, int QTR, int KK, int NI = 4, int READ_NEXT = 1, typename Hook>",
                 "template <typename T, int PTR, int QTR, int KK, int NI = 4, int READ_NEXT = 1, int WAITF = 1, typename Hook>")
        s = _sub(s, "    wait_frags(cur); // issued at least 8 MFMAs ago",
                 '    if constexpr (WAITF != 0) wait_frags(cur); else asm volatile("" : "+v"(cur.p[0]), "+v"(cur.p[1]), "+v"(cur.p[2]), '
                 '"+v"(cur.p[3]), "+v"(cur.q[0]), "+v"(cur.q[1]), "+v"(cur.q[2]), "+v"(cur.q[3]));')
        a, b = _k_step_body(s)
        body = s[a:b]
        read, waitf = ("1", f"({steady}) ? 0 : 1") if tag == "nowait" else (f"({steady}) ? 0 : 1", "1")
        for kk in "123":
            body = _sub(body, f"mma_step<T, WT, 0, {kk}, NI>(", f"mma_step<T, WT, 0, {kk}, NI, {read}, {waitf}>(")
        last_read = "(mode == 2 ? 0 : 1)" if tag == "nowait" else f"(mode == 2 || ({steady})) ? 0 : 1"
        body = _sub(body, "mma_step<T, WT, 0, 0, NI, (mode == 2 ? 0 : 1)>(", f"mma_step<T, WT, 0, 0, NI, {last_read}, {waitf}>(")
        s = s[:a] + body + s[b:]
    if tag == "nodma":
        a, b = _k_step_body(s)
        body = s[a:b]
        body = _sub(body, "                        issue_piece(kt_a, IC<DMA_N0 + G.value>{}, IC<(FULL.value != 0) ? 1 : 0>{});",
                    f"                        if constexpr (!({steady})) issue_piece(kt_a, IC<DMA_N0 + G.value>{{}}, IC<(FULL.value != 0) ? 1 : 0>{{}});")
        body = _sub(body, "                        if constexpr (G.value < DMA_N0) issue_piece(kt_b, G, FULL);",
                    f"                        if constexpr (G.value < DMA_N0 && !({steady})) issue_piece(kt_b, G, FULL);")
        s = s[:a] + body + s[b:]
    if tag == "lead2":
        a, b = _k_step_body(s)
        body = s[a:b]
        body = _sub(body, "                        issue_piece(kt_a, IC<DMA_N0 + G.value>{}, IC<(FULL.value != 0) ? 1 : 0>{});",
                    f"                        issue_piece(kt_a + (({steady}) ? 1 : 0), IC<DMA_N0 + G.value>{{}}, IC<(FULL.value != 0) ? 1 : 0>{{}});")
        s = s[:a] + body + s[b:]
        # the loads of the last steady steps reach one step further: the steady range ends one step earlier
        s = _sub(s, "                for (; kt + 2 < KT_full && kt < kt_end; ++kt) k_step(kt, IC<1>{}, IC<0>{});",
                 "                for (; kt + 3 < KT_full && kt < kt_end; ++kt) k_step(kt, IC<1>{}, IC<0>{});")
    return s


def build_one(tag: str) -> str:
    os.makedirs(OUT, exist_ok=True)
    src, obj, lib = (os.path.join(OUT, f"grouped_gemm_{tag}.{ext}") for ext in ("hip", "o", "so"))
    with open(src, "w") as f:
        f.write(make_source(tag))
    flags = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-fno-gpu-rdc", "-fvisibility=hidden", "-Xclang", "-target-feature",
             "-Xclang", "-packed-fp32-ops", "-DXMA_PST_TIMING", "-I", os.path.join(PKG, "csrc"), "-I", os.path.join(os.path.dirname(PKG), "include")]
    r = subprocess.run([HIPCC, *flags, "-c", src, "-o", obj], capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"{tag}: hipcc failed\n" + "\n".join(l for l in r.stderr.splitlines() if "error" in l))
    objs = [os.path.join(PKG, "build", f"{o}.o") for o in OTHER_OBJECTS]
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, obj, *objs], capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"{tag}: link failed (run build.py first)\n{r.stderr[-1500:]}")
    return lib


def run(workloads):
    sys.path.insert(0, HERE)
    import tile_phases

    for name in workloads:
        for tag in VARIANTS:
            lib = tile_phases.load(os.path.join(OUT, f"grouped_gemm_{tag}.so"))
            ops, _dw_ops, _keep = tile_phases.make_ops(lib, name)
            for what, (op, KT) in ops.items():
                if "SwiGLU backward" in what:
                    continue  # not among the three instantiations of the variants
                r = tile_phases.measure(lib, op, KT)
                print(f"{name} {what:24s} {tag:8s} {r['cycles_per_step']:6.0f} cycles per K step | clock {r['clock_ghz']:.3f} GHz | "
                      f"loop {r['phases_us'][2]:7.1f} us | launch {r['launch_us']:6.0f} us", flush=True)
            del ops, _keep


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "build":
        with ThreadPoolExecutor(max_workers=6) as pool:
            for lib in pool.map(build_one, VARIANTS):
                print("built", lib, flush=True)
    elif len(sys.argv) > 1 and sys.argv[1] == "run":
        run(sys.argv[2:] or ["c3", "c5"])
    else:
        sys.exit(__doc__)
