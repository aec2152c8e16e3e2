"""Offline build of libxma_rocm.so: hipcc cross-compiles the hand-written HIP
sources in csrc/ for gfx950 and links them into xma/rocm/libxma_rocm.so, which
the Python host loads with ctypes.  No torch headers, no JIT cache."""

from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor


HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OUT_DIR = os.path.join(HERE, "xma", "rocm")
LIB = os.path.join(OUT_DIR, "libxma_rocm.so")
SOURCES = ["api.hip", "routing.hip", "elementwise.hip", "grouped_gemm.hip", "grouped_gemm_staged.hip", "fp32.hip", "router.hip", "swiglu.hip", "bias.hip", "few_rows.hip", "diagnostics.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-fno-gpu-rdc",
    "-fvisibility=hidden",
    # keep the compiler from forming packed fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # per-kernel register, scratch and LDS figures on stderr (parsed below)
    "-Rpass-analysis=kernel-resource-usage",
    "-I", CSRC,
    "-I", INCLUDE,
]

# The grouped GEMM kernels keep 256 accumulators in AGPRs next to an almost full VGPR file and hand-placed waits around
# asynchronous inline-assembly loads: a register that the compiler spills inside the MFMA loop, behind those waits,
# could be stored before its load has arrived and corrupt data silently.  The build therefore reads the generated ISA of
# those kernels and fails if a scratch STORE sits between the first and the last MFMA of one of them (spills in front of
# the first MFMA, where nothing asynchronous is live, are harmless, and so is reloading such a value later), and says so
# if the compiler is not the version the kernels were written and measured with.
LOOP_NO_SCRATCH = {"grouped_gemm.hip": re.compile(r"grouped_gemm")}
TESTED_HIPCC = "7.2"
USAGE_REPORT = os.path.join(HERE, "build", "kernel_resource_usage.txt")


def _scratch_inside_mfma_loop(asm_path: str, which: re.Pattern) -> list[str]:
    """kernels matching `which` whose ISA has a scratch store between their first and last MFMA"""
    bad, name, first, last, scratch = [], None, None, None, []

    def close():
        if name and first is not None and any(first < n < last for n in scratch):
            bad.append(name)

    with open(asm_path) as f:
        for n, line in enumerate(f):
            m = re.match(r"^(_Z\w+):\s*(;.*)?$", line)
            if m:
                close()
                name = m.group(1) if which.search(m.group(1)) else None
                first, last, scratch = None, None, []
            elif name:
                if "v_mfma" in line:
                    first = n if first is None else first
                    last = n
                elif "scratch_store" in line:
                    scratch.append(n)
    close()
    return bad


def _resource_usage_from_asm(asm_path: str) -> dict[str, dict[str, str]]:
    """{kernel: {field: value}} from the kernel metadata at the end of a device ISA listing (a compile with -save-temps
    prints no resource remarks, so the kernels that the check below exists for are read from their listing)"""
    keys = {".vgpr_count": "VGPRs", ".agpr_count": "AGPRs", ".private_segment_fixed_size": "ScratchSize [bytes/lane]",
            ".group_segment_fixed_size": "LDS Size [bytes/block]", ".vgpr_spill_count": "VGPR spills",
            ".sgpr_spill_count": "SGPR spills", ".sgpr_count": "SGPRs"}
    out: dict[str, dict[str, str]] = {}
    cur: dict[str, str] = {}
    with open(asm_path) as f:
        for line in f:
            m = re.match(r"^\s+(?:- )?(\.[a-z_]+):\s+(\S+)\s*$", line)
            if not m:
                continue
            key, val = m.group(1), m.group(2)
            if key == ".agpr_count":  # first field of a kernel's record
                cur = {}
            if key in keys:
                cur[keys[key]] = val
            elif key == ".name" and val.startswith("_Z"):
                out[val] = cur
    for v in out.values():  # the VGPR figure of the remarks counts both files, as the occupancy rule does
        v.setdefault("Occupancy [waves/SIMD]", str(max(1, 512 // max(int(v.get("VGPRs", "512")), 1))))
    return out


def _resource_usage(stderr: str) -> dict[str, dict[str, str]]:
    """{kernel: {field: value}} from the -Rpass-analysis=kernel-resource-usage remarks"""
    out: dict[str, dict[str, str]] = {}
    cur = None
    for line in stderr.splitlines():
        m = re.search(r"remark:\s+(Function Name|[A-Za-z ]+(?: \[[^\]]*\])?):\s*(\S+)", line)
        if not m:
            continue
        key, val = m.group(1).strip(), m.group(2)
        if key == "Function Name":
            cur = out.setdefault(val, {})
        elif cur is not None:
            cur[key] = val
    return out


def _check_compiler(verbose: bool) -> None:
    r = subprocess.run([HIPCC, "--version"], capture_output=True, text=True)
    m = re.search(r"HIP version:\s*(\S+)", r.stdout)
    version = m.group(1) if m else "unknown"
    if not version.startswith(TESTED_HIPCC):
        print(f"build.py: warning: hipcc {version}, the kernels were written and measured with {TESTED_HIPCC}.x; "
              f"re-run the GPU parity tests before trusting this build", file=sys.stderr)
    elif verbose:
        print(f"hipcc {version}", flush=True)


def _compile(src: str, verbose: bool, defines: tuple[str, ...] = (), tag: str = "") -> str:
    obj = os.path.join(HERE, "build", src.replace(".hip", tag + ".o"))
    # keeps the device ISA next to the object (named after the source, so only the untagged build of a file may do this)
    extra = ["-save-temps=obj"] if src in LOOP_NO_SCRATCH and not tag else []
    cmd = [HIPCC, *FLAGS, *extra, *defines, "-c", os.path.join(CSRC, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    usage = _resource_usage(r.stderr)
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l and "kernel-resource-usage" not in l)
    err = re.sub(r"(?m)^\s*\d+ \|.*\n\s*\| \^\s*$\n?", "", err)  # source excerpts under the remarks
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if re.search(r"warning|error", err) and verbose:
        print(err, file=sys.stderr)
    if extra:
        asm = os.path.join(HERE, "build", src.replace(".hip", "-hip-amdgcn-amd-amdhsa-gfx950.s"))
        bad = _scratch_inside_mfma_loop(asm, LOOP_NO_SCRATCH[src])
        if bad:
            raise RuntimeError(f"{src}: scratch stores inside the MFMA loop of:\n  " + "\n  ".join(bad))
        usage = _resource_usage_from_asm(asm)
    return obj, usage


def build(verbose: bool = False) -> str:
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    os.makedirs(OUT_DIR, exist_ok=True)
    _check_compiler(verbose)
    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(lambda s: _compile(s, verbose), SOURCES))
    objs = [o for o, _ in results]
    with open(USAGE_REPORT, "w") as f:
        for _, usage in results:
            for k, v in usage.items():
                spills = f" spilled VGPRs {v['VGPR spills']}" if v.get("VGPR spills", "0") != "0" else ""
                f.write(f"{k}: VGPRs {v.get('VGPRs')} AGPRs {v.get('AGPRs')} scratch {v.get('ScratchSize [bytes/lane]')} "
                        f"LDS {v.get('LDS Size [bytes/block]')} occupancy {v.get('Occupancy [waves/SIMD]')}{spills}\n")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


TIMING_LIB = os.path.join(OUT_DIR, "libxma_rocm_timing.so")


def build_timing(verbose: bool = False, rebuild: bool = True) -> str:
    """A second library for diagnostics/tile_phases.py: grouped_gemm.hip compiled with -DXMA_PST_TIMING (the persistent
    GEMM kernel stamps the real-time counter and the shader clock counter at six points of every tile and behind every K
    step of one tile), linked with the objects of the normal build (rebuild=False: those of the last build()).
    Not part of build(): nothing in the product loads it."""
    if rebuild:
        build(verbose)
    obj, _ = _compile("grouped_gemm.hip", verbose, ("-DXMA_PST_TIMING",), "_timing")
    objs = [obj if s == "grouped_gemm.hip" else os.path.join(HERE, "build", s.replace(".hip", ".o")) for s in SOURCES]
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", TIMING_LIB, *objs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return TIMING_LIB


if __name__ == "__main__":
    if "--timing-only" in sys.argv[1:]:
        print(build_timing(verbose=True, rebuild=False))
    else:
        print(build_timing(verbose=True) if "--timing" in sys.argv[1:] else build(verbose=True))
