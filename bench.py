"""MoE hot-path benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c4|c5|c2|small_t|few_rows|copy|mfma_peak|library_gemm]

Default workload: the Mixtral-shaped layer (T=8192, H=4096, I=14336, E=8, top-2, packed SwiGLU, bf16).
A step is one forward + backward of the layer behind the gate: router (top-k + softmax + expert ids from the
given router logits), routing histogram/sort, grouped up-projection + SwiGLU, grouped down-projection, combine, and
all of their gradients down to the logits, on synthetic inputs (drawn on the CPU with torch.manual_seed(0), then
copied) that are resident in HBM before the timed region.  Prints ONE JSON line:

  value        tokens/s over the K timed steps (c2: routed ids/s)
  roofline     the dominant kernel against its roofline; `achieved` = algorithmic FLOPs (or bytes)
               of one launch / its average duration, timed live with events on the launch stream
  cpu_baseline the CPU oracle (plain torch restatement of the reference's torch path) on a bounded
               sample of the same workload, on this box's host cores
  kernels      per-kernel duration / throughput table (extra, for the record)
  other_configs (default workload only) c4, c5 and c2 measured in the same run and summarised
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "accelerated-model-architectures_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E

WORKLOADS = {
    # name: T, H, I, E, k, router bias std
    "c3": dict(T=8192, H=4096, I=14336, E=8, k=2, bias=0.0, label="Mixtral-shaped MoE layer fwd+bwd"),
    "c4": dict(T=16384, H=2048, I=1408, E=64, k=6, bias=1.5, label="fine-grained MoE fwd+bwd (skewed routing)"),
    "c5": dict(T=32768, H=2048, I=768, E=128, k=8, bias=0.0, label="many-expert MoE fwd+bwd"),
}


# HBM bytes per launch of the GEMM kernels of c3 and of c2's route, from two counter runs (FETCH_SIZE scaled by 2.0,
# WRITE_SIZE by 1.0: the factors a 1 GiB device copy, `--workload copy`, gives for the same counters).  bench.py cannot
# read hardware counters itself: the figures are copied from the profile named beside them and are NOT measured in this
# run; the roofline block carries the one of the kernel it names.
MEASURED_TRAFFIC_BYTES = {
    "c3": {
        "up_swiglu": 8.79e9,  # 7.38 GB fetched + 1.41 GB written (3.42 GB algorithmic)
        "down": 3.74e9,  # three launches: whole tiles, K slices of the last round, their sum
        "dx2_swiglu_bwd": 6.51e9,
        "dw2": 3.76e9,
        "dw1": 7.52e9,  # 5.64 GB fetched + 1.88 GB written (2.95 GB algorithmic)
        "dx1": 7.59e9,  # three launches
    },
    "c2": 92.2e6,  # route: unit histogram 18.9 MB + scan 0.6 MB + scatter 72.7 MB (36.1 MB fetched + 56.1 MB written)
}
TRAFFIC_SOURCE = "profiles/hbm_traffic_c3_c2_pmc.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE; a constant, not measured in this run)"


def _host_cpu() -> dict:
    """model name and logical CPU count of the host the CPU baseline runs on"""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cpu_model": model, "os_cpu_count": os.cpu_count()}


def _time_gpu(fn, iters: int, warmup: int = 2) -> float:
    """average milliseconds per call, events on the current (launch) stream"""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def _make_moe_inputs(cfg, device, seed=0):
    """module and inputs of a workload, drawn on the CPU from one seeded generator (so the CPU baseline and the device see
    the same bits) and copied to the device; weights expert by expert to bound the host memory"""
    from xma.functional import swiglu_packed
    from xma.layers import MoE

    g = torch.Generator().manual_seed(seed)
    T, H, I, E, k = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["k"]
    with torch.device("meta"):
        moe = MoE(E, k, H, I, swiglu_packed, True, add_bias=False, std=0.02)
    moe = moe.to_empty(device=device).to(torch.bfloat16)
    with torch.no_grad():
        for p in (moe.c_fc.weight, moe.c_proj.weight):
            for e in range(E):
                p[e].copy_((torch.randn(p.shape[1:], generator=g) * 0.02).to(p.dtype))
        moe.gate.weight.copy_((torch.randn(moe.gate.weight.shape, generator=g) * 0.02).to(torch.bfloat16))
        moe.c_fc.N_array.fill_(2 * I), moe.c_fc.K_array.fill_(H)
        moe.c_proj.N_array.fill_(H), moe.c_proj.K_array.fill_(I)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(device)
    logits = torch.randn(T, E, generator=g)
    if cfg["bias"]:
        logits = logits + cfg["bias"] * torch.randn(E, generator=g)
    logits = logits.to(device)
    vals, sel = logits.topk(k, dim=-1)
    rw = torch.softmax(vals.float(), dim=-1).to(torch.bfloat16)
    grad = torch.randn(T, H, generator=g).to(torch.bfloat16).to(device)
    return moe, x, logits, rw, sel, grad


def _kernel_table(moe, x, rw, sel, grad, cfg, iters):
    """per-kernel timings of the ops of one step, each launched alone in a loop"""
    from xma.layers.moe import rocm_implementation as R
    from xma.rocm import ops

    T, H, I, E, k = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["k"]
    Tk = T * k
    dev = x.device
    counts, offs, excl, se, ss = R.route(sel, E)
    w_fc, w_proj = moe.c_fc.weight.detach().permute(0, 2, 1), moe.c_proj.weight.detach().permute(0, 2, 1)
    z = torch.empty(Tk, 2 * I, device=dev, dtype=x.dtype)
    h = torch.empty(Tk, I, device=dev, dtype=x.dtype)
    eo = torch.empty(Tk, H, device=dev, dtype=x.dtype)
    y = torch.empty(T, H, device=dev, dtype=x.dtype)
    dz = torch.empty_like(z)
    d_rw = torch.empty_like(rw)
    dw_fc, dw_proj = torch.empty_like(w_fc), torch.empty_like(w_proj)
    flat_w = rw.view(-1)
    ids = sel.flatten()

    ops.up_projection_swiglu_rocm(x, w_fc, ss, offs, z, h, k)
    ops.scatter2scatter_rocm(h, w_proj, ss, offs, eo, None, 1, True, False)
    ops.down_projection_dx_swiglu_rocm(grad, w_proj.permute(0, 2, 1), ss, offs, z, dz, flat_w, k)

    table = {}

    def gemm(name, fn, flops):
        ms = _time_gpu(fn, iters)
        table[name] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1), "frac_mfma_peak": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                       "flops": flops}

    def mem(name, fn, nbytes):
        ms = _time_gpu(fn, iters * 6, warmup=3)
        table[name] = {"ms": round(ms, 4), "gbs": round(nbytes / ms / 1e6, 1), "frac_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                       "bytes": nbytes}

    f = 2.0 * Tk * H * I
    gemm("up_swiglu(grouped_gemm NT+SwiGLU)", lambda: ops.up_projection_swiglu_rocm(x, w_fc, ss, offs, z, h, k), 2 * f)
    gemm("down(grouped_gemm NT)", lambda: ops.scatter2scatter_rocm(h, w_proj, ss, offs, eo, None, 1, True, False), f)
    gdy = torch.empty(Tk, H, device=dev, dtype=x.dtype)
    ops.group_rocm(grad, ss, gdy, flat_w, k)
    if R._scale_activations_for_dw2(k, grad):
        # from four experts per token on the step's dX2 also writes w * h, and its dW2 reads dy through the index
        hs = torch.empty_like(h)
        gemm("dx2_swiglu_bwd(grouped_gemm NN, + w*h out)",
             lambda: ops.down_projection_dx_swiglu_scaled_act_rocm(grad, w_proj.permute(0, 2, 1), ss, offs, z, dz, hs, flat_w, k), f)
        gemm("dw2(grouped_gemm_dw, dy gathered)", lambda: ops.group_bwd_W_rocm(grad, hs, ss, offs, dw_proj, None, k, 0), f)
        del hs
    else:
        gemm("dx2_swiglu_bwd(grouped_gemm NN)",
             lambda: ops.down_projection_dx_swiglu_rocm(grad, w_proj.permute(0, 2, 1), ss, offs, z, dz, flat_w, k), f)
        gemm("dw2(grouped_gemm_dw)", lambda: ops.group_bwd_W_rocm(gdy, h, ss, offs, dw_proj, None, 0, 0), f)
    gemm("dw1(grouped_gemm_dw)", lambda: ops.group_bwd_W_rocm(dz, x, ss, offs, dw_fc, None, 0, k), 2 * f)
    gemm("dx1(grouped_gemm NN)", lambda: ops.scatter2scatter_rocm(dz, w_fc.permute(0, 2, 1), ss, offs, eo, None, 1, True, False), 2 * f)
    esz = 2
    # The HBM-bound kernels run on rotating sets of buffers that together exceed the 256 MB Infinity Cache, so that no
    # launch finds its operands cached by the one before ("cold" figures); index and weight vectors are shared.
    comb_bytes = Tk * H * esz + T * k * esz + T * H * esz
    nset = max(3, -(-(768 << 20) // comb_bytes))
    eos = [eo] + [torch.randn_like(eo) for _ in range(nset - 1)]
    ys = [torch.empty_like(y) for _ in range(nset)]
    grads = [grad] + [torch.randn_like(grad) for _ in range(nset - 1)]
    gdys = [gdy] + [torch.empty_like(gdy) for _ in range(nset - 1)]
    turn = [0]

    def rotating(fn):
        def call():
            turn[0] += 1
            fn(turn[0] % nset)
        return call

    mem("combine", rotating(lambda i: ops.combine_rocm(eos[i], rw, ys[i], k)), comb_bytes)
    mem("combine_bwd", rotating(lambda i: ops.combine_bwd_rocm(eos[i], grads[i], d_rw)), Tk * H * esz + T * H * esz + T * k * esz)
    mem("group(dy*w)" if not R._scale_activations_for_dw2(k, grad) else "group(dy*w) [not part of this step: dW2 takes w*h]", rotating(lambda i: ops.group_rocm(grads[i], ss, gdys[i], flat_w, k)),
        T * H * esz + Tk * H * esz + Tk * (8 + esz))
    # what the machine does with the plainest kernels on the same buffers: a device-to-device copy and a fill of Tk x H
    mem("plain copy of (Tk,H) [torch copy_]", rotating(lambda i: gdys[i].copy_(eos[i])), 2 * Tk * H * esz)
    mem("plain fill of (Tk,H) [torch fill_]", rotating(lambda i: gdys[i].fill_(1.0)), Tk * H * esz)
    notes = {"hbm_kernels": f"combine, combine_bwd, group(dy*w) and the two plain copy / fill lines timed on {nset} rotating buffer "
                            f"sets ({nset * comb_bytes >> 20} MiB, more than the Infinity Cache): cold figures; the plain "
                            f"lines are stock torch kernels, the rate a plain copy / fill of the same size reaches here"}
    del eos, ys, grads, gdys
    mem("route", lambda: R.route(sel, E), Tk * 8 + Tk * 8 + Tk * 8 + E * 20)
    # the router: top-k + softmax + ids from given logits (part of the timed step), and fused with the gate projection
    # (what MoE.forward runs), beside the reference's chain of stock ops
    lg = torch.randn(T, E, device=dev, dtype=torch.float32).to(x.dtype)
    r_w = torch.empty(T, k, device=dev, dtype=x.dtype)
    r_ids = torch.empty(T, k, device=dev, dtype=torch.int64)
    d_lg = torch.empty_like(lg)
    mem("router_topk(top-k+softmax+ids)", lambda: ops.router_topk_rocm(lg, r_w, r_ids), T * E * esz + T * k * (esz + 8))
    mem("router_topk_bwd", lambda: ops.router_topk_bwd_rocm(lg, r_ids, r_w, d_lg), 2 * T * E * esz + T * k * (esz + 8))
    mem("router_torch(topk+softmax+cast)", lambda: torch.softmax(lg.topk(k, dim=-1).values.float(), -1).to(x.dtype),
        T * E * esz + T * k * (esz + 8))
    wg = moe.gate.weight.detach()
    if ops.router_gate_topk_supported(H, E, k, x.dtype):
        r_ids32 = torch.empty(T, k, device=dev, dtype=torch.int32)
        r_lg = torch.empty(T, E, device=dev, dtype=x.dtype)
        gate_bytes = T * H * esz + E * H * esz + T * E * esz + T * k * (esz + 4)
        mem("gate+router_fused(gemm+top-k+softmax+ids)", lambda: ops.router_gate_topk_rocm(x, wg, r_lg, r_w, r_ids32), gate_bytes)
        mem("gate+router_torch(linear+topk+softmax+cast)",
            lambda: torch.softmax(torch.nn.functional.linear(x, wg).topk(k, dim=-1).values.float(), -1).to(x.dtype), gate_bytes)
    return table, notes


def measure_moe(args, cfg, name, cpu_baseline=True):
    from oracle import moe as oracle_moe
    from xma import KernelBackend

    from xma.layers.moe import rocm_implementation as R

    dev = torch.device("cuda:0")
    moe, x, logits, rw, sel, grad = _make_moe_inputs(cfg, dev)
    T, H, I, E, k = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["k"]
    xg = x.clone().requires_grad_()
    lg = logits.to(torch.bfloat16).requires_grad_()  # the router works in the activations' dtype, as behind the gate

    def step():
        for p in moe.parameters():
            p.grad = None
        xg.grad = None
        lg.grad = None
        w, ids = R.router_topk(lg, k, ids_dtype=torch.int32)
        y = moe._compute_experts(xg, w, ids, kernel_backend=KernelBackend.rocm)
        y.backward(grad)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # the whole layer as MoE.forward runs it (gate projection fused with the router), for the record
    def layer_step():
        for p in moe.parameters():
            p.grad = None
        xg.grad = None
        y, _ = moe(xg, kernel_backend=KernelBackend.rocm)
        y.backward(grad)

    for _ in range(2):
        layer_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(max(args.steps // 2, 1)):
        layer_step()
    torch.cuda.synchronize()
    layer_ms = (time.perf_counter() - t0) * 1e3 / max(args.steps // 2, 1)
    rw, sel = R.router_topk(lg.detach(), k)  # the routing the timed steps used (bf16 logits)
    counts = torch.bincount(sel.flatten(), minlength=E)

    table, notes = _kernel_table(moe, x, rw, sel, grad, cfg, args.kernel_iters)
    gemms = {n: v for n, v in table.items() if "tflops" in v}
    # the dominant kernel: the GEMM launch (group) that takes longest in this run
    dom = max(gemms, key=lambda n: gemms[n]["ms"])
    total_flops = sum(v["flops"] for v in gemms.values())
    total_ms = sum(v["ms"] for v in gemms.values())
    traffic = MEASURED_TRAFFIC_BYTES.get(name)
    dom_traffic = traffic.get(dom.split("(")[0]) if isinstance(traffic, dict) else None
    roofline = {
        "kernel": dom,
        "bound": "mfma",
        "achieved": gemms[dom]["tflops"],
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(gemms[dom]["tflops"] / PEAK_BF16_TFLOPS, 4),
        "traffic": dom_traffic,
        "traffic_source": TRAFFIC_SOURCE if dom_traffic else None,
        "all_gemms_tflops": round(total_flops / total_ms / 1e9, 1),
        "all_gemms_frac": round(total_flops / total_ms / 1e9 / PEAK_BF16_TFLOPS, 4),
        "gemm_fracs": {n.split("(")[0]: v["frac_mfma_peak"] for n, v in gemms.items()},
    }

    # CPU baseline: the oracle, bf16 like the reference's torch path, on the first T / cpu_fraction tokens with every other
    # dimension unchanged (same weights, bit-identical)
    cpu = None
    if cpu_baseline and not args.no_cpu_baseline:
        Ts = max(T // args.cpu_fraction, 1)
        w1, w2 = moe.c_fc.weight.detach().cpu(), moe.c_proj.weight.detach().cpu()
        xs, rws, sels, gs = x[:Ts].cpu(), rw[:Ts].cpu(), sel[:Ts].cpu(), grad[:Ts].cpu()
        reps = 2
        t1 = time.perf_counter()
        for _ in range(reps):
            oracle_moe.experts_forward_backward(xs, rws, sels, w1, w2, oracle_moe.swiglu_packed, gs)
        dt = (time.perf_counter() - t1) / reps
        cpu = {
            "value": round(Ts / dt, 1),
            "unit": "tokens/s",
            "cores": torch.get_num_threads(),
            **_host_cpu(),
            "kind": "port",
            "sample": f"fwd+bwd of the torch-path oracle in bf16 on the first {Ts} of {T} tokens (all other dimensions and "
                      f"the weights unchanged), mean of {reps} runs of {dt:.1f} s",
        }
        del w1, w2

    out = {
        "metric": "moe_fwd_bwd_tokens_per_s",
        "value": round(T / ms_per_step * 1e3, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{name}: {cfg['label']}, T={T} H={H} I={I} E={E} top-{k} packed SwiGLU bf16, x~N(0,1) W~N(0,0.02) "
                        f"logits~N(0,1){'+N(0,1.5) expert bias' if cfg['bias'] else ''}, upstream grad~N(0,1)",
            "tokens": T,
            "rows_per_expert_min_mean_max": [int(counts.min()), float(counts.float().mean()), int(counts.max())],
            "step_tflops": round(18.0 * T * k * H * I / ms_per_step / 1e9, 1),
            # what `value` and `ms_per_step` time: MoE._compute_experts behind given router logits (BASELINE's metric)
            "step": "router top-k/softmax/ids from the given logits + routing + experts fwd+bwd down to d_logits",
            # for the record, the whole layer: MoE.forward + backward with the gate projection fused into the router
            "whole_layer_ms": round(layer_ms, 4),
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
        "kernels": table,
        "notes": notes,
    }
    del moe, x, logits, rw, sel, grad, xg, lg
    torch.cuda.empty_cache()
    return out


def measure_routing(args, zipf, cpu_baseline=True):
    """configs[1]: continuous_count + routing on 4 Mi int32 ids over 64 experts (uniform; --zipf for the skewed run)"""
    from oracle import routing as oracle_routing
    from xma import KernelBackend
    from xma.functional import continuous_count
    from xma.layers.moe import rocm_implementation as R
    from xma.rocm import ops

    n, E = 4 * 1024 * 1024, 64
    g = torch.Generator().manual_seed(0)
    if zipf:
        p = torch.arange(1, E + 1, dtype=torch.float64) ** (-1.1)
        ids_cpu = torch.multinomial(p / p.sum(), n, replacement=True, generator=g).to(torch.int32)
    else:
        ids_cpu = torch.randint(0, E, (n,), generator=g, dtype=torch.int32)
    # rotate over enough distinct buffers to exceed the 256 MB Infinity Cache
    nbuf = 20
    bufs = [ids_cpu.cuda() for _ in range(nbuf)]
    it = [0]

    def step():
        it[0] += 1
        R.route(bufs[it[0] % nbuf], E)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    y = torch.zeros(E, dtype=torch.uint32, device="cuda")

    def hist():  # what the public functional runs: output from torch.empty, counts written by the kernels
        it[0] += 1
        continuous_count(bufs[it[0] % nbuf], E, kernel_backend=KernelBackend.rocm)

    def graph_ms(call, reps=20):
        """per-call time of `call(buffer)` replayed from one graph that holds a call per input buffer: GPU time without the
        host's launch overhead, which at these kernel sizes is larger than the kernels"""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            call(bufs[0])
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g_ = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g_):
            for b in bufs:
                call(b)
        return _time_gpu(g_.replay, reps, warmup=3) / len(bufs)

    route_graph_ms = graph_ms(lambda b: R.route(b, E))
    hist_graph_ms = graph_ms(lambda b: ops.continuous_count_set_rocm(b, y))
    hist_ms = _time_gpu(hist, args.kernel_iters * 10, warmup=5)

    def hist_op():  # the custom op alone, output preallocated (its scratch still comes from torch's allocator inside the op)
        it[0] += 1
        ops.continuous_count_set_rocm(bufs[it[0] % nbuf], y)

    hist_op_ms = _time_gpu(hist_op, args.kernel_iters * 10, warmup=5)
    hist_warm_ms = _time_gpu(lambda: ops.continuous_count_set_rocm(bufs[0], y), args.kernel_iters * 10, warmup=5)
    route_ms = _time_gpu(step, args.kernel_iters * 5, warmup=5)
    hist_bytes = n * 4 + E * 4
    route_bytes = n * 4 + n * 8 + n * 4 + E * 20
    # what the machine does with the plainest kernels at this size: a fill of the 12 B/id that route writes, and a copy
    # that moves as many bytes as route (half in, half out), each replayed from a graph like the calls above
    outs = [torch.empty(n * 12, dtype=torch.uint8, device="cuda") for _ in range(nbuf)]
    halves = [torch.empty(route_bytes // 2, dtype=torch.uint8, device="cuda") for _ in range(nbuf)]

    def ref_graph_ms(fn, reps=20):
        fn(0)
        torch.cuda.synchronize()
        g_ = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g_):
            for i in range(nbuf):
                fn(i)
        return _time_gpu(g_.replay, reps, warmup=3) / nbuf

    fill_ms = ref_graph_ms(lambda i: outs[i].view(torch.int32).fill_(1))
    copy_ms = ref_graph_ms(lambda i: halves[i].copy_(halves[(i + 1) % nbuf]))
    read_ms = ref_graph_ms(lambda i: halves[0][:64].copy_(bufs[i].view(torch.uint8)[:64]))  # launch floor of one kernel
    del outs, halves
    # the same kernels with the launch cost amortised: 64 Mi ids (16 times the configuration), two alternating buffers
    big_n = 64 * 1024 * 1024
    big = [torch.randint(0, E, (big_n,), dtype=torch.int32, device="cuda") for _ in range(2)]
    if zipf:
        for b in big:
            b.copy_(torch.multinomial((p / p.sum()).cuda().float(), big_n, replacement=True).to(torch.int32))
    big_y = torch.empty(E, dtype=torch.uint32, device="cuda")
    big_route_ms = _time_gpu(lambda: (it.__setitem__(0, it[0] + 1), R.route(big[it[0] % 2], E)), 10, warmup=2)
    big_hist_ms = _time_gpu(lambda: (it.__setitem__(0, it[0] + 1), ops.continuous_count_set_rocm(big[it[0] % 2], big_y)), 10, warmup=2)
    del big
    torch.cuda.empty_cache()
    reps, dt = 3, None
    if cpu_baseline and not args.no_cpu_baseline:
        t1 = time.perf_counter()
        for _ in range(reps):
            oracle_routing.route(ids_cpu.numpy(), E)
        dt = (time.perf_counter() - t1) / reps
    out = {
        "metric": "routing_ids_per_s",
        "value": round(n / ms_per_step * 1e3, 1),
        "unit": "ids/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int32",
        "data": "synthetic",
        "config": {"workload": f"c2: counts + offsets + stable permutation of {n} int32 ids over E={E}, "
                               f"{'Zipf(s=1.1)' if zipf else 'uniform'}, {nbuf} rotating input buffers"},
        "roofline": {
            "kernel": "route (3 kernels: unit histogram, scan, stable scatter), per call, replayed from a graph",
            "bound": "hbm",
            "achieved": round(route_bytes / route_graph_ms / 1e6, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(route_bytes / route_graph_ms / 1e6 / PEAK_HBM_GBS, 4),
            "traffic": None if zipf else MEASURED_TRAFFIC_BYTES["c2"],
            "traffic_source": None if zipf else TRAFFIC_SOURCE,
        },
        "cpu_baseline": None if dt is None else {
            "value": round(n / dt, 1), "unit": "ids/s", "cores": 1, **_host_cpu(), "kind": "port",
            "sample": f"numpy stable argsort + bincount + cumsum of the same {n} ids, mean of {reps}"},
        "kernels": {
            "continuous_count_cold": {"ms": round(hist_ms, 5), "gbs": round(hist_bytes / hist_ms / 1e6, 1),
                                      "frac_hbm_peak": round(hist_bytes / hist_ms / 1e6 / PEAK_HBM_GBS, 4), "bytes": hist_bytes},
            "continuous_count_op_cold": {"ms": round(hist_op_ms, 5), "note": "the custom op with a preallocated output, launched from Python"},
            "continuous_count_warm": {"ms": round(hist_warm_ms, 5), "gbs": round(hist_bytes / hist_warm_ms / 1e6, 1),
                                      "frac_hbm_peak": round(hist_bytes / hist_warm_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "route": {"ms": round(route_ms, 5), "gbs": round(route_bytes / route_ms / 1e6, 1), "bytes": route_bytes},
            "route_graph": {"ms": round(route_graph_ms, 5), "gbs": round(route_bytes / route_graph_ms / 1e6, 1),
                            "frac_hbm_peak": round(route_bytes / route_graph_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "continuous_count_graph": {"ms": round(hist_graph_ms, 5), "gbs": round(hist_bytes / hist_graph_ms / 1e6, 1),
                                       "frac_hbm_peak": round(hist_bytes / hist_graph_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "plain fill of 12 B/id [torch fill_, graph]": {"ms": round(fill_ms, 5), "gbs": round(n * 12 / fill_ms / 1e6, 1),
                                                                "frac_hbm_peak": round(n * 12 / fill_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "plain copy moving route's bytes [torch copy_, graph]": {
                "ms": round(copy_ms, 5), "gbs": round(route_bytes / copy_ms / 1e6, 1),
                "frac_hbm_peak": round(route_bytes / copy_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "one 64-byte copy kernel [graph]": {"ms": round(read_ms, 5)},
            "route_64Mi_ids": {"ms": round(big_route_ms, 5), "gbs": round(route_bytes * 16 / big_route_ms / 1e6, 1),
                               "frac_hbm_peak": round(route_bytes * 16 / big_route_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "continuous_count_64Mi_ids": {"ms": round(big_hist_ms, 5), "gbs": round(big_n * 4 / big_hist_ms / 1e6, 1),
                                          "frac_hbm_peak": round(big_n * 4 / big_hist_ms / 1e6 / PEAK_HBM_GBS, 4)},
        },
    }
    del bufs
    torch.cuda.empty_cache()
    return out


def _other_configs(args) -> dict:
    """The configurations beside the headline one, measured in the same process and summarised: c4 and c5 (a few steps and
    the per-kernel table each), c2 uniform and Zipf (route and continuous_count replayed from a graph)."""
    res = {}
    saved = (args.steps, args.warmup)
    args.steps, args.warmup = max(3, min(args.steps, 5)), 2
    for name in ("c4", "c5"):
        r = measure_moe(args, WORKLOADS[name], name, cpu_baseline=False)
        fr = r["roofline"]["gemm_fracs"]
        low = min(fr, key=fr.get)
        res[name] = {"ms_per_step": r["ms_per_step"], "tokens_per_s": r["value"], "step_tflops": r["config"]["step_tflops"],
                     "whole_layer_ms": r["config"]["whole_layer_ms"], "all_gemms_frac": r["roofline"]["all_gemms_frac"],
                     "gemm_fracs": fr, "lowest_gemm": low, "dominant_gemm": r["roofline"]["kernel"],
                     "rows_per_expert_min_mean_max": r["config"]["rows_per_expert_min_mean_max"],
                     "hbm_kernels_frac": {n.split("(")[0]: v["frac_hbm_peak"] for n, v in r["kernels"].items()
                                          if "frac_hbm_peak" in v and not n.startswith("plain")}}
    for label, zipf in (("c2_uniform", False), ("c2_zipf", True)):
        r = measure_routing(args, zipf, cpu_baseline=False)
        k = r["kernels"]
        res[label] = {"route_graph_us": round(k["route_graph"]["ms"] * 1e3, 2), "route_frac_hbm": k["route_graph"]["frac_hbm_peak"],
                      "continuous_count_graph_us": round(k["continuous_count_graph"]["ms"] * 1e3, 2),
                      "continuous_count_frac_hbm": k["continuous_count_graph"]["frac_hbm_peak"],
                      "continuous_count_functional_us": round(k["continuous_count_cold"]["ms"] * 1e3, 2),
                      "continuous_count_op_us": round(k["continuous_count_op_cold"]["ms"] * 1e3, 2),
                      "route_op_us": round(k["route"]["ms"] * 1e3, 2),
                      "route_64Mi_frac_hbm": k["route_64Mi_ids"]["frac_hbm_peak"],
                      "continuous_count_64Mi_frac_hbm": k["continuous_count_64Mi_ids"]["frac_hbm_peak"]}
    args.steps, args.warmup = saved
    return res


def run_small_t(args):
    """Latency of one forward + backward of the expert computation with a handful of tokens, the case the reference's
    own test runs (7 tokens, tests/layers/moe_test.py:107) at its two size points (moe_test.py:26-53), with 64, 192 and
    384 tokens (decoding batches), and C4's layer (64 experts) at 64, 512 and 1024 tokens: eager, replayed from a HIP
    graph (no host launch overhead), and the same graph with the 256 x 256 kernels only, beside the time the weights
    touched by the step need to stream through HBM once per use at 8 TB/s (forward, dX and the dW store: three uses);
    and the forward alone (router, routing, both projections, combine) from a graph, the step of a decoding loop."""
    from xma import KernelBackend, set_seed
    from xma.functional import swiglu_packed
    from xma.layers import MoE
    from xma.layers.moe import rocm_implementation as R
    from xma.rocm import ops as _ops

    res = {}
    # the reference test's two size points at 7 tokens and at decoding batches; C4's layer at three batch sizes
    for E, k, H, I, Ts in ((8, 2, 2048, 8192, (7, 64, 192, 384)), (128, 8, 576, 256, (7, 64, 192, 384)),
                           (64, 6, 2048, 1408, (64, 512, 1024))):
        set_seed(0)
        moe = MoE(E, k, H, I, swiglu_packed, True, add_bias=False, std=0.02).to(torch.bfloat16).cuda()
        for T in Ts:
            if args.only not in f"E{E}_k{k}_H{H}_I{I}_T{T}":
                continue
            x = torch.randn(T, H, device="cuda").to(torch.bfloat16).requires_grad_()
            lg = torch.randn(T, E, device="cuda").to(torch.bfloat16).requires_grad_()
            grad = torch.randn(T, H, device="cuda").to(torch.bfloat16)

            def step():
                for p_ in moe.parameters():
                    p_.grad = None
                x.grad = None
                lg.grad = None
                w, ids = R.router_topk(lg, k, ids_dtype=torch.int32)
                y = moe._compute_experts(x, w, ids, kernel_backend=KernelBackend.rocm)
                y.backward(grad)

            eager_ms = _time_gpu(step, max(args.steps, 20), warmup=5)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g_ = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g_):
                step()
            graph_ms = _time_gpu(g_.replay, max(args.steps, 20), warmup=5)
            few_rows_max, _ops.FEW_ROWS_MAX = _ops.FEW_ROWS_MAX, 0  # the same step through the 256 x 256 kernels only
            try:
                step()
                torch.cuda.synchronize()
                gt = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gt):
                    step()
                tiles_only_ms = _time_gpu(gt.replay, max(args.steps, 20), warmup=5)
            finally:
                _ops.FEW_ROWS_MAX = few_rows_max
            del gt

            def forward_only():
                with torch.no_grad():
                    w, ids = R.router_topk(lg, k, ids_dtype=torch.int32)
                    return moe._compute_experts(x, w, ids, kernel_backend=KernelBackend.rocm)

            forward_only()
            torch.cuda.synchronize()
            gf = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gf):
                forward_only()
            fwd_graph_ms = _time_gpu(gf.replay, max(args.steps, 20), warmup=5)
            _, sel = R.router_topk(lg.detach(), k)
            touched = int(torch.unique(sel).numel())
            wbytes = (2 * I * H + H * I) * 2  # both matrices of one expert
            stream_bytes = 2 * touched * wbytes + E * wbytes  # forward and dX read the touched experts, dW writes all
            res[f"E{E}_k{k}_H{H}_I{I}_T{T}"] = {
                "eager_ms": round(eager_ms, 4), "graph_ms": round(graph_ms, 4),
                "mfma_tiles_only_graph_ms": round(tiles_only_ms, 4), "experts_touched": touched,
                "gemm_kernels": {form: ("few_rows" if _ops._few_rows(T * k, E, torch.bfloat16, form) else "mfma tiles") for form in _ops.FEW_ROWS_PER_EXPERT},
                "forward_only_graph_ms": round(fwd_graph_ms, 4),
                "forward_only_weight_stream_ms_at_8TBs": round(touched * wbytes / PEAK_HBM_GBS / 1e6, 4),
                "weight_stream_ms_at_8TBs": round(stream_bytes / PEAK_HBM_GBS / 1e6, 4),
                "graph_over_stream": round(graph_ms / (stream_bytes / PEAK_HBM_GBS / 1e6), 2),
            }
        del moe
        torch.cuda.empty_cache()
    if not res:
        sys.exit(f"small_t: no case name contains {args.only!r}")
    first = next(iter(res.values()))
    print(json.dumps({"metric": "moe_small_t_fwd_bwd_latency_ms", "value": first["graph_ms"], "unit": "ms", "n_gpus": 1,
                      "steps": args.steps, "warmup": args.warmup, "ms_per_step": first["graph_ms"], "higher_is_better": False,
                      "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": "small_t: expert computation fwd+bwd (router top-k from given logits, routing, "
                                             "experts, combine and all gradients) at T = 7, 64, 192 and 384 on the reference test's two "
                                             "size points, bf16 packed SwiGLU"},
                      "results": res}))


def run_few_rows(args):
    """The six grouped GEMMs of one layer (E = 8, H = 2048, I = 8192, bf16) with R rows in every expert, R from 1 to 192:
    microseconds per launch from a graph of five launches, through the 256 x 256 MFMA kernels and through the kernels of
    the few-token regime (csrc/few_rows.hip), whatever the dispatch rule of the ops would pick.  Where the two columns
    cross is where the rule's limits come from (with routed, uneven tokens they sit lower: --workload small_t)."""
    from xma.rocm import ops

    E, H, I, dt = 8, 2048, 8192, torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(0)
    W1 = (torch.randn(E, 2 * I, H, device="cuda", generator=g) * 0.02).to(dt)
    W2 = (torch.randn(E, H, I, device="cuda", generator=g) * 0.02).to(dt)
    dW1, dW2 = torch.empty_like(W1), torch.empty_like(W2)

    def graph_us(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for _ in range(5):
                fn()
        return _time_gpu(gr.replay, 4, warmup=1) / 5 * 1e3

    res = {}
    for R in (1, 2, 4, 8, 16, 32, 64, 96, 128, 192):
        M = R * E
        ids = torch.arange(E, device="cuda").repeat_interleave(R)[torch.randperm(M, device="cuda", generator=g)]
        se, ss = ids.sort(stable=True)
        offs = torch.bincount(se, minlength=E).cumsum(0)
        x, dy = (torch.randn(M, H, device="cuda", generator=g).to(dt) for _ in range(2))
        hg = torch.randn(M, I, device="cuda", generator=g).to(dt)
        dzg, zg = (torch.randn(M, 2 * I, device="cuda", generator=g).to(dt) for _ in range(2))
        w = torch.rand(M, device="cuda", generator=g).to(dt)
        z, dz = torch.empty(M, 2 * I, device="cuda", dtype=dt), torch.empty(M, 2 * I, device="cuda", dtype=dt)
        h, out = torch.empty(M, I, device="cuda", dtype=dt), torch.empty(M, H, device="cuda", dtype=dt)
        gemms = {
            "up_swiglu": lambda: ops.up_projection_swiglu_rocm(x, W1.permute(0, 2, 1), ss, offs, z, h, 1, None),
            "down": lambda: ops.scatter2scatter_rocm(hg, W2.permute(0, 2, 1), ss, offs, out, w, 1, True, False),
            "dx1": lambda: ops.scatter2scatter_rocm(dzg, W1, ss, offs, out, None, 1, True, False),
            "dx2_swiglu_bwd": lambda: ops.down_projection_dx_swiglu_rocm(dy, W2, ss, offs, zg, dz, w, 1),
            "dw1": lambda: ops.group_bwd_W_rocm(dzg, x, ss, offs, dW1.permute(0, 2, 1), None, 0, 1),
            "dw2": lambda: ops.group_bwd_W_rocm(dy, hg, ss, offs, dW2.permute(0, 2, 1), None, 1, 0),
        }
        row = {}
        for name, fn in gemms.items():
            saved = (ops.FEW_ROWS_MAX, ops.FEW_ROWS_PER_EXPERT)
            try:
                ops.FEW_ROWS_MAX = 0  # the 256 x 256 kernels
                tiles = graph_us(fn)
                ops.FEW_ROWS_MAX, ops.FEW_ROWS_PER_EXPERT = 1 << 20, dict.fromkeys(saved[1], 1 << 20)  # the few-token kernels
                few = graph_us(fn)
            finally:
                ops.FEW_ROWS_MAX, ops.FEW_ROWS_PER_EXPERT = saved
            row[name] = {"mfma_tiles_us": round(tiles, 1), "few_rows_us": round(few, 1)}
        res[f"R{R}"] = row
        print(f"R={R}: " + "  ".join(f"{n} {v['mfma_tiles_us']:.0f}/{v['few_rows_us']:.0f}" for n, v in row.items()), file=sys.stderr, flush=True)
    first = res["R1"]["up_swiglu"]["few_rows_us"]
    print(json.dumps({"metric": "few_rows_up_projection_us", "value": first, "unit": "us", "n_gpus": 1, "steps": args.steps,
                      "warmup": args.warmup, "ms_per_step": first / 1e3, "higher_is_better": False, "dtype": "bf16",
                      "data": "synthetic",
                      "config": {"workload": "few_rows: the six grouped GEMMs of a layer of 8 experts, H = 2048, I = 8192, with R "
                                             "rows in every expert, 256 x 256 MFMA kernels beside the few-token kernels"},
                      "rules": {"rows_per_expert": dict(ops.FEW_ROWS_PER_EXPERT), "rows": ops.FEW_ROWS_MAX}, "results": res}))


def run_copy(args):
    """counter calibration: a plain device copy of known size (1 GiB read + 1 GiB written per launch), the kernel
    that FETCH_SIZE / WRITE_SIZE readings of the other workloads are scaled by"""
    nbytes = 1 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    ms = _time_gpu(lambda: dst.copy_(src), args.steps, warmup=args.warmup)
    print(json.dumps({"metric": "copy_gb_per_s", "value": round(2 * nbytes / ms / 1e6, 1), "unit": "GB/s", "n_gpus": 1,
                      "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
                      "config": {"workload": f"copy: torch copy_ of {nbytes} bytes (reads {nbytes}, writes {nbytes} per launch)"}}))


def run_mfma_peak(args):
    """What the matrix pipes sustain with nothing else going on: independent bf16 MFMAs from registers on every compute
    unit, once with random operands and once with all-zero operands (which toggle nothing and run at the full clock).
    The GEMM kernels' fractions of the 2.5 PFLOP/s figure are read beside the first number."""
    from xma.rocm import get_library
    from xma.rocm.loader import check

    lib = get_library()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    g = torch.Generator().manual_seed(0)
    rnd = (torch.rand(16 * 256 * 8, generator=g) * 4 - 2).to(torch.bfloat16).cuda()  # 8 bf16 per lane and fragment
    out = torch.empty(cus * 256, dtype=torch.float32, device="cuda")
    iters = 20000
    flops = 2.0 * 32 * 32 * 16 * 64 * 4 * cus * iters
    res = {}
    for label, ops_ in (("random_operands", rnd), ("zero_operands", torch.zeros_like(rnd))):
        def call():
            check(lib.xma_rocm_diag_mfma_stream(ops_.data_ptr(), iters, out.data_ptr(), cus,
                                                torch.cuda.current_stream().cuda_stream), "xma_rocm_diag_mfma_stream")
        ms = _time_gpu(call, max(args.steps, 3), warmup=max(args.warmup, 1))
        res[label] = {"ms": round(ms, 3), "tflops": round(flops / ms / 1e9, 1), "frac_of_2500": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    print(json.dumps({"metric": "mfma_only_bf16_tflops", "value": res["random_operands"]["tflops"], "unit": "TFLOP/s", "n_gpus": 1,
                      "steps": args.steps, "warmup": args.warmup, "ms_per_step": res["random_operands"]["ms"],
                      "higher_is_better": True, "dtype": "bf16",
                      "config": {"workload": f"mfma_peak: {iters} x 64 independent v_mfma_f32_32x32x16_bf16 per wave, 4 waves on "
                                             f"each of {cus} compute units, operands in registers, no memory traffic"},
                      "results": res}))


def run_library_gemm(args):
    """For comparison, not part of the product path: the stock dense bf16 GEMM of this PyTorch build (hipBLASLt) on the
    dense equivalents of the C3 GEMMs - every token through one expert's weights, no gather, no scatter, no activation -
    in the three operand forms the layer uses: x @ W^T (forward), dy @ W (dX) and dy^T @ x (dW).  Same value distribution
    as the layer's operands (activations ~ N(0, 1), weights ~ N(0, 0.02))."""
    g = torch.Generator(device="cuda").manual_seed(0)

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, device="cuda", generator=g) * std).to(torch.bfloat16)

    Tk, H, I = 16384, 4096, 14336
    res = {}

    def timed(name, fn, flops):
        ms = _time_gpu(fn, max(args.steps, 5), warmup=max(args.warmup, 2))
        res[name] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1), "frac_mfma_peak": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}

    x, w1 = rn(Tk, H), rn(2 * I, H, std=0.02)
    timed("up-projection form: x (Tk,H) @ W1 (2I,H)^T", lambda: torch.nn.functional.linear(x, w1), 4.0 * Tk * H * I)
    dz = rn(Tk, 2 * I)
    timed("dX1 form: dz (Tk,2I) @ W1 (2I,H)", lambda: dz @ w1, 4.0 * Tk * H * I)
    timed("dW1 form: dz (Tk,2I)^T @ x (Tk,H)", lambda: dz.t() @ x, 4.0 * Tk * H * I)
    del dz, w1
    h, w2 = rn(Tk, I), rn(H, I, std=0.02)
    timed("down-projection form: h (Tk,I) @ W2 (H,I)^T", lambda: torch.nn.functional.linear(h, w2), 2.0 * Tk * H * I)
    dy = rn(Tk, H)
    timed("dX2 form: dy (Tk,H) @ W2 (H,I)", lambda: dy @ w2, 2.0 * Tk * H * I)
    timed("dW2 form: dy (Tk,H)^T @ h (Tk,I)", lambda: dy.t() @ h, 2.0 * Tk * H * I)
    total_ms = sum(v["ms"] for v in res.values())
    print(json.dumps({"metric": "library_dense_gemm_tflops", "value": round(18.0 * Tk * H * I / total_ms / 1e9, 1),
                      "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(total_ms, 4),
                      "higher_is_better": True, "dtype": "bf16",
                      "config": {"workload": "library_gemm: stock dense bf16 GEMMs (torch -> hipBLASLt) on the dense equivalents of "
                                             "the six C3 GEMMs, Tk=16384 H=4096 I=14336, no routing and no epilogue work"},
                      "results": res}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5", "small_t", "few_rows", "copy", "mfma_peak", "library_gemm"])
    ap.add_argument("--zipf", action="store_true", help="c2 only: Zipf(s=1.1) ids instead of uniform")
    ap.add_argument("--kernel-iters", type=int, default=5)
    ap.add_argument("--cpu-fraction", type=int, default=1, help="CPU baseline runs on T / this many tokens")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="c3 only: leave out the summary of c4, c5 and c2")
    ap.add_argument("--only", default="", help="small_t only: run the cases whose name contains this text (e.g. E8_k2_H2048_I8192_T7)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus N with N > 1 is not supported (no collectives in the path)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a GPU")
    from xma.rocm import get_library

    get_library()
    if args.workload == "copy":
        run_copy(args)
    elif args.workload == "mfma_peak":
        run_mfma_peak(args)
    elif args.workload == "library_gemm":
        run_library_gemm(args)
    elif args.workload == "small_t":
        run_small_t(args)
    elif args.workload == "few_rows":
        run_few_rows(args)
    elif args.workload == "c2":
        print(json.dumps(measure_routing(args, args.zipf)))
    else:
        out = measure_moe(args, WORKLOADS[args.workload], args.workload)
        if args.workload == "c3" and not args.no_other_configs:
            out["other_configs"] = _other_configs(args)
        print(json.dumps(out))


if __name__ == "__main__":
    main()
