"""Expert-layer benchmark on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2]`` times K
passes of route -> permute -> SwiGLU FFN (grouped GEMM) -> combine over one
synthetic batch that is already resident in HBM, and prints ONE JSON line:
tokens/s of the whole step, the roofline record of the dominant kernel (the
gate-up grouped GEMM) measured with HIP events on the launch stream, the other
stages' rates, and the CPU path timed on the host cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_FP8_TFLOPS = 5000.0

# Bytes per launch of the dominant kernel that crossed the L2 boundary, from rocprofv3 --pmc runs of this script
# (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, the factors read off a 1 GiB copy in the same runs).  A bench run does not
# measure them: they are read off the committed summaries named here.  None = not measured.
MEASURED_TRAFFIC = {"C2": (3.500e9, "profiles/expert_layer_c2_hbm_traffic.md"),
                    "C3": (1.911e9, "profiles/expert_layer_c5_c4_c3_hbm_traffic.md"),
                    "C4": (1.418e9, "profiles/expert_layer_c5_c4_c3_hbm_traffic.md"),
                    "C5": (12.069e9, "profiles/expert_layer_c5_c4_c3_hbm_traffic.md")}


def _event_ms(fn, iters: int, warmup: int = 2, plug=None):
    """Average duration of ``fn`` in ms, HIP events on the current stream (the one
    the kernels are launched on).  ``plug`` is device work of a few ms enqueued first:
    the events and launches of a kernel that is shorter than its own host call then
    queue up behind it and the intervals hold no time spent waiting for the host."""
    import torch
    for _ in range(warmup):
        fn()
    if plug is not None:
        plug()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    stop = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    for i in range(iters):
        start[i].record()
        fn()
        stop[i].record()
    torch.cuda.synchronize()
    times = [s.elapsed_time(e) for s, e in zip(start, stop)]
    return sum(times) / len(times), min(times)


def _cpu_baseline(w, x, ids, gates, layer, budget_s: float = 12.0):
    """The CPU path (oracle/cpu_path.py) on a growing prefix of the batch until
    about ``budget_s`` seconds are spent; returns the record of the largest sample."""
    import torch
    from oracle import cpu_path
    # the threads the environment grants this process: OMP_NUM_THREADS where it is set (a GPU box shares its host
    # cores between its GPUs), every core otherwise; the host's own core count is reported beside it
    cores = torch.get_num_threads()
    w13 = layer.w13_weight.detach().cpu()
    w2 = layer.w2_weight.detach().cpu()
    xc, idc, gc = x.cpu(), ids.cpu(), gates.cpu()
    n = min(w.T, 64)
    spent = 0.0
    times = []
    while True:
        t0 = time.perf_counter()
        cpu_path.expert_layer(xc[:n], idc[:n], gc[:n], w13, w2)
        dt = time.perf_counter() - t0
        spent += dt
        if n < w.T and spent + 2.2 * dt <= budget_s:
            n = min(w.T, n * 2)       # grow the sample while it is cheap
            times = []
            continue
        times.append(dt)
        if spent + dt > budget_s or len(times) >= 50:
            break
    times.sort()
    dt = times[len(times) // 2]
    return {"value": n / dt, "unit": "tokens/s", "cores": cores, "host_cpu_count": os.cpu_count(), "kind": "port",
            "sample": f"first {n} of {w.T} tokens ({n * w.k} routed rows) through all {w.E} experts' full weights, "
                      f"median of {len(times)} passes, {dt:.2f} s each, {spent:.1f} s of CPU work in all; "
                      f"bf16 storage, torch CPU matmul (fp32 accumulate)"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="C2", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--variant", type=int, default=0, help="grouped GEMM tile variant (tuning)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--kernel-iters", type=int, default=10)
    ap.add_argument("--no-split", action="store_true",
                    help="grouped GEMMs without a workspace: the tiles of the last round are not cut along K (comparison)")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run a plain device copy of this many MiB (scales the FETCH_SIZE/WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the expert-worker path is built and measured on a single MI355X; "
              "run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    from disagmoe_amd import _lib, workloads
    from disagmoe_amd.grouped_gemm import backend as gg
    from disagmoe_amd.models.experts import MoEExperts, MoEExpertsFP8
    from disagmoe_amd.ops import memory

    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    _lib.load()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    w = workloads.WORKLOADS[args.config]
    gg.set_tile_variant(args.variant)

    ids_cpu, gates_cpu = workloads.make_routing(w)
    x = workloads.make_activations(w).to(dev)
    ids, gates = ids_cpu.to(dev), gates_cpu.to(dev)
    w13, w2 = workloads.make_weights(w, dev)
    if w.fp8:
        layer = MoEExpertsFP8(w13, w2)
        bf16_layer = None
    else:
        layer = MoEExperts.__new__(MoEExperts)
        torch.nn.Module.__init__(layer)
        layer.hidden_size, layer.intermediate_size, layer.num_experts, layer.tp_size = w.d, w.I, w.E, 1
        layer.w13_weight = torch.nn.Parameter(w13, requires_grad=False)
        layer.w2_weight = torch.nn.Parameter(w2, requires_grad=False)
        layer.enable_cache = False
        layer.gmm_cache_max_batch_size = 0
    # the layer's state block (MoEExperts.create_weights) and the stream's shared workspace
    if not w.fp8:
        layer._init_gemm_state(dev)
    gemm_state = dict(arguments_ptr=layer.arguments_ptr, workspace=None if args.no_split else gg.shared_workspace(dev))
    if args.no_split:
        layer._gemm_state = lambda: gemm_state
    torch.cuda.synchronize()

    # bf16: where the batch is small enough for it to pay, the gate-up kernel fetches the tokens' rows by their place in
    # the expert-sorted order and no permute kernel runs (the same result bit for bit)
    fetch_rows = (not w.fp8) and (not args.no_split) and layer.takes_rows(w.T, w.R)

    def step():
        if w.fp8:   # the routed rows are quantised on their way into the expert-sorted buffer
            mappings, batch_sizes, _ = memory.route_tokens(ids, w.E)
            xq, xs = memory.permute_quantize(x, mappings)
            y = layer.forward_quantized(w.R, xq, xs, batch_sizes)
        elif fetch_rows:
            mappings, batch_sizes, _, row_token = memory.route_tokens_with_sources(ids, w.E)
            y = layer.forward_rows(x, row_token, batch_sizes)
        else:
            mappings, batch_sizes, _ = memory.route_tokens(ids, w.E)
            permuted = memory.permute_tokens_cuda(x, mappings)
            y = layer.forward(w.R, permuted, batch_sizes)
        return memory.combine_tokens(y, mappings, gates)

    if args.copy_probe_mib > 0:
        src = torch.empty(args.copy_probe_mib << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # ---- per-kernel timing (HIP events on the launch stream) ----
    mappings, batch_sizes, _ = memory.route_tokens(ids, w.E)
    permuted = memory.permute_tokens_cuda(x, mappings)
    it = args.kernel_iters
    stages = {}
    # the row kernels take 5 - 100 us, less than the host needs to launch them from Python
    plug_a = torch.randn(8192, 8192, dtype=torch.bfloat16, device=dev)
    plug_c = torch.empty_like(plug_a)

    def plug():
        for _ in range(4):
            torch.mm(plug_a, plug_a, out=plug_c)

    ms, _ = _event_ms(lambda: memory.route_tokens(ids, w.E), it, plug=plug)
    stages["route"] = {"ms": ms, "GB/s": w.route_bytes / ms / 1e6}
    def gemm_ms(fn):
        """(ms per launch with 5 launches inside one event pair: what a profiler's kernel duration compares with; ms of
        one launch inside its own event pair, which holds the events' own packets as well)"""
        def many():
            for _ in range(5):
                fn()
        return _event_ms(many, max(2, it // 2))[0] / 5, _event_ms(fn, it)[0]

    def sustained_ms(fn, n=10):
        """ms per launch when n launches follow each other inside one event interval: a launch's ramp-up overlaps the
        drain of the one before it, as it does behind another kernel in a running step"""
        def many():
            for _ in range(n):
                fn()
        return _event_ms(many, max(2, it // 2), plug=plug)[0] / n

    def rotating_ms(call, inputs, n=12):
        """ms per launch when n launches follow each other inside one event interval, each on the next of several
        copies of the input and into the next of as many output buffers (the ring keeps the outputs alive, so the
        allocator hands out different blocks): more than the 256 MB Infinity Cache in all, so that no launch finds the
        bytes of the one before it in a cache"""
        ring = [None] * len(inputs)
        def many():
            for i in range(n):
                ring[i % len(inputs)] = call(inputs[i % len(inputs)])
        return _event_ms(many, max(2, it // 2), plug=plug)[0] / n

    n_sets = max(4, int(768e6 // ((w.T + w.R) * w.d * 2)) + 1)      # at least 768 MB under the timing loop
    n_sets = min(n_sets, 64)
    ms, _ = _event_ms(lambda: memory.permute_tokens_cuda(x, mappings), it, plug=plug)
    # "GB/s" counts a read and a write per routed row; the kernel reads a token once for its k copies ("moved")
    moved = (w.T + w.R) * w.d * 2 + 8.0 * w.R
    stages["permute"] = {"ms": ms, "GB/s": w.permute_bytes / ms / 1e6, "frac_hbm": w.permute_bytes / ms / 1e6 / PEAK_HBM_GBS,
                         "GB/s_moved": moved / ms / 1e6, "frac_hbm_moved": moved / ms / 1e6 / PEAK_HBM_GBS}
    ms = sustained_ms(lambda: memory.permute_tokens_cuda(x, mappings))
    stages["permute"].update({"ms_back_to_back": ms, "frac_hbm_moved_back_to_back": moved / ms / 1e6 / PEAK_HBM_GBS})
    xs = [x] + [x.clone() for _ in range(n_sets - 1)]
    ms = rotating_ms(lambda xi: memory.permute_tokens_cuda(xi, mappings), xs)
    stages["permute"].update({"ms_rotating_buffers": ms, "frac_hbm_moved_rotating_buffers": moved / ms / 1e6 / PEAK_HBM_GBS,
                              "rotating_sets": n_sets})
    del xs
    if w.fp8:
        xq, xs = gg.quantize_rows(permuted)
        h = gg.gmm_fp8_swiglu(xq, xs, layer.w13_q, layer.w13_scale, batch_sizes, **gemm_state)
        hq, hs = gg.quantize_rows(h)
        up_ms, up_single = gemm_ms(lambda: gg.gmm_fp8_swiglu(xq, xs, layer.w13_q, layer.w13_scale, batch_sizes, c=h, **gemm_state))
        y_buf = torch.empty((w.R, w.d), dtype=torch.bfloat16, device=dev)
        down_ms, down_single = gemm_ms(lambda: gg.gmm_fp8(hq, hs, layer.w2_q, layer.w2_scale, batch_sizes, c=y_buf, **gemm_state))
        q_ms, _ = _event_ms(lambda: gg.quantize_rows(h), it)
        stages["quant_rows"] = {"ms": q_ms, "GB/s": 3.0 * w.R * w.I / q_ms / 1e6}       # the [R, I] intermediate
        pq_ms, _ = _event_ms(lambda: memory.permute_quantize(x, mappings), it)
        stages["permute_quantize"] = {"ms": pq_ms, "GB/s": (2.0 * w.T + w.R) * w.d / pq_ms / 1e6}   # bytes actually moved
        peak = PEAK_FP8_TFLOPS
    else:
        h = gg.gmm_swiglu(permuted, layer.w13_weight, batch_sizes, **gemm_state)
        up_ms, up_single = gemm_ms(lambda: gg.gmm_swiglu(permuted, layer.w13_weight, batch_sizes, c=h, **gemm_state))
        y_buf = torch.empty((w.R, w.d), dtype=torch.bfloat16, device=dev)
        down_ms, down_single = gemm_ms(lambda: gg.gmm(h, layer.w2_weight, batch_sizes, c=y_buf, **gemm_state))
        peak = PEAK_BF16_TFLOPS
    up_flops = 2.0 * w.R * w.d * 2 * w.I
    down_flops = 2.0 * w.R * w.I * w.d
    # what the library launches for the two GEMMs, by its own account (kernel, tile rows, workgroups, tiles cut along K)
    ws_bytes = 0 if args.no_split else gemm_state["workspace"].numel()
    sizes_host = batch_sizes.cpu()
    plan_up = gg.launch_plan(w.R, w.E, w.d, w.I, swiglu=True, fp8=w.fp8, workspace_bytes=ws_bytes, batch_sizes=sizes_host)
    plan_down = gg.launch_plan(w.R, w.E, w.I, w.d, swiglu=False, fp8=w.fp8, workspace_bytes=ws_bytes, batch_sizes=sizes_host)
    kernel = (f"{plan_up['kernel']} ({'fp8 e4m3' if w.fp8 else 'bf16, [K, N] weights'}, tiles of {plan_up['tile_rows']} rows, "
              f"{plan_up['workgroups']} workgroups of {plan_up['wavefronts']} wavefronts): gate-up projection with fused SiLU*mul")
    if w.fp8:
        # yardstick, not part of the path: the vendor library's dense fp8 GEMM (torch._scaled_mm) of the gate-up launch's
        # flop count, one expert's quantised weights, unit scales; skipped (with the reason) where torch refuses it
        try:
            one = torch.ones((), dtype=torch.float32, device=dev)
            wq_t = layer.w13_q[0].t()                     # [d, 2I] column-major view of the K-contiguous [2I, d] weights
            lib_ms, _ = gemm_ms(lambda: torch._scaled_mm(xq, wq_t, scale_a=one, scale_b=one, out_dtype=torch.bfloat16))
            stages["library_dense_gemm"] = {"ms": lib_ms, "TFLOP/s": up_flops / lib_ms / 1e9, "frac_mfma": up_flops / lib_ms / 1e9 / peak,
                                            "what": "torch._scaled_mm (hipBLASLt, fp8 e4m3 x fp8 e4m3 -> bf16, unit scales) on [R, d] x "
                                                    "[d, 2I]: the flop count of the gate-up launch as one dense GEMM"}
            rows_e = w.R // w.E
            one_ms, _ = gemm_ms(lambda: torch._scaled_mm(xq[:rows_e], wq_t, scale_a=one, scale_b=one, out_dtype=torch.bfloat16))
            stages["library_gemm_one_expert"] = {"ms": one_ms, "TFLOP/s": up_flops / w.E / one_ms / 1e9,
                                                 "what": "the same library call on one expert's share of the rows, [R/E, d] x [d, 2I]: "
                                                         "repeated on ONE weight matrix, which the 256 MB Infinity Cache keeps"}

            def fp8_loop():
                for e in range(w.E):
                    torch._scaled_mm(xq[e * rows_e:(e + 1) * rows_e], layer.w13_q[e].t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
            loop_ms, _ = gemm_ms(fp8_loop)
            stages["library_gemm_loop_over_experts"] = {"ms": loop_ms, "TFLOP/s": up_flops / loop_ms / 1e9, "frac_mfma": up_flops / loop_ms / 1e9 / peak,
                                                        "what": "E library calls of R/E rows, each on its own expert's weights: the gate-up launch "
                                                                "on equal experts as a loop over the vendor's dense GEMM"}
        except Exception as err:   # noqa: BLE001 - a yardstick must not break the bench
            stages["library_dense_gemm"] = {"ms": None, "what": f"torch._scaled_mm refused: {str(err)[:160]}"}
    if not w.fp8:
        # yardstick, not part of the path: the vendor library's dense GEMM of the gate-up launch's flop count
        # ([R, d] x [d, 2I], one expert's weights, no SiLU*mul), timed the same way on the same box
        dense_c = torch.empty((w.R, 2 * w.I), dtype=torch.bfloat16, device=dev)
        lib_ms, _ = gemm_ms(lambda: torch.mm(permuted, layer.w13_weight[0], out=dense_c))
        stages["library_dense_gemm"] = {"ms": lib_ms, "TFLOP/s": up_flops / lib_ms / 1e9, "frac_mfma": up_flops / lib_ms / 1e9 / peak,
                                        "what": "torch.mm (hipBLASLt) on [R, d] x [d, 2I]: the flop count of the gate-up launch as "
                                                "one dense GEMM without the epilogue; a yardstick for what this chip sustains"}
        rows_e = w.R // w.E
        one_c = torch.empty((rows_e, 2 * w.I), dtype=torch.bfloat16, device=dev)
        one_ms, _ = gemm_ms(lambda: torch.mm(permuted[:rows_e], layer.w13_weight[0], out=one_c))
        stages["library_gemm_one_expert"] = {"ms": one_ms, "TFLOP/s": up_flops / w.E / one_ms / 1e9,
                                             "what": "the same library call on one expert's share of the rows, [R/E, d] x [d, 2I], repeated "
                                                     "on ONE weight matrix, which the 256 MB Infinity Cache keeps"}
        outs_e = [dense_c[e * rows_e:(e + 1) * rows_e] for e in range(w.E)]

        def bf16_loop():
            for e in range(w.E):
                torch.mm(permuted[e * rows_e:(e + 1) * rows_e], layer.w13_weight[e], out=outs_e[e])
        loop_ms, _ = gemm_ms(bf16_loop)
        stages["library_gemm_loop_over_experts"] = {"ms": loop_ms, "TFLOP/s": up_flops / loop_ms / 1e9, "frac_mfma": up_flops / loop_ms / 1e9 / peak,
                                                    "what": "E library calls of R/E rows, each on its own expert's weights: the gate-up launch on "
                                                            "equal experts as a loop over the vendor's dense GEMM"}
        del one_c, outs_e, dense_c
    stages["gemm_gate_up"] = {"ms": up_ms, "ms_single_launch": up_single, "TFLOP/s": up_flops / up_ms / 1e9, "frac_mfma": up_flops / up_ms / 1e9 / peak,
                              "launch": plan_up}
    stages["gemm_down"] = {"ms": down_ms, "ms_single_launch": down_single, "TFLOP/s": down_flops / down_ms / 1e9, "frac_mfma": down_flops / down_ms / 1e9 / peak,
                           "launch": plan_down}
    stages["gemm_total"] = {"ms": up_ms + down_ms, "TFLOP/s": w.gemm_flops / (up_ms + down_ms) / 1e9,
                            "frac_mfma": w.gemm_flops / (up_ms + down_ms) / 1e9 / peak}
    y = layer.forward(w.R, permuted, batch_sizes)
    ms, _ = _event_ms(lambda: memory.combine_tokens(y, mappings, gates), it, plug=plug)
    stages["combine"] = {"ms": ms, "GB/s": w.combine_bytes / ms / 1e6, "frac_hbm": w.combine_bytes / ms / 1e6 / PEAK_HBM_GBS}
    ms = sustained_ms(lambda: memory.combine_tokens(y, mappings, gates))
    stages["combine"].update({"ms_back_to_back": ms, "frac_hbm_back_to_back": w.combine_bytes / ms / 1e6 / PEAK_HBM_GBS})
    ys = [y] + [y.clone() for _ in range(n_sets - 1)]
    ms = rotating_ms(lambda yi: memory.combine_tokens(yi, mappings, gates), ys)
    stages["combine"].update({"ms_rotating_buffers": ms, "frac_hbm_rotating_buffers": w.combine_bytes / ms / 1e6 / PEAK_HBM_GBS,
                              "rotating_sets": n_sets})
    # yardstick, not part of the path: torch's device copy of the [R, d] rows over the same rotating buffers
    copy_bytes = 2.0 * w.R * w.d * 2
    dsts = [torch.empty_like(yi) for yi in ys]
    slot = [0]
    def copy_next(_):
        i = slot[0] = (slot[0] + 1) % len(ys)
        dsts[i].copy_(ys[i - 1])
        return None
    ms = rotating_ms(copy_next, ys)
    stages["library_device_copy"] = {"ms_rotating_buffers": ms, "GB/s": copy_bytes / ms / 1e6, "frac_hbm": copy_bytes / ms / 1e6 / PEAK_HBM_GBS,
                                     "what": "torch copy_ of [R, d] bf16 rows (read + write) over the rotating buffers: what a plain copy "
                                             "kernel sustains on this chip on bytes that no cache holds"}
    del ys, dsts

    # algorithmic bytes of the two GEMM launches: weights of the experts that have rows, the rows in, the rows out
    ws = 1 if w.fp8 else 2
    live = int((batch_sizes > 0).sum().item())
    up_bytes = live * w.d * 2.0 * w.I * ws + w.R * w.d * ws + w.R * w.I * 2
    down_bytes = live * w.I * float(w.d) * ws + w.R * w.I * ws + w.R * w.d * 2
    stages["gemm_gate_up"].update({"GB/s": up_bytes / up_ms / 1e6, "frac_hbm": up_bytes / up_ms / 1e6 / PEAK_HBM_GBS})
    stages["gemm_down"].update({"GB/s": down_bytes / down_ms / 1e6, "frac_hbm": down_bytes / down_ms / 1e6 / PEAK_HBM_GBS})

    achieved = up_flops / up_ms / 1e9
    traffic, traffic_source = MEASURED_TRAFFIC.get(args.config, (None, None))
    if args.no_split:
        traffic, traffic_source = None, None
    if up_flops / up_bytes < peak * 1e12 / (PEAK_HBM_GBS * 1e9):
        # fewer flops per byte than the ridge of the roofline (decode-sized batches): streaming the weights bounds it
        roofline = {"kernel": kernel, "bound": "hbm", "achieved": up_bytes / up_ms / 1e6, "peak": PEAK_HBM_GBS,
                    "unit": "GB/s", "frac": up_bytes / up_ms / 1e6 / PEAK_HBM_GBS,
                    "traffic": traffic, "traffic_source": traffic_source, "bytes_per_launch": up_bytes,
                    "flops_per_launch": up_flops, "avg_launch_ms": up_ms}
    else:
        roofline = {"kernel": kernel, "bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                    "frac": achieved / peak, "traffic": traffic, "traffic_source": traffic_source,
                    "flops_per_launch": up_flops, "avg_launch_ms": up_ms}

    record = {
        "metric": "expert-layer tokens/s (route + permute + grouped-GEMM SwiGLU FFN + combine)",
        "value": w.T / (ms_per_step / 1e3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp8_e4m3" if w.fp8 else "bf16", "data": "synthetic",
        "config": {"workload": w.name, "E": w.E, "d": w.d, "ffn": w.I, "T": w.T, "top_k": w.k,
                   "routed_rows": w.R, "routing": w.routing, "tile_variant": args.variant,
                   "permute": ("fetched by the gate-up kernel (dmoe_gmm_swiglu_rows): no permute launch in the timed step"
                               if fetch_rows else "fused with the row quantiser" if w.fp8 else "its own kernel"),
                   "tail_tiles_cut_along_k": not args.no_split},
        "roofline": roofline,
        "stage_timing": "ms = per launch with several launches inside one HIP event pair on the launch stream (5 for the "
                        "GEMMs; the row kernels' ms_back_to_back with 10), comparable with a profiler's kernel durations; "
                        "ms_single_launch / the row kernels' ms = one launch inside its own event pair, which also holds "
                        "the events' own packets and the launch's ramp-up on an idle chip; the row kernels' "
                        "ms_rotating_buffers = 12 launches back to back over rotating_sets copies of the input and as many "
                        "output buffers (more than the Infinity Cache holds)",
        "stages": {k: {kk: (round(vv, 5) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in stages.items()},
    }
    if not args.no_cpu:
        if w.fp8:
            record["cpu_baseline"] = {"value": None, "unit": "tokens/s", "cores": 0, "kind": "port",
                                      "sample": "not run: the CPU path has no fp8 form"}
        else:
            record["cpu_baseline"] = _cpu_baseline(w, x, ids, gates, layer)
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
