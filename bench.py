"""MoE-layer benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--headline-only] [--no-cpu-baseline]

A step is one forward of the MoE block (router -> dispatch -> grouped SwiGLU experts -> shared
expert -> combine) over one batch of synthetic hidden states already resident in HBM, weights
resident.  Prints ONE JSON line: the DeepSeek-V3 W8A16 workload the metric is quoted on, with the
same figures (tokens/s, roofline of the dominant kernel, routing GB/s, CPU baseline) for every
other synthetic workload under "workloads".  Per-stage durations come from events recorded on the
launch stream inside the timed steps.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_HBM_GBPS = 8000.0


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or platform.machine()


def cpu_baseline(w, blk, n_sample: int, passes: int = 3):
    """The reference's own algorithm (oracle/torch_blocks.py: fp32 gate, Python loop over experts,
    bf16 F.linear, per-call fp8 block dequantisation) timed on the host cores on a bounded sample
    of the same workload: the first n_sample tokens, same weights, same router.  One warm-up pass,
    then the median of `passes` timed passes."""
    import torch
    from moe_gen_amd import synthetic
    from oracle import torch_blocks as TB

    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1))
    torch.set_num_threads(threads)

    def host(lin):
        wt = lin.weight.data.cpu()
        if wt.dtype == torch.float8_e4m3fn:
            return (wt, lin.weight_scale_inv.data.cpu())
        return wt

    experts = [tuple(host(p) for p in ex.projections()) for ex in blk.experts]
    shared = None
    if w.S and w.family != "mixtral":
        shared = tuple(host(p) for p in blk.shared_experts.projections())
    gate_w = blk.gate.weight.data.cpu()
    x = synthetic.hidden_states(w, "cuda")[..., :, :].reshape(w.n, w.h)[:n_sample].cpu().view(1, n_sample, w.h)

    def run():
        if w.family == "mixtral":
            return TB.mixtral_block(x, gate_w, experts, w.k)
        bias = blk.gate.e_score_correction_bias.data.cpu() if w.family == "v3" else None
        return TB.deepseek_block(x, gate_w, bias, experts, shared, w.family, w.k, w.method, w.n_group,
                                 w.topk_group, w.norm, w.scale)

    run()                                            # warm-up: thread pool, allocator, page faults
    times = []
    for _ in range(passes):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[len(times) // 2]
    return {"value": n_sample / dt, "unit": "tokens/s", "cores": threads, "cpu": cpu_model(), "kind": "port",
            "sample": f"{'all' if n_sample == w.n else 'first ' + str(n_sample) + ' of'} {w.n} tokens of the same workload, all experts' weights; one warm-up pass, "
                      f"median of {passes} timed passes ({dt:.2f} s; all: {', '.join(f'{t:.2f}' for t in times)}); "
                      "stock-PyTorch CPU restatement of the reference block"}


def staged_run(w, blk, x, steps: int, routing_aware: bool = False, pool: int = 0, pageable: bool = False):
    """Second figure: the same block with every expert matrix in pinned host memory, delivered by
    the stager (cyclic prefetch on the copy stream, event hand-off) into a pool of `pool` slots while
    earlier experts are multiplied.  Three layers' worth of modules take turns, as in a model (with two, the
    layer before the current one is also the next one, and the engine's rule that drops what is left of the
    previous layer would throw away what it has just prefetched whenever the pool holds two layers).
    routing_aware: copy only the experts that received tokens, busiest first, once the per-expert
    counts are known (fewer bytes, but the copies cannot start before the router has run).
    pageable: the host copies of the weights are ORDINARY memory (a mapped weight segment that was not
    allocated pinned) and travel through the stager's ring of 8 pinned chunks of 32 MiB, filled by 8 host
    threads: the host holds the model once instead of twice."""
    import time as _t

    import torch
    from moe_gen_amd import StagedExpert, Stager

    E = w.E
    wdt = torch.float8_e4m3fn if w.fp8 else torch.bfloat16
    names = blk.experts[0].names
    shapes = {"routed_expert": {f"{n}.weight": (tuple(getattr(blk.experts[0], n).weight.shape), wdt) for n in names}}
    # the reference engine's prefill pool holds 20 routed experts (deepseekv3_initializer.py:912-916); a layer
    # with more experts runs in waves of half the pool while the other half is being filled
    n_slots = {"routed_expert": pool if pool > 0 else min(20, 2 * E)}
    has_shared = bool(w.S) and w.family != "mixtral"
    if has_shared:
        shapes["shared_expert"] = {f"{n}.weight": (tuple(getattr(blk.shared_experts, n).weight.shape), wdt) for n in names}
        n_slots["shared_expert"] = 2
    st = Stager(shapes, n_slots, device="cuda:0", model_type={"v3": "deepseek_v3", "v2": "deepseek_v2"}.get(w.family, "mixtral"),
                num_hidden_layers=64, num_local_experts=E, bounce_chunks=8 if pageable else 0, bounce_chunk_bytes=32 << 20,
                bounce_threads=8)
    layers = (10, 11, 12)
    if routing_aware:
        st.set_policy("routed_expert", "on_demand")

    def scales_of(mlp):
        if not w.fp8:
            return None
        return {f"{n}.weight_scale_inv": getattr(mlp, n).weight_scale_inv.data for n in names}

    staged = {}
    host = {}
    keep = (lambda t: t) if pageable else (lambda t: t.pin_memory())
    for e in range(E):
        host[e] = {f"{n}.weight": keep(getattr(blk.experts[e], n).weight.data.cpu()) for n in names}
    if has_shared:
        host["s"] = {f"{n}.weight": keep(getattr(blk.shared_experts, n).weight.data.cpu()) for n in names}
    for L in layers:
        for e in range(E):
            st.add_module(f"routed_expert_{L}_{e}", "routed_expert", host[e], pageable=pageable)
        if has_shared:
            st.add_module(f"shared_expert_{L}", "shared_expert", host["s"], pageable=pageable)
        staged[L] = ([StagedExpert(blk.experts[e], L, e, st, scales_of(blk.experts[e])) for e in range(E)],
                     StagedExpert(blk.shared_experts, L, -1, st, scales_of(blk.shared_experts)) if has_shared else None)
    resident_experts = blk.experts
    resident_shared = blk.shared_experts if has_shared else None
    import torch.nn as nn

    def step(i):
        ex, sh = staged[layers[i % len(layers)]]
        blk.experts = nn.ModuleList(ex)
        if has_shared:
            blk.shared_experts = sh
        return blk(x)

    blk.routing_aware_staging = routing_aware
    st.pump()
    for i in range(len(layers)):
        step(i)
    torch.cuda.synchronize()
    c0, b0 = st.stats()
    t0 = _t.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    dt = _t.perf_counter() - t0
    copies, nbytes = st.stats()
    if routing_aware:
        per_step = (nbytes - b0) / steps           # on-demand copies are issued inside the step they serve
    else:                                          # the cyclic prefetch runs ahead of the timed window
        per_step = nbytes / copies * (E + (1 if has_shared else 0))
    blk.routing_aware_staging = False
    blk.experts = resident_experts
    if has_shared:
        blk.shared_experts = resident_shared
    st.close()
    note = ("only experts with a non-zero token count are staged, busiest first, after the router has run"
            if routing_aware else
            "all expert weights re-staged from ordinary (pageable) host memory every step through 8 pinned chunks of 32 MiB"
            if pageable else
            "all expert weights re-staged from pinned host memory every step (the reference's policy)")
    return {"tokens_per_s": w.n * steps / dt, "ms_per_step": dt * 1e3 / steps,
            "host_to_hbm_gib_per_step": per_step / 2 ** 30, "host_to_hbm_gbps": per_step / (dt / steps) / 1e9,
            "note": note + "; bounded by the host link, not by the kernels"}


def staged_host_run(w, steps: int = 20, pool: int = 0):
    """Host-side cost of the staged path per layer call: a block with the workload's expert count and routing rules
    but small matrices (hidden 512, intermediate 256) and 64 tokens, so that the kernels take next to nothing, its
    experts behind an engine that hands out the RESIDENT weights (no copy, no PCIe) through the wrapper protocol
    with the reference's pool size.  What is timed is the Python / ctypes work of walking the layer in waves:
    get_weights / free_weights_buffer per expert, pointer tables and two grouped launches per wave (plus the one
    read of the per-expert counts, which waits for the router and the dispatch)."""
    import time as _t

    import torch
    import torch.nn as nn
    from moe_gen_amd import StagedExpert, synthetic

    w = w.scaled(n=64, h=512, I=256, seq=64)
    blk = synthetic.build_block(w, device="cuda:0", gen_device="cuda:0")
    names = blk.experts[0].names
    has_shared = bool(w.S) and w.family != "mixtral"
    n_slots = pool if pool > 0 else min(20, 2 * w.E)

    class ResidentEngine:
        stream_ordered_release = True

        def __init__(self):
            self.table = {}

        def pool_size(self, module_type):
            return n_slots if module_type == "routed_expert" else 1

        def get_weights(self, key):
            return self.table[key]

        def free_weights_buffer(self, key):
            pass

        def clear_expert_buffer(self, layer_idx, expert_idx):
            return 0

    eng = ResidentEngine()

    def scales_of(mlp):
        return {f"{n}.weight_scale_inv": getattr(mlp, n).weight_scale_inv.data for n in names} if w.fp8 else None

    L = 3
    staged = []
    for e, ex in enumerate(blk.experts):
        eng.table[f"routed_expert_{L}_{e}"] = {f"{n}.weight": getattr(ex, n).weight.data for n in names}
        staged.append(StagedExpert(ex, L, e, eng, scales_of(ex)))
    sh = None
    if has_shared:
        eng.table[f"shared_expert_{L}"] = {f"{n}.weight": getattr(blk.shared_experts, n).weight.data for n in names}
        sh = StagedExpert(blk.shared_experts, L, -1, eng, scales_of(blk.shared_experts))
    x = synthetic.hidden_states(w, "cuda:0")
    blk.experts = nn.ModuleList(staged)
    if has_shared:
        blk.shared_experts = sh
    for _ in range(3):
        blk(x)
    torch.cuda.synchronize()
    t0 = _t.perf_counter()
    for _ in range(steps):
        blk(x)
    t_host = _t.perf_counter() - t0                 # the calls have returned: everything is enqueued
    torch.cuda.synchronize()
    t_all = _t.perf_counter() - t0
    waves = -(-w.E // max(1, n_slots // 2)) if w.E > n_slots else 1
    return {"host_ms_per_layer": t_host * 1e3 / steps, "wall_ms_per_layer": t_all * 1e3 / steps, "waves_per_layer": waves,
            "pool_slots": n_slots, "tokens": 64, "hidden": w.h, "moe_intermediate": w.I,
            "note": "engine hands out resident weights (no copies), small matrices: Python / ctypes cost of the wave walk per layer call"}


def decoder_half_run(w, blk, x, steps: int):
    """The MLP half of a decoder layer around the block (post-attention RMSNorm, block, residual
    add): the library's fused form (one norm kernel, residual folded into the combine) against
    the same block with the norm and the add as separate passes."""
    import time as _t

    import torch
    from moe_gen_amd import norm_moe_residual, ops
    from moe_gen_amd.block import StageTimer

    ln = torch.ones(w.h, dtype=torch.bfloat16, device=x.device)
    first = lambda r: r[0] if isinstance(r, tuple) else r

    def fused():
        return first(norm_moe_residual(blk, x, ln, 1e-6))

    def separate():
        xn = ops.rmsnorm(x.view(-1, w.h), ln, 1e-6).view_as(x)
        return x + first(blk(xn))

    out = {}
    for name, fn in (("fused", fused), ("separate", separate)):
        fn(); fn()
        torch.cuda.synchronize()
        t0 = _t.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        out[name + "_ms_per_step"] = (_t.perf_counter() - t0) * 1e3 / steps
    def stage_means(fn):
        timer = StageTimer()
        blk.stage_timer = timer
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        blk.stage_timer = None
        return {k: sum(v) / len(v) for k, v in timer.totals_ms().items()}

    st_f, st_p = stage_means(fused), stage_means(lambda: blk(x))
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    xf = x.view(-1, w.h)
    a.record()
    for _ in range(steps):
        ops.rmsnorm(xf, ln, 1e-6)
    b.record()
    torch.cuda.synchronize()
    nh2 = 2.0 * w.n * w.h
    out["rmsnorm_kernel_ms"] = a.elapsed_time(b) / steps
    out["rmsnorm_kernel_gbps"] = 2 * nh2 / (out["rmsnorm_kernel_ms"] * 1e-3) / 1e9     # read x, write the normalised copy
    out["router_ms"] = st_p["router"]
    out["router_through_norm_ms"] = st_f["router"]        # norm folded into the router's read of the rows
    out["combine_ms"] = st_p["combine"]
    out["combine_residual_ms"] = st_f["combine"]
    out["combine_residual_gbps"] = (w.combine_bytes + nh2) / (st_f["combine"] * 1e-3) / 1e9
    return out


def calibrate(w, reps: int = 40):
    """Same-process, same-box yardsticks for the MFMA-bound launches of workload `w`: the vendor library's dense
    bf16 GEMM (torch.matmul) and this library's own grouped kernel on ONE dense group, both on the workload's
    gate/up shape ([rows, h] x [2I, h]^T) and down shape ([rows, I] x [h, I]^T) with rows = min(n k, 65536),
    random operands of the workload's distributions (the chip is power-limited under MFMA load, so operand
    values matter).  Boxes differ by several per cent in sustained clock; ratios against these figures carry over
    from box to box, absolute TFLOP/s do not."""
    import torch
    from moe_gen_amd import ops

    dev = "cuda:0"
    rows, h, inter = min(w.n * w.k, 65536), w.h, w.I
    g = torch.Generator(device=dev).manual_seed(1234)
    rnd = lambda shape, sd: (torch.randn(shape, generator=g, device=dev) * sd).to(torch.bfloat16)
    x, w_gu, w_d, act = rnd((rows, h), 1.0), rnd((2 * inter, h), 0.02), rnd((h, inter), 0.02), rnd((rows, inter), 0.05)
    c1 = torch.empty((rows, 2 * inter), dtype=torch.bfloat16, device=dev)
    c2 = torch.empty((rows, h), dtype=torch.bfloat16, device=dev)
    a2 = torch.empty((rows, inter), dtype=torch.bfloat16, device=dev)
    ptrs = ops.expert_pointers([w_gu[:inter]], [w_gu[inter:]], [w_d])
    off = torch.tensor([0, rows], dtype=torch.int32, device=dev)

    def timed(fn):
        # long enough (40 launches after 5 of warm-up, ~0.1 s) for the clock to settle under the load, as it
        # has in the timed passes of the block
        for _ in range(5):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    f_gu, f_d = 4.0 * rows * inter * h, 2.0 * rows * h * inter
    out = {"vendor_dense_tflops": f_gu / timed(lambda: torch.matmul(x, w_gu.t(), out=c1)) / 1e9,
           "own_dense_bf16_tflops": f_gu / timed(lambda: ops.grouped_swiglu(x, None, ptrs, off, rows, a2, c2, ops.PHASE_GATE_UP)) / 1e9}
    a2.copy_(act)
    out["vendor_dense_down_tflops"] = f_d / timed(lambda: torch.matmul(act, w_d.t(), out=c2)) / 1e9
    out["own_dense_bf16_down_tflops"] = f_d / timed(lambda: ops.grouped_swiglu(x, None, ptrs, off, rows, a2, c2, ops.PHASE_DOWN)) / 1e9
    out["shape"] = {"rows": rows, "gate_up": [rows, 2 * inter, h], "down": [rows, h, inter]}
    out["reps"] = reps
    del x, w_gu, w_d, act, c1, c2, a2
    torch.cuda.empty_cache()
    return out


# HBM traffic per launch of the dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (two runs; FETCH_SIZE scaled by 2.0, the factor a plain copy kernel of known size showed on this
# box, WRITE_SIZE by 1.0).  bench.py cannot run the profiler on itself: these are RECORDED figures,
# copied from the named summary under profiles/, for the workloads that were profiled; None elsewhere.
MEASURED_TRAFFIC = {"deepseek_v3_w8a16": (23.7e9, "profiles/pmc_traffic_deepseek_v3_w8a16_65536.md"),
                    # 3.03 GiB fetched + the 16 MiB of activations written
                    "mixtral_8x22b_decode": (3.27e9, "profiles/pmc_small_workloads_decode_and_v2_lite.md")}


def run_workload(name: str, args, with_cpu: bool):
    import torch
    from moe_gen_amd import synthetic
    from moe_gen_amd.block import StageTimer

    w = synthetic.WORKLOADS[name]
    if args.tokens:
        w = w.scaled(n=args.tokens)
    dev = "cuda:0"
    blk = synthetic.build_block(w, device=dev, gen_device=dev)
    blk.fused_gather = not args.materialize
    blk.join_shared = not args.no_join_shared
    x = synthetic.hidden_states(w, dev)
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        blk(x)
    torch.cuda.synchronize()
    mean_rows = w.n * w.k // w.E
    # which kernels a grouped GEMM call launches follows from the mean rows per expert (grouped_gemm.hip, launch_mt):
    # below 128 the one-workgroup-per-tile kernel alone; else both (on the former, bf16: experts of up to 192 rows;
    # fp8: what an expert's full 256-row tiles leave over, if at most 192 rows; either: the persistent kernel's last
    # round of tiles if it is at most half a round; most rows, and the time, on the latter)
    persistent = mean_rows >= 128 and w.E <= 512 and w.h % 128 == 0
    # yardsticks of this box, taken right before and right after the timed passes (MFMA-bound workloads)
    cal = [calibrate(w)] if persistent and not args.no_calibration else []

    # the timed region: exactly `steps` passes, nothing but the block's own launches on the stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        blk(x)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps
    tokens_per_s = w.n * args.steps / dt

    # the same steps once more with an event pair around every stage, for the per-kernel figures (the events
    # cost a step of a few kernels several per cent -- 0.92 -> 1.01 ms on the 256-token decode workload -- which is
    # why they stay out of the region `value` is taken from; on the headline workload the two agree within 0.1 %)
    timer = StageTimer()
    blk.stage_timer = timer
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        blk(x)
    torch.cuda.synchronize()
    ms_per_step_with_events = (time.perf_counter() - t0) * 1e3 / args.steps
    blk.stage_timer = None
    if cal:
        cal.append(calibrate(w))

    st = {k: sum(v) / len(v) for k, v in timer.totals_ms().items()}
    # dominant kernel: the fused gate/up SwiGLU GEMM.  With shared experts it is launched twice per
    # step (routed experts, shared expert; same kernel, different row counts): algorithmic FLOP per
    # launch and average launch duration are both averages over those launches.
    # (At small token counts the block runs a single shared expert as one more group of the routed call: then the
    # "routed" launches carry its rows too and there are no launches of its own.)
    joined = w.S > 0 and "shared_gate_up" not in st
    gu_flop = [4.0 * w.n * w.k * w.h * w.I + (4.0 * w.n * w.h * w.S * w.I if joined else 0.0)]
    gu_ms = [st["routed_gate_up"]]
    if "shared_gate_up" in st:
        gu_flop.append(4.0 * w.n * w.h * w.S * w.I)
        gu_ms.append(st["shared_gate_up"])
    flop_per_launch = sum(gu_flop) / len(gu_flop)
    ms_per_launch = sum(gu_ms) / len(gu_ms)
    achieved = flop_per_launch / (ms_per_launch * 1e-3) / 1e12
    gemm_ms = sum(st.get(k, 0.0) for k in ("routed_gate_up", "routed_down", "shared_gate_up", "shared_down"))
    gemm_tflops = (w.routed_flop + w.shared_flop) / (gemm_ms * 1e-3) / 1e12
    disp_bytes = w.dispatch_bytes if args.materialize else 4.0 * w.n * w.k
    pair = persistent
    wbytes = 3.0 * w.E * w.h * w.I * (1 if w.fp8 else 2)
    w8 = "true" if w.fp8 else "false"
    if persistent:
        roofline = {"bound": "mfma",
                    "kernel": f"grouped_gemm_persistent_kernel<SWIGLU=true,W8={w8}> (gate/up + SiLU*mul)"
                              + (f" + grouped_gemm_kernel<WN=4,SWIGLU=true,W8={w8}> for the "
                                 + ("rows past an expert's full 256-row tiles" if w.fp8 else "experts of one small tile")
                                 + " and a short last round of the persistent kernel: a call is this pair of launches, timed as one"
                                 if pair else ""),
                    "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / PEAK_BF16_TFLOPS, "traffic": MEASURED_TRAFFIC.get(name, (None, None))[0],
                    "traffic_source": (f"recorded from {MEASURED_TRAFFIC[name][1]} (rocprofv3 --pmc), not measured by this run"
                                       if name in MEASURED_TRAFFIC else None),
                    "frac_of_fp8_peak": achieved / PEAK_FP8_TFLOPS,
                    "launches_per_step": len(gu_ms), "avg_launch_ms": ms_per_launch,
                    "flop_per_launch": flop_per_launch}
        if cal:
            keys = ("vendor_dense_tflops", "own_dense_bf16_tflops", "vendor_dense_down_tflops", "own_dense_bf16_down_tflops")
            mean = {k: sum(c[k] for c in cal) / len(cal) for k in keys}
            rows = w.n * w.k + (w.n * w.S if joined else 0)
            routed_gu = 4.0 * rows * w.h * w.I / (st["routed_gate_up"] * 1e-3) / 1e12
            routed_dn = 2.0 * rows * w.h * w.I / (st["routed_down"] * 1e-3) / 1e12
            roofline["calibration"] = {**mean, "before_timed_passes": {k: cal[0][k] for k in keys},
                                       "after_timed_passes": {k: cal[1][k] for k in keys}, "shape": cal[0]["shape"],
                                       "reps": cal[0]["reps"],
                                       "what": "same process, same box: vendor library dense bf16 GEMM (torch.matmul) and this "
                                               "library's grouped kernel on one dense bf16 group, gate/up and down shapes of "
                                               "this workload, random operands; means of the runs before and after the timed passes"}
            # the dominant call (all its launches, routed and shared) against the vendor's dense GEMM of the same shape
            roofline["frac_of_vendor_dense"] = achieved / mean["vendor_dense_tflops"]
            roofline["own_dense_bf16_frac_of_vendor_dense"] = mean["own_dense_bf16_tflops"] / mean["vendor_dense_tflops"]
            roofline["routed_gate_up"] = {"tflops": routed_gu, "frac_of_vendor_dense": routed_gu / mean["vendor_dense_tflops"]}
            roofline["routed_down"] = {"tflops": routed_dn, "frac_of_vendor_dense": routed_dn / mean["vendor_dense_down_tflops"]}
    else:
        # few rows per expert: the launch streams every expert's gate and up matrix once and is bound by HBM.
        # Algorithmic bytes per launch: both matrices of every expert, the gathered token rows, the activations out.
        gu_bytes = 2.0 * w.E * w.h * w.I * (1 if w.fp8 else 2) + 2.0 * w.n * w.k * (w.h + w.I)
        if joined:                                   # (+ the shared expert's matrices, rows and activations)
            gu_bytes += 2.0 * w.S * w.h * w.I * (1 if w.fp8 else 2) + 2.0 * w.n * (w.h + w.S * w.I)
        gbps = gu_bytes / (st["routed_gate_up"] * 1e-3) / 1e9
        roofline = {"bound": "hbm",
                    "kernel": f"grouped_gemm_kernel<WN=4,SWIGLU=true,W8={w8}> (gate/up + SiLU*mul, one workgroup per tile)",
                    "achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": gbps / PEAK_HBM_GBPS,
                    "traffic": MEASURED_TRAFFIC.get(name, (None, None))[0],
                    "traffic_source": (f"recorded from {MEASURED_TRAFFIC[name][1]} (rocprofv3 --pmc), not measured by this run"
                                       if name in MEASURED_TRAFFIC else None),
                    "launches_per_step": 1, "avg_launch_ms": st["routed_gate_up"],
                    "bytes_per_launch": gu_bytes, "tflops": achieved}
    result = {
        "metric": "MoE-layer tokens/sec at DeepSeek-V3 W8A16 shape" if name == "deepseek_v3_w8a16"
                  else f"MoE-layer tokens/sec ({name})",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_with_stage_events": ms_per_step_with_events, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w.name, "tokens": w.n, "hidden": w.h, "experts": w.E, "top_k": w.k,
                   "moe_intermediate": w.I, "shared_experts": w.S,
                   "weights": "fp8-e4m3fn + 128x128 fp32 scales, dequantised to bf16 ahead of MFMA" if w.fp8 else "bf16",
                   "gather": "materialized" if args.materialize else "fused into the GEMM A-operand load"},
        "roofline": roofline,
        "pct_mfma_peak": {"all_expert_gemms_tflops": gemm_tflops, "of_bf16_peak": gemm_tflops / PEAK_BF16_TFLOPS,
                          "of_fp8_peak": gemm_tflops / PEAK_FP8_TFLOPS,
                          "weight_stream_gbps": wbytes / (gemm_ms * 1e-3) / 1e9},
        "routing_gbps": {"router": w.router_bytes / (st["router"] * 1e-3) / 1e9,
                         "dispatch": disp_bytes / (st["dispatch"] * 1e-3) / 1e9,
                         "combine": w.combine_bytes / (st["combine"] * 1e-3) / 1e9,
                         "of_hbm_peak": {"router": w.router_bytes / (st["router"] * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                                         "combine": w.combine_bytes / (st["combine"] * 1e-3) / 1e9 / PEAK_HBM_GBPS}},
        "stage_ms": st,
    }
    if args.decoder_half:
        result["decoder_half"] = decoder_half_run(w, blk, x, args.steps)
    if args.staged:
        result["staged"] = staged_run(w, blk, x, max(2, args.steps // 2), pool=args.staged_pool)
        result["staged_routing_aware"] = staged_run(w, blk, x, max(2, args.steps // 2), routing_aware=True, pool=args.staged_pool)
        result["staged_from_pageable_memory"] = staged_run(w, blk, x, max(2, args.steps // 2), pool=args.staged_pool, pageable=True)
        result["staged"]["pool_slots"] = result["staged_routing_aware"]["pool_slots"] = args.staged_pool or min(20, 2 * w.E)
        result["staged_host"] = staged_host_run(w, pool=args.staged_pool)
    if with_cpu:
        # full size where the workload is small (DeepSeek-V2-Lite 4096 tokens, the 256-token decode case),
        # a bounded sample of the first tokens elsewhere
        result["cpu_baseline"] = cpu_baseline(w, blk, w.n if w.n <= 4096 else min(args.cpu_sample, w.n))
    del blk, x
    torch.cuda.empty_cache()
    return result


def ceiling_run(args):
    """What this box leaves to ANY bf16 GEMM of the headline shapes, next to the grouped kernel's own
    dense (one-group) launch: (1) the registers-only MFMA loop of moe_gen_amd/csrc/probes/mfma_rate.hip,
    (2) the vendor library's dense bf16 GEMM (torch.matmul) and (3) the library's grouped SwiGLU
    kernels on one group of the same shape -- each with random and with all-zero operands.  The gap
    between zero and random operands is data-dependent power, paid in clock."""
    import subprocess

    probe = os.path.join(ROOT, "moe_gen_amd", "csrc", "build", "mfma_rate")
    if not os.path.exists(probe):
        sys.exit(f"{probe} is missing: build it with `make -C moe_gen_amd/csrc probes`")
    res = {"metric": "bf16 MFMA ceiling probes (DeepSeek-V3 MoE shapes)", "unit": "TFLOP/s", "peak": PEAK_BF16_TFLOPS}
    # (1) started as a child before this process touches the GPU
    txt = subprocess.run([probe, "10000"], check=True, capture_output=True, text=True, timeout=300).stdout
    regs = {}
    for line in txt.splitlines():
        f = line.split()
        if len(f) == 6 and f[0].startswith("mfma_"):
            regs.setdefault(f"{f[0]}/{f[1]}", []).append(float(f[4]))
    res["registers_only_mfma"] = {k: max(v) for k, v in regs.items()}

    import torch
    from moe_gen_amd import ops
    torch.cuda.set_device(0)
    dev = "cuda:0"
    n, h, inter = 65536, 7168, 2048
    reps = args.steps

    def timed(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    g = torch.Generator(device=dev).manual_seed(0)

    def tensor(shape, scale, zero):
        if zero:
            return torch.zeros(shape, dtype=torch.bfloat16, device=dev)
        return (torch.randn(shape, generator=g, device=dev) * scale).to(torch.bfloat16)

    vendor, ours = {}, {}
    for zero in (False, True):
        tag = "zero" if zero else "random"
        x = tensor((n, h), 1.0, zero)
        w_gu = tensor((2 * inter, h), 0.02, zero)             # gate and up as one dense matrix
        w_d = tensor((h, inter), 0.02, zero)
        act = tensor((n, inter), 0.05, zero)
        c1 = torch.empty((n, 2 * inter), dtype=torch.bfloat16, device=dev)
        c2 = torch.empty((n, h), dtype=torch.bfloat16, device=dev)
        ms = timed(lambda: torch.matmul(x, w_gu.t(), out=c1))
        vendor[f"gate_up_{n}x{2 * inter}x{h}/{tag}"] = 2.0 * n * 2 * inter * h / ms / 1e9
        ms = timed(lambda: torch.matmul(act, w_d.t(), out=c2))
        vendor[f"down_{n}x{h}x{inter}/{tag}"] = 2.0 * n * h * inter / ms / 1e9
        del c1
        ptrs = ops.expert_pointers([w_gu[:inter]], [w_gu[inter:]], [w_d])
        off = torch.tensor([0, n], dtype=torch.int32, device=dev)
        a2 = torch.empty((n, inter), dtype=torch.bfloat16, device=dev)
        ms = timed(lambda: ops.grouped_swiglu(x, None, ptrs, off, n, a2, c2, ops.PHASE_GATE_UP))
        ours[f"gate_up_swiglu_bf16/{tag}"] = 4.0 * n * inter * h / ms / 1e9
        a2.copy_(act)
        ms = timed(lambda: ops.grouped_swiglu(x, None, ptrs, off, n, a2, c2, ops.PHASE_DOWN))
        ours[f"down_bf16/{tag}"] = 2.0 * n * h * inter / ms / 1e9
        if not zero:                                          # the W8A16 path on the same shape
            q = [torch.randint(0, 120, s, generator=g, device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn)
                 for s in ((inter, h), (inter, h), (h, inter))]
            sc = [torch.full((-(-s[0] // 128), -(-s[1] // 128)), 1e-3, device=dev) for s in ((inter, h), (inter, h), (h, inter))]
            p8 = ops.expert_pointers([q[0]], [q[1]], [q[2]], [sc[0]], [sc[1]], [sc[2]])
            ms = timed(lambda: ops.grouped_swiglu(x, None, p8, off, n, a2, c2, ops.PHASE_GATE_UP))
            ours["gate_up_swiglu_w8a16/random"] = 4.0 * n * inter * h / ms / 1e9
            a2.copy_(act)
            ms = timed(lambda: ops.grouped_swiglu(x, None, p8, off, n, a2, c2, ops.PHASE_DOWN))
            ours["down_w8a16/random"] = 2.0 * n * h * inter / ms / 1e9
        del x, w_gu, w_d, act, c2, a2
        torch.cuda.empty_cache()
    res["vendor_dense_bf16_gemm"] = vendor
    res["grouped_kernel_one_group"] = ours
    res["device"] = torch.cuda.get_device_name(0)
    res["reps"] = reps
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="deepseek_v3_w8a16")
    ap.add_argument("--all-workloads", action="store_true", help="(default) every synthetic workload in the one JSON line")
    ap.add_argument("--headline-only", action="store_true", help="only the workload named by --workload")
    ap.add_argument("--tokens", type=int, default=0, help="override the token count (parity/debug only)")
    ap.add_argument("--no-join-shared", action="store_true", help="keep a single shared expert in a grouped call of "
                    "its own at every token count (by default it joins the routed call at small batches)")
    ap.add_argument("--materialize", action="store_true", help="gather rows into a sorted copy instead of "
                    "reading them through the row map inside the GEMM")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-calibration", action="store_true", help="skip the vendor-dense / own-dense GEMM yardsticks")
    ap.add_argument("--staged", action="store_true", help="also time the block with weights staged from pinned host memory")
    ap.add_argument("--staged-pool", type=int, default=0, help="routed-expert slots of the staging pool (default 20, the reference engine's prefill default)")
    ap.add_argument("--staged-host", action="store_true", help="only the host-side cost of the staged path per layer call")
    ap.add_argument("--decoder-half", action="store_true", help="also time RMSNorm + block + residual add, fused and separate")
    ap.add_argument("--cpu-sample", type=int, default=1024, help="tokens of the workload the CPU baseline runs")
    ap.add_argument("--ceiling", action="store_true", help="instead of the benchmark: registers-only MFMA rate, vendor dense "
                    "bf16 GEMM and this library's one-group launch at the headline shapes, random and zero operands")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1")
    if args.ceiling:
        return ceiling_run(args)

    import torch
    from moe_gen_amd import synthetic
    torch.cuda.set_device(0)
    result = run_workload(args.workload, args, not args.no_cpu_baseline)
    if not args.headline_only and args.workload == "deepseek_v3_w8a16" and not args.tokens:
        # the other synthetic configurations: same steps / warm-up, each timed on its own
        extra = argparse.Namespace(**{**vars(args), "staged": False, "decoder_half": False})
        result["workloads"] = [run_workload(n, extra, not args.no_cpu_baseline)
                               for n in synthetic.WORKLOADS if n != args.workload]
    print(json.dumps(result))


if __name__ == "__main__":
    main()
