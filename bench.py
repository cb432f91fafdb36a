"""MoE-layer benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

A step is one forward of the MoE block (router -> dispatch -> grouped SwiGLU experts -> shared
expert -> combine) over one batch of synthetic hidden states already resident in HBM, weights
resident.  Prints ONE JSON line.  Per-stage durations come from events recorded on the launch
stream inside the timed steps.
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


def cpu_baseline(w, blk, n_sample: int):
    """The reference's own algorithm (oracle/torch_blocks.py: fp32 gate, Python loop over experts,
    bf16 F.linear, per-call fp8 block dequantisation) timed on the host cores on a bounded sample
    of the same workload: the first n_sample tokens, same weights, same router."""
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

    t0 = time.perf_counter()
    run()
    dt = time.perf_counter() - t0
    return {"value": n_sample / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"first {n_sample} of {w.n} tokens of the same workload, all experts' weights, one pass "
                      f"({dt:.1f} s); stock-PyTorch CPU restatement of the reference block"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="deepseek_v3_w8a16")
    ap.add_argument("--tokens", type=int, default=0, help="override the token count (parity/debug only)")
    ap.add_argument("--materialize", action="store_true", help="gather rows into a sorted copy instead of "
                    "reading them through the row map inside the GEMM")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample", type=int, default=128)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1")

    import torch
    from moe_gen_amd import synthetic
    from moe_gen_amd.block import StageTimer

    w = synthetic.WORKLOADS[args.workload]
    if args.tokens:
        w = w.scaled(n=args.tokens)
    dev = "cuda:0"
    torch.cuda.set_device(0)
    blk = synthetic.build_block(w, device=dev, gen_device=dev)
    blk.fused_gather = not args.materialize
    x = synthetic.hidden_states(w, dev)
    torch.cuda.synchronize()

    for _ in range(args.warmup):
        blk(x)
    torch.cuda.synchronize()

    timer = StageTimer()
    blk.stage_timer = timer
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        blk(x)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    blk.stage_timer = None
    ms_per_step = dt * 1e3 / args.steps
    tokens_per_s = w.n * args.steps / dt

    st = {k: sum(v) / len(v) for k, v in timer.totals_ms().items()}
    # dominant kernel: the fused gate/up SwiGLU GEMM.  It is launched once for the routed experts
    # and once for the shared expert per step (same kernel, different row counts): algorithmic FLOP
    # per launch and average launch duration are both averages over those launches.
    gu_flop = [4.0 * w.n * w.k * w.h * w.I]
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
    result = {
        "metric": "MoE-layer tokens/sec at DeepSeek-V3 W8A16 shape" if args.workload == "deepseek_v3_w8a16"
                  else f"MoE-layer tokens/sec ({args.workload})",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": w.name, "tokens": w.n, "hidden": w.h, "experts": w.E, "top_k": w.k,
                   "moe_intermediate": w.I, "shared_experts": w.S, "weights": "fp8-e4m3fn+128x128 fp32 scales" if w.fp8 else "bf16",
                   "gather": "materialized" if args.materialize else "fused into the GEMM A-operand load"},
        "roofline": {"bound": "mfma", "kernel": "grouped_gemm_kernel<MT=4,SWIGLU,W8> (gate/up + SiLU*mul)",
                     "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None,
                     "frac_of_fp8_peak": achieved / PEAK_FP8_TFLOPS,
                     "launches_per_step": len(gu_ms), "avg_launch_ms": ms_per_launch},
        "pct_mfma_peak": {"all_expert_gemms_tflops": gemm_tflops, "of_bf16_peak": gemm_tflops / PEAK_BF16_TFLOPS,
                          "of_fp8_peak": gemm_tflops / PEAK_FP8_TFLOPS},
        "routing_gbps": {"router": w.router_bytes / (st["router"] * 1e-3) / 1e9,
                         "dispatch": disp_bytes / (st["dispatch"] * 1e-3) / 1e9,
                         "combine": w.combine_bytes / (st["combine"] * 1e-3) / 1e9,
                         "of_hbm_peak": {"router": w.router_bytes / (st["router"] * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                                         "combine": w.combine_bytes / (st["combine"] * 1e-3) / 1e9 / PEAK_HBM_GBPS}},
        "stage_ms": st,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, blk, min(args.cpu_sample, w.n))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
