"""Benchmark of the Muon optimizer step on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` times K full Muon steps (momentum, Newton-Schulz,
scaling, decay, update) over a Qwen3-8B-shaped 2-D parameter set (36 layers; q,o 4096x4096;
k,v 1024x4096; gate,up 12288x4096; down 4096x12288; bf16 params and grads, fp32 momentum;
lr 0.02, momentum 0.95 Nesterov, wd 0.01, 5 NS steps) with everything resident in HBM, and
prints ONE JSON line.  `value` is the algorithmic Newton-Schulz FLOPs of one step,
steps*(3 M^2 K + M^3) per matrix, divided by the whole step time.

The `roofline` object is for the dominant kernel (the B.X GEMM with the a.X epilogue): its
algorithmic FLOPs per launch over its mean launch time, measured with HIP events recorded
around every launch inside the timed region, against the dense bf16 MFMA peak.
`cpu_baseline` times the CPU oracle (a torch restatement of the reference step, test
infrastructure) on one matrix per shape bucket and scales by the bucket counts.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "Muon step ms + NS TFLOP/s (% bf16 MFMA peak), Qwen3-8B param set, 1 GPU"
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
# Mean HBM-side bytes (L2 misses plus write-backs) of one B.X launch in a full step of each workload:
# rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE over this script, each scaled by what the same counter
# reads for the 1 GiB copy of --calibrate-copy (one FETCH_SIZE unit = 2 KiB, one WRITE_SIZE unit = 1 KiB).
# A counter run cannot share a process with the event timing, so the figure is carried here.
BX_TRAFFIC_BYTES_PER_LAUNCH = {"qwen3-8b": 23.455e9 + 3.473e9}

WORKLOADS = {
    "qwen3-8b": dict(layers=36, shapes=dict(q=(4096, 4096), k=(1024, 4096), v=(1024, 4096), o=(4096, 4096),
                                            gate=(12288, 4096), up=(12288, 4096), down=(4096, 12288)),
                     pdtype="bf16", mdtype="f32"),
    "qwen2.5-0.5b": dict(layers=24, shapes=dict(q=(896, 896), k=(128, 896), v=(128, 896), o=(896, 896),
                                                gate=(4864, 896), up=(4864, 896), down=(896, 4864)),
                         pdtype="f32", mdtype="f32"),
    "qwen3-moe-30b-a3b": dict(layers=48, experts=128,
                              shapes=dict(q=(4096, 2048), k=(512, 2048), v=(512, 2048), o=(2048, 4096)),
                              expert_shapes=dict(gate=(768, 2048), up=(768, 2048), down=(2048, 768)),
                              pdtype="bf16", mdtype="f32"),
    # single large matrices: the per-kernel MFMA utilisation sweep
    "square-8192": dict(layers=1, shapes=dict(w=(8192, 8192)), pdtype="bf16", mdtype="f32"),
    "llama70b-mlp-28672x8192": dict(layers=1, shapes=dict(w=(28672, 8192)), pdtype="bf16", mdtype="f32"),
}
HP = dict(lr=0.02, momentum=0.95, nesterov=True, weight_decay=0.01, ns_steps=5, rms_scale=False)


def ns_flops(rows, cols, steps):
    M, K = min(rows, cols), max(rows, cols)
    return steps * (3.0 * M * M * K + 1.0 * M ** 3)


def matrix_list(w, layers):
    out = []
    for _ in range(layers):
        for name, s in w["shapes"].items():
            out.append(s)
        for name, s in w.get("expert_shapes", {}).items():
            out.extend([s] * w["experts"])
    return out


def cpu_baseline(w, layers, target_flops_per_step):
    """The CPU oracle on one matrix per shape bucket, scaled by the bucket counts."""
    import torch

    from oracle import muon_oracle as O

    torch.set_num_threads(max(1, min(16, os.cpu_count() or 1)))
    counts = {}
    for s in matrix_list(w, layers):
        counts[s] = counts.get(s, 0) + 1
    pd = torch.bfloat16 if w["pdtype"] == "bf16" else torch.float32
    total_s, sample = 0.0, []
    gen = torch.Generator().manual_seed(1)
    budget_s = 45.0
    t_begin = time.perf_counter()
    for s, cnt in sorted(counts.items(), key=lambda kv: ns_flops(*kv[0], 5)):
        if time.perf_counter() - t_begin > budget_s:
            # scale the largest measured bucket by FLOPs instead of running past the budget
            ref_s, ref_t = sample[-1]
            total_s += cnt * ref_t * ns_flops(*s, 5) / ns_flops(*ref_s, 5)
            continue
        p = (0.02 * torch.randn(*s, generator=gen)).to(pd)
        g = (1e-3 * torch.randn(*s, generator=gen)).to(pd)
        m = torch.zeros(*s, dtype=torch.float32)
        t0 = time.perf_counter()
        O.muon_step_matrix(p, g, m, lr=HP["lr"], weight_decay=HP["weight_decay"], beta=HP["momentum"],
                           nesterov=True, ns_steps=HP["ns_steps"], rms_scale=False)
        dt = time.perf_counter() - t0
        sample.append((s, dt))
        total_s += cnt * dt
    return {
        "value": target_flops_per_step / total_s / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "step_s_extrapolated": total_s,
        "sample": "one full Muon step of the torch CPU oracle per (rows, cols) bucket "
                  + ", ".join(f"{s[0]}x{s[1]}:{dt:.2f}s" for s, dt in sample)
                  + "; scaled by bucket counts (and by FLOPs for buckets past the time budget)",
    }


def extras(params, pd, dev, reps):
    """Gradient clipping over the Muon gradients and the AdamW fallback over a Qwen3-8B-shaped non-Muon group
    (embedding and lm_head 151936x4096, 73 norm vectors), each as achieved HBM bytes per second."""
    import torch

    from lmms_engine_amd import _abi
    from lmms_engine_amd.clip_grad import clip_grad_norm_
    from lmms_engine_amd.muon_utils import Muon

    gb = 2 if pd == torch.bfloat16 else 4
    shapes = [(151936, 4096), (151936, 4096)] + [(4096,)] * 73
    fb = [torch.nn.Parameter(torch.zeros(*s, dtype=pd, device=dev)) for s in shapes]
    for p in fb:
        p.grad = torch.full_like(p, 1e-3)
    opt = Muon([dict(params=fb, use_muon=False, lr=1e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.01)])
    opt.step()
    clip_grad_norm_(params, 1.0)
    torch.cuda.synchronize()
    _abi.timing_enable(True)
    for _ in range(reps):
        clip_grad_norm_(params, 1.0)
        opt.step()
    torch.cuda.synchronize()
    t = _abi.timing_read()
    _abi.timing_enable(False)
    n_muon = sum(p.numel() for p in params)
    n_fb = sum(p.numel() for p in fb)
    res = {}
    for name, nbytes in (("grad_norm", n_muon * gb), ("clip_scale", n_muon * 2 * gb), ("adamw_multi", n_fb * 7 * gb)):
        ms, cnt = t[name]
        if cnt:
            per = ms / reps
            res[name] = dict(ms_per_call=per, launches_per_call=cnt / reps, gbs=nbytes / (per * 1e-3) / 1e9,
                             frac_hbm_peak=nbytes / (per * 1e-3) / 1e9 / PEAK_HBM_GBS)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="qwen3-8b", choices=sorted(WORKLOADS))
    ap.add_argument("--layers", type=int, default=0, help="override the layer count (0 = the workload's own)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--workspace-limit-gib", type=float, default=0.0,
                    help="cap of the Newton-Schulz workspace (0 = the optimizer's default); smaller caps mean more, "
                         "smaller grouped launches")
    ap.add_argument("--extras", action="store_true",
                    help="also time the two neighbours of the Muon step, outside the timed region: gradient-norm clipping "
                         "over the same gradients and the AdamW fallback over an embedding + lm_head + norm-vector group")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device copy (a kernel of known traffic) so that FETCH_SIZE / WRITE_SIZE "
                         "readings of a rocprofv3 --pmc run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the Muon step on ONE GPU (no sharding, no collectives); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from lmms_engine_amd import _abi
    from lmms_engine_amd.muon_utils import Muon

    if not os.path.exists(_abi.LIB_PATH):
        from lmms_engine_amd.build import build_library

        build_library()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    w = WORKLOADS[args.workload]
    layers = args.layers or w["layers"]
    shapes = matrix_list(w, layers)
    pd = torch.bfloat16 if w["pdtype"] == "bf16" else torch.float32
    md = torch.float32 if w["mdtype"] == "f32" else None

    gen = torch.Generator(device=dev).manual_seed(1)
    params = []
    for s in shapes:
        params.append(torch.nn.Parameter((0.02 * torch.randn(*s, device=dev, generator=gen)).to(pd)))
    for p in params:
        p.grad = (1e-3 * torch.randn(*p.shape, device=dev, generator=gen)).to(pd)
    extra = dict(workspace_limit_bytes=int(args.workspace_limit_gib * (1 << 30))) if args.workspace_limit_gib > 0 else {}
    opt = Muon([dict(params=list(params), use_muon=True, **HP)], momentum_dtype=md if pd != torch.float32 else None, **extra)

    flops_step = sum(ns_flops(*s, HP["ns_steps"]) for s in shapes)
    elements = sum(s[0] * s[1] for s in shapes)

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        opt.step()
    torch.cuda.synchronize()
    if not args.no_kernel_timing:
        _abi.timing_enable(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        opt.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_step = dt / args.steps * 1e3
    kern = {}
    if not args.no_kernel_timing:
        kern = _abi.timing_read()
        _abi.timing_enable(False)

    # per-kernel algorithmic work of one step
    syrk_f = sum(HP["ns_steps"] * float(min(s)) ** 2 * max(s) for s in shapes)
    symp_f = sum(HP["ns_steps"] * float(min(s)) ** 3 for s in shapes)
    bx_f = 2.0 * syrk_f
    gb = 2 if pd == torch.bfloat16 else 4
    mom_bytes = elements * (gb + 2 * 4 + 2) if md == torch.float32 or pd == torch.float32 else elements * (3 * gb + 2)
    work = {"syrk": (syrk_f, "flop"), "sympoly": (symp_f, "flop"), "bx_axpy": (bx_f, "flop"),
            "momentum_norm": (mom_bytes, "byte"), "normalize": (elements * 4, "byte"),
            "apply_update": (elements * (2 + 2 * gb), "byte")}
    kernels = {}
    for name, (tot_ms, cnt) in kern.items():
        if cnt == 0 or name not in work:
            continue
        amount, kind = work[name]
        per_step_ms = tot_ms / args.steps
        rate = amount / (per_step_ms * 1e-3)
        if kind == "flop":
            kernels[name] = dict(ms_per_step=per_step_ms, launches_per_step=cnt / args.steps, tflops=rate / 1e12,
                                 frac_mfma_peak=rate / 1e12 / PEAK_BF16_TFLOPS)
        else:
            kernels[name] = dict(ms_per_step=per_step_ms, launches_per_step=cnt / args.steps, gbs=rate / 1e9,
                                 frac_hbm_peak=rate / 1e9 / PEAK_HBM_GBS)

    roofline = None
    if "bx_axpy" in kernels:
        tot_ms, cnt = kern["bx_axpy"]
        achieved = bx_f * args.steps / (tot_ms * 1e-3) / 1e12
        roofline = {"kernel": "gemm_nt_pp_kernel<256, 256, 2, 4, EPI_BX> (X' = a.X + B.X)", "bound": "mfma", "achieved": achieved,
                    "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                    "traffic": BX_TRAFFIC_BYTES_PER_LAUNCH.get(args.workload) if layers == w["layers"] else None,
                    "launches": cnt, "avg_launch_ms": tot_ms / cnt,
                    "algorithmic_flop_per_launch": bx_f * args.steps / cnt}
    gemm_ms = sum(kernels[k]["ms_per_step"] for k in ("syrk", "sympoly", "bx_axpy") if k in kernels)

    out = {
        "metric": METRIC,
        "value": flops_step / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{args.workload} 2-D parameter set, {layers} layers, {len(shapes)} matrices, "
                               f"{w['pdtype']} params/grads, fp32 momentum, full Muon step",
                   "elements": elements, "ns_steps": HP["ns_steps"], "grouped_buckets": len(set(shapes))},
        "ns_flop_per_step_algorithmic": flops_step,
        "pct_bf16_mfma_peak_whole_step": 100.0 * flops_step / (ms_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "ns_tflops_gemm_kernels_only": (flops_step / (gemm_ms * 1e-3) / 1e12) if gemm_ms else None,
        "kernels": kernels,
        "roofline": roofline,
    }
    if args.extras:
        out["extras"] = extras(params, pd, dev, args.steps)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, layers, flops_step)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
