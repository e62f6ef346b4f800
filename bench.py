"""Benchmark of the Muon optimizer step on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` times K full Muon steps (momentum, Newton-Schulz,
scaling, decay, update) over a Qwen3-8B-shaped 2-D parameter set (36 layers; q,o 4096x4096;
k,v 1024x4096; gate,up 12288x4096; down 4096x12288; bf16 params and grads, fp32 momentum;
lr 0.02, momentum 0.95 Nesterov, wd 0.01, 5 NS steps) with everything resident in HBM, and
prints ONE JSON line.  `value` is the algorithmic Newton-Schulz FLOPs of one step,
steps*(3 M^2 K + M^3) per matrix, divided by the whole step time.

The `roofline` object is for the dominant kernel (the persistent B.X GEMM with the a.X epilogue,
two fifths of the step): its algorithmic FLOPs per launch over its mean launch time, measured with
HIP events recorded around every launch inside the timed region, against the dense bf16 MFMA peak.
The one B.X launch in five that carries the parameter update is another kernel and has its own
entry under `kernels`.
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
# Mean HBM-side bytes (L2 misses plus write-backs) of one B.X launch in a full step: rocprofv3 --pmc FETCH_SIZE
# and --pmc WRITE_SIZE over this script, each scaled by what the same counter reads for the 1 GiB copy of
# --calibrate-copy.  A counter run cannot share a process with the event timing, so the figure lives in the
# tracked summary of that run, on a line
#   roofline.traffic workload=<name> bytes_per_launch=<float> gemm_nt_hip_blob=<git blob hash of gemm_nt.hip>
# and is reported only while the GEMM source is still the one it was measured on.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "muon_step_qwen3_8b_hbm_traffic.txt")
GEMM_SOURCE = os.path.join(ROOT, "lmms_engine_amd", "csrc", "gemm_nt.hip")


def git_blob_hash(path):
    """What `git hash-object` prints for the file."""
    import hashlib

    data = open(path, "rb").read()
    return hashlib.sha1(b"blob %d\0" % len(data) + data).hexdigest()


def recorded_traffic(workload):
    """bytes per launch of the persistent B.X kernel from the tracked counter summary, or None when absent or measured on other code."""
    try:
        cur = git_blob_hash(GEMM_SOURCE)
        for line in open(TRAFFIC_SUMMARY):
            if not line.lstrip("# ").startswith("roofline.traffic "):
                continue
            kv = dict(tok.split("=", 1) for tok in line.split()[1:] if "=" in tok)
            if kv.get("workload") == workload and kv.get("gemm_nt_hip_blob") == cur:
                return float(kv["bytes_per_launch"])
    except (OSError, ValueError, KeyError):
        pass
    return None

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

    # the GPU box gives one job 16 host cores, whatever os.cpu_count() shows there: the cap is the whole share
    torch.set_num_threads(max(1, min(16, os.cpu_count() or 1)))
    cpu_model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                cpu_model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
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
        "cpu_model": cpu_model,
        "host_cores_visible": os.cpu_count(),
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


def hbm_reference(dev, gib=2, reps=10):
    """What torch's own streaming kernels reach on this box, as bytes moved per second: a read-only reduction, an
    in-place multiply (one read and one write per element, the mix of the momentum kernel) and a copy (the mix of the
    normalisation).  The elementwise kernels of the step are to be read against these as well as against the 8 TB/s."""
    import torch

    n = gib << 28  # fp32 elements
    a = torch.empty(n, dtype=torch.float32, device=dev).normal_()
    b = torch.empty_like(a)
    nbytes = 4.0 * n
    res = {}
    for name, fn, moved in (("read_only_norm", lambda: torch.linalg.vector_norm(a), nbytes), ("in_place_multiply", lambda: a.mul_(1.0000001), 2 * nbytes),
                            ("copy", lambda: b.copy_(a), 2 * nbytes)):
        ms = _event_ms(fn, reps, torch, warm=2)
        res[name] = dict(gbs=moved / (ms * 1e-3) / 1e9, frac_hbm_peak=moved / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS)
    res["what"] = f"torch kernels over {gib} GiB fp32 buffers, {reps} calls each"
    return res


def _event_ms(fn, reps, torch, warm=1):
    """Mean milliseconds of fn() over `reps` calls after `warm` warm-up calls, from events on the current stream."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def gpu_oracle(params, moms, shapes, flops_step, reps=2):
    """The second baseline: the reference's own torch expressions (muon_utils.py:138-156, :188-189, :324-325) run
    unfused on the same GPU, one parameter at a time, with torch's bf16 matmul (hipBLASLt) for every product,
    X @ X.mT standing in for the Triton kernel.  Also the library GEMM alone on the shapes of the dominant kernel:
    B (M x M) @ X (M x K) in bf16, as dense TFLOP/s, to set beside the B.X kernel's figure."""
    import torch

    a, b, c = 3.4445, -4.7750, 2.0315
    beta, lr, wd, steps = HP["momentum"], HP["lr"], HP["weight_decay"], HP["ns_steps"]

    def one(p, m):
        g = p.grad if p.grad.dtype == m.dtype else p.grad.to(m.dtype)
        m.lerp_(g, 1 - beta)
        u = g.lerp(m, beta)
        X = u.bfloat16()
        if p.shape[0] > p.shape[1]:
            X = X.mT
        X = X / (X.norm(dim=(-2, -1), keepdim=True) + 1e-7)
        for _ in range(steps):
            A = X @ X.mT
            A2 = A @ A.mT
            B = b * A + c * A2
            X = a * X + B @ X
        if p.shape[0] > p.shape[1]:
            X = X.mT
        X = X * max(1, p.shape[0] / p.shape[1]) ** 0.5
        p.mul_(1 - lr * wd)
        p.add_(X.reshape(p.shape), alpha=-lr)

    def step():
        with torch.no_grad():
            for p, m in zip(params, moms):
                one(p, m)

    ms = _event_ms(step, reps, torch)
    dense = sum(HP["ns_steps"] * (4.0 * min(s) ** 2 * max(s) + 2.0 * min(s) ** 3) for s in shapes)
    out = {"what": "reference expressions unfused in torch on this GPU (hipBLASLt bf16 matmuls, dense products)",
           "ms_per_step": ms, "ns_tflops_algorithmic": flops_step / (ms * 1e-3) / 1e12,
           "ns_tflops_dense_executed": dense / (ms * 1e-3) / 1e12}
    dev = params[0].device
    lib_gemm = {}
    tot_f, tot_t = 0.0, 0.0
    counts = {}
    for s in shapes:
        mk = (min(s), max(s))
        counts[mk] = counts.get(mk, 0) + 1
    for (M, K), cnt in sorted(counts.items()):
        nb = max(1, min(cnt, 8, (2 << 30) // (M * K * 2)))
        Bm = torch.randn(nb, M, M, device=dev).bfloat16() * 0.05
        Xm = torch.randn(nb, M, K, device=dev).bfloat16() * 0.01
        t_bx = _event_ms(lambda: [torch.matmul(Bm[i], Xm[i]) for i in range(nb)], 5, torch)
        t_xx = _event_ms(lambda: [torch.matmul(Xm[i], Xm[i].mT) for i in range(nb)], 5, torch)
        f = 2.0 * M * M * K * nb
        lib_gemm[f"{M}x{K}"] = {"matrices": nb, "B@X_tflops": f / (t_bx * 1e-3) / 1e12,
                                "X@X.mT_tflops_dense": f / (t_xx * 1e-3) / 1e12}
        tot_f += 2.0 * M * M * K * cnt
        tot_t += t_bx * 1e-3 / nb * cnt
        del Bm, Xm
    out["library_gemm"] = lib_gemm
    out["library_B@X_tflops_weighted"] = tot_f / tot_t / 1e12
    return out


def operand_power(dev, M=4096, K=12288, nb=16, reps=10):
    """The three product entry points on operands of one size, filled (a) with independent random values of the
    magnitude the iteration sees and (b) with one constant: same kernels, same bytes, same instruction stream.
    The difference is what the operand data costs (the part lowers its clock under matrix-pipe load)."""
    import torch

    from lmms_engine_amd import _abi

    lib = _abi.lib()
    nx, na = lib.muon_hip_blocked_elems(M, K), lib.muon_hip_blocked_elems(M, M)
    X = torch.empty(nb * nx, dtype=torch.bfloat16, device=dev)
    Xo = torch.empty_like(X)
    A = torch.empty(nb * na, dtype=torch.bfloat16, device=dev)
    Bm = torch.empty_like(A)
    ctr = torch.zeros(_abi.PPX_COUNTER_BYTES, dtype=torch.uint8, device=dev)  # tile counters of the persistent kernel
    res = {}
    for label in ("random", "constant"):
        if label == "random":
            X.copy_((torch.randn(nb * nx, device=dev) * (1.0 / K ** 0.5)).bfloat16())
            A.copy_((torch.randn(nb * na, device=dev) * (1.0 / M ** 0.5)).bfloat16())
        else:
            X.fill_(1.0 / 128)
            A.fill_(1.0 / 64)
        calls = {
            "syrk": (lambda: _abi.check(lib.muon_hip_syrk_bf16(X.data_ptr(), Bm.data_ptr(), M, K, nb, -1, ctr.data_ptr(), _abi.stream_ptr(dev))),
                     float(M) * M * K * nb),
            "sympoly": (lambda: _abi.check(lib.muon_hip_sympoly_bf16(A.data_ptr(), Bm.data_ptr(), M, nb, -4.775, 2.0315, -1,
                                                                     ctr.data_ptr(), _abi.stream_ptr(dev))), float(M) ** 3 * nb),
            "bx_axpy": (lambda: _abi.check(lib.muon_hip_bx_axpy_bf16(A.data_ptr(), X.data_ptr(), Xo.data_ptr(), M, K, nb, 3.4445,
                                                                     -1, ctr.data_ptr(), _abi.stream_ptr(dev))), 2.0 * M * M * K * nb),
        }
        res[label] = {}
        for name, (fn, flop) in calls.items():
            ms = _event_ms(fn, reps, torch)
            res[label][name] = {"ms": ms, "tflops": flop / (ms * 1e-3) / 1e12,
                                "frac_mfma_peak": flop / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
    res["shape"] = f"{nb} matrices {M}x{K}"
    return res


def mfma_probe(dev, iters=40000, reps=25):
    """Loops of nothing but MFMAs (muon_probe_mfma of libmuon_probe.so, a measurement library beside the product's):
    both instruction shapes, operands with random mantissas and constant operands.  The sustained rate is what the
    part's power management leaves of the 2.5 PFLOP/s."""
    import ctypes

    import torch

    from lmms_engine_amd import _abi
    from lmms_engine_amd.build import PROBE_LIB

    lib = ctypes.CDLL(PROBE_LIB)
    lib.muon_probe_mfma.restype = ctypes.c_int
    lib.muon_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                    ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    n = 256 * 12 * 512 * 16 // 2
    sink = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    res = {}
    for label in ("random", "constant"):
        ops = (torch.randn(n, device=dev) * 0.02).bfloat16() if label == "random" else torch.full((n,), 0.0078125, dtype=torch.bfloat16, device=dev)
        res[label] = {}
        for shape, name in ((0, "v_mfma_f32_32x32x16_bf16"), (1, "v_mfma_f32_16x16x32_bf16")):
            flop = ctypes.c_double()
            def fn():
                rc = lib.muon_probe_mfma(ops.data_ptr(), sink.data_ptr(), shape, iters, ctypes.byref(flop), _abi.stream_ptr(dev))
                assert rc == 0, f"muon_probe_mfma failed ({rc})"

            # about half a second of back-to-back launches behind a warm-up of the same kind: the clock follows
            # the power drawn over tens of milliseconds
            ms = _event_ms(fn, reps, torch, warm=8)
            res[label][name] = {"ms": ms, "tflops": flop.value / (ms * 1e-3) / 1e12}
    res["what"] = f"{reps} launches of {iters} iterations each after 8 warm-up launches, per instruction and operand content"
    return res


def stream_probe(dev, gib=2, reps=4):
    """Streaming rate of plain kernels (muon_probe_stream of libmuon_probe.so) against the number of XCDs that take part:
    a read, a read and a write in place, a copy.  One XCD alone and all eight together bound what the elementwise kernels
    of the step can reach on this box."""
    import ctypes

    import torch

    from lmms_engine_amd import _abi
    from lmms_engine_amd.build import PROBE_LIB

    lib = ctypes.CDLL(PROBE_LIB)
    lib.muon_probe_stream.restype = ctypes.c_int
    lib.muon_probe_stream.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                      ctypes.c_void_p]
    nbytes = gib << 30
    a = torch.zeros(nbytes // 4, dtype=torch.float32, device=dev)
    b = torch.zeros_like(a)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    res = {}
    for mode, name in ((0, "read_only"), (1, "in_place"), (2, "copy")):
        res[name] = {}
        for nx in (1, 2, 4, 8):
            def fn():
                rc = lib.muon_probe_stream(a.data_ptr(), b.data_ptr(), nbytes, mode, nx, sink.data_ptr(), _abi.stream_ptr(dev))
                assert rc == 0, f"muon_probe_stream failed ({rc})"

            ms = _event_ms(fn, reps, torch, warm=2)
            moved = nbytes * (1 if mode == 0 else 2)
            res[name][f"{nx}_xcds"] = dict(gbs=moved / (ms * 1e-3) / 1e9, frac_hbm_peak=moved / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS)
    res["what"] = f"{gib} GiB buffers, fp32x4 accesses, {reps} launches per point; workgroup b runs on XCD b % 8"
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
    ap.add_argument("--hip-graph", action="store_true",
                    help="record one step into a HIP graph after the warm-up and time its replays (no per-kernel timing)")
    ap.add_argument("--workspace-limit-gib", type=float, default=0.0,
                    help="cap of the Newton-Schulz workspace (0 = the optimizer's default); smaller caps mean more, "
                         "smaller grouped launches")
    ap.add_argument("--extras", action="store_true",
                    help="also time the two neighbours of the Muon step, outside the timed region: gradient-norm clipping "
                         "over the same gradients and the AdamW fallback over an embedding + lm_head + norm-vector group")
    ap.add_argument("--no-hbm-reference", action="store_true",
                    help="skip the streaming rates of torch's own kernels on this box (after the timed region)")
    ap.add_argument("--no-gpu-oracle", action="store_true",
                    help="skip the second baseline (the reference's expressions unfused in torch on this GPU, and the "
                         "library bf16 GEMM on the shapes of the dominant kernel), which runs after the timed region")
    ap.add_argument("--operand-power", action="store_true",
                    help="also time the three product entry points on random and on constant operands of one size")
    ap.add_argument("--operand-power-only", action="store_true",
                    help="run only the --operand-power measurement (for counter runs)")
    ap.add_argument("--stream-probe-only", action="store_true",
                    help="run only the streaming-rate measurement against the number of active XCDs")
    ap.add_argument("--gemm-config", type=int, default=-1,
                    help="force one GEMM tile configuration (MUON_HIP_CFG_*; -1 = chosen per kernel and shape)")
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
    if args.gemm_config >= 0:
        _abi.check(_abi.lib().muon_hip_set_gemm_config(args.gemm_config), "set_gemm_config")
    if args.operand_power_only:
        print(json.dumps({"operand_power": operand_power(dev), "mfma_probe": mfma_probe(dev)}))
        return
    if args.stream_probe_only:
        print(json.dumps({"stream_probe": stream_probe(dev)}))
        return
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
    step_fn = opt.step
    if args.hip_graph:
        args.no_kernel_timing = True  # events around every launch do not record into a graph
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            opt.step()
        step_fn = graph.replay
        torch.cuda.synchronize()
    if not args.no_kernel_timing:
        # Event pairs for every launch of the timed region exist before it starts (one more warm-up step counts the
        # launches of a step), so that a timed launch costs two event records and nothing else.
        _abi.timing_enable(True, reserve=1 << 16)
        step_fn()
        torch.cuda.synchronize()
        per_step = sum(cnt for _, cnt in _abi.timing_read().values())
        _abi.timing_enable(True, reserve=per_step * args.steps + 64)
    # one event per step boundary on the stream the kernels run on: per-step times for the median and the minimum
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step_fn()
        marks[i + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_step = dt / args.steps * 1e3
    step_ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    ms_median = step_ms[len(step_ms) // 2] if len(step_ms) % 2 else 0.5 * (step_ms[len(step_ms) // 2 - 1] + step_ms[len(step_ms) // 2])
    kern = {}
    if not args.no_kernel_timing:
        kern = _abi.timing_read()
        untimed = _abi.lib().muon_hip_timing_untimed()
        _abi.timing_enable(False)
        assert untimed == 0, f"{untimed} launches ran without events: the pool was too small"

    # per-kernel algorithmic work of one step
    syrk_f = sum(HP["ns_steps"] * float(min(s)) ** 2 * max(s) for s in shapes)
    symp_f = sum(HP["ns_steps"] * float(min(s)) ** 3 for s in shapes)
    bx_f = 2.0 * syrk_f
    gb = 2 if pd == torch.bfloat16 else 4
    mom_bytes = elements * (gb + 2 * 4 + 2) if md == torch.float32 or pd == torch.float32 else elements * (3 * gb + 2)
    # With at least one iteration the parameters are updated by the epilogue of the last B.X of the step (its time is
    # inside bx_axpy) and the update kernel does not run: it appears below only if it was launched.
    upd_elements = elements
    # The launch that carries the update (one of the ns_steps B.X launches of every chunk) is timed on its own: it is
    # another kernel, with the parameter's bytes in its epilogue.
    folded = kern.get("bx_axpy_update", (0.0, 0))[1] > 0
    bx_plain_f = bx_f * (HP["ns_steps"] - 1) / HP["ns_steps"] if folded else bx_f
    work = {"syrk": (syrk_f, "flop"), "sympoly": (symp_f, "flop"), "bx_axpy": (bx_plain_f, "flop"),
            "bx_axpy_update": (bx_f - bx_plain_f, "flop"),
            "momentum_norm": (mom_bytes, "byte"), "normalize": (elements * 4, "byte"),
            "apply_update": (upd_elements * (2 + 2 * gb), "byte")}
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
        achieved = bx_plain_f * args.steps / (tot_ms * 1e-3) / 1e12
        roofline = {"kernel": "gemm_nt_ppx_kernel<EPI_BX>: X' = a.X + B.X, the persistent kernel (the first ns_steps - 1 of the "
                              "B.X launches of every chunk; the last one, which carries the parameter update in its "
                              "epilogue, is another kernel: kernels.bx_axpy_update)",
                    "bound": "mfma", "achieved": achieved,
                    "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                    "traffic": recorded_traffic(args.workload) if layers == w["layers"] else None,
                    "launches": cnt, "avg_launch_ms": tot_ms / cnt,
                    "algorithmic_flop_per_launch": bx_plain_f * args.steps / cnt}
    gemm_ms = sum(kernels[k]["ms_per_step"] for k in ("syrk", "sympoly", "bx_axpy", "bx_axpy_update") if k in kernels)

    out = {
        "metric": METRIC,
        "value": flops_step / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "ms_per_step_median": ms_median,
        "ms_per_step_min": step_ms[0],
        "ms_per_step_max": step_ms[-1],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{args.workload} 2-D parameter set, {layers} layers, {len(shapes)} matrices, "
                               f"{w['pdtype']} params/grads, fp32 momentum, full Muon step",
                   "elements": elements, "ns_steps": HP["ns_steps"], "grouped_buckets": len(set(shapes)),
                   "launch": "replays of one step recorded into a HIP graph" if args.hip_graph else "eager"},
        "ns_flop_per_step_algorithmic": flops_step,
        "pct_bf16_mfma_peak_whole_step": 100.0 * flops_step / (ms_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "ns_tflops_gemm_kernels_only": (flops_step / (gemm_ms * 1e-3) / 1e12) if gemm_ms else None,
        "kernels": kernels,
        "roofline": roofline,
    }
    if args.extras:
        out["extras"] = extras(params, pd, dev, args.steps)
    if args.operand_power:
        out["operand_power"] = operand_power(dev)
        out["mfma_probe"] = mfma_probe(dev)
    if not args.no_hbm_reference:
        out["hbm_reference"] = hbm_reference(dev)
    if not args.no_gpu_oracle:
        moms = [opt.state[p]["momentum_buffer"] for p in params]
        out["gpu_oracle"] = gpu_oracle(params, moms, shapes, flops_step)
        if roofline is not None:
            out["gpu_oracle"]["bx_axpy_kernel_tflops"] = roofline["achieved"]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, layers, flops_step)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
