"""Shared builders for the parity tests: seeded inputs in the generation order the
benchmark configs fix (for layer: for name in q,k,v,o,gate,up,down: weight; then per step
the same nested order for grads)."""
import ctypes

import numpy as np
import torch

QWEN25_05B = dict(layers=24, q=(896, 896), k=(128, 896), v=(128, 896), o=(896, 896), gate=(4864, 896),
                  up=(4864, 896), down=(896, 4864))
QWEN3_8B = dict(layers=36, q=(4096, 4096), k=(1024, 4096), v=(1024, 4096), o=(4096, 4096), gate=(12288, 4096),
                up=(12288, 4096), down=(4096, 12288))
NAMES = ["q", "k", "v", "o", "gate", "up", "down"]
MUON_HP = dict(lr=0.02, momentum=0.95, nesterov=True, weight_decay=0.01, ns_steps=5, rms_scale=False)


def rel_fro(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def make_param_set(spec, layers, seed, steps, dtype=torch.float32):
    """CPU tensors: list of (name, weight) and per-step list of grads, fixed generation order."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    weights = []
    for l in range(layers):
        for n in NAMES:
            weights.append((f"layers.{l}.{n}", (0.02 * torch.randn(*spec[n], generator=gen)).to(dtype)))
    grads = []
    for _ in range(steps):
        grads.append([(1e-3 * torch.randn(*w.shape, generator=gen)).to(dtype) for _, w in weights])
    return weights, grads


def bf16_from_u16(arr: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(arr.astype(np.uint16).view(np.int16).copy()).view(torch.bfloat16)


def u16_from_bf16(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def c_newton_schulz(lib, G: torch.Tensor, steps: int) -> torch.Tensor:
    """oracle/muon_oracle.c's orc_newton_schulz on an fp32 CPU matrix."""
    rows, cols = G.shape
    Gc = G.detach().float().contiguous().numpy()
    out = np.zeros((rows, cols), dtype=np.uint16)
    lib.orc_newton_schulz(Gc.ctypes.data_as(ctypes.c_void_p), rows, cols, steps, ctypes.c_double(3.4445),
                          ctypes.c_double(-4.7750), ctypes.c_double(2.0315), out.ctypes.data_as(ctypes.c_void_p))
    return bf16_from_u16(out)


PARITY_REPORT = []


def report_parity(line: str) -> None:
    """Print a measured parity figure now and keep it for the end-of-run summary (tests/conftest.py), so that it
    shows in the output of a quiet run, where the stdout of passing tests is dropped."""
    print(line, flush=True)
    PARITY_REPORT.append(line)
