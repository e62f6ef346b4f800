"""CPU restatement of lmms-engine's Muon optimizer step.  TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP path: only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import it.  Nothing in the lmms_engine_amd package does.

It restates, in plain torch CPU ops, what the reference computes in
src/lmms_engine/utils/muon_utils.py.  Two spellings are kept side by side:

* ``literal=True``  follows the reference's own torch expressions (``b * buf1 + c * buf2``,
  ``X / (X.norm(...) + 1e-7)`` ...) with ``X @ X.mT`` standing in for the Triton
  ``mmt_kernel`` (muon_utils.py:28-92), whose contract is bf16 in, fp32 accumulate
  (:70), one rounding to bf16 (:80), lower triangle mirrored from the upper (:89-92).
* ``literal=False`` spells every bf16 rounding point out with fp32 arithmetic, which is
  what the HIP epilogues implement.  tests/test_oracle.py requires both spellings to be
  bit-identical, so a mis-stated rounding point fails there.

Parity status: the reference's tests hold no golden vector for Muon (no test executes it),
so every function here is pinned by what the mathematics fixes instead: closed forms,
the SVD polynomial identity, invariants, fp64 brute force on tiny inputs, torch library
routines (torch.lerp, torch.optim.AdamW) and an independent plain-C restatement
(oracle/muon_oracle.c).  See tests/test_oracle.py for each check.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import Tensor

# muon_utils.py:137
NS_COEFFS = (3.4445, -4.7750, 2.0315)


def bf(x: Tensor) -> Tensor:
    """Round to bf16 (RNE) and return as fp32 values."""
    return x.to(torch.bfloat16).to(torch.float32)


def _f32(x: float) -> float:
    """A python double as the fp32 'opmath' scalar ATen kernels see."""
    return torch.tensor(x, dtype=torch.float32).item()


def mmt(X: Tensor) -> Tensor:
    """bf16 X (M,K) -> bf16 X·Xᵀ, fp32 accumulate, exactly symmetric.

    Follows matmul_transpose_assign / mmt_kernel (muon_utils.py:95-119, 28-92): only
    tiles with pid_m <= pid_n are computed and the transposed tile is copied below the
    diagonal, so the result is symmetric bit for bit.
    """
    assert X.dtype == torch.bfloat16 and X.ndim == 2
    Xf = X.float()
    A = (Xf @ Xf.mT).to(torch.bfloat16)
    return torch.triu(A) + torch.triu(A, 1).mT


def frobenius_denominator(X: Tensor) -> Tensor:
    """bf16 scalar d = bf(bf(‖X‖_F) + 1e-7) (muon_utils.py:146).

    Tensor.norm on a bf16 tensor accumulates in fp32 and returns bf16; the add of 1e-7
    is a bf16 add.
    """
    n = X.float().pow(2).sum().sqrt().to(torch.bfloat16)
    return (n.float() + _f32(1e-7)).to(torch.bfloat16)


def newton_schulz(G: Tensor, steps: int = 5, literal: bool = False) -> Tensor:
    """fast_newtonschulz (muon_utils.py:129-156). Returns bf16, shape of G."""
    assert G.ndim == 2
    a, b, c = NS_COEFFS
    X = G.to(torch.bfloat16)  # :138
    transposed = G.size(-2) > G.size(-1)  # :139
    if transposed:
        X = X.mT
    if literal:
        X = X / (X.norm(dim=(-2, -1), keepdim=True) + 1e-7)  # :146
        for _ in range(steps):
            buf1 = mmt(X.contiguous())  # :149
            buf2 = mmt(buf1)  # :150
            B = b * buf1 + c * buf2  # :151
            X = a * X + B @ X  # :152
    else:
        af, bf_, cf = _f32(a), _f32(b), _f32(c)
        d = frobenius_denominator(X)
        X = (X.float() / d.float()).to(torch.bfloat16)
        for _ in range(steps):
            A = mmt(X.contiguous())
            A2 = mmt(A)
            t1 = bf(A.float() * bf_)
            t2 = bf(A2.float() * cf)
            B = bf(t1 + t2)
            BX = bf(B @ X.float())
            aX = bf(X.float() * af)
            X = (aX + BX).to(torch.bfloat16)
    if transposed:
        X = X.mT
    return X


def apply_momentum(grad: Tensor, momentum: Tensor, beta: float, nesterov: bool) -> Tensor:
    """In place, as muon_update does (muon_utils.py:188-189).

    Same-dtype case: literally the reference's two lerp_ calls.  Mixed case (bf16 grad,
    fp32 momentum -- an extension the reference cannot express because lerp_ refuses
    mixed dtypes): the grad is upcast to fp32 first and the blend stays fp32.
    Returns the update (the blended grad when nesterov, else the momentum buffer).
    """
    if grad.dtype != momentum.dtype:
        assert momentum.dtype == torch.float32
        g = grad.float()
        momentum.lerp_(g, 1 - beta)
        return g.lerp_(momentum, beta) if nesterov else momentum
    momentum.lerp_(grad, 1 - beta)
    return grad.lerp_(momentum, beta) if nesterov else momentum


def lerp_closed_form(start: Tensor, end: Tensor, weight: float) -> Tensor:
    """ATen's lerp formula in fp64, for checking apply_momentum.

    weight < 0.5: start + w(end-start); else end - (end-start)(1-w), w taken as fp32.
    """
    w = _f32(weight)
    s, e = start.double(), end.double()
    if abs(w) < 0.5:
        return s + w * (e - s)
    return e - (e - s) * (1.0 - w)


def scale_factor(rows: int, cols: int, rms_scale: bool) -> float:
    """apply_scaling's multiplier (muon_utils.py:167-175) as a python double."""
    if rms_scale:
        return 0.2 * (max(cols, rows)) ** 0.5
    return max(1, rows / cols) ** 0.5


def apply_scaling(update: Tensor, rms_scale: bool) -> Tensor:
    """In place on the (bf16) NS output; one rounding in the tensor's dtype."""
    update *= scale_factor(update.size(-2), update.size(-1), rms_scale)
    return update


def param_update(param: Tensor, update: Tensor, lr: float, weight_decay: float) -> None:
    """SingelDeviceWork.start's tail (muon_utils.py:324-325), in place.

    For a bf16 parameter the add is spelled out: ATen's GPU add kernel keeps `alpha` in fp32
    opmath, while its CPU kernel narrows alpha to bf16 first (measured: -0.02 becomes
    -0.02002).  The reference runs on a GPU, so the GPU arithmetic is the one restated.
    """
    param.mul_(1 - lr * weight_decay)
    update = update.reshape(param.shape)
    if param.dtype == torch.float32:
        param.add_(update, alpha=-lr)
    else:
        param.copy_((param.float() + _f32(-lr) * update.float()).to(param.dtype))


def muon_step_matrix(
    param: Tensor,
    grad: Tensor,
    momentum: Tensor,
    lr: float = 0.02,
    weight_decay: float = 0.0,
    beta: float = 0.95,
    nesterov: bool = True,
    ns_steps: int = 5,
    rms_scale: bool = True,
    literal: bool = False,
) -> Tensor:
    """One Muon step for one 2-D parameter, in place on param / grad / momentum.

    Keyword-correct semantics (ns_steps iterations, nesterov flag) as the reference's
    FSDP path passes them (muon_utils.py:261); the single-device call site swaps the two
    positionally (:316-323), which `reference_bug_compat_args` below reproduces.
    Returns the scaled orthogonalised update (bf16).
    """
    assert param.ndim == 2
    u = apply_momentum(grad, momentum, beta, nesterov)
    o = newton_schulz(u, steps=ns_steps, literal=literal)
    o = apply_scaling(o, rms_scale)
    param_update(param, o, lr, weight_decay)
    return o


def reference_bug_compat_args(nesterov, ns_steps):
    """What muon_update receives from SingelDeviceWork.start (muon_utils.py:316-323 into :186).

    The call passes (momentum, nesterov, ns_steps, rms_scale) positionally into
    (beta, ns_steps, nesterov, rms_scale): ns_steps <- nesterov (range(True) is one
    iteration, range(False) none) and nesterov <- ns_steps (truthy unless 0).
    Returns (effective nesterov, effective ns_steps).
    """
    return bool(ns_steps), int(bool(nesterov))


def adam_update(grad: Tensor, buf1: Tensor, buf2: Tensor, step: int, betas, eps: float, literal: bool = False) -> Tensor:
    """muon_utils.py:178-183.

    `literal=True` is the reference's text evaluated by torch on the CPU.  The default restates what the same
    text computes on a GPU, where ATen evaluates tensor / python-scalar as tensor * float(1.0 / scalar), the reciprocal
    taken in double precision (its CPU kernel divides); the two differ by at most one fp32 ulp before the rounding to the tensor dtype.  The GPU
    form is pinned by a device-side test against torch itself (tests/test_gpu_torch_device.py).
    """
    buf1.lerp_(grad, 1 - betas[0])
    buf2.lerp_(grad.square(), 1 - betas[1])
    if literal:
        buf1c = buf1 / (1 - betas[0] ** step)
        buf2c = buf2 / (1 - betas[1] ** step)
    else:
        inv1 = torch.tensor(1.0 / (1 - betas[0] ** step), dtype=torch.float32)
        inv2 = torch.tensor(1.0 / (1 - betas[1] ** step), dtype=torch.float32)
        buf1c = (buf1.float() * inv1).to(buf1.dtype)
        buf2c = (buf2.float() * inv2).to(buf2.dtype)
    return buf1c / (buf2c.sqrt() + eps)


def adamw_step_tensor(param, grad, exp_avg, exp_avg_sq, step, lr, betas, eps, weight_decay) -> None:
    """Adam branch of step_fsdp (muon_utils.py:468-477), in place. `step` is already incremented."""
    upd = adam_update(grad, exp_avg, exp_avg_sq, step, betas, eps)
    param_update(param, upd, lr, weight_decay)


class OracleMuon:
    """Step-level restatement of Muon.step_fsdp on one device (muon_utils.py:434-482).

    Holds its own param/momentum copies on the CPU.  `groups` uses the reference's group
    dict layout after Muon.__init__ has filled the defaults.
    """

    def __init__(self, groups, momentum_dtype: Optional[torch.dtype] = None, literal: bool = False):
        self.groups = groups
        self.state = {}
        self.momentum_dtype = momentum_dtype
        self.literal = literal
        self.last_updates = {}

    def step(self):
        for gi, group in enumerate(self.groups):
            for pi, p in enumerate(group["params"]):
                key = (gi, pi)
                g = p.grad if p.grad is not None else torch.zeros_like(p)
                st = self.state.setdefault(key, {})
                if group["use_muon"]:
                    assert p.ndim == 2, p.shape
                    if not st:
                        st["momentum_buffer"] = torch.zeros_like(p, dtype=self.momentum_dtype or p.dtype)
                    with torch.no_grad():
                        o = muon_step_matrix(
                            p,
                            g.clone(),
                            st["momentum_buffer"],
                            lr=group["lr"],
                            weight_decay=group["weight_decay"],
                            beta=group["momentum"],
                            nesterov=group["nesterov"],
                            ns_steps=group["ns_steps"],
                            rms_scale=group["rms_scale"],
                            literal=self.literal,
                        )
                    self.last_updates[key] = o
                else:
                    if not st:
                        st["exp_avg"] = torch.zeros_like(p)
                        st["exp_avg_sq"] = torch.zeros_like(p)
                        st["step"] = 0
                    st["step"] += 1
                    with torch.no_grad():
                        adamw_step_tensor(
                            p, g, st["exp_avg"], st["exp_avg_sq"], st["step"],
                            group["lr"], group["betas"], group["eps"], group["weight_decay"],
                        )


def svd_polynomial(G: Tensor, steps: int = 5) -> Tensor:
    """Exact-arithmetic value of the NS chain: U φ^steps(Σ) Vᵀ for G/‖G‖_F = UΣVᵀ.

    φ(σ) = aσ + bσ³ + cσ⁵.  fp64; a sanity bound for newton_schulz, not the parity bound
    (bf16 roundings move the result by a few percent).
    """
    a, b, c = NS_COEFFS
    Gd = G.double()
    Gd = Gd / Gd.norm()
    U, S, Vh = torch.linalg.svd(Gd, full_matrices=False)
    for _ in range(steps):
        S = a * S + b * S**3 + c * S**5
    return (U * S) @ Vh


def ns_flops(rows: int, cols: int, steps: int = 5, dense: bool = False) -> float:
    """Algorithmic NS FLOPs: steps·(3M²K + M³); dense-equivalent steps·(4M²K + 2M³)."""
    M, K = min(rows, cols), max(rows, cols)
    if dense:
        return steps * (4.0 * M * M * K + 2.0 * M**3)
    return steps * (3.0 * M * M * K + 1.0 * M**3)
