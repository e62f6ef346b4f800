"""Muon optimizer step on one MI355X: the host side.

Mirrors the public surface of the reference module
/root/reference/src/lmms_engine/utils/muon_utils.py (same names, argument meaning, group
and state layout, error behaviour) so that `from ... import Muon` can be pointed here and
the trainer's optimizer factory (src/lmms_engine/train/hf/trainer.py:459-465) works unchanged.
All arithmetic runs in hand-written gfx950 kernels behind the C ABI of libmuon_hip.so
(include/muon_hip.h); torch supplies device memory and streams only.  There is no
fallback: tensors that are not on a GPU, or a missing library, raise.

Differences from the reference, all deliberate:
  * step() dispatches each stage once per bucket of same-shape parameters (pointer tables,
    batched kernels) instead of once per parameter.
  * keyword-correct hyper-parameters: `ns_steps` iterations and the `nesterov` flag mean what
    they say.  The reference's single-device call site passes them swapped positionally
    (muon_utils.py:316-323 into :186); `reference_bug_compat=True` reproduces that.
  * p.grad is not overwritten with the Nesterov blend unless `write_back_grad=True`.
  * the Newton-Schulz workspace is kept between steps (`keep_workspace=False` or `release_workspace()` frees it).
  * `momentum_dtype=torch.float32` keeps an fp32 momentum buffer for bf16 parameters (the
    reference always uses the parameter's dtype, muon_utils.py:450).
"""
from __future__ import annotations

import logging
from collections import OrderedDict, deque
from itertools import chain
from typing import Optional, Protocol

import torch
from torch import Tensor
from torch.distributed.tensor import DTensor

from . import _abi

logger = logging.getLogger(__name__)

NS_COEFFS = (3.4445, -4.7750, 2.0315)  # muon_utils.py:137

# Cap of the Newton-Schulz workspace one grouped launch may use; buckets that need more are cut into chunks.
# Measured on the Qwen3-8B-shaped set: 2 / 3.2 / 4.2 / 5 / 6.5 / 8.5 GiB give 357.9 / 353.2 / 352.0 / 351.4 / 351.6 /
# 352.2 ms per step: up to about 4 GiB larger chunks land the triangular tile counts of X.Xt on whole rounds of the compute
# units (15 matrices 4096x12288 = 2040 tiles = 7.97 rounds, where 7 gave 3.72), past that a.X + B.X loses what chunks of a few
# large matrices gain from the memory-side cache.  4 GiB is the smallest cap within 0.2 % of the best.
DEFAULT_WORKSPACE_LIMIT = 4 << 30

_noted_semantics = False


def _note_keyword_semantics() -> None:
    """Once per process: this optimizer is not arithmetic-identical to the reference's single-device call site."""
    global _noted_semantics
    if _noted_semantics:
        return
    _noted_semantics = True
    logger.warning(
        "Muon (MI355X build): ns_steps and nesterov are honoured as named. The reference's single-device call site "
        "passes them swapped (one Newton-Schulz iteration, Nesterov always on); pass reference_bug_compat=True to "
        "reproduce that trajectory."
    )


_MUON_KEYS = {"params", "lr", "momentum", "weight_decay", "use_muon", "rms_scale", "nesterov", "ns_steps"}
_ADAM_KEYS = {"params", "lr", "betas", "eps", "weight_decay", "use_muon"}


# --------------------------------------------------------------------------------------
# device plumbing
# --------------------------------------------------------------------------------------
def _require_cuda(t: Tensor, name: str) -> None:
    if not t.is_cuda:
        raise _abi.MuonHipError(f"{name} must live on a GPU: this build has no CPU path (got device {t.device})")


def _workspace(nbytes: int, device) -> Tensor:
    # 256-byte alignment comes with torch's caching allocator (512-byte granularity)
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def _pointer_table(tensors, device, cache=None, key=None) -> Tensor:
    """Device table of the tensors' base pointers.  With a cache (a _TableCache), a table whose pointers have not changed
    since the last call under `key` is handed back as it is: no host allocation and no copy, which is what lets a step
    over static tensors be recorded into a HIP graph (and saves the copy otherwise)."""
    ptrs = tuple(t.data_ptr() for t in tensors)
    if cache is not None:
        hit = cache.tables.get(key)
        if hit is not None and hit[0] == ptrs and hit[1].device == device:
            return hit[1]
    if torch.cuda.is_current_stream_capturing():
        # A miss under capture would record a copy out of a host buffer that is freed when this call returns, and
        # replace a table that an earlier recording may still read.
        raise _abi.MuonHipError(
            "Muon.step under HIP graph capture needs the pointer tables of an earlier eager step: parameters, grads "
            "and momentum buffers must keep their addresses (run an eager step first and do not re-allocate grads, "
            "e.g. zero_grad(set_to_none=False))"
        )
    host = torch.tensor(ptrs, dtype=torch.int64, pin_memory=True)
    table = host.to(device, non_blocking=True)
    if cache is not None:
        cache.replace(key, ptrs, table)
    return table


class _TableCache:
    """Pointer tables of the last step, per bucket chunk.  A table that a later step replaces is kept alive for a while
    instead of going back to the allocator: a HIP graph recorded earlier may still read it."""

    KEEP = 64  # replaced tables kept alive (a few KB each)

    def __init__(self):
        self.tables = {}   # key -> (pointers, device table)
        self.retired = []

    def __len__(self):
        return len(self.tables)

    def replace(self, key, ptrs, table) -> None:
        old = self.tables.get(key)
        if old is not None:
            self.retired.append(old[1])
            del self.retired[:-self.KEEP]
        self.tables[key] = (ptrs, table)


def scale_factor(rows: int, cols: int, rms_scale: bool) -> float:
    """The python double apply_scaling multiplies by (muon_utils.py:167-175)."""
    if rms_scale:
        return 0.2 * (max(cols, rows)) ** 0.5
    return max(1, rows / cols) ** 0.5


# --------------------------------------------------------------------------------------
# functional surface (muon_utils.py:95-192)
# --------------------------------------------------------------------------------------
def matmul_transpose_assign(d_in: Tensor, d_out: Tensor) -> None:
    """d_out = d_in @ d_in.T on the symmetric MFMA kernel (muon_utils.py:95-119)."""
    assert d_in.is_cuda, "Input `d_in` must be a CUDA tensor"
    assert d_out.is_cuda, "Input `d_out` must be a CUDA tensor"
    assert d_in.device == d_out.device, "Inputs `d_in` and `d_out` must be on the same CUDA device"
    assert d_in.dtype == d_out.dtype, "Inputs must have the same data type"
    assert d_in.ndim == 2, "Input `d_in` must be a 2D tensor"
    assert d_out.ndim == 2, "Input `d_out` must be a 2D tensor"
    assert (
        d_in.size(0) == d_out.size(0) == d_out.size(1)
    ), "First dimension of `d_in` must match first and second dimension of `d_out`"
    if d_in.dtype != torch.bfloat16:
        raise TypeError(f"the MI355X kernel multiplies bfloat16 operands, got {d_in.dtype}")
    M, K = d_in.shape
    tile = 256 if (M % 256 == 0 and M >= 512) else 128
    cfg = _abi.CFG_AUTO  # the library picks the kernel for the padded size
    Mp, Kp = -(-M // tile) * tile, -(-K // tile) * tile
    lib = _abi.lib()
    with torch.cuda.device(d_in.device):
        s = _abi.stream_ptr(d_in.device)
        src = d_in.contiguous()
        x = torch.empty(lib.muon_hip_blocked_elems(Mp, Kp), dtype=torch.bfloat16, device=d_in.device)
        a = torch.empty(lib.muon_hip_blocked_elems(Mp, Mp), dtype=torch.bfloat16, device=d_in.device)
        _abi.check(lib.muon_hip_pack_bf16(src.data_ptr(), 0, K, M, K, x.data_ptr(), Mp, Kp, 1, s), "pack")
        _abi.check(lib.muon_hip_syrk_bf16(x.data_ptr(), a.data_ptr(), Mp, Kp, 1, cfg, None, s), "syrk")
        out = d_out if d_out.is_contiguous() else torch.empty_like(d_out, memory_format=torch.contiguous_format)
        _abi.check(lib.muon_hip_unpack_bf16(a.data_ptr(), Mp, Mp, out.data_ptr(), 0, M, M, M, 1, s), "unpack")
        if out is not d_out:
            d_out.copy_(out)


def get_autotune_config():
    """muon_utils.py:13-25 lists the Triton tile shapes the autotuner tries.  The HIP kernels are not autotuned:
    this returns the fixed tile configurations the launcher chooses between by shape."""
    return [
        dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, num_stages=2, num_warps=4, config=_abi.CFG_128_PIPE),
        dict(BLOCK_SIZE_M=256, BLOCK_SIZE_N=256, BLOCK_SIZE_K=64, num_stages=2, num_warps=8, config=_abi.CFG_256_PIPE),
        dict(BLOCK_SIZE_M=256, BLOCK_SIZE_N=256, BLOCK_SIZE_K=32, num_stages=4, num_warps=8, config=_abi.CFG_256_PINGPONG),
        dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=32, num_stages=4, num_warps=8, config=_abi.CFG_128_PINGPONG),
        dict(BLOCK_SIZE_M=256, BLOCK_SIZE_N=256, BLOCK_SIZE_K=32, num_stages=4, num_warps=8, config=_abi.CFG_256_PERSIST),
    ]


class _MmtKernel:
    """Stands where the reference keeps its Triton kernel object (muon_utils.py:28-92) so that code which
    launches it as `mmt_kernel[grid](x, y, M, K, stride_xm, stride_xk, stride_ym, stride_yn)` keeps working:
    the launch runs the symmetric MFMA kernel through matmul_transpose_assign; the grid is ignored."""

    def __getitem__(self, grid):
        def launch(x, y, M, K, stride_xm, stride_xk, stride_ym, stride_yn, **meta):
            src = torch.as_strided(x, (M, K), (stride_xm, stride_xk))
            dst = torch.as_strided(y, (M, M), (stride_ym, stride_yn))
            matmul_transpose_assign(src, dst)

        return launch


mmt_kernel = _MmtKernel()


def matmul_transpose(d_in: Tensor) -> Tensor:
    M, _ = d_in.shape
    d_out = torch.empty((M, M), device=d_in.device, dtype=d_in.dtype)
    matmul_transpose_assign(d_in, d_out)
    return d_out


def fast_newtonschulz(G: Tensor, steps: int = 5) -> Tensor:
    """Newton-Schulz orthogonalisation (muon_utils.py:129-156); returns bf16 in G's shape.

    G is 2-D, or 3-D [batch, rows, cols] for a stack of same-shape matrices (an extension:
    one grouped dispatch per stage).
    """
    assert G.ndim >= 2, f"Gradient must be a 2D tensor, but got {G.shape}"
    _require_cuda(G, "G")
    if G.ndim > 3:
        raise ValueError(f"expected a 2-D matrix or a 3-D stack, got shape {tuple(G.shape)}")
    batch = G.size(0) if G.ndim == 3 else 1
    rows, cols = G.size(-2), G.size(-1)
    Gc = G.contiguous()
    if Gc.dtype in (torch.float16, torch.float64):
        # G.bfloat16() (muon_utils.py:138) converts these through fp32: fp16 -> fp32 is exact, fp64 -> fp32 is the
        # rounding torch's own conversion makes first
        Gc = Gc.float()
    lib = _abi.lib()
    a, b, c = NS_COEFFS
    with torch.cuda.device(G.device):
        ws = _workspace(_abi.workspace_bytes(rows, cols, batch), G.device)
        out = torch.empty(G.shape, dtype=torch.bfloat16, device=G.device)
        s = _abi.stream_ptr(G.device)
        _abi.check(lib.muon_hip_cast_norm(Gc.data_ptr(), _abi.dtype_code(Gc.dtype), ws.data_ptr(), rows, cols, batch, s),
                   "cast_norm")
        _abi.check(lib.muon_hip_ns_grouped(ws.data_ptr(), rows, cols, batch, int(steps), a, b, c, s), "ns_grouped")
        _abi.check(lib.muon_hip_ns_output(ws.data_ptr(), rows, cols, batch, int(steps), out.data_ptr(), s), "ns_output")
    return out


def _row_major(t: Tensor) -> Tensor:
    """t itself when its strides are row-major, else a row-major copy (the caller writes it back)."""
    return t if t.is_contiguous() else t.detach().contiguous()


def apply_momentum(grad: Tensor, momentum: Tensor, beta: float, nesterov: bool) -> Tensor:
    """In place on both tensors, as muon_utils.py:159-164; returns the update.  Tensors whose strides are not
    row-major go through row-major copies that are written back."""
    _require_cuda(grad, "grad")
    gc, mc = _row_major(grad), _row_major(momentum)
    g2 = gc.view(len(gc), -1) if gc.ndim == 4 else gc
    assert g2.ndim == 2 and momentum.shape == grad.shape
    rows, cols = g2.shape
    with torch.cuda.device(grad.device):
        ws = _workspace(_abi.workspace_bytes(rows, cols, 1), grad.device)
        gt, mt = _pointer_table([gc], grad.device), _pointer_table([mc], grad.device)
        _abi.check(
            _abi.lib().muon_hip_momentum_norm(gt.data_ptr(), mt.data_ptr(), _abi.dtype_code(grad.dtype),
                                              _abi.dtype_code(momentum.dtype), ws.data_ptr(), rows, cols, 1,
                                              float(beta), int(bool(nesterov)), 1, _abi.stream_ptr(grad.device)),
            "momentum_norm",
        )
        if gc is not grad:
            grad.copy_(gc)
        if mc is not momentum:
            momentum.copy_(mc)
    update = grad if nesterov else momentum
    if update.ndim == 4:
        update = update.reshape(len(update), -1)
    return update


def apply_scaling(grad: Tensor, rms_scale: bool = False) -> Tensor:
    """muon_utils.py:167-175, in place, one rounding in grad's dtype.  step() fuses this into the update kernel;
    this is the stand-alone helper."""
    _require_cuda(grad, "grad")
    gc = _row_major(grad)
    with torch.cuda.device(grad.device):
        _abi.check(
            _abi.lib().muon_hip_scale(gc.data_ptr(), _abi.dtype_code(grad.dtype), grad.numel(),
                                      float(scale_factor(grad.size(-2), grad.size(-1), rms_scale)),
                                      _abi.stream_ptr(grad.device)),
            "scale",
        )
        if gc is not grad:
            grad.copy_(gc)
    return grad


def adam_update(grad: Tensor, buf1: Tensor, buf2: Tensor, step: int, betas, eps: float) -> Tensor:
    """muon_utils.py:178-183: both moment buffers move in place, the bias-corrected update is returned."""
    _require_cuda(grad, "grad")
    if not (grad.dtype == buf1.dtype == buf2.dtype):
        raise TypeError("adam_update: grad and both moment buffers must share one dtype")
    if grad.shape != buf1.shape or grad.shape != buf2.shape:
        raise ValueError("adam_update: the moment buffers must have the gradient's shape")
    g, b1, b2 = _row_major(grad), _row_major(buf1), _row_major(buf2)
    out = torch.empty_like(b1)
    with torch.cuda.device(grad.device):
        _abi.check(
            _abi.lib().muon_hip_adam_update(g.data_ptr(), b1.data_ptr(), b2.data_ptr(), out.data_ptr(),
                                            _abi.dtype_code(grad.dtype), grad.numel(), int(step), float(betas[0]),
                                            float(betas[1]), float(eps), _abi.stream_ptr(grad.device)),
            "adam_update",
        )
        if b1 is not buf1:
            buf1.copy_(b1)
        if b2 is not buf2:
            buf2.copy_(b2)
    return out


def muon_update(grad, momentum, beta=0.95, ns_steps=5, nesterov=True, rms_scale=False):
    """muon_utils.py:186-192: momentum, Newton-Schulz, scaling; returns the bf16 update."""
    update = apply_momentum(grad, momentum, beta, nesterov)
    update = fast_newtonschulz(update, steps=ns_steps)
    return apply_scaling(update, rms_scale)


# --------------------------------------------------------------------------------------
# grouped launcher
# --------------------------------------------------------------------------------------
_cu_counts = {}  # device index -> compute units, as the library reads them from the runtime


def _cu_count(device) -> int:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _cu_counts:
        with torch.cuda.device(idx):
            _cu_counts[idx] = _abi.device_shape()[0]
    return _cu_counts[idx]


def _pick_chunk(n: int, cap: int, rows: int, cols: int, cus: int = 256) -> int:
    """Matrices per grouped launch for a bucket of n: at most `cap` (what the workspace limit holds, and never more
    than the 65535 matrices one library call takes) and at least half of it, chosen so that the tile counts of the
    three products leave the last round of the `cus` compute units (one 256x256 workgroup each) as full as possible.  A launch of t tiles runs ceil(t / cus) rounds (a last
    round of at most 64 tiles is cut into quarter tiles and costs about 0.6 of a round) plus about a third of a
    round of ramp-up and tail; a tile of X.Xt costs ~K, one of b.A + c.A.A and of a.X + B.X ~M."""
    cap = min(cap, 65535)
    if cap >= n or cap <= 2:
        return max(1, min(n, cap))
    M, K = min(rows, cols), max(rows, cols)
    if M % 256 or M < 512:
        return cap  # 128-tiles: many small tiles, rounds hardly matter
    T, TN = M // 256, -(-K // 256)
    tri, rect = T * (T + 1) // 2, T * TN

    def rounds(t):
        full, rest = divmod(t, cus)
        return full + (0.0 if rest == 0 else 0.6 if rest <= cus // 4 and full > 0 else 1.0)

    def cost(nb):
        return (rounds(tri * nb) + 0.35) * (K + M) + (rounds(rect * nb) + 0.35) * M

    best, best_cost = cap, None
    for nb in range(max(1, cap // 2), min(n, cap) + 1):
        chunks, last = divmod(n, nb)
        c = chunks * cost(nb) + (cost(last) if last else 0.0)
        if best_cost is None or c < best_cost * (1 - 1e-9):
            best, best_cost = nb, c
    return best


def _muon_bucket_step(params, grads, moms, group, ns_steps, nesterov, write_back_grad, ws_holder, ws_limit, tables=None):
    """All stages of the Muon step for same-shape, same-dtype parameters on one device."""
    p0 = params[0]
    rows, cols = p0.shape
    dev = p0.device
    lib = _abi.lib()
    pd, gd, md = _abi.dtype_code(p0.dtype), _abi.dtype_code(grads[0].dtype), _abi.dtype_code(moms[0].dtype)
    a, b, c = NS_COEFFS
    scale = scale_factor(rows, cols, group["rms_scale"])
    n = len(params)
    per = _abi.workspace_bytes(rows, cols, 1)
    chunk = _pick_chunk(n, max(1, min(ws_limit // per, 65535)), rows, cols, _cu_count(dev))
    with torch.cuda.device(dev):
        s = _abi.stream_ptr(dev)
        for lo in range(0, n, chunk):
            hi = min(n, lo + chunk)
            nb = hi - lo
            need = _abi.workspace_bytes(rows, cols, nb)
            ws = ws_holder.get(dev)
            if ws is None or ws.numel() < need:
                ws_holder[dev] = None
                ws = ws_holder[dev] = _workspace(need, dev)
            table = _pointer_table(params[lo:hi] + grads[lo:hi] + moms[lo:hi], dev, tables,
                                   (id(group), dev, rows, cols, p0.dtype, grads[0].dtype, moms[0].dtype, lo))
            base = table.data_ptr()
            _abi.check(
                lib.muon_hip_step_grouped(
                    base, base + 8 * nb, base + 16 * nb, pd, gd, md, ws.data_ptr(), rows, cols, nb,
                    float(group["lr"]), float(group["weight_decay"]), float(group["momentum"]), int(bool(nesterov)),
                    int(ns_steps), float(scale), a, b, c, int(bool(write_back_grad)), s,
                ),
                "step_grouped",
            )


# --------------------------------------------------------------------------------------
# Work protocol (muon_utils.py:195-328)
# --------------------------------------------------------------------------------------
class Work(Protocol):
    def __init__(self, param, state, group, index: int):
        ...

    def start(self):
        ...

    def finish(self):
        ...


class _MeshWorkUnavailable:
    """Distributed variants need collectives; this build runs on one GPU only."""

    def __init__(self, param, state, group, index: int):
        raise NotImplementedError("not implemented")


class Fsdp1dWork(_MeshWorkUnavailable):
    """Muon work for an FSDP2 1-D mesh (muon_utils.py:206-275): gather to an owner rank,
    orthogonalise there, scatter back.  Not built here; the owner-side computation is
    fast_newtonschulz on the gathered matrix."""


class TpFsdp2dWork(_MeshWorkUnavailable):
    """Muon work for TP + FSDP mesh (a stub in the reference too, muon_utils.py:278-284)."""


class EpFsdp2dWork(_MeshWorkUnavailable):
    """Muon work for EP mesh (stub, muon_utils.py:287-293)."""


class TpEpFsdp3dWork(_MeshWorkUnavailable):
    """Muon work for TP + EP mesh (stub, muon_utils.py:296-302)."""


class SingelDeviceWork:
    """Muon step for one parameter on one device (muon_utils.py:305-328): a bucket of one."""

    def __init__(self, param, state, group, index: int):
        self.param = param
        self.state = state
        self.group = group
        self.reference_bug_compat = False
        self.write_back_grad = False

    def start(self):
        g = self.group
        ns_steps, nesterov = g["ns_steps"], g["nesterov"]
        if self.reference_bug_compat:
            ns_steps, nesterov = int(bool(g["nesterov"])), bool(g["ns_steps"])
        _muon_bucket_step([self.param], [self.param.grad], [self.state["momentum_buffer"]], g, ns_steps, nesterov,
                          self.write_back_grad, {}, 1 << 62)

    def finish(self):
        pass


# --------------------------------------------------------------------------------------
# the optimizer (muon_utils.py:331-482)
# --------------------------------------------------------------------------------------
class Muon(torch.optim.Optimizer):
    def __init__(
        self,
        param_groups,
        defaults=dict(lr=0.02),
        is_deepspeed_enabled=False,
        *,
        momentum_dtype: Optional[torch.dtype] = None,
        reference_bug_compat: bool = False,
        write_back_grad: bool = False,
        workspace_limit_bytes: int = DEFAULT_WORKSPACE_LIMIT,
        keep_workspace: bool = True,
    ):
        self.is_deepspeed_enabled = is_deepspeed_enabled
        self.momentum_dtype = momentum_dtype
        self.reference_bug_compat = reference_bug_compat
        self.write_back_grad = write_back_grad
        self.workspace_limit_bytes = int(workspace_limit_bytes)
        self.keep_workspace = bool(keep_workspace)
        self._workspaces = {}
        self._pointer_tables = _TableCache()  # per bucket chunk: the device pointer table of the last step
        self._recorded = False     # a step has been recorded into a HIP graph: workspace and tables must stay
        if not reference_bug_compat and not is_deepspeed_enabled:
            _note_keyword_semantics()
        for group in param_groups:
            assert "use_muon" in group
            if group["use_muon"]:
                # largest first; python's sort is stable, ties keep their order
                group["params"] = sorted(group["params"], key=lambda x: x.size(), reverse=True)
                group["lr"] = group.get("lr", 0.02)
                group["momentum"] = group.get("momentum", 0.95)
                group["weight_decay"] = group.get("weight_decay", 0)
                rms_scale = group.get("rms_scale", True)
                if self.is_deepspeed_enabled and rms_scale:
                    logger.warning("rms_scale for Muon is not supported in deepspeed, setting rms_scale to False")
                    rms_scale = False
                group["rms_scale"] = rms_scale
                nesterov = group.get("nesterov", True)
                if self.is_deepspeed_enabled and not nesterov:
                    # the reference warns that it will force True and then stores False; kept as is
                    logger.warning("disabled nesterov for Muon is not supported in deepspeed, setting nesterov to True")
                    nesterov = False
                group["nesterov"] = nesterov
                group["ns_steps"] = group.get("ns_steps", 5)
                assert set(group.keys()) == _MUON_KEYS
            else:
                group["lr"] = group.get("lr", 3e-4)
                group["betas"] = group.get("betas", (0.9, 0.95))
                group["eps"] = group.get("eps", 1e-10)
                group["weight_decay"] = group.get("weight_decay", 0)
                assert set(group.keys()) == _ADAM_KEYS
        super().__init__(param_groups, defaults=defaults)

    def _get_work_class(self, p: torch.Tensor) -> tuple[type[Work], int]:
        """Work class and prefetch depth by mesh dimension (muon_utils.py:374-386)."""
        if isinstance(p, DTensor):
            if p.device_mesh.ndim == 1:
                return Fsdp1dWork, 8
            elif p.device_mesh.ndim == 2:
                return TpFsdp2dWork, 8
            else:
                raise ValueError(f"Unsupported mesh dimension: {p.device_mesh.ndim}")
        else:
            return SingelDeviceWork, 1

    @torch.no_grad()
    def step(self, closure=None):
        if self.is_deepspeed_enabled:
            return self.step_deepspeed(closure)
        else:
            return self.step_fsdp(closure)

    @torch.no_grad()
    def step_deepspeed(self, closure=None):
        """muon_utils.py:395-432.  Under DeepSpeed the orthogonalised update already sits in p.grad, so a Muon group
        only decays and updates (:405-407); the Adam groups run the same arithmetic as step_fsdp (the reference
        imports DeepSpeed's copy of adam_update there, the formula of :178-183)."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        lib = _abi.lib()
        for group in self.param_groups:
            if group["use_muon"]:
                for p in group["params"]:
                    _require_cuda(p, "a Muon parameter")
                    u = p.grad.reshape(p.shape)
                    u = u if u.is_contiguous() else u.contiguous()
                    pc = p if p.is_contiguous() else p.detach().contiguous()  # row-major copy, written back below
                    with torch.cuda.device(p.device):
                        _abi.check(
                            lib.muon_hip_decay_update(pc.data_ptr(), _abi.dtype_code(p.dtype), u.data_ptr(),
                                                      _abi.dtype_code(u.dtype), p.numel(), float(group["lr"]),
                                                      float(group["weight_decay"]), _abi.stream_ptr(p.device)),
                            "decay_update",
                        )
                    if pc is not p:
                        p.copy_(pc)
            else:
                self._adam_group_step(group)
        return loss

    def release_workspace(self) -> None:
        """Drop the Newton-Schulz workspace (it is re-allocated by the next step): for callers that want the
        memory back between optimizer steps, e.g. for activations.  A HIP graph recorded from step() holds the
        workspace's address, so after a recording the workspace stays until `forget_recordings()` says that no such
        graph will be replayed any more."""
        if self._recorded:
            raise RuntimeError("a recorded HIP graph replays into this workspace: call forget_recordings() once the "
                               "graph is gone, then release_workspace()")
        self._workspaces.clear()

    def forget_recordings(self) -> None:
        """Declare that no HIP graph recorded from step() will be replayed again."""
        self._recorded = False

    def _adam_group_step(self, group) -> None:
        items = []
        for p in group["params"]:
            if p.grad is None:
                p.grad = torch.zeros_like(p)
            state = self.state[p]
            if len(state) == 0:
                state["exp_avg"] = torch.zeros_like(p)
                state["exp_avg_sq"] = torch.zeros_like(p)
                state["step"] = 0
            state["step"] += 1
            items.append((p, p.grad, state["exp_avg"], state["exp_avg_sq"], state["step"]))
        _adamw_group(items, group)

    def load_state_dict(self, state_dict) -> None:
        """torch casts every floating state tensor to the parameter's dtype on load; put an
        fp32 momentum buffer back when `momentum_dtype` asks for one."""
        super().load_state_dict(state_dict)
        if self.momentum_dtype is None:
            return
        saved_ids = chain.from_iterable(g["params"] for g in state_dict["param_groups"])
        params = chain.from_iterable(g["params"] for g in self.param_groups)
        for sid, p in zip(saved_ids, params):
            st = state_dict["state"].get(sid)
            if st is not None and "momentum_buffer" in st:
                self.state[p]["momentum_buffer"] = st["momentum_buffer"].to(device=p.device, dtype=self.momentum_dtype)

    def _init_muon_state(self, p: Tensor) -> dict:
        state = self.state[p]
        if len(state) == 0:
            state["momentum_buffer"] = torch.zeros_like(p, dtype=self.momentum_dtype or p.dtype)
        return state

    @torch.no_grad()
    def step_fsdp(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        dq: deque[Work] = deque()
        if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
            if not self.keep_workspace:
                raise RuntimeError("recording a step into a HIP graph needs keep_workspace=True: replays use the workspace")
            self._recorded = True
        for group in self.param_groups:
            if group["use_muon"]:
                buckets: "OrderedDict[tuple, list]" = OrderedDict()
                strided = []
                for i, p in enumerate(group["params"]):
                    assert p.ndim == 2, p.shape
                    if p.grad is None:
                        p.grad = torch.zeros_like(p)
                    state = self._init_muon_state(p)
                    class_work, prefetch_factor = self._get_work_class(p)
                    if class_work is not SingelDeviceWork:
                        work = class_work(p, state, group, i)
                        work.start()
                        dq.append(work)
                        if len(dq) > prefetch_factor:
                            dq.popleft().finish()
                        continue
                    _require_cuda(p, "a Muon parameter")
                    # The kernels read row-major tensors.  A parameter, gradient or momentum buffer with other strides
                    # (the reference's torch expressions take any) steps through row-major copies that are written back.
                    g = p.grad if p.grad.is_contiguous() else p.grad.contiguous()
                    m = state["momentum_buffer"]
                    pc = p if p.is_contiguous() else p.detach().contiguous()
                    mc = m if m.is_contiguous() else m.contiguous()
                    if pc is not p or mc is not m or (g is not p.grad and self.write_back_grad):
                        strided.append((p, pc, m, mc, g))
                    key = (p.device, tuple(p.shape), p.dtype, g.dtype, m.dtype)
                    buckets.setdefault(key, []).append((pc, g, mc))
                ns_steps, nesterov = group["ns_steps"], group["nesterov"]
                if self.reference_bug_compat:
                    ns_steps, nesterov = int(bool(group["nesterov"])), bool(group["ns_steps"])
                for items in buckets.values():
                    ps, gs, ms = (list(t) for t in zip(*items))
                    _muon_bucket_step(ps, gs, ms, group, ns_steps, nesterov, self.write_back_grad, self._workspaces,
                                      self.workspace_limit_bytes, self._pointer_tables)
                for p, pc, m, mc, g in strided:
                    if pc is not p:
                        p.copy_(pc)
                    if mc is not m:
                        m.copy_(mc)
                    if g is not p.grad and self.write_back_grad:
                        p.grad.copy_(g)
            else:
                self._adam_group_step(group)

        if not self.keep_workspace:
            self.release_workspace()
        for work in dq:
            work.finish()

        return loss


def _adamw_group(items, group: dict) -> None:
    """The Adam branch of step_fsdp (muon_utils.py:458-477) for a whole parameter group: one launch per
    (device, dtype) over all its tensors.  Every parameter carries its own step, so the two bias
    corrections travel as per-tensor doubles."""
    from .multi_tensor import TensorListTable

    buckets: "OrderedDict[tuple, list]" = OrderedDict()
    strided = []  # tensors with other than row-major strides step through row-major copies that are written back
    for p, grad, e1, e2, step in items:
        _require_cuda(p, "an AdamW parameter")
        if e1.dtype != p.dtype or e2.dtype != p.dtype:
            raise NotImplementedError("AdamW-fallback state must have the parameter's dtype")
        if p.numel() == 0:
            continue
        g = grad
        if g.dtype != p.dtype or not g.is_contiguous():
            g = g.to(p.dtype).contiguous()
        if not (p.is_contiguous() and e1.is_contiguous() and e2.is_contiguous()):
            pairs = [(t, t if t.is_contiguous() else t.detach().contiguous()) for t in (p, e1, e2)]
            strided.extend(pr for pr in pairs if pr[0] is not pr[1])
            p, e1, e2 = (c for _, c in pairs)
        buckets.setdefault((p.device, p.dtype), []).append((p, g, e1, e2, step))
    b1, b2 = float(group["betas"][0]), float(group["betas"][1])
    for (dev, dt), its in buckets.items():
        ps, gs, e1s, e2s, steps = (list(t) for t in zip(*its))
        with torch.cuda.device(dev):
            tab = TensorListTable([ps, gs, e1s, e2s], doubles=[[1 - b1 ** st for st in steps], [1 - b2 ** st for st in steps]])
            _abi.check(
                _abi.lib().muon_hip_adamw_multi(
                    *tab.role_ptrs, tab.numel_ptr, tab.chunk_start_ptr, *tab.double_ptrs, tab.n, tab.chunks,
                    _abi.dtype_code(dt), float(group["lr"]), b1, b2, float(group["eps"]), float(group["weight_decay"]),
                    _abi.stream_ptr(dev),
                ),
                "adamw_multi",
            )
    for t, c in strided:
        t.copy_(c)


def _adamw_tensor(p: Tensor, grad: Tensor, exp_avg: Tensor, exp_avg_sq: Tensor, step: int, group: dict) -> None:
    """adam_update + decoupled decay + update (muon_utils.py:178-183, :468-477) in one kernel."""
    _require_cuda(p, "an AdamW parameter")
    if not (p.is_contiguous() and exp_avg.is_contiguous() and exp_avg_sq.is_contiguous()):
        raise NotImplementedError("AdamW-fallback parameters and state must be contiguous")
    g = grad
    if g.dtype != p.dtype or not g.is_contiguous():
        g = g.to(p.dtype).contiguous()
    with torch.cuda.device(p.device):
        _abi.check(
            _abi.lib().muon_hip_adamw(
                p.data_ptr(), g.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(), _abi.dtype_code(p.dtype),
                p.numel(), int(step), float(group["lr"]), float(group["betas"][0]), float(group["betas"][1]),
                float(group["eps"]), float(group["weight_decay"]), _abi.stream_ptr(p.device),
            ),
            "adamw",
        )
