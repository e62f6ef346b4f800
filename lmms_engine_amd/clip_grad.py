"""Gradient-norm clipping on one GPU, the call that precedes `optimizer.step()`.

Mirror of `fsdp2_clip_grad_norm_` (src/lmms_engine/utils/fsdp2_utils.py:234-255) when no process
group is active: torch's `_get_total_norm` followed by `_clip_grads_with_norm_`.  The norm of every
gradient, the norm of those norms and the in-place scaling each run as one multi-tensor kernel per
dtype; nothing synchronises the host unless `error_if_nonfinite` asks for the value.
"""
from __future__ import annotations

from collections import OrderedDict

import torch
from torch import Tensor

from . import _abi
from .multi_tensor import TensorListTable


@torch.no_grad()
def clip_grad_norm_(parameters, max_norm, norm_type=2.0, error_if_nonfinite=False, foreach=None) -> Tensor:
    """Same signature and return value (the total norm, a 0-d tensor on the gradients' device) as
    fsdp2_clip_grad_norm_.  `norm_type` is any order torch.linalg.vector_norm takes: 2 (the default), 1, 0, inf and
    -inf have reductions of their own, every other p is (sum |x|^p)^(1/p) accumulated in fp32 as torch does.
    `foreach` is accepted and ignored (every call is one launch per dtype)."""
    if isinstance(parameters, Tensor):
        parameters = [parameters]
    else:
        parameters = list(parameters)
    norm_type = float(norm_type)
    if norm_type != norm_type:
        raise ValueError("norm_type is NaN")
    grads = [p.grad for p in parameters if p.grad is not None]
    if len(grads) == 0:
        return torch.tensor(0.0)  # what _get_total_norm returns for an empty list
    for g in grads:
        if not g.is_cuda:
            raise _abi.MuonHipError(f"gradients must live on a GPU: this build has no CPU path (got {g.device})")
    dev = grads[0].device
    groups: "OrderedDict[torch.dtype, list]" = OrderedDict()
    strided = []  # gradients with other than row-major strides are scaled through a row-major copy that is written back
    for g in grads:
        if g.device != dev:
            raise NotImplementedError("gradients on several devices")
        c = g if g.is_contiguous() else g.contiguous()
        if c is not g:
            strided.append((g, c))
        groups.setdefault(g.dtype, []).append(c)
    lib = _abi.lib()
    # torch stacks the per-tensor norms of all dtype groups; stacking promotes, so the total has the widest dtype
    out_dtype = torch.float32 if torch.float32 in groups else torch.bfloat16
    n_total = len(grads)
    with torch.cuda.device(dev):
        s = _abi.stream_ptr(dev)
        norms = torch.empty(n_total, dtype=torch.float32, device=dev)
        total_f32 = torch.empty(1, dtype=torch.float32, device=dev)
        total = torch.empty((), dtype=out_dtype, device=dev)
        tables, off = [], 0
        for dt, gs in groups.items():
            tab = TensorListTable([gs])
            tables.append((dt, tab))
            if tab.chunks > 0:
                partials = torch.empty(tab.chunks, dtype=torch.float32, device=dev)
                _abi.check(lib.muon_hip_grad_norms(tab.role_ptrs[0], tab.numel_ptr, tab.chunk_start_ptr, tab.n, tab.chunks,
                                                   _abi.dtype_code(dt), norm_type, partials.data_ptr(), norms.data_ptr() + 4 * off, s),
                           "grad_norms")
            else:
                norms[off:off + tab.n].zero_()
            off += tab.n
        _abi.check(lib.muon_hip_total_norm(norms.data_ptr(), n_total, _abi.dtype_code(out_dtype), norm_type, total_f32.data_ptr(),
                                           total.data_ptr(), s), "total_norm")
        if error_if_nonfinite and not bool(torch.isfinite(total)):
            raise RuntimeError(
                f"The total norm of order {norm_type} for gradients from `parameters` is non-finite, so it "
                "cannot be clipped. To disable this error and scale the gradients by the non-finite norm anyway, "
                "set `error_if_nonfinite=False`")
        for dt, tab in tables:
            if tab.chunks > 0:
                _abi.check(lib.muon_hip_clip_scale(tab.role_ptrs[0], tab.numel_ptr, tab.chunk_start_ptr, tab.n, tab.chunks,
                                                   _abi.dtype_code(dt), total_f32.data_ptr(), _abi.dtype_code(out_dtype),
                                                   float(max_norm), s), "clip_scale")
        for g, c in strided:
            g.copy_(c)
    return total


fsdp2_clip_grad_norm_ = clip_grad_norm_
