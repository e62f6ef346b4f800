"""Device-side description of a list of tensors for the multi-tensor kernels of libmuon_hip.

One pinned host buffer holds, as int64 words, the base pointers of every tensor role (one row
per role: parameters, grads, ...), the element counts, the first-chunk index of every tensor
(n + 1 entries) and any per-tensor doubles (bit patterns); one asynchronous copy puts it on
the device.  The layout is the one include/muon_hip.h documents for muon_hip_adamw_multi,
muon_hip_grad_norms and muon_hip_clip_scale.
"""
from __future__ import annotations

import struct
from typing import Sequence

import torch
from torch import Tensor

from . import _abi


class TensorListTable:
    def __init__(self, roles: Sequence[Sequence[Tensor]], doubles: Sequence[Sequence[float]] = ()):
        n = len(roles[0])
        assert n > 0 and all(len(r) == n for r in roles) and all(len(d) == n for d in doubles)
        first = roles[0][0]
        for r in roles:
            for t, ref in zip(r, roles[0]):
                if not t.is_cuda:
                    raise _abi.MuonHipError(f"tensors must live on a GPU: this build has no CPU path (got {t.device})")
                if t.device != first.device or t.dtype != first.dtype or t.numel() != ref.numel():
                    raise ValueError("a tensor list holds tensors of one device and dtype; roles must match in size")
                if not t.is_contiguous():
                    raise NotImplementedError("multi-tensor kernels need contiguous tensors")
        self.n = n
        self.device = first.device
        self.dtype = first.dtype
        numel = [t.numel() for t in roles[0]]
        starts = [0]
        for ne in numel:
            starts.append(starts[-1] + (ne + _abi.MULTI_CHUNK - 1) // _abi.MULTI_CHUNK)
        self.chunks = starts[-1]
        words = []
        for r in roles:
            words.extend(t.data_ptr() for t in r)
        words.extend(numel)
        words.extend(starts)
        for d in doubles:
            words.extend(struct.unpack("<q", struct.pack("<d", float(v)))[0] for v in d)
        host = torch.tensor(words, dtype=torch.int64, pin_memory=True)
        self.table = host.to(self.device, non_blocking=True)
        self._keep = (host, [list(r) for r in roles])  # the tensors stay alive while kernels may read them
        base, k = self.table.data_ptr(), len(roles)
        self.role_ptrs = [base + 8 * n * i for i in range(k)]
        self.numel_ptr = base + 8 * n * k
        self.chunk_start_ptr = self.numel_ptr + 8 * n
        self.double_ptrs = [self.chunk_start_ptr + 8 * (n + 1) + 8 * n * i for i in range(len(doubles))]
