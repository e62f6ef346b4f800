"""ctypes binding of libmuon_hip.so (the C ABI declared in include/muon_hip.h).

The library is loaded lazily, on the first call that needs it, and a missing library is an
error: there is no fallback implementation.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_int, c_long, c_size_t, c_void_p, POINTER

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmuon_hip.so")

F32, BF16 = 0, 1
CFG_AUTO, CFG_128_PIPE, CFG_256_PIPE, CFG_256_PINGPONG, CFG_128_PINGPONG, CFG_256_PERSIST = -1, 0, 1, 2, 3, 4
GEMM_CONFIGS = list(range(4))
K_MOMENTUM, K_NORMALIZE, K_SYRK, K_SYMPOLY, K_BX, K_UPDATE, K_ADAMW, K_ADAMW_MULTI, K_GRAD_NORM, K_CLIP_SCALE = range(10)
KERNEL_NAMES = ["momentum_norm", "normalize", "syrk", "sympoly", "bx_axpy", "apply_update", "adamw", "adamw_multi",
                "grad_norm", "clip_scale", "bx_axpy_update"]
MULTI_CHUNK = 16384  # MUON_HIP_MULTI_CHUNK
STATIC_MAX_CHUNKS = 1 << 20  # MUON_HIP_STATIC_MAX_CHUNKS
PPX_COUNTER_BYTES = 576  # MUON_HIP_PPX_COUNTER_BYTES

# name -> (restype, argtypes); mirrors include/muon_hip.h one to one
SIGNATURES = {
    "muon_hip_version": (c_int, []),
    "muon_hip_last_error": (c_char_p, []),
    "muon_hip_geometry": (c_int, [c_int, c_int] + [POINTER(c_int)] * 5),
    "muon_hip_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "muon_hip_set_gemm_config": (c_int, [c_int]),
    "muon_hip_momentum_norm": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_double,
                                       c_int, c_int, c_void_p]),
    "muon_hip_cast_norm": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "muon_hip_normalize": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p]),
    "muon_hip_ns_grouped": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_double, c_double, c_double, c_void_p]),
    "muon_hip_apply_update": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_double, c_double,
                                      c_double, c_void_p]),
    "muon_hip_ns_output": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "muon_hip_step_grouped": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int,
                                      c_double, c_double, c_double, c_int, c_int, c_double, c_double, c_double,
                                      c_double, c_int, c_void_p]),
    "muon_hip_blocked_elems": (c_long, [c_int, c_int]),
    "muon_hip_pack_bf16": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "muon_hip_unpack_bf16": (c_int, [c_void_p, c_int, c_int, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p]),
    "muon_hip_syrk_bf16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "muon_hip_sympoly_bf16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_double, c_double, c_int, c_void_p, c_void_p]),
    "muon_hip_bx_axpy_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_double, c_int, c_void_p,
                                      c_void_p]),
    "muon_hip_adamw": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_double, c_double,
                               c_double, c_double, c_double, c_void_p]),
    "muon_hip_adam_update": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_double, c_double,
                                     c_double, c_void_p]),
    "muon_hip_scale": (c_int, [c_void_p, c_int, c_long, c_double, c_void_p]),
    "muon_hip_decay_update": (c_int, [c_void_p, c_int, c_void_p, c_int, c_long, c_double, c_double, c_void_p]),
    "muon_hip_adamw_multi": (c_int, [c_void_p] * 8 + [c_int, c_long, c_int] + [c_double] * 5 + [c_void_p]),
    "muon_hip_grad_norms": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_double, c_void_p, c_void_p, c_void_p]),
    "muon_hip_grad_norms_static": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_double, c_void_p, c_void_p]),
    "muon_hip_total_norm": (c_int, [c_void_p, c_int, c_int, c_double, c_void_p, c_void_p, c_void_p]),
    "muon_hip_clip_scale": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_void_p, c_int, c_double,
                                    c_void_p]),
    "muon_hip_device_shape": (c_int, [POINTER(c_int), POINTER(c_int)]),
    "muon_hip_timing_reserve": (c_int, [c_long]),
    "muon_hip_timing_untimed": (c_long, []),
    "muon_hip_timing_enable": (c_int, [c_int]),
    "muon_hip_timing_read": (c_int, [c_int, POINTER(c_double), POINTER(c_long)]),
}

_lib = None


class MuonHipError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MuonHipError(
                f"{LIB_PATH} is missing: build it with `python -m lmms_engine_amd.build` "
                "(hipcc, gfx950). There is no fallback path."
            )
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        msg = lib().muon_hip_last_error().decode()
        raise MuonHipError(f"{what or 'muon_hip'} failed (code {rc}): {msg}")


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise TypeError(f"libmuon_hip supports float32 and bfloat16 tensors, got {dt}")


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def geometry(rows: int, cols: int):
    out = [c_int() for _ in range(5)]
    check(lib().muon_hip_geometry(rows, cols, *[ctypes.byref(o) for o in out]), "geometry")
    M, K, Mp, Kp, tile = (o.value for o in out)
    return dict(M=M, K=K, Mp=Mp, Kp=Kp, tile=tile)


def workspace_bytes(rows: int, cols: int, batch: int) -> int:
    n = lib().muon_hip_workspace_bytes(rows, cols, batch)
    if n == 0:
        raise MuonHipError(f"workspace_bytes({rows}, {cols}, {batch}): " + lib().muon_hip_last_error().decode())
    return n


def device_shape():
    """(compute units, XCDs) of the current device."""
    cus, xcds = c_int(), c_int()
    check(lib().muon_hip_device_shape(ctypes.byref(cus), ctypes.byref(xcds)), "device_shape")
    return cus.value, xcds.value


def timing_enable(on: bool, reserve: int = 0) -> None:
    """Switch per-kernel event timing on or off; `reserve` event pairs are created first, so that none has to be
    created while the clock runs (launches beyond the pool go untimed and are counted by muon_hip_timing_untimed)."""
    if on and reserve:
        check(lib().muon_hip_timing_enable(0), "timing_enable")
        check(lib().muon_hip_timing_reserve(int(reserve)), "timing_reserve")
    check(lib().muon_hip_timing_enable(int(on)), "timing_enable")


def timing_read():
    """{kernel name: (total_ms, launches)} since timing was enabled; waits for the events."""
    out = {}
    for kid, name in enumerate(KERNEL_NAMES):
        ms, cnt = c_double(), c_long()
        check(lib().muon_hip_timing_read(kid, ctypes.byref(ms), ctypes.byref(cnt)), "timing_read")
        out[name] = (ms.value, cnt.value)
    return out
