"""MI355X-native Muon optimizer step (drop-in for lmms_engine.utils.muon_utils)."""
from .muon_utils import (  # noqa: F401
    Muon,
    SingelDeviceWork,
    Work,
    adam_update,
    apply_momentum,
    apply_scaling,
    fast_newtonschulz,
    matmul_transpose,
    matmul_transpose_assign,
    muon_update,
)

__all__ = [
    "Muon",
    "SingelDeviceWork",
    "Work",
    "adam_update",
    "apply_momentum",
    "apply_scaling",
    "fast_newtonschulz",
    "matmul_transpose",
    "matmul_transpose_assign",
    "muon_update",
]
