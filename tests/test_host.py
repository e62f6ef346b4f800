"""Host-side contract of the Muon drop-in, checked without a GPU: constructor defaults,
asserts and sort order (muon_utils.py:332-372), work-class dispatch (:374-386), the loud
failure when tensors are not on a GPU, and that libmuon_hip.so loads and exports every
symbol include/muon_hip.h declares (no compute calls here)."""
import ctypes
import os
import re

import pytest
import torch

from lmms_engine_amd import _abi, muon_utils
from lmms_engine_amd.muon_utils import Muon

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def P(*shape):
    return torch.nn.Parameter(torch.zeros(*shape))


def test_muon_group_defaults_and_keys():
    g = dict(params=[P(4, 3)], use_muon=True)
    opt = Muon([g])
    assert g["lr"] == 0.02 and g["momentum"] == 0.95 and g["weight_decay"] == 0
    assert g["rms_scale"] is True and g["nesterov"] is True and g["ns_steps"] == 5
    assert set(g.keys()) == {"params", "lr", "momentum", "weight_decay", "use_muon", "rms_scale", "nesterov", "ns_steps"}
    assert opt.defaults == dict(lr=0.02) and opt.is_deepspeed_enabled is False
    assert opt.param_groups[0] is g or opt.param_groups[0]["params"][0] is g["params"][0]


def test_adam_group_defaults_and_keys():
    g = dict(params=[P(7)], use_muon=False)
    Muon([g])
    assert g["lr"] == 3e-4 and g["betas"] == (0.9, 0.95) and g["eps"] == 1e-10 and g["weight_decay"] == 0
    assert set(g.keys()) == {"params", "lr", "betas", "eps", "weight_decay", "use_muon"}


def test_given_values_are_kept():
    g = dict(params=[P(4, 3)], use_muon=True, lr=1e-3, momentum=0.9, weight_decay=0.1, rms_scale=False, nesterov=False,
             ns_steps=3)
    Muon([g], defaults=dict(lr=1e-3))
    assert (g["lr"], g["momentum"], g["weight_decay"], g["rms_scale"], g["nesterov"], g["ns_steps"]) == (1e-3, 0.9, 0.1, False, False, 3)


def test_asserts():
    with pytest.raises(AssertionError):
        Muon([dict(params=[P(4, 3)])])  # use_muon missing
    with pytest.raises(AssertionError):
        Muon([dict(params=[P(4, 3)], use_muon=True, betas=(0.9, 0.95))])  # foreign key in a Muon group
    with pytest.raises(AssertionError):
        Muon([dict(params=[P(4)], use_muon=False, momentum=0.9)])  # foreign key in an Adam group


def test_params_sorted_by_size_descending_and_stable():
    ps = [P(2, 3), P(5, 1), P(2, 3), P(5, 4)]
    opt = Muon([dict(params=list(ps), use_muon=True)])
    got = opt.param_groups[0]["params"]
    assert [tuple(p.shape) for p in got] == [(5, 4), (5, 1), (2, 3), (2, 3)]
    assert got[2] is ps[0] and got[3] is ps[2], "ties keep their order"


def test_trainer_factory_shaped_groups_with_empty_lists():
    """The four dicts Trainer.create_optimizer builds (train/hf/trainer.py:417-448), some empty."""
    w, e = P(8, 8), P(10)
    groups = [
        dict(params=[], use_muon=True, lr=1e-3, momentum=0.95, weight_decay=0.01),
        dict(params=[w], use_muon=True, lr=1e-3, momentum=0.95, weight_decay=0.0),
        dict(params=[], use_muon=False, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01),
        dict(params=[e], use_muon=False, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0),
    ]
    opt = Muon(groups, defaults=dict(lr=1e-3), is_deepspeed_enabled=False)
    assert len(opt.param_groups) == 4
    sd = opt.state_dict()
    assert sd["state"] == {} and [g["params"] for g in sd["param_groups"]] == [[], [0], [], [1]]


def test_deepspeed_quirks_kept():
    g = dict(params=[P(4, 3)], use_muon=True, nesterov=False)
    opt = Muon([g], is_deepspeed_enabled=True)
    assert g["rms_scale"] is False, "DeepSpeed forces rms_scale off"
    assert g["nesterov"] is False, "the reference warns but keeps False"
    g["params"][0].grad = torch.zeros(4, 3)
    with pytest.raises(_abi.MuonHipError, match="no CPU path"):
        opt.step()  # dispatches to step_deepspeed, which has no CPU path either


# every top-level name of the reference module (muon_utils.py:13, 33, 95, 122, 129, 159, 167, 178, 186, 195, 206,
# 278, 287, 296, 305, 331)
REFERENCE_MODULE_NAMES = [
    "get_autotune_config", "mmt_kernel", "matmul_transpose_assign", "matmul_transpose", "fast_newtonschulz",
    "apply_momentum", "apply_scaling", "adam_update", "muon_update", "Work", "Fsdp1dWork", "TpFsdp2dWork",
    "EpFsdp2dWork", "TpEpFsdp3dWork", "SingelDeviceWork", "Muon",
]


def test_module_substitution_is_name_complete(monkeypatch):
    """Installing this module under the reference's import path: `from lmms_engine.utils.muon_utils import Muon`
    (train/hf/trainer.py:459) then resolves here, and so does every other public name of the reference module."""
    import importlib
    import sys
    import types

    pkg, sub = types.ModuleType("lmms_engine"), types.ModuleType("lmms_engine.utils")
    pkg.utils, sub.muon_utils = sub, muon_utils
    monkeypatch.setitem(sys.modules, "lmms_engine", pkg)
    monkeypatch.setitem(sys.modules, "lmms_engine.utils", sub)
    monkeypatch.setitem(sys.modules, "lmms_engine.utils.muon_utils", muon_utils)
    mod = importlib.import_module("lmms_engine.utils.muon_utils")
    assert mod is muon_utils
    from lmms_engine.utils.muon_utils import Muon as Swapped  # the factory's own import line

    assert Swapped is Muon
    for name in REFERENCE_MODULE_NAMES:
        assert hasattr(mod, name), f"{name} is a public name of the reference module"
    import inspect

    assert list(inspect.signature(mod.adam_update).parameters) == ["grad", "buf1", "buf2", "step", "betas", "eps"]
    assert list(inspect.signature(mod.muon_update).parameters) == ["grad", "momentum", "beta", "ns_steps", "nesterov", "rms_scale"]
    assert list(inspect.signature(mod.apply_momentum).parameters) == ["grad", "momentum", "beta", "nesterov"]
    assert list(inspect.signature(mod.Muon.__init__).parameters)[:4] == ["self", "param_groups", "defaults", "is_deepspeed_enabled"]
    assert len(mod.get_autotune_config()) == 5


def test_keyword_semantics_are_announced_once(caplog):
    import logging

    muon_utils._noted_semantics = False
    with caplog.at_level(logging.WARNING, logger=muon_utils.logger.name):
        Muon([dict(params=[P(4, 3)], use_muon=True)])
        Muon([dict(params=[P(4, 3)], use_muon=True)])
    assert sum("reference_bug_compat" in r.message for r in caplog.records) == 1
    caplog.clear()
    muon_utils._noted_semantics = False
    with caplog.at_level(logging.WARNING, logger=muon_utils.logger.name):
        Muon([dict(params=[P(4, 3)], use_muon=True)], reference_bug_compat=True)
    assert not caplog.records


def test_work_class_dispatch():
    opt = Muon([dict(params=[P(4, 3)], use_muon=True)])
    cls, prefetch = opt._get_work_class(torch.zeros(2, 2))
    assert cls is muon_utils.SingelDeviceWork and prefetch == 1
    for stub in (muon_utils.Fsdp1dWork, muon_utils.TpFsdp2dWork, muon_utils.EpFsdp2dWork, muon_utils.TpEpFsdp3dWork):
        with pytest.raises(NotImplementedError):
            stub(None, None, None, 0)


def test_cpu_tensors_fail_loudly():
    p = P(4, 3)
    p.grad = torch.zeros(4, 3)
    opt = Muon([dict(params=[p], use_muon=True)])
    with pytest.raises(_abi.MuonHipError, match="no CPU path"):
        opt.step()
    q = P(5)
    q.grad = torch.zeros(5)
    with pytest.raises(_abi.MuonHipError, match="no CPU path"):
        Muon([dict(params=[q], use_muon=False)]).step()
    with pytest.raises(_abi.MuonHipError):
        muon_utils.fast_newtonschulz(torch.zeros(4, 4))
    with pytest.raises(AssertionError):
        muon_utils.matmul_transpose(torch.zeros(4, 4, dtype=torch.bfloat16))


def test_non_2d_muon_param_asserts_before_any_kernel():
    p = P(5)
    p.grad = torch.zeros(5)
    with pytest.raises(AssertionError):
        Muon([dict(params=[p], use_muon=True)]).step()


def test_scale_factor():
    assert muon_utils.scale_factor(4864, 896, False) == (4864 / 896) ** 0.5
    assert muon_utils.scale_factor(896, 4864, False) == 1.0
    assert muon_utils.scale_factor(896, 4864, True) == 0.2 * 4864 ** 0.5


def test_missing_library_is_an_error(monkeypatch):
    monkeypatch.setattr(_abi, "_lib", None)
    monkeypatch.setattr(_abi, "LIB_PATH", "/nonexistent/libmuon_hip.so")
    with pytest.raises(_abi.MuonHipError, match="no fallback"):
        _abi.lib()


# ---- the C ABI ----------------------------------------------------------------------------
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "muon_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(muon_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 17
    lib = ctypes.CDLL(_abi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/muon_hip.h but not exported"
    assert set(names) == set(_abi.SIGNATURES), "the ctypes table mirrors the header one to one"


def test_host_only_entry_points():
    lib = _abi.lib()
    assert lib.muon_hip_version() >= 100
    geo = _abi.geometry(896, 4864)
    assert geo == dict(M=896, K=4864, Mp=896, Kp=4864, tile=128)
    geo = _abi.geometry(12288, 4096)
    assert (geo["M"], geo["K"], geo["tile"]) == (4096, 12288, 256)
    assert _abi.geometry(100, 300) == dict(M=100, K=300, Mp=128, Kp=384, tile=128)
    w1, w2 = _abi.workspace_bytes(896, 4864, 1), _abi.workspace_bytes(896, 4864, 2)
    assert w1 >= 4 * 896 * 4864 + 4 * 896 * 896 and w1 < w2 <= 2 * w1 + 4096  # X twice, A, B (bf16)
    assert lib.muon_hip_workspace_bytes(0, 4, 1) == 0 and b"positive" in lib.muon_hip_last_error()
    assert lib.muon_hip_set_gemm_config(99) == -1
    assert lib.muon_hip_set_gemm_config(_abi.CFG_256_PIPE) == 0
    try:
        assert _abi.geometry(896, 4864)["tile"] == 256 and _abi.geometry(896, 4864)["Mp"] == 1024
    finally:
        assert lib.muon_hip_set_gemm_config(_abi.CFG_AUTO) == 0
    with pytest.raises(TypeError):
        _abi.dtype_code(torch.float16)


def test_clip_grad_norm_host_behaviour():
    """What clip_grad_norm_ decides before any kernel runs: the empty cases return what torch's
    _get_total_norm returns, a NaN order and CPU gradients are refused (no fallback path)."""
    from lmms_engine_amd import _abi, clip_grad

    out = clip_grad.clip_grad_norm_([], 1.0)
    assert out.item() == 0.0 and out.device.type == "cpu"
    p = torch.nn.Parameter(torch.zeros(4))
    assert clip_grad.clip_grad_norm_(p, 1.0).item() == 0.0  # a bare tensor is accepted; no grad yet
    p.grad = torch.ones(4)
    with pytest.raises(ValueError):
        clip_grad.clip_grad_norm_([p], 1.0, norm_type=float("nan"))
    for norm_type in (3.0, 1.0, float("inf")):
        with pytest.raises(_abi.MuonHipError):
            clip_grad.clip_grad_norm_([p], 1.0, norm_type=norm_type)
    with pytest.raises(_abi.MuonHipError):
        clip_grad.clip_grad_norm_([p], 1.0)
    assert torch.equal(p.grad, torch.ones(4))  # untouched
    assert clip_grad.fsdp2_clip_grad_norm_ is clip_grad.clip_grad_norm_


def test_tensor_list_table_rejects_cpu_tensors():
    from lmms_engine_amd import _abi
    from lmms_engine_amd.multi_tensor import TensorListTable

    with pytest.raises(_abi.MuonHipError):
        TensorListTable([[torch.zeros(3)]])
    assert _abi.MULTI_CHUNK == 16384


def test_argument_errors_are_reported_before_any_launch():
    """Every entry point rejects what it cannot run with a negative code and a message, before it
    touches the device (so this runs without one)."""
    lib = _abi.lib()
    EINVAL, ESHAPE = -1, -2
    ws = 0x1000  # never dereferenced: every call below is rejected on its arguments
    tbl = 0x2000
    F32, BF16 = _abi.dtype_code(torch.float32), _abi.dtype_code(torch.bfloat16)

    def rejected(rc, code, needle):
        assert rc == code, (rc, lib.muon_hip_last_error())
        assert needle in lib.muon_hip_last_error().decode(), lib.muon_hip_last_error()

    rejected(lib.muon_hip_momentum_norm(tbl, tbl, F32, F32, None, 8, 8, 1, 0.95, 1, 0, None), EINVAL, "workspace is null")
    rejected(lib.muon_hip_momentum_norm(tbl, tbl, F32, F32, ws + 8, 8, 8, 1, 0.95, 1, 0, None), EINVAL, "256-byte aligned")
    rejected(lib.muon_hip_momentum_norm(None, tbl, F32, F32, ws, 8, 8, 1, 0.95, 1, 0, None), EINVAL, "pointer table")
    rejected(lib.muon_hip_momentum_norm(tbl, tbl, F32, BF16, ws, 8, 8, 1, 0.95, 1, 0, None), EINVAL, "dtypes")
    rejected(lib.muon_hip_momentum_norm(tbl, tbl, F32, F32, ws, 8, 8, 70000, 0.95, 1, 0, None), ESHAPE, "65535")
    rejected(lib.muon_hip_cast_norm(None, F32, ws, 8, 8, 1, None), EINVAL, "bad input")
    rejected(lib.muon_hip_cast_norm(tbl, 7, ws, 8, 8, 1, None), EINVAL, "bad input")
    rejected(lib.muon_hip_ns_grouped(ws, 8, 8, 1, -1, 1.0, 1.0, 1.0, None), EINVAL, "steps")
    rejected(lib.muon_hip_ns_grouped(ws, 0, 8, 1, 5, 1.0, 1.0, 1.0, None), EINVAL, "positive")
    rejected(lib.muon_hip_apply_update(None, F32, ws, 8, 8, 1, 5, 1.0, 0.02, 0.0, None), EINVAL, "bad pointer table")
    rejected(lib.muon_hip_apply_update(tbl, 9, ws, 8, 8, 1, 5, 1.0, 0.02, 0.0, None), EINVAL, "dtype")
    rejected(lib.muon_hip_ns_output(ws, 8, 8, 1, 5, None, None), EINVAL, "output pointer")
    rejected(lib.muon_hip_step_grouped(tbl, tbl, tbl, F32, F32, F32, None, 8, 8, 1, 0.02, 0.0, 0.95, 1, 5, 1.0,
                                       3.4445, -4.775, 2.0315, 0, None), EINVAL, "workspace is null")
    assert lib.muon_hip_blocked_elems(256, 48) == 0 and b"multiple of 32" in lib.muon_hip_last_error()
    assert lib.muon_hip_blocked_elems(300, 64) == 2 * 2 * 8192
    rejected(lib.muon_hip_pack_bf16(None, 0, 64, 8, 64, tbl, 256, 64, 1, None), EINVAL, "null tensor")
    rejected(lib.muon_hip_pack_bf16(tbl, 0, 32, 8, 64, tbl, 256, 64, 1, None), ESHAPE, "pack")
    rejected(lib.muon_hip_unpack_bf16(tbl, 256, 48, tbl, 0, 64, 8, 48, 1, None), ESHAPE, "unpack")
    rejected(lib.muon_hip_syrk_bf16(tbl, tbl, 256, 300, 1, _abi.CFG_AUTO, None, None), ESHAPE, "multiples")
    rejected(lib.muon_hip_syrk_bf16(tbl, tbl, 512, 512, 1, 17, None, None), EINVAL, "unknown GEMM configuration")
    rejected(lib.muon_hip_syrk_bf16(None, tbl, 512, 512, 1, _abi.CFG_AUTO, None, None), EINVAL, "null operand")
    rejected(lib.muon_hip_sympoly_bf16(tbl, tbl, 512, 1, 1.0, 1.0, _abi.CFG_AUTO, None, None), EINVAL, "aliased")
    rejected(lib.muon_hip_bx_axpy_bf16(tbl, tbl + 64, tbl + 64, 512, 512, 1, 1.0, _abi.CFG_AUTO, None, None), EINVAL, "alias")
    rejected(lib.muon_hip_bx_axpy_bf16(tbl, tbl + 64, tbl + 128, 512, 640, 1, 1.0, _abi.CFG_256_PINGPONG, None, None),
             ESHAPE, "multiples")
    rejected(lib.muon_hip_adamw(None, tbl, tbl, tbl, F32, 4, 1, 1e-3, 0.9, 0.95, 1e-8, 0.0, None), EINVAL, "null tensor")
    rejected(lib.muon_hip_adamw(tbl, tbl, tbl, tbl, F32, 4, 0, 1e-3, 0.9, 0.95, 1e-8, 0.0, None), EINVAL, "step")
    assert lib.muon_hip_adamw(tbl, tbl, tbl, tbl, F32, 0, 1, 1e-3, 0.9, 0.95, 1e-8, 0.0, None) == 0  # empty tensor
    rejected(lib.muon_hip_adam_update(tbl, tbl, None, tbl, F32, 4, 1, 0.9, 0.95, 1e-8, None), EINVAL, "null tensor")
    rejected(lib.muon_hip_adam_update(tbl, tbl, tbl, tbl, F32, 4, 0, 0.9, 0.95, 1e-8, None), EINVAL, "step")
    rejected(lib.muon_hip_scale(None, F32, 4, 2.0, None), EINVAL, "null tensor")
    rejected(lib.muon_hip_scale(tbl, 5, 4, 2.0, None), EINVAL, "dtype")
    rejected(lib.muon_hip_decay_update(tbl, BF16, tbl, F32, 4, 0.02, 0.0, None), EINVAL, "fp32 update")
    rejected(lib.muon_hip_decay_update(None, F32, tbl, F32, 4, 0.02, 0.0, None), EINVAL, "null tensor")
    rejected(lib.muon_hip_adamw_multi(tbl, tbl, tbl, tbl, tbl, tbl, tbl, tbl, 0, 1, F32, 1e-3, 0.9, 0.95, 1e-8, 0.0,
                                      None), EINVAL, "at least one tensor")
    rejected(lib.muon_hip_adamw_multi(tbl, tbl, tbl, tbl, tbl, tbl, None, tbl, 1, 1, F32, 1e-3, 0.9, 0.95, 1e-8, 0.0,
                                      None), EINVAL, "null table")
    rejected(lib.muon_hip_grad_norms(tbl, tbl, None, 1, 1, F32, 2.0, tbl, tbl, None), EINVAL, "null tensor-list")
    rejected(lib.muon_hip_grad_norms(tbl, tbl, tbl, 1, 1, F32, 2.0, None, tbl, None), EINVAL, "null output")
    rejected(lib.muon_hip_total_norm(tbl, 0, F32, 2.0, tbl, tbl, None), EINVAL, "empty list")
    rejected(lib.muon_hip_total_norm(tbl, 1, F32, float("nan"), tbl, tbl, None), EINVAL, "norm_type is NaN")
    rejected(lib.muon_hip_grad_norms(tbl, tbl, tbl, 1, 1, F32, float("nan"), tbl, tbl, None), EINVAL, "norm_type is NaN")
    rejected(lib.muon_hip_clip_scale(tbl, tbl, tbl, 1, 1, F32, None, F32, 1.0, None), EINVAL, "null total")
    rejected(lib.muon_hip_clip_scale(tbl, tbl, tbl, 1, 1 << 31, F32, tbl, F32, 1.0, None), ESHAPE, "chunks exceed")
    rejected(lib.muon_hip_timing_read(99, None, None), EINVAL, "kernel id")
    rejected(lib.muon_hip_syrk_bf16(tbl, tbl + 64, 512, 512, 1, _abi.CFG_AUTO, tbl + 8, None), EINVAL, "64-byte aligned")
    rejected(lib.muon_hip_timing_reserve(-1), EINVAL, "can be reserved")
    rejected(lib.muon_hip_grad_norms_static(tbl, tbl, tbl, 1, (1 << 20) + 1, F32, 2.0, tbl, None), ESHAPE, "built-in scratch")
    rejected(lib.muon_hip_grad_norms_static(tbl, tbl, tbl, 1, 1, F32, 2.0, None, None), EINVAL, "null output")


def test_chunk_choice_lands_on_whole_rounds():
    """Matrices per grouped launch: never beyond the workspace cap (a hard limit) or the 65535 matrices a library call
    takes, whole rounds of the 256 compute units where the shape allows, never more than the bucket holds, never zero."""
    pick = muon_utils._pick_chunk
    assert pick(12288, 260, 768, 2048) == 256  # 6 and 24 tiles per matrix: 6 and 24 whole rounds
    assert pick(12288, 248, 768, 2048) <= 248
    assert pick(200000, 65535, 37, 53) == 65535 and pick(200000, 1 << 20, 37, 53) == 65535
    assert pick(200000, 70000, 768, 2048) <= 65535
    assert pick(5, 248, 768, 2048) == 5 and pick(1, 7, 4096, 12288) == 1 and pick(100, 1, 4096, 4096) == 1
    for n, cap, rows, cols in ((72, 15, 4096, 4096), (72, 7, 12288, 4096), (36, 7, 4096, 12288), (24, 91, 896, 4864)):
        nb = pick(n, cap, rows, cols)
        assert 1 <= nb <= min(n, cap)


def test_persistent_tile_handout_model():
    """A host model of how the persistent GEMM kernel hands out tiles (csrc/gemm_nt.hip: two static rounds per workgroup,
    then one atomic counter per XCD; virtual ids mapped to tiles by xcd_remap of csrc/common.h), for device shapes other
    than the 256 compute units / 8 XCDs of a whole MI355X as well: whatever order the workgroups ask in, every tile is
    computed exactly once, and a counter never hands out more than one id past the end per workgroup."""
    import random

    XCD_CHUNK = 32

    def xcd_remap(pid, nblocks, shift):
        span = XCD_CHUNK << shift
        full = nblocks // span * span
        if pid >= full:
            return pid
        xcd, local = pid & ((1 << shift) - 1), pid >> shift
        return (((local // XCD_CHUNK) << shift) + xcd) * XCD_CHUNK + local % XCD_CHUNK

    rng = random.Random(7)
    for cus, shift in ((256, 3), (128, 2), (64, 1), (32, 0), (304, 3)):
        for total in (cus + 1, 2 * cus, 2 * cus + 1, 5 * cus + 37, 17 * cus, 9216):
            grid = min(total, cus)
            assert grid % (1 << shift) == 0
            # the remap is a bijection of the virtual ids onto the tiles
            assert sorted(xcd_remap(p, total, shift) for p in range(total)) == list(range(total))
            counters = [0] * (1 << shift)
            done = []
            # workgroup state: (current id, next id); a workgroup asks for the id after next while it has a next tile
            wgs = {b: [b, b + grid] for b in range(grid)}
            active = list(wgs)
            while active:
                b = rng.choice(active)  # any interleaving
                cur, nxt = wgs[b]
                done.append(cur)
                if nxt >= total:
                    active.remove(b)
                    continue
                xcd = b & ((1 << shift) - 1)
                fetched = counters[xcd]
                counters[xcd] += 1
                wgs[b] = [nxt, ((2 * (grid >> shift) + fetched) << shift) + xcd]
            assert sorted(done) == list(range(total)), (cus, shift, total)
            assert sum(counters) <= total  # bounded: nobody spins on the counters
