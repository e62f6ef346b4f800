"""Pins the CPU oracle (oracle/muon_oracle.py and oracle/muon_oracle.c) without the GPU.

The reference's tests contain no Muon vector, so each oracle function is checked against
what the mathematics fixes: closed forms, the SVD polynomial identity, invariants, fp64
brute force, library routines (torch.lerp, torch.optim.AdamW) and the independent plain-C
restatement.  Each check is chosen so that a plausible mistake (dropped term, wrong sign,
transposed operand, missing rounding) fails it.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import muon_oracle as O
from tests.helpers import MUON_HP, bf16_from_u16, c_newton_schulz, make_param_set, rel_fro, u16_from_bf16

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _randn(rows, cols, seed):
    return torch.randn(rows, cols, generator=torch.Generator().manual_seed(seed))


# ---- Newton-Schulz ---------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(64, 160), (160, 64), (33, 47), (16, 16)])
def test_explicit_rounding_points_equal_literal_torch_expressions(shape):
    G = _randn(*shape, seed=1)
    for steps in (0, 1, 5):
        assert torch.equal(O.newton_schulz(G, steps, literal=False), O.newton_schulz(G, steps, literal=True))


def test_explicit_vs_literal_large_k_differ_only_by_accumulation_order():
    G = _randn(128, 896, seed=2)
    assert rel_fro(O.newton_schulz(G, 1, literal=False), O.newton_schulz(G, 1, literal=True)) < 1e-3
    assert rel_fro(O.newton_schulz(G, 5, literal=False), O.newton_schulz(G, 5, literal=True)) < 1.3e-2


@pytest.mark.parametrize("shape", [(64, 160), (160, 64), (33, 47)])
def test_c_restatement_bit_identical_on_small_shapes(oracle_c, shape):
    G = _randn(*shape, seed=3)
    for steps in (0, 1, 2, 5):
        assert torch.equal(c_newton_schulz(oracle_c, G, steps), O.newton_schulz(G, steps))


def test_c_restatement_large_k(oracle_c):
    G = _randn(128, 896, seed=4)
    one_c, one_t = c_newton_schulz(oracle_c, G, 1), O.newton_schulz(G, 1)
    assert (one_c != one_t).float().mean().item() < 1e-3  # a few elements round the other way
    assert rel_fro(c_newton_schulz(oracle_c, G, 5), O.newton_schulz(G, 5)) < 1.3e-2


@pytest.mark.parametrize("shape", [(64, 160), (160, 64), (128, 896), (200, 200)])
def test_svd_polynomial_identity(shape):
    """Exact arithmetic gives U phi^5(S) Vt; bf16 rounding moves it by a few percent only.
    A wrong coefficient, sign or operand order is off by O(1)."""
    G = _randn(*shape, seed=5)
    assert rel_fro(O.newton_schulz(G, 5), O.svd_polynomial(G, 5)) < 5e-2
    assert rel_fro(O.newton_schulz(G, 1), O.svd_polynomial(G, 1)) < 1e-2


def test_invariants():
    G = _randn(96, 240, seed=6)
    out = O.newton_schulz(G, 5)
    assert out.dtype == torch.bfloat16 and out.shape == G.shape
    # transpose rule: NS(Gt) = NS(G)t exactly (the same operand X is formed either way)
    assert torch.equal(O.newton_schulz(G.mT.contiguous(), 5), out.mT)
    # power-of-two scaling leaves every bf16 operand unchanged
    assert torch.equal(O.newton_schulz(G * 8.0, 5), out)
    # zero in, zero out, no NaN (the 1e-7 guard)
    z = O.newton_schulz(torch.zeros(8, 12), 5)
    assert torch.count_nonzero(z) == 0
    # singular values land in the polynomial's fixed-point band
    sv = torch.linalg.svdvals(out.double())
    assert sv.min() > 0.55 and sv.max() < 1.25
    assert abs(out.double().norm().item() / 96 ** 0.5 - 1.0) < 0.25


def test_brute_force_fp64_tiny():
    """16x24 with every product formed in fp64 and rounded at the stated points."""
    G = _randn(16, 24, seed=7)
    a, b, c = (torch.tensor(v, dtype=torch.float32).double() for v in O.NS_COEFFS)
    X = G.bfloat16().double()
    n = X.pow(2).sum().sqrt().float().bfloat16()
    d = (n.float() + torch.tensor(1e-7, dtype=torch.float32)).bfloat16().double()
    r = lambda t: t.float().bfloat16().double()  # noqa: E731
    X = r(X / d)
    for _ in range(5):
        A = r(X @ X.mT)
        A2 = r(A @ A)
        B = r(r(b * A) + r(c * A2))
        X = r(r(a * X) + r(B @ X))
    got = O.newton_schulz(G, 5).double()
    assert (got != X).double().mean().item() < 0.02 and rel_fro(got, X) < 2e-3


def test_rounding_points_are_discriminated():
    """Changing one rounding point moves the result by more than accumulation-order noise does:
    the 2e-2 parity bar can tell the two apart."""
    G = _randn(896, 4864, seed=0)
    base = O.newton_schulz(G, 5)
    a, b, c = (O._f32(v) for v in O.NS_COEFFS)

    def variant(fuse_b=False, f64_acc=False):
        X = G.bfloat16()
        X = (X.float() / O.frobenius_denominator(X).float()).bfloat16()
        for _ in range(5):
            if f64_acc:
                A = (X.double() @ X.double().mT).bfloat16()
                A2 = (A.double() @ A.double()).bfloat16()
            else:
                A, A2 = O.mmt(X), None
                A2 = O.mmt(A)
            if fuse_b:
                B = O.bf(A.float() * b + A2.float() * c)
            else:
                B = O.bf(O.bf(A.float() * b) + O.bf(A2.float() * c))
            BX = (B.double() @ X.double()).float() if f64_acc else B @ X.float()
            X = (O.bf(X.float() * a) + O.bf(BX)).bfloat16()
        return X

    noise = rel_fro(variant(f64_acc=True), base)
    moved = rel_fro(variant(fuse_b=True), base)
    assert noise < 1.3e-2, noise
    assert moved > 1.5e-2 and moved > 1.5 * noise, (moved, noise)


def test_mmt_contract():
    X = _randn(40, 72, seed=8).bfloat16()
    A = O.mmt(X)
    assert torch.equal(A, A.mT)
    ref = X.double() @ X.double().mT
    assert ((A.double() - ref).abs() <= ref.abs() * 2.0 ** -8 + 1e-6).all()


def test_golden_ns_vectors_reproduce():
    data = np.load(os.path.join(GOLDEN, "ns_small.npz"))
    assert len(data.files) == 10
    for key in data.files:
        _, shape, seed, steps = key.split("_")
        rows, cols = (int(v) for v in shape.split("x"))
        G = _randn(rows, cols, seed=int(seed[4:]))
        got = O.newton_schulz(G, int(steps[5:]))
        want = bf16_from_u16(data[key])
        if max(rows, cols) <= 256:
            assert (got != want).float().mean().item() < 1e-3, key  # BLAS blocking may flip a rare rounding
        assert rel_fro(got, want) < 1.3e-2, key


def test_golden_step_vectors_reproduce():
    from tests.golden.make_fixtures import STEP_SPEC

    data = np.load(os.path.join(GOLDEN, "step_small.npz"))
    weights, grads = make_param_set(STEP_SPEC, layers=1, seed=7, steps=3)
    params = [torch.nn.Parameter(w.clone()) for _, w in weights]
    groups = [dict(params=sorted(params, key=lambda x: x.size(), reverse=True), use_muon=True, **MUON_HP)]
    orc = O.OracleMuon(groups)
    for step in range(3):
        for p, g in zip(params, grads[step]):
            p.grad = g.clone()
        orc.step()
        for j in range(len(params)):
            assert rel_fro(orc.last_updates[(0, j)], bf16_from_u16(data[f"step{step}_update{j}"])) < 1.3e-2
    for j, p in enumerate(groups[0]["params"]):
        assert rel_fro(orc.state[(0, j)]["momentum_buffer"], torch.from_numpy(data[f"final_momentum{j}"])) < 1e-6
        assert rel_fro(p.detach(), torch.from_numpy(data[f"final_param{j}"])) < 1e-3


# ---- momentum ---------------------------------------------------------------------------
@pytest.mark.parametrize("nesterov", [True, False])
def test_momentum_closed_form_and_c(oracle_c, nesterov):
    gen = torch.Generator().manual_seed(9)
    g, m = torch.randn(50, 70, generator=gen), torch.randn(50, 70, generator=gen)
    g0, m0 = g.clone(), m.clone()
    u = O.apply_momentum(g, m, 0.95, nesterov)
    m_ref = O.lerp_closed_form(m0, g0, 1 - 0.95)
    u_ref = O.lerp_closed_form(g0, m_ref, 0.95) if nesterov else m_ref
    assert rel_fro(m, m_ref) < 1e-6 and rel_fro(u, u_ref) < 1e-6
    if nesterov:
        assert u.data_ptr() == g.data_ptr(), "the reference blends into the grad in place"
    # plain mathematics: m' = 0.95 m + 0.05 g ; u = 0.05 g + 0.95 m'
    assert rel_fro(m, 0.95 * m0.double() + 0.05 * g0.double()) < 1e-6
    mc, uc = m0.numpy().copy(), np.zeros((50, 70), dtype=np.float32)
    oracle_c.orc_momentum(g0.numpy().ctypes.data_as(ctypes.c_void_p), mc.ctypes.data_as(ctypes.c_void_p),
                          uc.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(g0.numel()), ctypes.c_double(0.95),
                          int(nesterov))
    assert rel_fro(torch.from_numpy(mc), m) < 2e-7 and rel_fro(torch.from_numpy(uc), u) < 2e-7


def test_momentum_mixed_dtype_extension():
    gen = torch.Generator().manual_seed(10)
    g = torch.randn(20, 30, generator=gen).bfloat16()
    m = torch.randn(20, 30, generator=gen)
    m0 = m.clone()
    u = O.apply_momentum(g, m, 0.95, True)
    assert u.dtype == torch.float32 and m.dtype == torch.float32
    assert rel_fro(m, 0.95 * m0.double() + 0.05 * g.double()) < 1e-6


# ---- scaling and update -----------------------------------------------------------------
def test_scale_factor_closed_forms():
    assert O.scale_factor(4864, 896, False) == (4864 / 896) ** 0.5
    assert O.scale_factor(896, 4864, False) == 1.0
    assert O.scale_factor(896, 4864, True) == 0.2 * 4864 ** 0.5 == O.scale_factor(4864, 896, True)


@pytest.mark.parametrize("pdtype", [torch.float32, torch.bfloat16])
def test_scale_and_update_closed_form_and_c(oracle_c, pdtype):
    gen = torch.Generator().manual_seed(11)
    p = (0.02 * torch.randn(60, 20, generator=gen)).to(pdtype)
    o = torch.randn(60, 20, generator=gen).bfloat16()
    p0, o0 = p.clone(), o.clone()
    s = O.apply_scaling(o, False)
    O.param_update(p, s, 0.02, 0.01)
    sc = (60 / 20) ** 0.5
    os_ref = (o0.float() * torch.tensor(sc, dtype=torch.float32)).bfloat16()
    assert torch.equal(s, os_ref)
    p_ref = p0.double() * (1 - 0.02 * 0.01) - 0.02 * os_ref.double()
    assert rel_fro(p, p_ref) < (1e-6 if pdtype == torch.float32 else 4e-3)
    ob = u16_from_bf16(o0)
    if pdtype == torch.float32:
        pc = p0.numpy().copy()
        oracle_c.orc_scale_update_f32(pc.ctypes.data_as(ctypes.c_void_p), ob.ctypes.data_as(ctypes.c_void_p),
                                      ctypes.c_size_t(p0.numel()), ctypes.c_double(sc), ctypes.c_double(0.02),
                                      ctypes.c_double(0.01))
        assert rel_fro(torch.from_numpy(pc), p) < 2e-7
    else:
        pc = u16_from_bf16(p0)
        oracle_c.orc_scale_update_bf16(pc.ctypes.data_as(ctypes.c_void_p), ob.ctypes.data_as(ctypes.c_void_p),
                                       ctypes.c_size_t(p0.numel()), ctypes.c_double(sc), ctypes.c_double(0.02),
                                       ctypes.c_double(0.01))
        assert torch.equal(bf16_from_u16(pc), p)
    assert torch.equal(bf16_from_u16(ob), s)


# ---- AdamW fallback ---------------------------------------------------------------------
def test_adamw_matches_torch_optim(oracle_c):
    gen = torch.Generator().manual_seed(12)
    w = torch.randn(300, generator=gen)
    p_t = torch.nn.Parameter(w.clone())
    ref = torch.optim.AdamW([p_t], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    p, e1, e2 = w.clone(), torch.zeros(300), torch.zeros(300)
    pc, e1c, e2c = w.numpy().copy(), np.zeros(300, np.float32), np.zeros(300, np.float32)
    for step in range(1, 6):
        g = torch.randn(300, generator=gen)
        p_t.grad = g.clone()
        ref.step()
        O.adamw_step_tensor(p, g.clone(), e1, e2, step, 1e-3, (0.9, 0.999), 1e-8, 0.01)
        gc = g.numpy().copy()
        oracle_c.orc_adamw_f32(pc.ctypes.data_as(ctypes.c_void_p), gc.ctypes.data_as(ctypes.c_void_p),
                               e1c.ctypes.data_as(ctypes.c_void_p), e2c.ctypes.data_as(ctypes.c_void_p),
                               ctypes.c_size_t(300), step, ctypes.c_double(1e-3), ctypes.c_double(0.9),
                               ctypes.c_double(0.999), ctypes.c_double(1e-8), ctypes.c_double(0.01))
    # torch's AdamW puts eps after dividing sqrt(v) by sqrt(bias correction): identical algebra up to rounding
    assert rel_fro(p, p_t.detach()) < 1e-6
    assert rel_fro(torch.from_numpy(pc), p) < 1e-6
    assert rel_fro(torch.from_numpy(e1c), e1) < 1e-6 and rel_fro(torch.from_numpy(e2c), e2) < 1e-6


def test_reference_bug_compat_args():
    assert O.reference_bug_compat_args(nesterov=True, ns_steps=5) == (True, 1)
    assert O.reference_bug_compat_args(nesterov=False, ns_steps=5) == (True, 0)
    assert O.reference_bug_compat_args(nesterov=True, ns_steps=0) == (False, 1)
    assert list(range(True)) == [0] and list(range(False)) == []


def test_ns_flops_formula():
    assert O.ns_flops(896, 4864) == 5 * (3 * 896 ** 2 * 4864 + 896 ** 3)
    assert O.ns_flops(4864, 896) == O.ns_flops(896, 4864)
    assert O.ns_flops(896, 4864, dense=True) == 5 * (4 * 896 ** 2 * 4864 + 2 * 896 ** 3)
