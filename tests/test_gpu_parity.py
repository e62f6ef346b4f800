"""Parity of the HIP path (through the C ABI) against the CPU oracle.  GPU box only.

Tolerances (from the task statement): orthogonalised update within 2e-2 relative Frobenius
error of the oracle computed in the same bf16 iteration order; fp32 momentum within 1e-6
relative.  Single GEMMs are held to one bf16 ulp of the fp64 product, and to bitwise
symmetry.
"""
import copy
import ctypes

import pytest
import torch

from tests.helpers import MUON_HP, NAMES, QWEN25_05B, make_param_set, rel_fro, report_parity

pytestmark = pytest.mark.gpu

NS_TOL = 2e-2
MOM_TOL = 1e-6


@pytest.fixture(scope="module")
def env():
    assert torch.cuda.is_available(), "these tests need the GPU box"
    from lmms_engine_amd import _abi, muon_utils
    from oracle import muon_oracle

    lib = _abi.lib()  # raises if libmuon_hip.so is missing
    assert lib.muon_hip_version() >= 100
    dev = torch.device("cuda:0")
    # tile counters for the single-GEMM entry points: zero before the first use, left zero by every launch
    ctr = torch.zeros(_abi.PPX_COUNTER_BYTES, dtype=torch.uint8, device=dev)
    return dict(abi=_abi, mu=muon_utils, O=muon_oracle, lib=lib, dev=dev, ctr=ctr, ctr_ptr=ctr.data_ptr())


def _ulp_diff_bf16(a: torch.Tensor, b: torch.Tensor) -> int:
    """Largest distance in bf16 representable steps (sign-magnitude mapped to a line)."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
        neg = i >= 0x8000
        return torch.where(neg, 0x8000 - i, i)
    return (key(a.cpu()) - key(b.cpu())).abs().max().item()


def _assert_product_close(got, ref64, absprod):
    """One bf16 rounding of an fp32-accumulated product: within a bf16 ulp of the exact value
    plus the accumulation error bound (which dominates where the sum cancels)."""
    tol = ref64.abs() * 2.0 ** -8 + absprod * 2.0 ** -20
    bad = (got.double().cpu() - ref64).abs() > tol
    assert not bad.any(), f"{int(bad.sum())} elements outside one bf16 ulp"


CFGS = list(range(5))


def _pack(env, t):
    """[batch, rows, cols] bf16 on the device -> blocked buffer (shapes here are whole tiles already)."""
    lib, abi = env["lib"], env["abi"]
    batch, rows, cols = t.shape
    t = t.contiguous()
    out = torch.full((batch * lib.muon_hip_blocked_elems(rows, cols),), float("nan"), dtype=torch.bfloat16, device=t.device)
    abi.check(lib.muon_hip_pack_bf16(t.data_ptr(), rows * cols, cols, rows, cols, out.data_ptr(), rows, cols, batch, 0))
    return out


def _blocked_nan(env, batch, rows, cols):
    n = batch * env["lib"].muon_hip_blocked_elems(rows, cols)
    return torch.full((n,), float("nan"), dtype=torch.bfloat16, device=env["dev"])


def _unpack(env, buf, batch, rows, cols):
    lib, abi = env["lib"], env["abi"]
    out = torch.empty(batch, rows, cols, dtype=torch.bfloat16, device=buf.device)
    abi.check(lib.muon_hip_unpack_bf16(buf.data_ptr(), rows, cols, out.data_ptr(), rows * cols, cols, rows, cols, batch, 0))
    torch.cuda.synchronize()
    return out.cpu()


def test_pack_unpack_round_trip_and_layout(env):
    """The blocked layout is what include/muon_hip.h states: element (r, c) at
    ((r/256)*cb + c/32)*8192 + (r%256)*32 + c%32, zero padded."""
    lib, abi, dev = env["lib"], env["abi"], env["dev"]
    g = torch.Generator().manual_seed(3)
    rows, cols, rp, cp, batch = 300, 200, 384, 256, 2
    t = torch.randn(batch, rows, cols + 8, generator=g).bfloat16().to(dev)  # row pitch 208 > cols
    n = lib.muon_hip_blocked_elems(rp, cp)
    assert n == 2 * 8 * 8192
    buf = torch.full((batch * n,), float("nan"), dtype=torch.bfloat16, device=dev)
    abi.check(lib.muon_hip_pack_bf16(t.data_ptr(), rows * (cols + 8), cols + 8, rows, cols, buf.data_ptr(), rp, cp, batch, 0))
    torch.cuda.synchronize()
    host, src = buf.cpu().view(batch, n), t.cpu()  # rows 384..511 of the last row of blocks are never touched
    r = torch.arange(rp).view(-1, 1).expand(rp, cp)
    c = torch.arange(cp).view(1, -1).expand(rp, cp)
    idx = ((r // 256) * (cp // 32) + c // 32) * 8192 + (r % 256) * 32 + c % 32
    for b in range(batch):
        img = host[b][idx]
        assert not torch.isnan(img).any()
        assert torch.equal(img[:rows, :cols], src[b, :, :cols])
        assert (img[rows:, :] == 0).all() and (img[:, cols:] == 0).all()
    out = torch.full((batch, rows, cols + 3), 7.0, dtype=torch.bfloat16, device=dev)
    abi.check(lib.muon_hip_unpack_bf16(buf.data_ptr(), rp, cp, out.data_ptr(), rows * (cols + 3), cols + 3, rows, cols, batch, 0))
    torch.cuda.synchronize()
    assert torch.equal(out.cpu()[:, :, :cols], src[:, :, :cols]) and (out.cpu()[:, :, cols:] == 7.0).all()
    assert lib.muon_hip_blocked_elems(256, 100) == 0 and lib.muon_hip_pack_bf16(t.data_ptr(), 0, 8, 300, 200, buf.data_ptr(), rp, cp, 1, 0) == -2


@pytest.mark.parametrize("cfg", CFGS)
@pytest.mark.parametrize("M,K,batch", [(256, 256, 1), (512, 768, 2), (768, 256, 3)])
def test_syrk_matches_fp64_and_is_symmetric(env, cfg, M, K, batch):
    print(f"syrk cfg={cfg} M={M} K={K} batch={batch}", flush=True)
    g = torch.Generator().manual_seed(10 + cfg)
    X = torch.randn(batch, M, K, generator=g).bfloat16()
    Xb = _pack(env, X.to(env["dev"]))
    Ab = _blocked_nan(env, batch, M, M)
    env["abi"].check(env["lib"].muon_hip_syrk_bf16(Xb.data_ptr(), Ab.data_ptr(), M, K, batch, cfg, env["ctr_ptr"], 0))
    A = _unpack(env, Ab, batch, M, M)
    assert torch.equal(A, A.mT), "X·Xᵀ must be symmetric bit for bit"
    ref64 = (X.double() @ X.double().mT)
    _assert_product_close(A, ref64, X.double().abs() @ X.double().abs().mT)
    assert rel_fro(A, ref64) < 3e-3


@pytest.mark.parametrize("cfg", CFGS)
def test_sympoly_rounding_points(env, cfg):
    print(f"sympoly cfg={cfg}", flush=True)
    O = env["O"]
    g = torch.Generator().manual_seed(20 + cfg)
    M, batch = 512, 2
    X = (torch.randn(batch, M, 1024, generator=g) / 32).bfloat16()
    A = torch.stack([O.mmt(X[i]) for i in range(batch)])
    Ab = _pack(env, A.to(env["dev"]))
    Bb = _blocked_nan(env, batch, M, M)
    a, b, c = O.NS_COEFFS
    env["abi"].check(env["lib"].muon_hip_sympoly_bf16(Ab.data_ptr(), Bb.data_ptr(), M, batch, b, c, cfg, env["ctr_ptr"], 0))
    B = _unpack(env, Bb, batch, M, M)
    assert torch.equal(B, B.mT)
    for i in range(batch):
        A2 = O.mmt(A[i])
        ref = O.bf(O.bf(A[i].float() * O._f32(b)) + O.bf(A2.float() * O._f32(c))).bfloat16()
        # accumulation order may flip the rounding of A·A in rare elements; everything after is exact
        frac = (B[i] != ref).float().mean().item()
        assert frac < 2e-2, frac
        assert rel_fro(B[i], ref) < 4e-3


@pytest.mark.parametrize("cfg", CFGS)
@pytest.mark.parametrize("M,K", [(256, 768), (512, 256)])
def test_bx_axpy_rounding_points(env, cfg, M, K):
    print(f"bx cfg={cfg} M={M} K={K}", flush=True)
    O = env["O"]
    g = torch.Generator().manual_seed(30 + cfg)
    batch = 2
    X = (torch.randn(batch, M, K, generator=g) / 16).bfloat16()
    Bm = (torch.randn(batch, M, M, generator=g) / 16).bfloat16()
    Bm = torch.triu(Bm) + torch.triu(Bm, 1).mT  # the kernel is specified for symmetric B
    dev = env["dev"]
    Xb, Bb, Xo = _pack(env, X.to(dev)), _pack(env, Bm.to(dev)), _blocked_nan(env, batch, M, K)
    a = O.NS_COEFFS[0]
    env["abi"].check(env["lib"].muon_hip_bx_axpy_bf16(Bb.data_ptr(), Xb.data_ptr(), Xo.data_ptr(), M, K, batch, a, cfg, env["ctr_ptr"], 0))
    Xo = _unpack(env, Xo, batch, M, K)
    for i in range(batch):
        ref = (O.bf(X[i].float() * O._f32(a)) + O.bf(Bm[i].float() @ X[i].float())).bfloat16()
        assert (Xo[i] != ref).float().mean().item() < 2e-2
        assert rel_fro(Xo[i], ref) < 4e-3


def test_split_tail_is_bitwise_the_plain_kernel(env):
    """A tile count just above a multiple of the 256 CUs makes the ping-pong configuration cut the last tiles into
    128x128 quarters.  Every output element still sums its products in ascending k, so the result equals the
    two-stage 256-tile kernel's bit for bit (which never splits)."""
    lib, abi, dev, O = env["lib"], env["abi"], env["dev"], env["O"]
    g = torch.Generator().manual_seed(77)
    # X.Xt: 10 triangular tiles x 26 matrices = 260; b.A + c.A.A likewise; a.X + B.X: 4 x 2 tiles x 33 = 264
    M, K, batch = 1024, 256, 26
    Xb = _pack(env, (torch.randn(batch, M, K, generator=g) / 16).bfloat16().to(dev))
    outs = []
    for cfg in (abi.CFG_256_PINGPONG, abi.CFG_256_PIPE):
        Ab, Bb = _blocked_nan(env, batch, M, M), _blocked_nan(env, batch, M, M)
        abi.check(lib.muon_hip_syrk_bf16(Xb.data_ptr(), Ab.data_ptr(), M, K, batch, cfg, env["ctr_ptr"], 0))
        abi.check(lib.muon_hip_sympoly_bf16(Ab.data_ptr(), Bb.data_ptr(), M, batch, O.NS_COEFFS[1], O.NS_COEFFS[2], cfg, env["ctr_ptr"], 0))
        outs.append((_unpack(env, Ab, batch, M, M), _unpack(env, Bb, batch, M, M)))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    assert torch.equal(outs[0][0], outs[0][0].mT) and not torch.isnan(outs[0][1]).any()
    M, K, batch = 1024, 512, 33
    Xb = _pack(env, (torch.randn(batch, M, K, generator=g) / 16).bfloat16().to(dev))
    Bm = (torch.randn(batch, M, M, generator=g) / 16).bfloat16()
    Bb = _pack(env, (torch.triu(Bm) + torch.triu(Bm, 1).mT).to(dev))
    outs = []
    for cfg in (abi.CFG_256_PINGPONG, abi.CFG_256_PIPE):
        Xo = _blocked_nan(env, batch, M, K)
        abi.check(lib.muon_hip_bx_axpy_bf16(Bb.data_ptr(), Xb.data_ptr(), Xo.data_ptr(), M, K, batch, O.NS_COEFFS[0], cfg, env["ctr_ptr"], 0))
        outs.append(_unpack(env, Xo, batch, M, K))
    assert torch.equal(outs[0], outs[1]) and not torch.isnan(outs[0]).any()


def test_persistent_bx_is_bitwise_the_one_tile_kernel(env):
    """The persistent configuration of a.X + B.X walks several tiles per workgroup (two static rounds, then tiles from
    per-XCD counters), prefetches the next tile behind an epilogue that needs no LDS and re-uses its counters launch
    after launch.  It adds the same products in the same order as the one-tile ping-pong kernel: X' must agree bit for
    bit with the two-stage kernel (whose epilogue goes through LDS), on tile counts of exactly two rounds, of several
    rounds, with a ragged last round, and with 8 k-tiles (the shortest reduction it takes); three launches in a row
    (the counters must be back at zero)."""
    lib, abi, dev, O = env["lib"], env["abi"], env["dev"], env["O"]
    g = torch.Generator().manual_seed(78)
    a_c = O.NS_COEFFS[0]
    # rectangular tiles M/256 * K/256 per matrix: 512, 1280, 1320 (= 5 rounds + 40), 270 (= 1 round + 14), 768
    for M, K, batch in ((512, 512, 128), (512, 1024, 160), (768, 2048, 55), (256, 256 * 27, 10), (1024, 256, 192)):
        print(f"persistent vs one-tile: M={M} K={K} batch={batch}", flush=True)
        Xb = _pack(env, (torch.randn(batch, M, K, generator=g) / 16).bfloat16().to(dev))
        Bm = (torch.randn(batch, M, M, generator=g) / 16).bfloat16()
        Bb = _pack(env, (torch.triu(Bm) + torch.triu(Bm, 1).mT).to(dev))
        res = []
        for cfg in (abi.CFG_256_PIPE, abi.CFG_256_PERSIST, abi.CFG_256_PERSIST, abi.CFG_256_PERSIST):
            Xo = _blocked_nan(env, batch, M, K)
            abi.check(lib.muon_hip_bx_axpy_bf16(Bb.data_ptr(), Xb.data_ptr(), Xo.data_ptr(), M, K, batch, a_c, cfg, env["ctr_ptr"], 0))
            torch.cuda.synchronize()
            assert not env["ctr"].any(), "a persistent launch leaves its tile counters zero"
            res.append(Xo.clone())
        for rep in (1, 2, 3):
            assert not torch.isnan(res[rep].float()).any(), rep
            assert torch.equal(res[0], res[rep]), f"M={M} K={K} batch={batch}, launch {rep}"
        # without a counter buffer the same configuration runs the one-tile kernels
        Xo = _blocked_nan(env, batch, M, K)
        abi.check(lib.muon_hip_bx_axpy_bf16(Bb.data_ptr(), Xb.data_ptr(), Xo.data_ptr(), M, K, batch, a_c, abi.CFG_256_PERSIST, None, 0))
        torch.cuda.synchronize()
        assert torch.equal(res[0], Xo)


def test_persistent_symmetric_products_are_bitwise_the_two_stage_kernel(env):
    """X.Xt and b.A + c.A.A with reductions of at most 2048 run in the persistent kernel when a launch has more tiles
    than compute units: triangular tile lists, diagonal tiles in which every wave skips the fragments below the
    diagonal, and an epilogue that transposes in registers instead of LDS.  Both outputs must agree bit for bit with
    the two-stage kernel (whole diagonal tiles, epilogue through LDS) and with the one-tile ping-pong kernel, be symmetric
    bit for bit, and stay so on three launches in a row; tile counts with a ragged last round, 8 k-tiles (the shortest reduction) and 64 (the longest)."""
    lib, abi, dev, O = env["lib"], env["abi"], env["dev"], env["O"]
    g = torch.Generator().manual_seed(79)
    _, b_c, c_c = O.NS_COEFFS
    # triangular tiles T(T+1)/2 per matrix with T = M/256: 330, 300, 300, 288, 280
    for M, K, batch in ((768, 2048, 55), (512, 256, 100), (1024, 1024, 30), (2048, 512, 8), (1792, 1280, 10)):
        print(f"persistent symmetric vs two-stage: M={M} K={K} batch={batch}", flush=True)
        Xb = _pack(env, (torch.randn(batch, M, K, generator=g) / 16).bfloat16().to(dev))
        res = []
        for cfg in (abi.CFG_256_PIPE, abi.CFG_256_PINGPONG, abi.CFG_256_PERSIST, abi.CFG_256_PERSIST, abi.CFG_256_PERSIST):
            A = _blocked_nan(env, batch, M, M)
            B = _blocked_nan(env, batch, M, M)
            abi.check(lib.muon_hip_syrk_bf16(Xb.data_ptr(), A.data_ptr(), M, K, batch, cfg, env["ctr_ptr"], 0))
            abi.check(lib.muon_hip_sympoly_bf16(A.data_ptr(), B.data_ptr(), M, batch, b_c, c_c, cfg, env["ctr_ptr"], 0))
            torch.cuda.synchronize()
            assert not env["ctr"].any(), "a persistent launch leaves its tile counters zero"
            res.append((A.clone(), B.clone()))
        for rep in (1, 2, 3, 4):  # the one-tile ping-pong kernel, then the persistent one three times
            for name, ref, got in (("syrk", res[0][0], res[rep][0]), ("sympoly", res[0][1], res[rep][1])):
                assert not torch.isnan(got.float()).any(), (name, rep)
                assert torch.equal(ref, got), f"{name} M={M} K={K} batch={batch}, launch {rep}"
        Bd = _unpack(env, res[1][1], batch, M, M)
        assert torch.equal(Bd, Bd.mT.contiguous())


def test_gemm_entry_points_reject_bad_shapes(env):
    lib, abi = env["lib"], env["abi"]
    x = torch.zeros(256 * 256, dtype=torch.bfloat16, device=env["dev"])
    assert lib.muon_hip_syrk_bf16(x.data_ptr(), x.data_ptr(), 200, 256, 1, 0, env["ctr_ptr"], 0) == -2
    assert b"multiples" in lib.muon_hip_last_error()
    assert lib.muon_hip_syrk_bf16(x.data_ptr(), x.data_ptr(), 128, 128, 1, abi.CFG_256_PIPE, env["ctr_ptr"], 0) == -2  # 128 is not a 256-tile
    assert lib.muon_hip_syrk_bf16(None, x.data_ptr(), 256, 256, 1, 0, env["ctr_ptr"], 0) == -1
    assert lib.muon_hip_syrk_bf16(x.data_ptr(), x.data_ptr(), 256, 256, 1, 99, env["ctr_ptr"], 0) == -1
    with pytest.raises(abi.MuonHipError):
        abi.check(lib.muon_hip_bx_axpy_bf16(x.data_ptr(), x.data_ptr(), None, 256, 256, 1, 1.0, 0, env["ctr_ptr"], 0))
    assert lib.muon_hip_bx_axpy_bf16(x.data_ptr(), x.data_ptr(), x.data_ptr(), 256, 256, 1, 1.0, 0, env["ctr_ptr"], 0) == -1  # in place


NS_SHAPES = [(64, 160), (160, 64), (33, 47), (100, 300), (300, 100), (128, 896), (896, 128), (256, 256), (512, 1024)]


@pytest.mark.parametrize("rows,cols", NS_SHAPES)
def test_newton_schulz_small_shapes(env, rows, cols):
    print(f"ns rows={rows} cols={cols}", flush=True)
    O, mu = env["O"], env["mu"]
    G = torch.randn(rows, cols, generator=torch.Generator().manual_seed(rows * 1000 + cols))
    ref = O.newton_schulz(G, 5)
    got = mu.fast_newtonschulz(G.to(env["dev"]), 5)
    assert got.dtype == torch.bfloat16 and got.shape == G.shape
    assert rel_fro(got, ref) <= NS_TOL
    for steps in (0, 1, 2):
        assert rel_fro(mu.fast_newtonschulz(G.to(env["dev"]), steps), O.newton_schulz(G, steps)) <= 2e-3


def test_newton_schulz_random_shapes_scales_and_step_counts(env):
    """Forty seeded draws of (rows, cols, input scale, iteration count) through fast_newtonschulz against the oracle:
    single rows and columns, ragged edges, both orientations, 128- and 256-tile buckets, inputs from 1e-3 to 50 times
    N(0,1) (the normalisation removes the scale), 0 to 5 iterations; bound 2e-2 relative Frobenius error as stated for
    five iterations."""
    import random
    O, mu = env["O"], env["mu"]
    rng = random.Random(1234)
    worst = 0.0
    for trial in range(40):
        rows = rng.choice([1, 7, 33, 64, 100, 128, 200, 256, 300, 384, 512, 640, 768, 896, 1024])
        cols = rng.choice([1, 9, 47, 64, 96, 128, 250, 256, 384, 512, 700, 768, 1024, 1536])
        steps = rng.choice([0, 1, 3, 5])
        scale = rng.choice([1e-3, 1.0, 50.0])
        print(f"random ns trial {trial}: {rows}x{cols} steps {steps} scale {scale}", flush=True)
        G = torch.randn(rows, cols, generator=torch.Generator().manual_seed(trial)) * scale
        err = rel_fro(mu.fast_newtonschulz(G.to(env["dev"]), steps), O.newton_schulz(G, steps))
        worst = max(worst, err)
        assert err <= NS_TOL, (rows, cols, steps, scale, err)
    print(f"worst error over the random draws: {worst:.3e}", flush=True)


def test_newton_schulz_config1(env):
    """Benchmark config 1: 896x4864 fp32 N(0,1) from seed 0, five bf16 iterations."""
    print("ns config 1", flush=True)
    O, mu = env["O"], env["mu"]
    G = torch.randn(896, 4864, generator=torch.Generator().manual_seed(0))
    ref = O.newton_schulz(G, 5)
    got = mu.fast_newtonschulz(G.to(env["dev"]), 5)
    err = rel_fro(got, ref)
    report_parity(f"config 1 (896x4864 fp32, seed 0, 5 iterations): NS-output error {err:.3e} (bound {NS_TOL})")
    assert err <= NS_TOL
    got_t = mu.fast_newtonschulz(G.mT.contiguous().to(env["dev"]), 5)
    assert rel_fro(got_t, O.newton_schulz(G.mT.contiguous(), 5)) <= NS_TOL
    # every tile configuration gives the same answer up to accumulation order
    for cfg in CFGS:
        env["abi"].check(env["lib"].muon_hip_set_gemm_config(cfg))
        try:
            assert rel_fro(mu.fast_newtonschulz(G.to(env["dev"]), 5), ref) <= NS_TOL
        finally:
            env["lib"].muon_hip_set_gemm_config(-1)


def test_newton_schulz_zero_and_scale(env):
    mu = env["mu"]
    Z = torch.zeros(96, 200, device=env["dev"])
    out = mu.fast_newtonschulz(Z, 5)
    assert torch.count_nonzero(out).item() == 0 and torch.isfinite(out.float()).all()
    G = torch.randn(128, 384, generator=torch.Generator().manual_seed(5)).to(env["dev"])
    a, b = mu.fast_newtonschulz(G, 5), mu.fast_newtonschulz(G * 4.0, 5)  # power-of-two scale: identical bf16 inputs
    assert rel_fro(a, b) < 2e-2
    # G.bfloat16() takes any floating dtype (muon_utils.py:138): fp16 and fp64 inputs give what their bf16 image gives
    H = G.half()
    assert torch.equal(mu.fast_newtonschulz(H, 5), mu.fast_newtonschulz(H.bfloat16(), 5))
    D = G.double()
    assert torch.equal(mu.fast_newtonschulz(D, 5), mu.fast_newtonschulz(D.bfloat16(), 5))


def test_newton_schulz_batched_matches_single_bitwise(env):
    mu = env["mu"]
    G = torch.randn(5, 128, 320, generator=torch.Generator().manual_seed(6)).to(env["dev"])
    stacked = mu.fast_newtonschulz(G, 5)
    for i in range(5):
        assert torch.equal(stacked[i], mu.fast_newtonschulz(G[i], 5))
    assert torch.equal(stacked, mu.fast_newtonschulz(G, 5)), "run-to-run determinism"


@pytest.mark.parametrize("rows,cols,batch", [(96, 200, 1), (200, 96, 2), (33, 47, 1), (512, 1024, 1)])
def test_normalize_stage_on_its_own(env, rows, cols, batch):
    """muon_hip_normalize after the first stage: X = bf(bf(G) / bf(bf(||bf(G)||_F) + 1e-7)) element for element
    (muon_utils.py:138-146), the same through muon_hip_ns_grouped with no iterations, zero stays zero."""
    print(f"normalize rows={rows} cols={cols} batch={batch}", flush=True)
    lib, abi, dev = env["lib"], env["abi"], env["dev"]
    G = torch.randn(batch, rows, cols, generator=torch.Generator().manual_seed(rows + cols + batch))
    G[-1, 0, :5] = 0.0
    X = G.bfloat16()
    d = (X.float().pow(2).sum(dim=(-2, -1), keepdim=True).sqrt().bfloat16() + 1e-7).bfloat16()  # bf16 norm, bf16 add
    ref = (X / d).bfloat16()
    assert torch.equal(ref, (X / (X.norm(dim=(-2, -1), keepdim=True) + 1e-7))), "the literal torch expression"
    Gd = G.to(dev)
    ws = torch.empty(abi.workspace_bytes(rows, cols, batch), dtype=torch.uint8, device=dev)
    out = [torch.full((batch, rows, cols), float("nan"), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    for o, via_ns in zip(out, (False, True)):
        abi.check(lib.muon_hip_cast_norm(Gd.data_ptr(), abi.dtype_code(Gd.dtype), ws.data_ptr(), rows, cols, batch, 0))
        if via_ns:
            abi.check(lib.muon_hip_ns_grouped(ws.data_ptr(), rows, cols, batch, 0, 3.4445, -4.775, 2.0315, 0))
        else:
            abi.check(lib.muon_hip_normalize(ws.data_ptr(), rows, cols, batch, 0))
        abi.check(lib.muon_hip_ns_output(ws.data_ptr(), rows, cols, batch, 0, o.data_ptr(), 0))
    torch.cuda.synchronize()
    assert torch.equal(out[0], out[1])
    # the device sums the squares in another order than torch, so for an unlucky sum the bf16 norm lands on the
    # neighbouring value and every element moves by up to one part in 256; otherwise the result is exact
    assert torch.equal(out[0].cpu(), ref) or rel_fro(out[0], ref) < 4.5e-3


@pytest.mark.parametrize("gdt,mdt", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                     (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("nesterov", [True, False])
@pytest.mark.parametrize("shape", [(64, 96), (37, 53)])
def test_momentum_stage(env, gdt, mdt, nesterov, shape):
    O, mu = env["O"], env["mu"]
    gen = torch.Generator().manual_seed(7)
    g = torch.randn(*shape, generator=gen).to(gdt)
    m = torch.randn(*shape, generator=gen).to(mdt)
    g_ref, m_ref = g.clone(), m.clone()
    u_ref = O.apply_momentum(g_ref, m_ref, 0.95, nesterov)
    gd, md = g.to(env["dev"]), m.to(env["dev"])
    u = mu.apply_momentum(gd, md, 0.95, nesterov)
    assert rel_fro(md, m_ref) <= (MOM_TOL if mdt == torch.float32 else 1e-3)
    if mdt == torch.float32 and gdt == torch.float32:
        assert rel_fro(u, u_ref) <= MOM_TOL
    else:
        assert rel_fro(u.float(), u_ref.float()) <= 4e-3  # u is stored in the grad's bf16


def _ns_via_stages(env, grads, moms, beta=0.95, nesterov=True, steps=5):
    """The unscaled Newton-Schulz output of a bucket, read from the workspace: muon_hip_momentum_norm ->
    muon_hip_ns_grouped -> muon_hip_ns_output on device tensors `grads` and `moms` (same shape; the momentum
    buffers move in place).  Returns a dense bf16 [batch, rows, cols] tensor."""
    lib, abi, dev = env["lib"], env["abi"], env["dev"]
    rows, cols = grads[0].shape
    nb = len(grads)
    ws = torch.empty(abi.workspace_bytes(rows, cols, nb), dtype=torch.uint8, device=dev)
    table = torch.tensor([t.data_ptr() for t in list(grads) + list(moms)], dtype=torch.int64, device=dev)
    out = torch.full((nb, rows, cols), float("nan"), dtype=torch.bfloat16, device=dev)
    a, b, c = env["O"].NS_COEFFS
    abi.check(lib.muon_hip_momentum_norm(table.data_ptr(), table.data_ptr() + 8 * nb, abi.dtype_code(grads[0].dtype),
                                         abi.dtype_code(moms[0].dtype), ws.data_ptr(), rows, cols, nb, beta, int(nesterov), 0, 0))
    abi.check(lib.muon_hip_ns_grouped(ws.data_ptr(), rows, cols, nb, steps, a, b, c, 0))
    abi.check(lib.muon_hip_ns_output(ws.data_ptr(), rows, cols, nb, steps, out.data_ptr(), 0))
    torch.cuda.synchronize()
    return out


def _build_opts(env, weights, hp, dtype, momentum_dtype=None, adam=None):
    """GPU optimizer from this package and the CPU oracle on copies of the same tensors."""
    mu, O = env["mu"], env["O"]
    dev = env["dev"]
    gp = [torch.nn.Parameter(w.clone().to(dtype).to(dev)) for _, w in weights]
    cp = [torch.nn.Parameter(w.clone().to(dtype)) for _, w in weights]
    ggroups = [dict(params=list(gp), use_muon=True, **hp)]
    cgroups = [dict(params=list(cp), use_muon=True, **hp)]
    if adam is not None:
        ga = [torch.nn.Parameter(w.clone().to(dev)) for w in adam]
        ca = [torch.nn.Parameter(w.clone()) for w in adam]
        ahp = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-10, weight_decay=0.01)
        ggroups.append(dict(params=ga, use_muon=False, **ahp))
        cgroups.append(dict(params=ca, use_muon=False, **ahp))
    opt = mu.Muon(ggroups, momentum_dtype=momentum_dtype)
    # the oracle works on the groups after the constructor sorted and filled them
    corder = sorted(cp, key=lambda x: x.size(), reverse=True)
    cgroups[0]["params"] = corder
    orc = O.OracleMuon(cgroups, momentum_dtype=momentum_dtype)
    return opt, orc, gp, cp


def _check_step(opt, orc, gp, cp, grads, dtype, p_tol, env=None):
    """One step on both sides; returns the worst update / momentum / parameter error.  The update error of an
    fp32 parameter is recovered from the parameter delta.  A bf16 parameter's delta is mostly its own rounding,
    so there the orthogonalised update is read directly: the stage entry points run on copies of the same
    gradient and momentum before the optimizer steps (pass `env`)."""
    dev = gp[0].device
    for p, c, g in zip(gp, cp, grads):
        p.grad = g.clone().to(dtype).to(dev)
        c.grad = g.clone().to(dtype)
    before = [p.detach().clone() for p in gp]
    staged = {}
    if dtype != torch.float32:
        assert env is not None
        for gi, group in enumerate(opt.param_groups):
            if not group["use_muon"]:
                continue
            for p in group["params"]:
                st = opt.state.get(p, {})
                m0 = st["momentum_buffer"].clone() if "momentum_buffer" in st else torch.zeros_like(
                    p, dtype=opt.momentum_dtype or p.dtype)
                o = _ns_via_stages(env, [p.grad.clone()], [m0], beta=group["momentum"], nesterov=group["nesterov"],
                                   steps=group["ns_steps"])[0]
                sc = env["mu"].scale_factor(p.shape[0], p.shape[1], group["rms_scale"])
                staged[p] = (o.float() * env["O"]._f32(sc)).bfloat16()
    opt.step()
    orc.step()
    torch.cuda.synchronize()
    worst_u = worst_m = worst_p = 0.0
    for gi, group in enumerate(orc.groups):
        if not group["use_muon"]:
            continue
        for pi, c in enumerate(group["params"]):
            p = opt.param_groups[gi]["params"][pi]
            assert p.shape == c.shape
            m_gpu = opt.state[p]["momentum_buffer"]
            m_cpu = orc.state[(gi, pi)]["momentum_buffer"]
            worst_m = max(worst_m, rel_fro(m_gpu, m_cpu))
            # recover the applied update from the parameter delta: o = (p_old*(1-lr*wd) - p_new)/lr
            idx = next(i for i, q in enumerate(gp) if q is p)
            lr, wd = group["lr"], group["weight_decay"]
            o_cpu = orc.last_updates[(gi, pi)].float()
            o_gpu = (before[idx].double().cpu() * (1 - lr * wd) - p.detach().double().cpu()) / lr
            if dtype == torch.float32:
                worst_u = max(worst_u, rel_fro(o_gpu, o_cpu))
            else:
                worst_u = max(worst_u, rel_fro(staged[p], o_cpu))
            worst_p = max(worst_p, rel_fro(p.detach(), c.detach()))
    return worst_u, worst_m, worst_p


def test_full_step_small_param_set_three_steps(env):
    """A 2-layer slice of the Qwen2.5-0.5B-shaped set (benchmark config 2 hyper-parameters),
    three consecutive steps, fp32 everything, plus a small AdamW-fallback group."""
    print("full step, 2 layers x 3 steps", flush=True)
    weights, grads = make_param_set(QWEN25_05B, layers=2, seed=1, steps=3)
    adam = [torch.randn(896, generator=torch.Generator().manual_seed(3)), torch.randn(1000, 64, generator=torch.Generator().manual_seed(4))]
    opt, orc, gp, cp = _build_opts(env, weights, MUON_HP, torch.float32, adam=adam)
    ga, ca = opt.param_groups[1]["params"], orc.groups[1]["params"]
    for step in range(3):
        for p, c in zip(ga, ca):
            g = torch.randn(*c.shape, generator=torch.Generator().manual_seed(100 + step))
            p.grad, c.grad = g.to(env["dev"]), g.clone()
        wu, wm, wp = _check_step(opt, orc, gp, cp, grads[step], torch.float32, None)
        report_parity(f"config 2 slice (2 layers, fp32) step {step}: update {wu:.3e} momentum {wm:.3e} param {wp:.3e}")
        assert wu <= NS_TOL and wm <= MOM_TOL
        assert wp <= 2e-3  # params move by lr*update each step; 2e-2 of that, relative to ||p||
        for ai, (p, c) in enumerate(zip(ga, ca)):
            assert rel_fro(p.detach(), c.detach()) <= 1e-6
            assert rel_fro(opt.state[p]["exp_avg"], orc.state[(1, ai)]["exp_avg"]) <= 1e-6
            assert rel_fro(opt.state[p]["exp_avg_sq"], orc.state[(1, ai)]["exp_avg_sq"]) <= 1e-6


@pytest.mark.parametrize("momentum_dtype", [None, torch.float32])
def test_full_step_bf16_params(env, momentum_dtype):
    """bf16 parameters and grads; momentum in bf16 (the reference's behaviour) or fp32."""
    spec = dict(q=(256, 256), k=(128, 256), v=(128, 256), o=(256, 256), gate=(640, 256), up=(640, 256), down=(256, 640))
    weights, grads = make_param_set(spec, layers=2, seed=11, steps=2, dtype=torch.bfloat16)
    opt, orc, gp, cp = _build_opts(env, weights, MUON_HP, torch.bfloat16, momentum_dtype=momentum_dtype)
    for step in range(2):
        wu, wm, wp = _check_step(opt, orc, gp, cp, grads[step], torch.bfloat16, None, env=env)
        report_parity(f"bf16 params (momentum {momentum_dtype}) step {step}: update {wu:.3e} momentum {wm:.3e} param {wp:.3e}")
        assert wu <= NS_TOL
        assert wm <= (MOM_TOL if momentum_dtype == torch.float32 else 1e-3)
        assert wp <= 4e-3  # a few bf16 roundings of p differ where the update differs


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_full_step_ragged_and_tall_shapes(env, dtype):
    """Shapes that are not whole tiles, not multiples of 8 and taller than wide (the update is then the transpose
    of the Newton-Schulz operand and goes through the transposing kernels), two steps each."""
    names = ["tall_odd", "wide_odd", "tall", "tall_vec", "square_odd", "thin"]
    shapes = [(53, 37), (37, 53), (300, 100), (640, 256), (129, 129), (1000, 8)]
    gen = torch.Generator().manual_seed(17)
    weights = [(n, 0.02 * torch.randn(*s, generator=gen)) for n, s in zip(names, shapes)]
    opt, orc, gp, cp = _build_opts(env, weights, MUON_HP, dtype, momentum_dtype=torch.float32 if dtype == torch.bfloat16 else None)
    for step in range(2):
        grads = [1e-3 * torch.randn(*s, generator=gen) for s in shapes]
        wu, wm, wp = _check_step(opt, orc, gp, cp, grads, dtype, None, env=env)
        print(f"ragged {dtype} step {step}: update {wu:.3e} momentum {wm:.3e} param {wp:.3e}", flush=True)
        assert wm <= MOM_TOL and wu <= NS_TOL
        if dtype == torch.float32:
            assert wp <= 2e-3  # params move by lr*update; 2e-2 of that relative to ||p||
        else:
            assert wp <= 4e-3


@pytest.mark.parametrize("hp", [
    dict(lr=0.05, momentum=0.9, nesterov=False, weight_decay=0.0, ns_steps=5, rms_scale=True),
    dict(lr=0.01, momentum=0.8, nesterov=True, weight_decay=0.1, ns_steps=1, rms_scale=True),
    dict(lr=0.02, momentum=0.95, nesterov=True, weight_decay=0.01, ns_steps=3, rms_scale=False),
    dict(lr=0.02, momentum=0.3, nesterov=False, weight_decay=0.01, ns_steps=4, rms_scale=False),
    dict(lr=0.02, momentum=0.95, nesterov=True, weight_decay=0.01, ns_steps=0, rms_scale=False),
], ids=lambda h: f"ns{h['ns_steps']}-{'nest' if h['nesterov'] else 'plain'}-{'rms' if h['rms_scale'] else 'ratio'}-b{h['momentum']}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_full_step_hyperparameters_against_the_oracle(env, hp, dtype):
    """Every hyper-parameter of a Muon group away from the benchmark's value: no Nesterov blend, momentum below 0.5 (the
    other branch of ATen's lerp), both scalings, no decay, 0 / 1 / 3 / 4 iterations (with none the update kernel runs,
    otherwise the parameter is updated inside the last product), on wide, tall and ragged shapes, two steps each."""
    names = ["wide", "tall", "square", "tall_ragged", "wide_ragged"]
    shapes = [(128, 384), (384, 128), (256, 256), (210, 77), (90, 250)]
    gen = torch.Generator().manual_seed(23)
    weights = [(n, 0.02 * torch.randn(*s, generator=gen)) for n, s in zip(names, shapes)]
    opt, orc, gp, cp = _build_opts(env, weights, hp, dtype, momentum_dtype=torch.float32 if dtype == torch.bfloat16 else None)
    for step in range(2):
        grads = [1e-3 * torch.randn(*s, generator=gen) for s in shapes]
        wu, wm, wp = _check_step(opt, orc, gp, cp, grads, dtype, None, env=env)
        print(f"hyper-parameters {hp} {dtype} step {step}: update {wu:.3e} momentum {wm:.3e} param {wp:.3e}", flush=True)
        assert wm <= MOM_TOL
        # fewer iterations leave less room for accumulation-order noise to grow; none is the rounded blend itself
        assert wu <= (NS_TOL if hp["ns_steps"] >= 4 else 4e-3)
        assert wp <= (2e-3 if dtype == torch.float32 else 4e-3) * max(1.0, hp["lr"] / 0.02) * (3.0 if hp["rms_scale"] else 1.0)


def test_grouped_equals_per_matrix_bitwise(env):
    mu = env["mu"]
    weights, grads = make_param_set(dict(QWEN25_05B, q=(256, 256), o=(256, 256), k=(128, 256), v=(128, 256),
                                         gate=(512, 256), up=(512, 256), down=(256, 512)), layers=2, seed=5, steps=1)
    dev = env["dev"]
    pa = [torch.nn.Parameter(w.clone().to(dev)) for _, w in weights]
    pb = [torch.nn.Parameter(w.clone().to(dev)) for _, w in weights]
    for p, q, g in zip(pa, pb, grads[0]):
        p.grad, q.grad = g.to(dev), g.to(dev)
    opt = mu.Muon([dict(params=pa, use_muon=True, **MUON_HP)])
    opt.step()
    group = dict(opt.param_groups[0])
    for q in pb:
        st = {"momentum_buffer": torch.zeros_like(q)}
        w = mu.SingelDeviceWork(q, st, group, 0)
        w.start()
        w.finish()
    torch.cuda.synchronize()
    for p, q in zip(pa, pb):
        assert torch.equal(p.detach(), q.detach())


@pytest.mark.parametrize("pdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols,batch", [(256, 384, 3), (37, 53, 2), (100, 300, 2), (512, 1024, 2), (768, 2048, 3), (64, 64, 1),
                                             (384, 256, 3), (53, 37, 2), (300, 100, 2), (1024, 512, 2), (2048, 768, 3), (1000, 520, 2),
                                             # more tiles than compute units: the persistent kernel carries the update
                                             (512, 1024, 40), (768, 2048, 24), (700, 1000, 30)])
def test_folded_update_equals_the_staged_sequence_bitwise(env, pdtype, rows, cols, batch):
    """muon_hip_step_grouped lets the epilogue of the last B.X apply the scaled update to the parameter without writing
    the final X': directly when the parameter has X's orientation (rows <= cols), through a transposing gather out of
    LDS when it is X's transpose (rows > cols).  The stage entry points run the same arithmetic through the stand-alone
    update kernel (itself bit-identical to torch on the device): parameters and momentum must come out equal bit for
    bit, ragged shapes, both orientations and both parameter dtypes included."""
    print(f"folded update {pdtype} {rows}x{cols} x{batch}", flush=True)
    lib, abi, mu, dev = env["lib"], env["abi"], env["mu"], env["dev"]
    gen = torch.Generator().manual_seed(rows * 13 + cols)
    gdt = torch.bfloat16 if pdtype == torch.bfloat16 else torch.float32
    p0 = [(0.02 * torch.randn(rows, cols, generator=gen)).to(pdtype).to(dev) for _ in range(batch)]
    g0 = [(1e-3 * torch.randn(rows, cols, generator=gen)).to(gdt).to(dev) for _ in range(batch)]
    m0 = [(1e-3 * torch.randn(rows, cols, generator=gen)).to(dev) for _ in range(batch)]
    a, b, c = env["O"].NS_COEFFS
    lr, wd, beta, steps = 0.02, 0.01, 0.95, 5
    scale = mu.scale_factor(rows, cols, True)
    outs = []
    for fused in (True, False):
        p, g, m = [t.clone() for t in p0], [t.clone() for t in g0], [t.clone() for t in m0]
        ws = torch.empty(abi.workspace_bytes(rows, cols, batch), dtype=torch.uint8, device=dev)
        table = torch.tensor([t.data_ptr() for t in p + g + m], dtype=torch.int64, device=dev)
        tp, tg, tm = table.data_ptr(), table.data_ptr() + 8 * batch, table.data_ptr() + 16 * batch
        codes = (abi.dtype_code(pdtype), abi.dtype_code(gdt), abi.F32)
        if fused:
            abi.check(lib.muon_hip_step_grouped(tp, tg, tm, *codes, ws.data_ptr(), rows, cols, batch, lr, wd, beta, 1, steps,
                                                scale, a, b, c, 0, 0))
        else:
            abi.check(lib.muon_hip_momentum_norm(tg, tm, codes[1], codes[2], ws.data_ptr(), rows, cols, batch, beta, 1, 0, 0))
            abi.check(lib.muon_hip_ns_grouped(ws.data_ptr(), rows, cols, batch, steps, a, b, c, 0))
            abi.check(lib.muon_hip_apply_update(tp, codes[0], ws.data_ptr(), rows, cols, batch, steps, scale, lr, wd, 0))
        torch.cuda.synchronize()
        outs.append((p, m))
    for i in range(batch):
        assert torch.equal(outs[0][1][i], outs[1][1][i])
        assert torch.equal(outs[0][0][i], outs[1][0][i]), f"matrix {i}: {(outs[0][0][i] != outs[1][0][i]).sum().item()} elements differ"
        assert not torch.equal(outs[0][0][i], p0[i]), "the parameter moved"


def test_grouped_equals_per_matrix_bitwise_on_256_tiles(env):
    """The same for shapes whose short side is a whole number of 256-tiles (ping-pong and split-tail kernels) and
    for the expert shapes 768x2048 / 2048x768 (128-tiles): bf16 parameters, fp32 momentum, three matrices per
    bucket against three launches of one."""
    mu, dev = env["mu"], env["dev"]
    spec = dict(q=(512, 512), k=(768, 2048), v=(768, 2048), o=(512, 512), gate=(2048, 768), up=(1024, 512), down=(512, 1024))
    weights, grads = make_param_set(spec, layers=3, seed=15, steps=1, dtype=torch.bfloat16)
    pa = [torch.nn.Parameter(w.clone().to(dev)) for _, w in weights]
    pb = [torch.nn.Parameter(w.clone().to(dev)) for _, w in weights]
    for p, q, g in zip(pa, pb, grads[0]):
        p.grad, q.grad = g.to(dev), g.to(dev)
    opt = mu.Muon([dict(params=pa, use_muon=True, **MUON_HP)], momentum_dtype=torch.float32)
    opt.step()
    group = dict(opt.param_groups[0])
    for q in pb:
        st = {"momentum_buffer": torch.zeros_like(q, dtype=torch.float32)}
        w = mu.SingelDeviceWork(q, st, group, 0)
        w.start()
        w.finish()
    torch.cuda.synchronize()
    for (name, _), p, q in zip(weights, pa, pb):
        assert torch.equal(p.detach(), q.detach()), name


def _chunk_plan(env, rows, cols, n, cap):
    """(workspace limit that holds `cap` matrices of the shape, matrices per launch the optimizer then takes)."""
    per = env["abi"].workspace_bytes(rows, cols, 1)
    limit = cap * per + per // 2
    assert limit // per == cap
    return limit, env["mu"]._pick_chunk(n, cap, rows, cols)


@pytest.mark.parametrize("rows,cols,n,cap,kernel", [
    (2048, 2048, 23, 8, "persistent"),   # 36 + 36 + 64 tiles a matrix: all three products of a chunk of 8 walk tiles
    (2048, 1024, 7, 3, "transposed"),    # rows > cols on 256-tiles: the update goes through the transposing gather
    (640, 384, 10, 4, "128-tiles"),      # short side no whole number of 256-tiles, transposed and ragged
])
def test_chunked_bucket_equals_the_unchunked_twin_bitwise(env, rows, cols, n, cap, kernel):
    """The reference steps one parameter at a time (muon_utils.py:443-456); here a bucket larger than the workspace
    limit is cut into chunks that share one workspace, each with a cached device pointer table keyed by its first
    index.  A bucket of n same-shape matrices under a limit that holds `cap` of them must run as at least three chunks
    with a ragged last one and leave parameters and momentum bit-equal to a twin that runs the bucket in one launch,
    over three steps (the second and third find the tables of the step before), and within the parity bounds of the
    CPU oracle on the first, a middle and the last matrix.  The workspace never exceeds the limit."""
    print(f"chunked dispatch {rows}x{cols} x{n}, cap {cap} ({kernel})", flush=True)
    mu, O, dev = env["mu"], env["O"], env["dev"]
    limit, chunk = _chunk_plan(env, rows, cols, n, cap)
    nchunks = -(-n // chunk)
    assert nchunks >= 3 and n % chunk != 0, (chunk, nchunks)
    if kernel == "persistent":
        T = rows // 256
        assert chunk * T * (T + 1) // 2 > 256 and chunk * T * (cols // 256) > 256  # more tiles than compute units
    gen = torch.Generator().manual_seed(rows + 3 * cols + n)
    w0 = [(0.02 * torch.randn(rows, cols, generator=gen)).bfloat16() for _ in range(n)]
    hp = dict(MUON_HP)
    twins = []
    for lim in (limit, 1 << 40):
        ps = [torch.nn.Parameter(w.clone().to(dev)) for w in w0]
        twins.append((ps, mu.Muon([dict(params=list(ps), use_muon=True, **hp)], momentum_dtype=torch.float32,
                                  workspace_limit_bytes=lim)))
    sample = sorted({0, n // 2, n - 1})
    cw = {i: w0[i].clone() for i in sample}
    cm = {i: torch.zeros(rows, cols) for i in sample}
    for step in range(3):
        grads = [(1e-3 * torch.randn(rows, cols, generator=gen)).bfloat16() for _ in range(n)]
        for ps, opt in twins:
            for p, g in zip(ps, grads):
                p.grad = g.to(dev)
            opt.step()
        torch.cuda.synchronize()
        (pa, oa), (pb, ob) = twins
        assert len(oa._pointer_tables) == nchunks
        assert oa._workspaces[dev].numel() <= limit < ob._workspaces[dev].numel()
        for i in range(n):
            assert torch.equal(pa[i].detach(), pb[i].detach()), f"step {step}, matrix {i}: parameter"
            assert torch.equal(oa.state[pa[i]]["momentum_buffer"], ob.state[pb[i]]["momentum_buffer"]), f"step {step}, matrix {i}: momentum"
        sc = O._f32(mu.scale_factor(rows, cols, False))
        for i in sample:
            # the orthogonalised update itself: the stage entry points on the same gradient and the momentum before the step
            got = _ns_via_stages(env, [grads[i].to(dev)], [cm[i].to(dev)])[0]
            o = O.muon_step_matrix(cw[i], grads[i].clone(), cm[i], lr=hp["lr"], weight_decay=hp["weight_decay"],
                                   beta=hp["momentum"], nesterov=True, ns_steps=5, rms_scale=False)
            wu, wm = rel_fro((got.float() * sc).bfloat16(), o), rel_fro(oa.state[pa[i]]["momentum_buffer"], cm[i])
            report_parity(f"chunked dispatch {rows}x{cols} step {step} matrix {i}: update {wu:.3e} momentum {wm:.3e}")
            assert wu <= NS_TOL and wm <= MOM_TOL
            assert rel_fro(pa[i].detach(), cw[i]) <= 4e-3


def test_chunked_bucket_follows_a_group_whose_tensors_change(env):
    """A cached pointer table must miss when the tensors behind a chunk change: between steps one parameter leaves the
    group (every later matrix moves up one place, across chunk boundaries), the gradients move to fresh addresses, and
    the parameter comes back.  The chunked optimizer stays bit-equal to the twin that runs one launch per bucket."""
    mu, dev = env["mu"], env["dev"]
    rows, cols, n, cap = 512, 768, 11, 4
    limit, chunk = _chunk_plan(env, rows, cols, n, cap)
    assert -(-n // chunk) >= 3
    gen = torch.Generator().manual_seed(77)
    w0 = [(0.02 * torch.randn(rows, cols, generator=gen)) for _ in range(n)]
    twins = []
    for lim in (limit, 1 << 40):
        ps = [torch.nn.Parameter(w.clone().to(dev)) for w in w0]
        twins.append((ps, mu.Muon([dict(params=list(ps), use_muon=True, **MUON_HP)], workspace_limit_bytes=lim)))
    keep = []  # old gradients stay alive, so that new ones cannot land on their addresses
    members = [list(range(n)), [i for i in range(n) if i != 2], list(range(n)), list(reversed(range(n)))]
    for step, idx in enumerate(members):
        grads = [1e-3 * torch.randn(rows, cols, generator=gen) for _ in range(n)]
        for ps, opt in twins:
            opt.param_groups[0]["params"] = [ps[i] for i in idx]
            for p, g in zip(ps, grads):
                p.grad = g.to(dev)
                keep.append(p.grad)
            opt.step()
        torch.cuda.synchronize()
        (pa, oa), (pb, ob) = twins
        for i in range(n):
            assert torch.equal(pa[i].detach(), pb[i].detach()), f"step {step}, matrix {i}"
            if pa[i] in oa.state:
                assert torch.equal(oa.state[pa[i]]["momentum_buffer"], ob.state[pb[i]]["momentum_buffer"])
    # matrix 2 sat out one step: it differs from a matrix that took all four, i.e. the steps really followed `members`
    assert not torch.equal(twins[0][0][2].detach(), w0[2].to(dev))


BUCKET_SHAPES = [(4096, 4096), (1024, 4096), (12288, 4096), (4096, 12288),      # Qwen3-8B (benchmark config 3)
                 (768, 2048), (2048, 768), (512, 2048), (4096, 2048), (2048, 4096)]  # Qwen3-MoE-30B-A3B (config 5)


@pytest.mark.parametrize("rows,cols", BUCKET_SHAPES)
def test_bucket_shapes_grouped_ns_output_within_bound(env, rows, cols):
    """Every bucket shape of the two bf16 benchmark configurations in a grouped launch (bf16 gradients, fp32
    momentum, several matrices): the orthogonalised update itself, read from the workspace after
    muon_hip_momentum_norm -> muon_hip_ns_grouped -> muon_hip_ns_output, per matrix within 2e-2 relative
    Frobenius error of (a) fast_newtonschulz's own torch expressions (muon_utils.py:138-156) evaluated on the
    device for every matrix, with torch's fp32-accumulated product standing in for the Triton kernel, and (b) the
    CPU oracle for the first matrix."""
    O, dev = env["O"], env["dev"]
    batch = 6 if rows * cols <= 2048 * 2048 else 2
    print(f"bucket {rows}x{cols} batch={batch}", flush=True)
    gen = torch.Generator().manual_seed(rows * 3 + cols)
    g = [(1e-3 * torch.randn(rows, cols, generator=gen)).bfloat16() for _ in range(batch)]
    m = [1e-3 * torch.randn(rows, cols, generator=gen) for _ in range(batch)]
    gd, md = [t.to(dev) for t in g], [t.to(dev) for t in m]
    m_ref = [t.clone() for t in md]
    out = _ns_via_stages(env, gd, md)
    assert torch.isfinite(out).all()
    torch.set_num_threads(16)
    worst = 0.0
    for i in range(batch):
        # the blend the extension defines for (bf16 g, fp32 m): gradient upcast, fp32 lerps
        gf = gd[i].float()
        m_ref[i].lerp_(gf, 1 - 0.95)
        u = gf.lerp_(m_ref[i], 0.95)
        assert torch.equal(md[i], m_ref[i]), "fp32 momentum is the device lerp, bit for bit"
        ref_dev = O.newton_schulz(u, 5, literal=True)
        e_dev = rel_fro(out[i], ref_dev)
        line = f"  matrix {i}: vs torch on device {e_dev:.3e}"
        assert e_dev <= NS_TOL, (rows, cols, i, e_dev)
        worst = max(worst, e_dev)
        if i == 0:
            e_cpu = rel_fro(out[i], O.newton_schulz(u.cpu(), 5))
            line += f", vs CPU oracle {e_cpu:.3e}"
            assert e_cpu <= NS_TOL, (rows, cols, e_cpu)
            worst = max(worst, e_cpu)
        print(line, flush=True)
    report_parity(f"bucket {rows}x{cols} x{batch} grouped (bf16 g, fp32 m): worst NS-output error {worst:.3e} (bound {NS_TOL})")


def test_module_substitution_factory_groups_and_checkpoint_round_trip(env, tmp_path, monkeypatch):
    """The integration recipe end to end: the module installed as lmms_engine.utils.muon_utils, the optimizer
    built through that import from the four groups Trainer.create_optimizer makes (train/hf/trainer.py:417-465),
    stepped on the GPU, and its state_dict sent through torch.save / torch.load (weights only, as a checkpoint
    is read back) into a fresh optimizer that then continues bit-identically, fp32 momentum included."""
    import sys
    import types

    mu, dev = env["mu"], env["dev"]
    pkg, sub = types.ModuleType("lmms_engine"), types.ModuleType("lmms_engine.utils")
    pkg.utils, sub.muon_utils = sub, mu
    monkeypatch.setitem(sys.modules, "lmms_engine", pkg)
    monkeypatch.setitem(sys.modules, "lmms_engine.utils", sub)
    monkeypatch.setitem(sys.modules, "lmms_engine.utils.muon_utils", mu)
    from lmms_engine.utils.muon_utils import Muon

    assert Muon is mu.Muon

    def model(seed):
        gen = torch.Generator().manual_seed(seed)
        mk = lambda *s: torch.nn.Parameter((0.02 * torch.randn(*s, generator=gen)).bfloat16().to(dev))
        return dict(q=mk(256, 256), up=mk(640, 256), down=mk(256, 640), emb=mk(1000, 64), norm=mk(256))

    def factory(ps, **extra):
        lr = 1e-3
        groups = [
            dict(params=[ps["q"]], use_muon=True, lr=lr, momentum=0.95, weight_decay=0.01),
            dict(params=[ps["up"], ps["down"]], use_muon=True, lr=lr, momentum=0.95, weight_decay=0.0),
            dict(params=[ps["emb"]], use_muon=False, lr=lr, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01),
            dict(params=[ps["norm"]], use_muon=False, lr=lr, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0),
        ]
        return Muon(groups, defaults=dict(lr=lr), is_deepspeed_enabled=False, **extra)

    def set_grads(ps, seed):
        gen = torch.Generator().manual_seed(seed)
        for p in ps.values():
            p.grad = (1e-3 * torch.randn(*p.shape, generator=gen)).bfloat16().to(dev)

    ps = model(1)
    opt = factory(ps, momentum_dtype=torch.float32)
    for step in range(2):
        set_grads(ps, 10 + step)
        opt.step()
    path = tmp_path / "optimizer.pt"
    torch.save(opt.state_dict(), path)
    sd = torch.load(path, map_location=dev, weights_only=True)
    assert sd["state"][0]["momentum_buffer"].dtype == torch.float32
    assert sd["state"][3]["step"] == 2 and set(sd["state"][3]) == {"exp_avg", "exp_avg_sq", "step"}
    ps2 = {k: torch.nn.Parameter(v.detach().clone()) for k, v in ps.items()}
    opt2 = factory(ps2, momentum_dtype=torch.float32)
    opt2.load_state_dict(sd)
    for p, q in zip(ps.values(), ps2.values()):
        if p.ndim == 2 and p is not ps["emb"]:
            assert opt2.state[q]["momentum_buffer"].dtype == torch.float32
            assert torch.equal(opt2.state[q]["momentum_buffer"], opt.state[p]["momentum_buffer"])
    set_grads(ps, 99)
    set_grads(ps2, 99)
    opt.step()
    opt2.step()
    torch.cuda.synchronize()
    for k in ps:
        assert torch.equal(ps[k].detach(), ps2[k].detach()), k
    # releasing the workspace between steps changes nothing but the memory held
    opt.release_workspace()
    assert opt._workspaces == {}
    set_grads(ps, 100)
    set_grads(ps2, 100)
    opt.step()
    opt2.step()
    for k in ps:
        assert torch.equal(ps[k].detach(), ps2[k].detach()), k


def test_muon_step_replays_from_a_hip_graph(env):
    """A step over static tensors records into a HIP graph (the pointer tables of the last step are reused, so nothing is
    allocated or copied while recording) and every replay equals the eager step of a twin optimizer bit for bit: four
    replays, each followed by the twin's eager step and a synchronisation.  The set holds buckets that run the persistent
    kernels (their tile counters are taken at record time and must come back to zero after every replay), a transposed
    bucket and a 128-tile one."""
    dev, mu = env["dev"], env["mu"]
    shapes = [(768, 2048)] * 60 + [(1024, 512)] * 4 + [(384, 640)] * 3

    def make():
        g = torch.Generator().manual_seed(5)
        ps = [torch.nn.Parameter((torch.randn(r, c, generator=g) * 0.02).bfloat16().to(dev)) for r, c in shapes]
        for p in ps:
            p.grad = (torch.randn(p.shape, generator=g) * 0.01).bfloat16().to(dev)
        opt = mu.Muon([dict(params=ps, use_muon=True, lr=0.02, momentum=0.95, weight_decay=0.01, rms_scale=False)],
                      momentum_dtype=torch.float32)
        return ps, opt

    (pa, oa), (pb, ob) = make(), make()
    for _ in range(2):  # state, workspace and pointer tables exist after the first steps
        oa.step()
        ob.step()
    torch.cuda.synchronize()
    # Per-kernel timing left switched on does not leak event records into the recording: launches under capture go
    # untimed and are counted as such.
    abi = env["abi"]
    abi.timing_enable(True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        oa.step()
    assert abi.lib().muon_hip_timing_untimed() > 0
    assert sum(cnt for _, cnt in abi.timing_read().values()) == 0
    abi.timing_enable(False)
    for rep in range(4):
        print(f"graph replay {rep}", flush=True)
        graph.replay()
        ob.step()
        torch.cuda.synchronize()
        for i, (p, q) in enumerate(zip(pa, pb)):
            assert torch.equal(p, q), (rep, i, shapes[i])
            assert torch.equal(oa.state[p]["momentum_buffer"], ob.state[q]["momentum_buffer"]), (rep, i)
    # the recording replays into the optimizer's workspace: it cannot be released while the graph may run again
    with pytest.raises(RuntimeError, match="recorded"):
        oa.release_workspace()
    del graph
    oa.forget_recordings()
    oa.release_workspace()
    ob.release_workspace()
    oa.step()  # and the next eager step allocates it again
    ob.step()
    torch.cuda.synchronize()
    assert all(torch.equal(p, q) for p, q in zip(pa, pb))


def test_two_optimizers_on_two_streams_one_replaying_a_graph(env):
    """Two optimizers step at the same time on two streams, one of them replaying a recorded HIP graph: everything their
    kernels share (operands, norms, the tile counters of the persistent kernels) lives in each optimizer's own
    workspace, so neither can take the other's tiles.  Three rounds, no synchronisation between the two streams inside
    a round; parameters and momentum must equal those of twins that run the same steps one after the other.  Buckets:
    expert-shaped matrices (all three products persistent), a transposed one, a 128-tile one."""
    dev, mu = env["dev"], env["mu"]
    shapes = [(768, 2048)] * 60 + [(1024, 512)] * 4 + [(384, 640)] * 3

    def make(seed):
        g = torch.Generator().manual_seed(seed)
        ps = [torch.nn.Parameter((torch.randn(r, c, generator=g) * 0.02).bfloat16().to(dev)) for r, c in shapes]
        for p in ps:
            p.grad = (torch.randn(p.shape, generator=g) * 0.01).bfloat16().to(dev)
        opt = mu.Muon([dict(params=ps, use_muon=True, lr=0.02, momentum=0.95, weight_decay=0.01, rms_scale=False)],
                      momentum_dtype=torch.float32)
        return ps, opt

    # (a, b) run concurrently, a from a graph; (c, d) are their serial twins
    (pa, oa), (pb, ob), (pc, oc), (pd, od) = make(5), make(6), make(5), make(6)
    for _ in range(2):
        for o in (oa, ob, oc, od):
            o.step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        oa.step()
    s1, s2 = torch.cuda.Stream(dev), torch.cuda.Stream(dev)
    for rep in range(3):
        print(f"two streams, round {rep}", flush=True)
        with torch.cuda.stream(s1):
            graph.replay()
        with torch.cuda.stream(s2):
            ob.step()
        oc.step()
        od.step()
        torch.cuda.synchronize()
        for name, ps, opt, qs, ref in (("graph", pa, oa, pc, oc), ("eager", pb, ob, pd, od)):
            for i, (p, q) in enumerate(zip(ps, qs)):
                assert torch.equal(p, q), (name, rep, i, shapes[i])
                assert torch.equal(opt.state[p]["momentum_buffer"], ref.state[q]["momentum_buffer"]), (name, rep, i)


def test_step_under_capture_refuses_tensors_that_moved(env):
    """Recording a step needs the device pointer tables of an earlier eager step.  When a tensor behind a table has moved
    (here a gradient re-allocated after the eager steps), the step raises instead of recording a copy out of a host
    buffer that is gone by the time the graph replays."""
    dev, mu = env["dev"], env["mu"]
    g = torch.Generator().manual_seed(9)
    ps = [torch.nn.Parameter((torch.randn(256, 384, generator=g) * 0.02).to(dev)) for _ in range(3)]
    for p in ps:
        p.grad = (torch.randn(p.shape, generator=g) * 0.01).to(dev)
    opt = mu.Muon([dict(params=ps, use_muon=True, **MUON_HP)])
    opt.step()
    opt.step()
    torch.cuda.synchronize()
    keep = ps[0].grad  # stays alive, so the clone lands elsewhere
    ps[0].grad = keep.clone()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(env["abi"].MuonHipError, match="capture"):
        with torch.cuda.graph(graph):
            opt.step()
    torch.cuda.synchronize()
    opt.step()  # eager steps go on as before
    torch.cuda.synchronize()


def test_strided_parameters_and_state_step_like_row_major_ones(env):
    """The reference's torch expressions take parameters of any strides (muon_utils.py:324-325, :476-477).  A Muon
    parameter that is a transposed view (its momentum buffer, made by zeros_like, then has the same strides), a
    parameter with a strided gradient, and an AdamW parameter that is a transposed view step through row-major copies:
    values must equal those of row-major twins bit for bit over two steps, and the strides must survive."""
    mu, dev = env["mu"], env["dev"]
    gen = torch.Generator().manual_seed(61)
    w = [0.02 * torch.randn(256, 384, generator=gen), 0.02 * torch.randn(384, 256, generator=gen), 0.02 * torch.randn(96, 40, generator=gen)]
    e = torch.randn(50, 30, generator=gen)

    def as_t_view(t):  # same values, column-major storage
        return t.to(dev).t().contiguous().t()

    pa = [torch.nn.Parameter(w[0].to(dev)), torch.nn.Parameter(w[1].to(dev)), torch.nn.Parameter(w[2].to(dev))]
    pb = [torch.nn.Parameter(as_t_view(w[0])), torch.nn.Parameter(w[1].to(dev)), torch.nn.Parameter(as_t_view(w[2]))]
    ea, eb = torch.nn.Parameter(e.to(dev)), torch.nn.Parameter(as_t_view(e))
    assert not pb[0].is_contiguous() and not eb.is_contiguous()
    ahp = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-10, weight_decay=0.01)
    oa = mu.Muon([dict(params=list(pa), use_muon=True, **MUON_HP), dict(params=[ea], use_muon=False, **ahp)], write_back_grad=True)
    ob = mu.Muon([dict(params=list(pb), use_muon=True, **MUON_HP), dict(params=[eb], use_muon=False, **ahp)], write_back_grad=True)
    for step in range(2):
        gs = [1e-3 * torch.randn(*t.shape, generator=gen) for t in w]
        ge = torch.randn(50, 30, generator=gen)
        for p, q, g in zip(pa, pb, gs):
            p.grad = g.to(dev)
            q.grad = as_t_view(g) if q is not pb[0] else g.to(dev)  # strided gradients for the row-major and one strided parameter
        ea.grad, eb.grad = ge.to(dev), as_t_view(ge)
        oa.step()
        ob.step()
        torch.cuda.synchronize()
        for p, q in zip(pa + [ea], pb + [eb]):
            assert torch.equal(p.detach(), q.detach()), (step, tuple(p.shape))
        for p, q in zip(pa, pb):
            assert torch.equal(oa.state[p]["momentum_buffer"], ob.state[q]["momentum_buffer"])
            assert torch.equal(p.grad, q.grad)  # write_back_grad: the blend reaches a strided gradient too
        assert torch.equal(oa.state[ea]["exp_avg_sq"], ob.state[eb]["exp_avg_sq"])
    assert pb[0].stride() == (1, 256) and ob.state[pb[0]]["momentum_buffer"].stride() == (1, 256) and eb.stride() == (1, 50)


def test_reference_bug_compat_and_rms_scale(env):
    """The reference's single-device call site runs range(True) = 1 NS iteration; the flag reproduces it."""
    mu, O = env["mu"], env["O"]
    dev = env["dev"]
    w = torch.randn(96, 160, generator=torch.Generator().manual_seed(8)) * 0.02
    g = torch.randn(96, 160, generator=torch.Generator().manual_seed(9)) * 1e-3
    p = torch.nn.Parameter(w.clone().to(dev))
    p.grad = g.clone().to(dev)
    opt = mu.Muon([dict(params=[p], use_muon=True, lr=0.02, weight_decay=0.0)], reference_bug_compat=True)
    assert opt.param_groups[0]["rms_scale"] is True
    opt.step()
    c, m = w.clone(), torch.zeros_like(w)
    nesterov, ns_steps = O.reference_bug_compat_args(nesterov=True, ns_steps=5)
    O.muon_step_matrix(c, g.clone(), m, lr=0.02, weight_decay=0.0, beta=0.95, nesterov=nesterov, ns_steps=ns_steps, rms_scale=True)
    assert rel_fro((p.detach().cpu() - w), (c - w)) <= 5e-3


def test_state_dict_layout_and_resume(env):
    mu = env["mu"]
    dev = env["dev"]
    shapes = [(2, 3), (5, 1), (2, 3), (5, 4)]
    ps = [torch.nn.Parameter(torch.randn(*s, device=dev)) for s in shapes]
    emb = torch.nn.Parameter(torch.randn(10, device=dev))

    def make(params, e):
        return mu.Muon([dict(params=list(params), use_muon=True, lr=0.01), dict(params=[e], use_muon=False)])

    opt = make(ps, emb)
    assert [tuple(p.shape) for p in opt.param_groups[0]["params"]] == [(5, 4), (5, 1), (2, 3), (2, 3)]
    assert opt.state_dict()["state"] == {}, "state is created lazily"
    for p in ps + [emb]:
        p.grad = torch.randn_like(p)
    ps[1].grad = None  # a missing grad becomes zeros
    opt.step()
    assert ps[1].grad is not None and torch.count_nonzero(ps[1].grad).item() == 0
    sd = copy.deepcopy(opt.state_dict())  # state_dict() hands out the live tensors
    assert set(sd.keys()) == {"state", "param_groups"}
    assert sd["param_groups"][0]["params"] == [0, 1, 2, 3] and sd["param_groups"][1]["params"] == [4]
    assert set(sd["param_groups"][0].keys()) == {"params", "lr", "momentum", "weight_decay", "use_muon", "rms_scale", "nesterov", "ns_steps"}
    assert set(sd["param_groups"][1].keys()) == {"params", "lr", "betas", "eps", "weight_decay", "use_muon"}
    for i in range(4):
        assert set(sd["state"][i].keys()) == {"momentum_buffer"}
    assert set(sd["state"][4].keys()) == {"exp_avg", "exp_avg_sq", "step"} and sd["state"][4]["step"] == 1
    # resume: a fresh optimizer over clones + load_state_dict continues identically
    ps2 = [torch.nn.Parameter(p.detach().clone()) for p in ps]
    emb2 = torch.nn.Parameter(emb.detach().clone())
    opt2 = make(ps2, emb2)
    opt2.load_state_dict(sd)
    for p, q in zip(ps + [emb], ps2 + [emb2]):
        gr = torch.randn_like(p)
        p.grad, q.grad = gr, gr.clone()
    opt.step()
    opt2.step()
    for p, q in zip(ps + [emb], ps2 + [emb2]):
        assert torch.equal(p.detach(), q.detach())
    assert opt2.state_dict()["state"][4]["step"] == 2


def test_fp32_momentum_survives_load_state_dict(env):
    mu = env["mu"]
    dev = env["dev"]
    p = torch.nn.Parameter(torch.randn(64, 64, device=dev).bfloat16())
    p.grad = torch.randn(64, 64, device=dev).bfloat16()
    opt = mu.Muon([dict(params=[p], use_muon=True)], momentum_dtype=torch.float32)
    opt.step()
    sd = opt.state_dict()
    assert sd["state"][0]["momentum_buffer"].dtype == torch.float32
    opt2 = mu.Muon([dict(params=[p], use_muon=True)], momentum_dtype=torch.float32)
    opt2.load_state_dict(sd)
    m2 = opt2.state[p]["momentum_buffer"]
    assert m2.dtype == torch.float32 and torch.equal(m2, sd["state"][0]["momentum_buffer"])


def test_closure_and_asserts(env):
    mu = env["mu"]
    dev = env["dev"]
    p = torch.nn.Parameter(torch.randn(8, 8, device=dev))
    opt = mu.Muon([dict(params=[p], use_muon=True)])
    calls = []

    def closure():
        assert torch.is_grad_enabled()
        loss = (p * p).sum()
        loss.backward()
        calls.append(1)
        return loss

    out = opt.step(closure)
    assert calls == [1] and out is not None
    bad = torch.nn.Parameter(torch.randn(8, device=dev))
    bad.grad = torch.zeros_like(bad)
    opt_bad = mu.Muon([dict(params=[bad], use_muon=True)])
    with pytest.raises(AssertionError):
        opt_bad.step()


def test_matmul_transpose_api(env):
    mu = env["mu"]
    X = torch.randn(200, 328, generator=torch.Generator().manual_seed(12)).bfloat16()
    out = mu.matmul_transpose(X.to(env["dev"])).cpu()
    ref = X.double() @ X.double().mT
    assert out.shape == (200, 200) and torch.equal(out, out.mT)
    _assert_product_close(out, ref, X.double().abs() @ X.double().abs().mT)
    with pytest.raises(AssertionError):
        mu.matmul_transpose_assign(X, torch.empty(200, 200, dtype=torch.bfloat16))  # CPU tensors


def test_config2_full_size_sampled_parity(env):
    """Benchmark config 2 at full size (24 layers, 168 matrices, 3 steps) on the GPU; the
    oracle checks layer 0 and layer 23 (matrices are independent, so a sample is exact)."""
    print("config 2 full size", flush=True)
    mu, O = env["mu"], env["O"]
    dev = env["dev"]
    weights, grads = make_param_set(QWEN25_05B, layers=24, seed=1, steps=3)
    gp = [torch.nn.Parameter(w.clone().to(dev)) for _, w in weights]
    opt = mu.Muon([dict(params=list(gp), use_muon=True, **MUON_HP)])
    sample = [i for i, (n, _) in enumerate(weights) if n.startswith("layers.0.") or n.startswith("layers.23.")]
    cw = {i: weights[i][1].clone() for i in sample}
    cm = {i: torch.zeros_like(weights[i][1]) for i in sample}
    for step in range(3):
        for p, g in zip(gp, grads[step]):
            p.grad = g.to(dev)
        before = {i: gp[i].detach().clone() for i in sample}
        opt.step()
        torch.cuda.synchronize()
        for i in sample:
            o = O.muon_step_matrix(cw[i], grads[step][i].clone(), cm[i], **{k: MUON_HP[k] for k in ("lr", "weight_decay", "nesterov", "ns_steps", "rms_scale")}, beta=MUON_HP["momentum"])
            lr, wd = MUON_HP["lr"], MUON_HP["weight_decay"]
            o_gpu = (before[i].double().cpu() * (1 - lr * wd) - gp[i].detach().double().cpu()) / lr
            assert rel_fro(o_gpu, o.float()) <= NS_TOL, (step, weights[i][0])
            assert rel_fro(opt.state[gp[i]]["momentum_buffer"], cm[i]) <= MOM_TOL
        # size-independent property on every matrix: the orthogonalised update has singular values near 1,
        # so ||o||_F^2 is close to min(rows, cols) (times the shape scale squared)
    for i, p in enumerate(gp):
        assert torch.isfinite(p).all()


def _sv_band(out: torch.Tensor, probes: int = 8):
    """Size-independent property of an orthogonalised matrix: five quintic iterations put every
    singular value in about [0.55, 1.25], so ||out^T v|| / ||v|| (rows <= cols) stays in that band for
    any v, and ||out||_F^2 / min(rows, cols) is the mean squared singular value.  fp64 on the CPU."""
    o = out.double().cpu()
    if o.shape[0] > o.shape[1]:
        o = o.mT
    gen = torch.Generator().manual_seed(5)
    v = torch.randn(o.shape[0], probes, dtype=torch.float64, generator=gen)
    ratio = (o.mT @ v).norm(dim=0) / v.norm(dim=0)
    return ratio.min().item(), ratio.max().item(), (o.norm() ** 2 / o.shape[0]).item()


@pytest.mark.parametrize("rows,cols", [(4096, 12288), (8192, 8192), (28672, 8192)])
def test_full_size_newton_schulz(env, rows, cols):
    """Benchmark config 3's largest shape and config 4's two matrices (N(0,1), seed 2, 5 iterations)
    at full size: against the oracle on the host cores, and through properties that do not need it
    (transpose equivariance and power-of-two scale invariance are exact; singular values land in the band)."""
    print(f"full-size NS {rows}x{cols}", flush=True)
    mu, O = env["mu"], env["O"]
    G = torch.randn(rows, cols, generator=torch.Generator().manual_seed(2))
    Gd = G.to(env["dev"])
    out = mu.fast_newtonschulz(Gd, steps=5)
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and out.shape == (rows, cols) and torch.isfinite(out).all()
    out_t = mu.fast_newtonschulz(Gd.mT.contiguous(), steps=5)
    if rows != cols:
        assert torch.equal(out_t, out.mT)  # the transpose rule makes both calls run the same arithmetic
    else:
        assert rel_fro(out_t, out.mT) <= NS_TOL  # a square matrix is iterated as given: equal only up to rounding
    out_s = mu.fast_newtonschulz(Gd * 8.0, steps=5)
    assert torch.equal(out_s, out)
    lo, hi, mean_sq = _sv_band(out)
    print(f"  sv probe band [{lo:.3f}, {hi:.3f}], mean s^2 {mean_sq:.3f}", flush=True)
    assert 0.5 <= lo and hi <= 1.3 and 0.4 <= mean_sq <= 1.4
    torch.set_num_threads(16)
    ref = O.newton_schulz(G, 5)
    err = rel_fro(out, ref)
    report_parity(f"full-size NS {rows}x{cols} (N(0,1), seed 2): error vs oracle {err:.3e} (bound {NS_TOL})")
    assert err <= NS_TOL


def test_config3_one_layer_full_step(env):
    """Benchmark config 3 shapes (Qwen3-8B layer: bf16 params and grads, fp32 momentum), two layers so that
    every bucket is a grouped launch; the oracle steps every matrix of layer 0 for two steps."""
    print("config 3 layer", flush=True)
    from tests.helpers import QWEN3_8B

    mu, O, dev = env["mu"], env["O"], env["dev"]
    weights, grads = make_param_set(QWEN3_8B, layers=2, seed=1, steps=2, dtype=torch.bfloat16)
    gp = [torch.nn.Parameter(w.clone().to(dev)) for _, w in weights]
    opt = mu.Muon([dict(params=list(gp), use_muon=True, **MUON_HP)], momentum_dtype=torch.float32)
    sample = [i for i, (n, _) in enumerate(weights) if n.startswith("layers.0.")]
    cw = {i: weights[i][1].clone() for i in sample}
    cm = {i: torch.zeros(weights[i][1].shape, dtype=torch.float32) for i in sample}
    torch.set_num_threads(16)
    lr, wd = MUON_HP["lr"], MUON_HP["weight_decay"]
    for step in range(2):
        for p, g in zip(gp, grads[step]):
            p.grad = g.to(dev)
        opt.step()
        torch.cuda.synchronize()
        for i in sample:
            O.muon_step_matrix(cw[i], grads[step][i].clone(), cm[i], lr=lr, weight_decay=wd, beta=MUON_HP["momentum"],
                               nesterov=True, ns_steps=5, rms_scale=False)
            assert rel_fro(opt.state[gp[i]]["momentum_buffer"], cm[i]) <= MOM_TOL, (step, weights[i][0])
            # parameters are bf16: the two sides may round a few elements to neighbouring values
            wp = rel_fro(gp[i], cw[i])
            print(f"  step {step} {weights[i][0]}: param {wp:.3e}", flush=True)
            assert wp <= 4e-3, (step, weights[i][0])


def test_config5_moe_layer_sampled_parity(env):
    """Benchmark config 5 shapes (Qwen3-MoE-30B-A3B: 128 experts x (gate, up 768x2048; down 2048x768) plus
    attention q 4096x2048, k, v 512x2048, o 2048x4096; grads N(0, 1e-3) seed 3, bf16 params, fp32 momentum):
    one full layer, 388 matrices in 5 grouped buckets; the oracle steps a sample out of every bucket."""
    print("config 5 layer", flush=True)
    mu, O, dev = env["mu"], env["O"], env["dev"]
    gen = torch.Generator().manual_seed(3)
    shapes = [("q", (4096, 2048)), ("k", (512, 2048)), ("v", (512, 2048)), ("o", (2048, 4096))]
    for e in range(128):
        shapes += [(f"e{e}.gate", (768, 2048)), (f"e{e}.up", (768, 2048)), (f"e{e}.down", (2048, 768))]
    weights = [(n, (0.02 * torch.randn(*s, generator=gen)).bfloat16()) for n, s in shapes]
    grads = [(1e-3 * torch.randn(*s, generator=gen)).bfloat16() for _, s in shapes]
    gp = [torch.nn.Parameter(w.clone().to(dev)) for _, w in weights]
    for p, g in zip(gp, grads):
        p.grad = g.to(dev)
    opt = mu.Muon([dict(params=list(gp), use_muon=True, **MUON_HP)], momentum_dtype=torch.float32)
    before = [p.detach().clone() for p in gp]
    opt.step()
    torch.cuda.synchronize()
    lr, wd = MUON_HP["lr"], MUON_HP["weight_decay"]
    names = [n for n, _ in weights]
    sample = [names.index(n) for n in ("q", "k", "o", "e0.gate", "e0.down", "e77.up", "e127.gate", "e127.down")]
    for i in sample:
        w, m = weights[i][1].clone(), torch.zeros(weights[i][1].shape, dtype=torch.float32)
        O.muon_step_matrix(w, grads[i].clone(), m, lr=lr, weight_decay=wd, beta=MUON_HP["momentum"], nesterov=True,
                           ns_steps=5, rms_scale=False)
        assert rel_fro(opt.state[gp[i]]["momentum_buffer"], m) <= MOM_TOL, names[i]
        assert rel_fro(gp[i], w) <= 4e-3, names[i]
    # every matrix moved by an update whose size matches an orthogonalised one:
    # ||dp||_F ~ lr * sqrt(min(rows, cols)) * sqrt(max(1, rows / cols)), up to the bf16 rounding of p
    for i, p in enumerate(gp):
        assert torch.isfinite(p).all()
        d = (p.detach().float() - before[i].float() * (1 - lr * wd)).norm().item() / lr
        r = d / (min(p.shape) ** 0.5) / max(1.0, p.shape[0] / p.shape[1]) ** 0.5
        assert 0.5 <= r <= 1.3, (names[i], r)


def test_golden_vectors_on_gpu(env):
    """The committed golden vectors (tests/golden/, written by make_fixtures.py from the oracle)."""
    import os

    import numpy as np

    from tests.golden.make_fixtures import STEP_SPEC
    from tests.helpers import bf16_from_u16

    mu = env["mu"]
    gdir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    data = np.load(os.path.join(gdir, "ns_small.npz"))
    for key in data.files:
        _, shape, seed, steps = key.split("_")
        rows, cols = (int(v) for v in shape.split("x"))
        G = torch.randn(rows, cols, generator=torch.Generator().manual_seed(int(seed[4:])))
        got = mu.fast_newtonschulz(G.to(env["dev"]), int(steps[5:]))
        assert rel_fro(got, bf16_from_u16(data[key])) <= (NS_TOL if steps == "steps5" else 2e-3), key
    data = np.load(os.path.join(gdir, "step_small.npz"))
    weights, grads = make_param_set(STEP_SPEC, layers=1, seed=7, steps=3)
    params = [torch.nn.Parameter(w.clone().to(env["dev"])) for _, w in weights]
    opt = mu.Muon([dict(params=list(params), use_muon=True, **MUON_HP)])
    lr, wd = MUON_HP["lr"], MUON_HP["weight_decay"]
    for step in range(3):
        for p, g in zip(params, grads[step]):
            p.grad = g.to(env["dev"])
        before = [p.detach().clone() for p in opt.param_groups[0]["params"]]
        opt.step()
        for j, p in enumerate(opt.param_groups[0]["params"]):
            o_gpu = (before[j].double().cpu() * (1 - lr * wd) - p.detach().double().cpu()) / lr
            assert rel_fro(o_gpu, bf16_from_u16(data[f"step{step}_update{j}"])) <= NS_TOL
    for j, p in enumerate(opt.param_groups[0]["params"]):
        assert rel_fro(opt.state[p]["momentum_buffer"], torch.from_numpy(data[f"final_momentum{j}"])) <= MOM_TOL
        assert rel_fro(p.detach(), torch.from_numpy(data[f"final_param{j}"])) <= 2e-3
