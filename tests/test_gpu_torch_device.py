"""The elementwise stages of the HIP path against torch itself ON THE DEVICE, bit for bit.  GPU box only.

The reference's momentum, normalisation, scaling, update and Adam lines are plain torch expressions
(/root/reference/src/lmms_engine/utils/muon_utils.py:146, :160-161, :170-174, :179-183, :188-189, :324-325,
:406-407); run on GPU tensors by torch-ROCm they are a library oracle for the arithmetic the reference performs
where it actually runs: GPU ATen keeps `alpha` of add_ in fp32, contracts lerp into one fma, divides tensor by
tensor with a correctly rounded fp32 division and turns tensor / python-scalar into a multiplication by the
scalar's fp32 reciprocal.  Every test here requires torch.equal, for (bf16, bf16) and (fp32, fp32) tensors.

The GEMM chain is compared with the same expressions on the device too (torch's bf16 matmul in place of the
Triton kernel), to the 2e-2 relative Frobenius bound, in tests/test_gpu_parity.py.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def env():
    assert torch.cuda.is_available(), "these tests need the GPU box"
    from lmms_engine_amd import _abi, muon_utils

    _abi.lib()
    return dict(abi=_abi, mu=muon_utils, lib=_abi.lib(), dev=torch.device("cuda:0"))


def _mismatch(a, b):
    ne = a != b
    return f"{int(ne.sum())} of {a.numel()} elements differ, first at {ne.flatten().nonzero()[:3].flatten().tolist()}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nesterov", [True, False])
@pytest.mark.parametrize("beta", [0.95, 0.9, 0.3])
@pytest.mark.parametrize("shape", [(512, 1024), (37, 53)])
def test_momentum_pair_is_torch_lerp_on_device(env, dtype, nesterov, beta, shape):
    """muon_update's two lerp_ calls (muon_utils.py:188-189); beta = 0.3 takes the other branch of ATen's formula
    in both calls."""
    print(f"momentum {dtype} nesterov={nesterov} beta={beta} {shape}", flush=True)
    mu, dev = env["mu"], env["dev"]
    gen = torch.Generator().manual_seed(41)
    g = (1e-3 * torch.randn(*shape, generator=gen)).to(dtype).to(dev)
    m = (1e-3 * torch.randn(*shape, generator=gen)).to(dtype).to(dev)
    g_ref, m_ref = g.clone(), m.clone()
    m_ref.lerp_(g_ref, 1 - beta)
    u_ref = g_ref.lerp_(m_ref, beta) if nesterov else m_ref
    u = mu.apply_momentum(g, m, beta, nesterov)  # writes the blend back into g, as the reference does
    torch.cuda.synchronize()
    assert torch.equal(m, m_ref), _mismatch(m, m_ref)
    assert torch.equal(u, u_ref), _mismatch(u, u_ref)
    assert torch.equal(g, g_ref), "the gradient holds the blend (nesterov) or is untouched"


def _exact_norm_matrix(rows, cols, gen):
    """Entries from {+-0.5, +-1, +-2}: every partial sum of squares is exact in fp32 whatever the order, so the
    device and torch agree on the norm and the test isolates the division."""
    mag = torch.tensor([0.5, 1.0, 2.0])[torch.randint(0, 3, (rows, cols), generator=gen)]
    sign = torch.randint(0, 2, (rows, cols), generator=gen).float() * 2 - 1
    return mag * sign


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,cols,batch", [(96, 200, 1), (200, 96, 2), (512, 1024, 2), (33, 47, 1)])
def test_normalize_is_the_torch_expression_on_device(env, dtype, rows, cols, batch):
    """X = G.bfloat16(); X / (X.norm(dim=(-2, -1), keepdim=True) + 1e-7) (muon_utils.py:138, :146)."""
    print(f"normalize {dtype} {rows}x{cols} batch={batch}", flush=True)
    lib, abi, dev = env["lib"], env["abi"], env["dev"]
    gen = torch.Generator().manual_seed(rows + cols)
    G = torch.stack([_exact_norm_matrix(rows, cols, gen) for _ in range(batch)]).to(dtype).to(dev)
    X = G.bfloat16()
    ref = X / (X.norm(dim=(-2, -1), keepdim=True) + 1e-7)
    ws = torch.empty(abi.workspace_bytes(rows, cols, batch), dtype=torch.uint8, device=dev)
    out = torch.full((batch, rows, cols), float("nan"), dtype=torch.bfloat16, device=dev)
    abi.check(lib.muon_hip_cast_norm(G.data_ptr(), abi.dtype_code(dtype), ws.data_ptr(), rows, cols, batch, 0))
    abi.check(lib.muon_hip_normalize(ws.data_ptr(), rows, cols, batch, 0))
    abi.check(lib.muon_hip_ns_output(ws.data_ptr(), rows, cols, batch, 0, out.data_ptr(), 0))
    torch.cuda.synchronize()
    assert torch.equal(out, ref), _mismatch(out, ref)


@pytest.mark.parametrize("pdtype", DTYPES)
@pytest.mark.parametrize("rows,cols", [(256, 384), (384, 256), (37, 53), (300, 100)])
@pytest.mark.parametrize("rms_scale", [False, True])
def test_apply_update_is_the_torch_expressions_on_device(env, pdtype, rows, cols, rms_scale):
    """apply_scaling (muon_utils.py:167-175) and param.mul_ / param.add_(update, alpha=-lr) (:324-325) on a bf16
    update; rows > cols goes through the transposing kernel."""
    print(f"apply_update {pdtype} {rows}x{cols} rms={rms_scale}", flush=True)
    lib, abi, mu, dev = env["lib"], env["abi"], env["mu"], env["dev"]
    gen = torch.Generator().manual_seed(rows * 7 + cols)
    G = torch.randn(rows, cols, generator=gen).to(dev)
    p = (0.02 * torch.randn(rows, cols, generator=gen)).to(pdtype).to(dev)
    lr, wd = 0.02, 0.01
    ws = torch.empty(abi.workspace_bytes(rows, cols, 1), dtype=torch.uint8, device=dev)
    O = torch.empty(rows, cols, dtype=torch.bfloat16, device=dev)
    abi.check(lib.muon_hip_cast_norm(G.data_ptr(), abi.F32, ws.data_ptr(), rows, cols, 1, 0))
    abi.check(lib.muon_hip_normalize(ws.data_ptr(), rows, cols, 1, 0))
    abi.check(lib.muon_hip_ns_output(ws.data_ptr(), rows, cols, 1, 0, O.data_ptr(), 0))  # what the update kernel reads
    # the reference's lines, on the device
    p_ref = p.clone()
    update = O.clone()
    if rms_scale:
        update *= 0.2 * (max(update.shape[1], update.shape[0])) ** 0.5
    else:
        update *= max(1, update.size(-2) / update.size(-1)) ** 0.5
    p_ref.mul_(1 - lr * wd)
    p_ref.add_(update.reshape(p_ref.shape), alpha=-lr)
    table = torch.tensor([p.data_ptr()], dtype=torch.int64, device=dev)
    abi.check(lib.muon_hip_apply_update(table.data_ptr(), abi.dtype_code(pdtype), ws.data_ptr(), rows, cols, 1, 0,
                                        mu.scale_factor(rows, cols, rms_scale), lr, wd, 0))
    torch.cuda.synchronize()
    assert torch.equal(p, p_ref), _mismatch(p, p_ref)
    # the stand-alone helper is the same multiplication
    scaled = mu.apply_scaling(O.clone(), rms_scale)
    assert torch.equal(scaled, update), _mismatch(scaled, update)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1000, 16384 * 3 + 5])
def test_adam_update_is_the_torch_expressions_on_device(env, dtype, n):
    """adam_update (muon_utils.py:178-183) over several steps, then the whole Adam branch (:468-477) through the
    multi-tensor kernel and through the single-tensor entry point."""
    print(f"adam {dtype} n={n}", flush=True)
    mu, lib, abi, dev = env["mu"], env["lib"], env["abi"], env["dev"]
    gen = torch.Generator().manual_seed(n)
    betas, eps, lr, wd = (0.9, 0.95), 1e-8, 1e-3, 0.1
    e1, e2 = torch.zeros(n, dtype=dtype, device=dev), torch.zeros(n, dtype=dtype, device=dev)
    r1, r2 = e1.clone(), e2.clone()
    for step in range(1, 5):
        g = (1e-2 * torch.randn(n, generator=gen)).to(dtype).to(dev)
        # reference text
        r1.lerp_(g, 1 - betas[0])
        r2.lerp_(g.square(), 1 - betas[1])
        buf1c = r1 / (1 - betas[0] ** step)
        buf2c = r2 / (1 - betas[1] ** step)
        ref = buf1c / (buf2c.sqrt() + eps)
        got = mu.adam_update(g, e1, e2, step, betas, eps)
        torch.cuda.synchronize()
        assert torch.equal(e1, r1) and torch.equal(e2, r2), (step, _mismatch(e1, r1), _mismatch(e2, r2))
        assert torch.equal(got, ref), (step, _mismatch(got, ref))
    # the optimizer's Adam branch: multi-tensor kernel
    w = (0.02 * torch.randn(n, generator=gen)).to(dtype).to(dev)
    p = torch.nn.Parameter(w.clone())
    q = w.clone()
    opt = mu.Muon([dict(params=[p], use_muon=False, lr=lr, betas=betas, eps=eps, weight_decay=wd)])
    s1, s2 = torch.zeros_like(q), torch.zeros_like(q)
    p1, t1, t2 = w.clone(), torch.zeros_like(q), torch.zeros_like(q)
    for step in range(1, 4):
        g = (1e-2 * torch.randn(n, generator=gen)).to(dtype).to(dev)
        p.grad = g.clone()
        opt.step()
        s1.lerp_(g, 1 - betas[0])
        s2.lerp_(g.square(), 1 - betas[1])
        update = (s1 / (1 - betas[0] ** step)) / ((s2 / (1 - betas[1] ** step)).sqrt() + eps)
        q.mul_(1 - lr * wd)
        q.add_(update, alpha=-lr)
        abi.check(lib.muon_hip_adamw(p1.data_ptr(), g.data_ptr(), t1.data_ptr(), t2.data_ptr(), abi.dtype_code(dtype), n,
                                     step, lr, betas[0], betas[1], eps, wd, 0))
        torch.cuda.synchronize()
        assert torch.equal(p.detach(), q), (step, _mismatch(p.detach(), q))
        assert torch.equal(p1, q), (step, _mismatch(p1, q))
        assert torch.equal(opt.state[p]["exp_avg"], s1) and torch.equal(opt.state[p]["exp_avg_sq"], s2)


def test_decay_update_of_an_fp32_parameter_by_a_bf16_update(env):
    """muon_utils.py:324-325 with the types of the fp32 configurations: fp32 parameter, bf16 update."""
    lib, abi, dev = env["lib"], env["abi"], env["dev"]
    gen = torch.Generator().manual_seed(19)
    for n in (1000, 8 * 4096 + 3):
        p = (0.02 * torch.randn(n, generator=gen)).to(dev)
        u = torch.randn(n, generator=gen).bfloat16().to(dev)
        ref = p.clone()
        ref.mul_(1 - 0.02 * 0.01)
        ref.add_(u, alpha=-0.02)
        abi.check(lib.muon_hip_decay_update(p.data_ptr(), abi.F32, u.data_ptr(), abi.BF16, n, 0.02, 0.01, 0))
        torch.cuda.synchronize()
        assert torch.equal(p, ref), _mismatch(p, ref)


@pytest.mark.parametrize("pdtype,udtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16)])
def test_step_deepspeed_is_the_torch_expressions_on_device(env, pdtype, udtype):
    """The Muon branch of step_deepspeed (muon_utils.py:405-407): decay and update with p.grad as the update; the
    Adam group of the same optimizer runs the Adam branch."""
    mu, dev = env["mu"], env["dev"]
    gen = torch.Generator().manual_seed(9)
    w = (0.02 * torch.randn(96, 160, generator=gen)).to(pdtype).to(dev)
    u = torch.randn(96, 160, generator=gen).to(udtype).to(dev)
    e = torch.randn(50, generator=gen).to(dev)
    p, q = torch.nn.Parameter(w.clone()), torch.nn.Parameter(e.clone())
    p.grad, q.grad = u.clone(), torch.ones_like(e)
    opt = mu.Muon([dict(params=[p], use_muon=True, lr=0.02, weight_decay=0.01), dict(params=[q], use_muon=False)],
                  is_deepspeed_enabled=True)
    opt.step()
    torch.cuda.synchronize()
    ref = w.clone()
    ref.mul_(1 - 0.02 * 0.01)
    ref.add_(u.reshape(ref.shape), alpha=-0.02)
    assert torch.equal(p.detach(), ref), _mismatch(p.detach(), ref)
    assert opt.state[q]["step"] == 1 and not torch.equal(q.detach(), e)


@pytest.mark.parametrize("dtype", DTYPES)
def test_functional_helpers_take_strided_tensors(env, dtype):
    """The reference's helpers are torch expressions and take tensors of any strides (muon_utils.py:159-183); here
    such tensors go through row-major copies that are written back, so the views still hold the results."""
    print(f"strided helpers {dtype}", flush=True)
    mu, dev = env["mu"], env["dev"]
    gen = torch.Generator().manual_seed(5)
    rows, cols, beta = 96, 160, 0.95

    def pair(scale):
        dense = (scale * torch.randn(rows, cols, generator=gen)).to(dtype).to(dev)
        wide = torch.zeros(rows, 2 * cols, dtype=dtype, device=dev)
        view = wide[:, ::2]          # strided with gaps
        view.copy_(dense)
        return dense, view

    g, gv = pair(1e-3)
    m, mt = pair(1e-3)
    mv = mt.t().contiguous().t()     # dense, column-major
    assert not gv.is_contiguous() and not mv.is_contiguous()
    u = mu.apply_momentum(g, m, beta, True)
    uv = mu.apply_momentum(gv, mv, beta, True)
    torch.cuda.synchronize()
    assert uv is gv and torch.equal(uv, u) and torch.equal(mv, m)
    s, sv = pair(1.0)
    assert mu.apply_scaling(sv, True) is sv
    assert torch.equal(sv, mu.apply_scaling(s, True))
    gr, grv = pair(1e-2)
    e1, e1v = pair(1e-3)
    e2, e2v = pair(1e-3)
    e2.abs_()
    e2v.abs_()
    out = mu.adam_update(gr, e1, e2, 3, (0.9, 0.95), 1e-8)
    outv = mu.adam_update(grv, e1v, e2v, 3, (0.9, 0.95), 1e-8)
    torch.cuda.synchronize()
    assert torch.equal(outv, out) and torch.equal(e1v, e1) and torch.equal(e2v, e2)
    with pytest.raises(ValueError):
        mu.adam_update(gr, e1[:4], e2, 3, (0.9, 0.95), 1e-8)
