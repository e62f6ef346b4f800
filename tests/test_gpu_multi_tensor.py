"""Multi-tensor kernels on the GPU against library oracles on the CPU: the AdamW fallback over a
whole group (oracle: the CPU restatement of the reference's Adam branch) and gradient-norm
clipping (oracle: torch.nn.utils.clip_grad_norm_ itself on CPU copies, the routine the reference
calls, utils/fsdp2_utils.py:234-255).

Tolerances: fp32 results within 1e-6 relative; bf16 results are compared as values, exact
unless stated (the only inexact step is the fp32 sum of squares, whose order differs)."""
import pytest
import torch

from tests.helpers import rel_fro

pytestmark = pytest.mark.gpu

SIZES = [(1,), (7,), (8,), (1000,), (16384,), (16385,), (50000,), (300, 64), (0,), (3, 5, 7)]


@pytest.fixture(scope="module")
def env():
    assert torch.cuda.is_available(), "these tests need the GPU box"
    from lmms_engine_amd import _abi, clip_grad, muon_utils
    from oracle import muon_oracle

    _abi.lib()
    return dict(abi=_abi, mu=muon_utils, clip=clip_grad, O=muon_oracle, dev=torch.device("cuda:0"))


def _misaligned(shape, dtype, dev, gen):
    """A contiguous tensor whose base pointer is not 16-byte aligned (a view one element into a buffer)."""
    n = 1
    for s in shape:
        n *= s
    buf = torch.zeros(n + 1, dtype=dtype, device=dev)
    v = buf[1:].view(*shape)
    v.copy_(torch.randn(*shape, generator=gen).to(dtype))
    assert v.data_ptr() % 16 != 0 and v.is_contiguous()
    return v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_adamw_group_ragged_sizes_and_steps(env, dtype):
    """1-D, tiny, chunk-boundary, empty, 3-D and misaligned tensors in one group; the second step runs with
    different per-tensor step counts (a parameter that joined later)."""
    print("adamw group", dtype, flush=True)
    mu, O, dev = env["mu"], env["O"], env["dev"]
    gen = torch.Generator().manual_seed(21)
    ps = [torch.nn.Parameter((0.02 * torch.randn(*s, generator=gen)).to(dtype).to(dev)) for s in SIZES]
    ps.append(torch.nn.Parameter(_misaligned((1001,), dtype, dev, gen)))
    hp = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    opt = mu.Muon([dict(params=list(ps), use_muon=False, **hp)])
    cp = [p.detach().cpu().clone() for p in ps]
    ce1 = [torch.zeros_like(c) for c in cp]
    ce2 = [torch.zeros_like(c) for c in cp]
    steps = [0] * len(ps)
    for it in range(3):
        grads = [(1e-2 * torch.randn(*p.shape, generator=gen)).to(dtype) for p in ps]
        for p, g in zip(ps, grads):
            p.grad = g.to(dev)
        if it == 1:  # desynchronise the step counters
            opt.state[ps[3]]["step"] += 5
            steps[3] += 5
        opt.step()
        torch.cuda.synchronize()
        for i in range(len(ps)):
            steps[i] += 1
            if cp[i].numel():
                O.adamw_step_tensor(cp[i], grads[i].clone(), ce1[i], ce2[i], steps[i], hp["lr"], hp["betas"], hp["eps"],
                                    hp["weight_decay"])
            st = opt.state[ps[i]]
            assert st["step"] == steps[i]
            if dtype == torch.float32:
                assert rel_fro(st["exp_avg"], ce1[i]) <= 1e-6 and rel_fro(st["exp_avg_sq"], ce2[i]) <= 1e-6
                assert rel_fro(ps[i], cp[i]) <= 1e-6
            else:
                assert torch.equal(st["exp_avg"].cpu(), ce1[i]) and torch.equal(st["exp_avg_sq"].cpu(), ce2[i]), (it, i)
                assert torch.equal(ps[i].detach().cpu(), cp[i]), (it, i)


def _clip_case(env, dtypes, scale, max_norm, seed=5, sizes=SIZES, misaligned=True):
    dev = env["dev"]
    gen = torch.Generator().manual_seed(seed)
    ps = []
    for i, s in enumerate(sizes):
        dt = dtypes[i % len(dtypes)]
        p = torch.nn.Parameter(torch.zeros(*s, dtype=dt, device=dev))
        p.grad = (scale * torch.randn(*s, generator=gen)).to(dt).to(dev)
        ps.append(p)
    if misaligned:
        p = torch.nn.Parameter(torch.zeros(1001, dtype=dtypes[0], device=dev))
        p.grad = _misaligned((1001,), dtypes[0], dev, gen)
        ps.append(p)
    ps.append(torch.nn.Parameter(torch.zeros(4, dtype=dtypes[0], device=dev)))  # no grad: skipped
    cpu = [torch.nn.Parameter(torch.zeros(p.shape, dtype=p.dtype)) for p in ps]
    for c, p in zip(cpu, ps):
        c.grad = None if p.grad is None else p.grad.detach().cpu().clone()
    before = [None if p.grad is None else p.grad.detach().clone() for p in ps]
    got = env["clip"].clip_grad_norm_(ps, max_norm)
    torch.cuda.synchronize()
    ref = torch.nn.utils.clip_grad_norm_(cpu, max_norm, foreach=False)
    return ps, cpu, before, got, ref


@pytest.mark.parametrize("dtypes", [(torch.float32,), (torch.bfloat16,), (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("scale,max_norm", [(1.0, 1.0), (1e-4, 1.0), (3.0, 0.5)])
def test_clip_grad_norm_matches_torch(env, dtypes, scale, max_norm):
    print("clip", dtypes, scale, max_norm, flush=True)
    ps, cpu, before, got, ref = _clip_case(env, dtypes, scale, max_norm)
    assert got.dtype == ref.dtype and got.device.type == "cuda" and got.ndim == 0
    if got.dtype == torch.float32:
        assert abs(got.item() - ref.item()) <= 1e-6 * ref.item()
    else:
        assert got.item() == ref.item()
    for p, c, b in zip(ps, cpu, before):
        if p.grad is None:
            assert c.grad is None
            continue
        if p.grad.numel() == 0:
            continue
        if p.grad.dtype == torch.float32:
            assert rel_fro(p.grad, c.grad) <= 1e-6
        else:
            assert torch.equal(p.grad.cpu(), c.grad)
        if ref.item() + 1e-6 <= max_norm and got.dtype == torch.float32:
            assert torch.equal(p.grad, b)  # coefficient clamps to exactly 1: untouched bits


def test_clip_grad_norm_edge_cases(env):
    clip, dev = env["clip"], env["dev"]
    assert clip.clip_grad_norm_([], 1.0).item() == 0.0
    p = torch.nn.Parameter(torch.zeros(10, device=dev))
    assert clip.clip_grad_norm_(p, 1.0).item() == 0.0  # no grads at all
    p.grad = torch.full((10,), float("inf"), device=dev)
    with pytest.raises(RuntimeError, match="non-finite"):
        clip.clip_grad_norm_([p], 1.0, error_if_nonfinite=True)
    out = clip.clip_grad_norm_([p], 1.0)  # scales by the non-finite norm, as torch does
    assert torch.isinf(out) and torch.isnan(p.grad).all()
    with pytest.raises(ValueError):
        clip.clip_grad_norm_([p], 1.0, norm_type=float("nan"))
    p.grad = torch.tensor([1.0, float("nan"), 3.0] + [0.0] * 7, device=dev)
    assert torch.isnan(clip.clip_grad_norm_([p], 1.0, norm_type=float("inf")))  # a NaN is the largest, as in torch.max
    q = torch.nn.Parameter(torch.zeros(4))
    q.grad = torch.ones(4)
    with pytest.raises(env["abi"].MuonHipError):
        clip.clip_grad_norm_([q], 1.0)  # CPU gradients: no fallback
    assert clip.fsdp2_clip_grad_norm_ is clip.clip_grad_norm_


@pytest.mark.parametrize("dtypes", [(torch.float32,), (torch.bfloat16,), (torch.float32, torch.bfloat16)])
def test_clip_grad_norm_infinity_norm_and_strided_gradients(env, dtypes):
    """norm_type=inf (fsdp2_clip_grad_norm_ forwards any norm_type to torch, utils/fsdp2_utils.py:244-254): the largest
    magnitude over all gradients, exact in any order, so the total and the scaled gradients must equal torch's on the
    CPU (fp32 gradients to 1e-6: the coefficient's reciprocal).  Gradients that are transposed or sliced views step
    through a row-major copy and are written back in place."""
    clip, dev = env["clip"], env["dev"]
    gen = torch.Generator().manual_seed(41)
    shapes = [(300, 70), (16384 * 2 + 5,), (9,), (64, 33)]
    ps, cpu = [], []
    for i, s in enumerate(shapes):
        dt = dtypes[i % len(dtypes)]
        g = (2.5 * torch.randn(*s, generator=gen)).to(dt)
        if i == 0:   # a transposed view: dense, not row-major
            gd, gc = g.to(dev).t().contiguous().t(), g.clone()
        elif i == 3:  # a column slice: strided with gaps
            wide_d, wide_c = torch.zeros(64, 66, dtype=dt, device=dev), torch.zeros(64, 66, dtype=dt)
            gd, gc = wide_d[:, ::2], wide_c[:, ::2]
            gd.copy_(g.to(dev))
            gc.copy_(g)
        else:
            gd, gc = g.to(dev), g.clone()
        assert (i in (0, 3)) == (not gd.is_contiguous())
        p, c = torch.nn.Parameter(torch.zeros(*s, dtype=dt, device=dev)), torch.nn.Parameter(torch.zeros(*s, dtype=dt))
        p.grad, c.grad = gd, gc
        ps.append(p)
        cpu.append(c)
    for it, (norm_type, max_norm) in enumerate(((float("inf"), 1.0), (2.0, 0.5), (float("inf"), 100.0))):
        got = clip.clip_grad_norm_(ps, max_norm, norm_type=norm_type)
        ref = torch.nn.utils.clip_grad_norm_(cpu, max_norm, norm_type=norm_type, foreach=False)
        torch.cuda.synchronize()
        assert got.dtype == ref.dtype
        # exact while both sides hold the same gradients: always in bf16, in fp32 until the first scaling
        if got.dtype == torch.bfloat16 or it == 0:
            assert got.item() == ref.item(), (norm_type, got.item(), ref.item())
        else:
            assert abs(got.item() - ref.item()) <= 1e-6 * ref.item()
        for i, (p, c) in enumerate(zip(ps, cpu)):
            assert (i in (0, 3)) == (not p.grad.is_contiguous())  # scaled in place: the views are still views
            if p.grad.dtype == torch.float32:
                assert rel_fro(p.grad, c.grad) <= 1e-6
            else:
                assert torch.equal(p.grad.cpu(), c.grad)


@pytest.mark.parametrize("dtypes", [(torch.float32,), (torch.bfloat16,), (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("norm_type", [1.0, 0.0, float("-inf"), 3.0, 0.5, 1.5])
def test_clip_grad_norm_other_orders(env, dtypes, norm_type):
    """Every other order fsdp2_clip_grad_norm_ can forward (utils/fsdp2_utils.py:244-254): the reductions of
    torch.linalg.vector_norm by order (sum of magnitudes, count of non-zeros, smallest magnitude, (sum |x|^p)^(1/p)),
    per tensor in fp32 rounded to the tensor's dtype, then over the per-tensor norms.  Against torch on the CPU: the
    count and the smallest magnitude exactly; the sums to 1e-5 in fp32 (another order of additions, another power
    routine) and to one bf16 step where the result is rounded to bf16."""
    print("clip order", norm_type, dtypes, flush=True)
    clip, dev = env["clip"], env["dev"]
    gen = torch.Generator().manual_seed(43)
    shapes = [(300, 70), (16384 * 2 + 5,), (9,), (64, 33), (3, 16384)]
    ps, cpu = [], []
    for i, s in enumerate(shapes):
        dt = dtypes[i % len(dtypes)]
        g = (0.5 * torch.randn(*s, generator=gen)).to(dt)
        g.view(-1)[::7] = 0  # zeros for the count; the smallest magnitude is then 0 for the larger tensors
        if i == 2:
            g = g.abs() + 0.25  # one tensor without zeros
        p, c = torch.nn.Parameter(torch.zeros(*s, dtype=dt, device=dev)), torch.nn.Parameter(torch.zeros(*s, dtype=dt))
        p.grad, c.grad = g.to(dev), g.clone()
        ps.append(p)
        cpu.append(c)
    for max_norm in (0.75, 1e9):
        got = clip.clip_grad_norm_(ps, max_norm, norm_type=norm_type)
        ref = torch.nn.utils.clip_grad_norm_(cpu, max_norm, norm_type=norm_type, foreach=False)
        torch.cuda.synchronize()
        assert got.dtype == ref.dtype
        if norm_type in (0.0, float("-inf")):
            assert got.item() == ref.item(), (norm_type, got.item(), ref.item())
        else:
            tol = 2.0 ** -7 if got.dtype == torch.bfloat16 else 1e-5
            assert abs(got.item() - ref.item()) <= tol * abs(ref.item()), (norm_type, got.item(), ref.item())
        for p, c in zip(ps, cpu):
            tol = 2.0 ** -6 if torch.bfloat16 in dtypes else 2e-5   # the coefficient is rounded to the norm's dtype
            assert rel_fro(p.grad, c.grad) <= tol, (norm_type, rel_fro(p.grad, c.grad))
            c.grad.copy_(p.grad.cpu())  # both sides go on from the same gradients


def test_clip_grad_norm_full_size(env):
    """A Qwen3-8B layer's worth of bf16 gradients (218 M elements): the total against torch on the CPU, and the
    size-independent property that clipping to c leaves a norm of c (to bf16 accuracy)."""
    print("clip full size", flush=True)
    from tests.helpers import NAMES, QWEN3_8B

    clip, dev = env["clip"], env["dev"]
    gen = torch.Generator(device=dev).manual_seed(9)
    ps = []
    for n in NAMES:
        p = torch.nn.Parameter(torch.empty(*QWEN3_8B[n], dtype=torch.bfloat16, device=dev))
        p.grad = (1e-3 * torch.randn(*QWEN3_8B[n], device=dev, generator=gen)).bfloat16()
        ps.append(p)
    cpu_grads = [p.grad.cpu() for p in ps]
    ref = torch.nn.utils.clip_grad.get_total_norm(cpu_grads) if hasattr(torch.nn.utils.clip_grad, "get_total_norm") \
        else torch.nn.utils.clip_grad._get_total_norm(cpu_grads)
    got = clip.clip_grad_norm_(ps, 1.0)
    assert abs(got.item() - ref.item()) <= 2.0 ** -7 * ref.item()  # one bf16 step
    after = clip.clip_grad_norm_(ps, 1e9)
    assert abs(after.item() - 1.0) <= 2e-2
