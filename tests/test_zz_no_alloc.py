"""muon_hip_grad_norms_static, the entry point that allocates nothing, through the C ABI against
muon_hip_grad_norms with a caller-allocated scratch buffer: the per-tensor norms must be identical bit for
bit, on two calls in a row, the second with a smaller input (the built-in array keeps the first call's
contents).  Collected last on purpose."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _norms(lib, abi, table, dtype, dev, static):
    norms = torch.full((table.n,), float("nan"), dtype=torch.float32, device=dev)
    if static:
        abi.check(lib.muon_hip_grad_norms_static(table.role_ptrs[0], table.numel_ptr, table.chunk_start_ptr, table.n,
                                                 table.chunks, abi.dtype_code(dtype), 2.0, norms.data_ptr(), 0), "static")
    else:
        partials = torch.full((table.chunks,), float("nan"), dtype=torch.float32, device=dev)
        abi.check(lib.muon_hip_grad_norms(table.role_ptrs[0], table.numel_ptr, table.chunk_start_ptr, table.n,
                                          table.chunks, abi.dtype_code(dtype), 2.0, partials.data_ptr(), norms.data_ptr(), 0),
                  "caller scratch")
    torch.cuda.synchronize()
    return norms


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_scratch_entry_point_matches_caller_scratch(dtype):
    assert torch.cuda.is_available(), "this test needs the GPU box"
    from lmms_engine_amd import _abi as abi
    from lmms_engine_amd.multi_tensor import TensorListTable

    lib, dev = abi.lib(), torch.device("cuda:0")
    gen = torch.Generator().manual_seed(33)
    big = [(300, 1000), (16384 * 5 + 3,), (7,), (64, 64, 9), (1 << 20,)]
    small = [(1000,), (3, 5), (16385,)]
    for shapes in (big, small):  # second call: fewer tensors, fewer chunks
        print(f"no-alloc grad norms {dtype} {shapes}", flush=True)
        grads = [torch.randn(*s, generator=gen).to(dtype).to(dev) for s in shapes]
        table = TensorListTable([grads])
        a = _norms(lib, abi, table, dtype, dev, static=False)
        b = _norms(lib, abi, table, dtype, dev, static=True)
        assert torch.isfinite(a).all() and torch.equal(a, b), (a, b)
        ref = torch.stack([g.float().norm() for g in grads])
        assert torch.allclose(a, ref, rtol=1e-2 if dtype == torch.bfloat16 else 1e-5)
    # the limit is enforced before anything is launched
    rc = lib.muon_hip_grad_norms_static(table.role_ptrs[0], table.numel_ptr, table.chunk_start_ptr, table.n,
                                        abi.STATIC_MAX_CHUNKS + 1, abi.dtype_code(dtype), 2.0, a.data_ptr(), 0)
    assert rc == -2 and b"built-in scratch" in lib.muon_hip_last_error()
