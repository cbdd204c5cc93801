"""The entry point that allocates nothing (mvit_grad_sumsq_static) against mvit_grad_sumsq, through the C ABI."""

import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _table(grads):
    from mi355_vit import _lib
    from mi355_vit.optim import _NO_SHADOW, _build_table

    rows = [(0, g.data_ptr(), 0, 0, g.numel(), 0, 0.0, 0.0, 0.0, 0.0) + _NO_SHADOW for g in grads]
    table, n_chunks = _build_table(rows)
    return torch.from_numpy(table.view(np.uint8)).to(DEV), len(rows), n_chunks, _lib.load()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_sum_of_squares_equals_the_workspace_entry_point(dtype):
    from mi355_vit import _lib

    print(f"[case] mvit_grad_sumsq_static {dtype}", flush=True)
    g = torch.Generator().manual_seed(3)
    code = _lib.BF16 if dtype == torch.bfloat16 else _lib.F32
    stream = torch.cuda.current_stream().cuda_stream
    # two calls in a row on the shared array, the second with a smaller input (fewer chunks than the first left behind)
    for shapes in ([(8192 * 40 + 17,), (300, 257), (1280,), (64, 3420)], [(5000,), (3,)]):
        grads = [(torch.randn(s, generator=g) * 3.0).to(dtype).to(DEV) for s in shapes]
        table, n, n_chunks, lib = _table(grads)
        partial = torch.empty(n_chunks, dtype=torch.float32, device=DEV)
        ref = torch.zeros(1, dtype=torch.float64, device=DEV)
        out = torch.zeros(1, dtype=torch.float64, device=DEV)
        _lib.check(lib.mvit_grad_sumsq(table.data_ptr(), n, n_chunks, partial.data_ptr(), ref.data_ptr(), code, stream), "mvit_grad_sumsq")
        # the call itself takes no device memory: the driver's free-memory figure is the same before and after it
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        _lib.check(lib.mvit_grad_sumsq_static(table.data_ptr(), n, n_chunks, out.data_ptr(), code, stream), "mvit_grad_sumsq_static")
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert out.item() == ref.item() and out.item() > 0.0
        exact = sum(float(x.double().pow(2).sum()) for x in grads)
        assert abs(out.item() - exact) <= 1e-6 * exact


def test_static_scratch_rejects_sizes_beyond_its_maximum():
    from mi355_vit import _lib

    lib = _lib.load()
    dummy = torch.zeros(16, dtype=torch.float64, device=DEV)
    rc = lib.mvit_grad_sumsq_static(dummy.data_ptr(), 1, _lib.SUMSQ_STATIC_MAX_CHUNKS + 1, dummy.data_ptr(), _lib.F32, torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and b"exceed the built-in scratch" in lib.mvit_last_error()
