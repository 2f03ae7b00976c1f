"""The allocation-free column sum (`pf_colsum_accumulate_static`: partial rows in a device array
built into the library) against `pf_colsum_accumulate` with a caller workspace, through the C ABI:
bit-exact, on two calls in a row, the second with a smaller input (the array keeps the first
call's contents)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(lib, x, rows, cols, ld, seed_acc):
    from pfeife_amd.hip import dtype_code

    s = torch.cuda.current_stream().cuda_stream
    n_ws = int(lib.pf_colreduce_workspace(rows, cols))
    ws = torch.empty(n_ws, device="cuda", dtype=torch.float32)
    acc_ref = seed_acc.clone()
    acc_new = seed_acc.clone()
    assert lib.pf_colsum_accumulate(x.data_ptr(), dtype_code(x.dtype), rows, cols, ld, acc_ref.data_ptr(),
                                    ws.data_ptr(), 0, s) == 0, lib.pf_last_error()
    before = torch.cuda.memory_allocated()
    assert lib.pf_colsum_accumulate_static(x.data_ptr(), dtype_code(x.dtype), rows, cols, ld, acc_new.data_ptr(),
                                           s) == 0, lib.pf_last_error()
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return acc_ref, acc_new


def test_static_scratch_column_sum_matches_workspace_version():
    from pfeife_amd import hip

    lib = hip.load()
    assert lib.pf_init(0) == 0, lib.pf_last_error()
    g = torch.Generator().manual_seed(3)
    # first call: the headline's bias-gradient shape (3152 token rows x 4096 columns, fp16)
    x1 = torch.randn(3152, 4096, generator=g).to(torch.float16).cuda()
    a1 = torch.randn(4096, generator=g).cuda()
    ref, new = _both(lib, x1, 3152, 4096, 4096, a1)
    assert torch.equal(ref, new)
    torch.testing.assert_close(new, a1 + x1.float().sum(0), rtol=1e-4, atol=1e-2)
    # second call, smaller and ragged (rows not a multiple of the row chunk, a leading dimension
    # larger than the column count, fp32): stale partials of the first call must not leak in
    x2 = torch.randn(197, 264, generator=g).cuda()
    a2 = torch.zeros(200, device="cuda")
    ref, new = _both(lib, x2, 197, 200, 264, a2)
    assert torch.equal(ref, new)
    torch.testing.assert_close(new, x2[:, :200].sum(0), rtol=1e-5, atol=1e-4)


def test_static_scratch_rejects_oversized_problems():
    from pfeife_amd import hip

    lib = hip.load()
    assert lib.pf_init(0) == 0
    cap = int(lib.pf_colsum_static_capacity())
    rows, cols = 65536, 16384
    assert int(lib.pf_colsum_partials(rows)) * cols > cap
    x = torch.zeros(8, device="cuda")   # never read: the size check comes first
    acc = torch.zeros(8, device="cuda")
    rc = lib.pf_colsum_accumulate_static(x.data_ptr(), 0, rows, cols, cols, acc.data_ptr(), None)
    assert rc == -1
    assert b"exceed the built-in scratch" in lib.pf_last_error()
