"""The entry point that allocates nothing, `kr_rmsnorm_bwd_add_noalloc`, called through the C ABI:
its results must equal `kr_rmsnorm_bwd_add`'s bit for bit (same kernels, the partial rows of the
weight gradient in the library's own device array instead of a caller workspace), on two calls in
a row of which the second is smaller (the array keeps the first call's contents)."""

import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a HIP device")]
DEV = "cuda"


def _free_device_bytes():
    """Free device memory as the HIP runtime itself counts it (hipMemGetInfo): unlike torch's own
    counters this also moves when a library calls hipMalloc / hipFree behind torch's back."""
    torch.cuda.synchronize()
    return torch.cuda.mem_get_info()[0]


def _case(lib, rows, cols, with_residual, seed, symbol_known=True):
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    x = torch.randn(rows, cols, generator=g).to(DEV, bf)
    dy = torch.randn(rows, cols, generator=g).to(DEV, bf)
    res = torch.randn(rows, cols, generator=g).to(DEV, bf) if with_residual else None
    gamma = (1 + 0.1 * torch.randn(cols, generator=g)).to(DEV, bf)
    rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    stream = torch.cuda.current_stream().cuda_stream
    res_ptr = res.data_ptr() if res is not None else None
    res_ld = cols if res is not None else 0

    dx_a, dg_a = torch.empty_like(x), torch.empty_like(gamma)
    ws = torch.empty(lib.kr_rmsnorm_bwd_workspace_bytes(rows, cols), dtype=torch.uint8, device=DEV)
    rc = lib.kr_rmsnorm_bwd_add(dy.data_ptr(), x.data_ptr(), rstd.data_ptr(), gamma.data_ptr(), res_ptr,
                                dx_a.data_ptr(), dg_a.data_ptr(), ws.data_ptr(), rows, cols, cols, cols,
                                res_ld, cols, stream)
    assert rc == 0
    dx_b, dg_b = torch.empty_like(x), torch.empty_like(gamma)
    before, before_torch = _free_device_bytes(), torch.cuda.memory_allocated()
    rc = lib.kr_rmsnorm_bwd_add_noalloc(dy.data_ptr(), x.data_ptr(), rstd.data_ptr(), gamma.data_ptr(), res_ptr,
                                        dx_b.data_ptr(), dg_b.data_ptr(), rows, cols, cols, cols,
                                        res_ld, cols, stream)
    assert rc == 0
    after = _free_device_bytes()
    assert torch.cuda.memory_allocated() == before_torch
    if symbol_known:     # the first call on a device looks the array's address up, which may load the code object
        assert after == before, f"free device memory moved by {before - after} bytes across the call"
    assert torch.equal(dx_a, dx_b) and torch.equal(dg_a, dg_b)
    return dg_b


def test_noalloc_rmsnorm_backward_equals_the_workspace_entry_point():
    from kareus_amd.backend.hip import load_library

    lib = load_library()
    print("case rows=4096 cols=4096 residual", flush=True)
    big = _case(lib, 4096, 4096, True, seed=1, symbol_known=False)      # 512 partial rows of 4096 columns
    print("case rows=70 cols=1376 plain", flush=True)
    small = _case(lib, 70, 1376, False, seed=2)     # smaller: 18 partial rows; the rest keeps the old contents
    print("case rows=300 cols=8192 residual", flush=True)
    _case(lib, 300, 8192, True, seed=3)             # the widest row the device array holds
    assert torch.isfinite(big.float()).all() and torch.isfinite(small.float()).all()
    # wider rows than the device array holds are refused, nothing is launched
    rc = lib.kr_rmsnorm_bwd_add_noalloc(16, 16, 16, 16, None, 16, 16, 4, 8200, 8200, 8200, 0, 8200, None)
    assert rc == -2
    # no place for the weight gradient: refused (the partial rows live where the caller cannot read them)
    t = torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV)
    r = torch.ones(8, dtype=torch.float32, device=DEV)
    rc = lib.kr_rmsnorm_bwd_add_noalloc(t.data_ptr(), t.data_ptr(), r.data_ptr(), t.data_ptr(), None, t.data_ptr(),
                                        None, 8, 64, 64, 64, 0, 64, None)
    assert rc == -1
