"""``dmf_colsum_static``: the entry point that allocates nothing (its partial sums
live in a device array inside the library).  Called through the C ABI and
compared with ``dmf_colsum`` -- same kernels, so the same bits -- on two calls in
a row, the second on a smaller input (the array keeps the first call's contents),
plus the size limit."""
import ctypes

import pytest
import torch

from dmf_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_FLOATS = 1 << 20   # DMF_COLSUM_STATIC_MAX_FLOATS (include/dmf_block.h)


def _both(lib, x, out_dtype):
    rows, C = x.shape
    code = {torch.float32: _lib.DMF_ATTN_F32, torch.bfloat16: _lib.DMF_ATTN_BF16}
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(int(lib.dmf_block_workspace_floats(3, 1, rows, C)), dtype=torch.float32, device=DEV)
    ref = torch.empty(C, dtype=out_dtype, device=DEV)
    got = torch.full((C,), float("nan"), dtype=out_dtype, device=DEV)
    assert lib.dmf_colsum(x.data_ptr(), ref.data_ptr(), ws.data_ptr(), rows, C, code[x.dtype], code[out_dtype], stream) == 0
    assert lib.dmf_colsum_static(x.data_ptr(), got.data_ptr(), rows, C, code[x.dtype], code[out_dtype], stream) == 0
    torch.cuda.synchronize()
    return got, ref


def test_colsum_static_matches_colsum_on_two_calls_in_a_row(lib):
    g = torch.Generator().manual_seed(11)
    # a Linear bias gradient at the DMFT-XL/2 shape (8192 tokens x 4608 features), then a smaller, ragged one
    for rows, C, dtype, out_dtype in ((8192, 4608, torch.bfloat16, torch.float32), (777, 1152, torch.bfloat16, torch.bfloat16),
                                      (130, 72, torch.float32, torch.float32)):
        print(f"case rows{rows} C{C} {dtype} -> {out_dtype}", flush=True)
        x = torch.randn(rows, C, generator=g).to(dtype).to(DEV)
        got, ref = _both(lib, x, out_dtype)
        assert torch.equal(got, ref)
        exact = x.double().sum(0)
        assert float((got.double() - exact).norm() / exact.norm()) <= (1e-6 if out_dtype == torch.float32 else 4e-3)


def test_colsum_static_refuses_what_does_not_fit(lib):
    rows, C = 64 * (MAX_FLOATS // 4608 + 1), 4608          # one chunk of rows too many
    x = torch.zeros(8, device=DEV)                          # never read: the call is refused before any launch
    out = torch.full((C,), 7.0, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.dmf_colsum_static(x.data_ptr(), out.data_ptr(), rows, C, _lib.DMF_ATTN_F32, _lib.DMF_ATTN_F32, stream)
    assert rc == -9 and b"scratch" in lib.dmf_attn_strerror(rc)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
    # the largest problem that fits is accepted
    rows = 64 * (MAX_FLOATS // 4608)
    x = torch.ones(rows, C, device=DEV, dtype=torch.bfloat16)
    out = torch.empty(C, device=DEV)
    assert lib.dmf_colsum_static(x.data_ptr(), out.data_ptr(), rows, C, _lib.DMF_ATTN_BF16, _lib.DMF_ATTN_F32, stream) == 0
    torch.cuda.synchronize()
    assert bool((out == rows).all())
