"""The entry point that allocates nothing: pdw_dwconv_wgrad_static (partial sums in a static device buffer of the
library) against pdw_dwconv_wgrad with a caller-supplied workspace, through the C ABI: bitwise the same weight
gradient, on two calls in a row, the second with a smaller input."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(shape, k, dtype, seed):
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    B, H, W, C = shape
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=gen).to(dtype).cuda()
    gy = torch.randn(*shape, generator=gen).to(dtype).cuda()
    code = _lib.dtype_code(dtype)
    geo = (B, H, W, C, k, k, 1, 1, k // 2, k // 2, 1, 1)
    need = L.pdw_dwconv_wgrad_workspace_bytes(*geo, code)
    assert 0 < need <= L.pdw_static_scratch_bytes()
    ws = torch.empty(need // 4 + 1, device="cuda", dtype=torch.float32)
    ref = torch.empty(k, k, C, device="cuda", dtype=dtype)
    got = torch.full((k, k, C), float("nan"), device="cuda", dtype=dtype)
    stream = _lib.stream_ptr(x.device)
    _lib.check(L.pdw_dwconv_wgrad(x.data_ptr(), gy.data_ptr(), ref.data_ptr(), ws.data_ptr(), ws.numel() * 4, *geo,
                                  code, stream), "pdw_dwconv_wgrad")
    torch.cuda.synchronize()
    # the device's own free-byte count (hipMemGetInfo): torch's allocator statistics would not see a hipMalloc or
    # hipFree made inside the library
    before, reserved = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    _lib.check(L.pdw_dwconv_wgrad_static(x.data_ptr(), gy.data_ptr(), got.data_ptr(), *geo, code, stream),
               "pdw_dwconv_wgrad_static")
    during = torch.cuda.mem_get_info()[0]
    torch.cuda.synchronize()
    assert torch.cuda.memory_reserved() == reserved
    assert during == before and torch.cuda.mem_get_info()[0] == before
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got, ref), f"{shape} k={k} {dtype}: max diff {(got.float() - ref.float()).abs().max().item()}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_wgrad_two_calls(dtype):
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    assert L.pdw_static_scratch_bytes() == 32 << 20
    _lib.check(L.pdw_static_scratch_init(), "pdw_static_scratch_init")
    _both((8, 56, 56, 64), 13, dtype, 1)    # a large problem first ...
    _both((2, 20, 23, 24), 7, dtype, 2)     # ... then a smaller one on the same buffer: stale partials beyond it
    _both((3, 28, 30, 40), 9, dtype, 3)


def test_static_scratch_rejects_oversize_and_deferral():
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    code = _lib.dtype_code(torch.bfloat16)
    big = (64, 224, 224, 1024, 17, 17, 1, 1, 8, 8, 1, 1)
    assert L.pdw_dwconv_wgrad_workspace_bytes(*big, code) > L.pdw_static_scratch_bytes()
    assert L.pdw_dwconv_wgrad_static(1, 1, 1, *big, code, None) != 0
    assert b"static buffer holds" in L.pdw_last_error()
    small = (2, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1)
    _lib.check(L.pdw_reduce_defer_begin(), "begin")
    try:
        assert L.pdw_dwconv_wgrad_static(1, 1, 1, *small, code, None) != 0
        assert b"pdw_reduce_defer_begin" in L.pdw_last_error()
    finally:
        _lib.check(L.pdw_reduce_defer_flush(None), "flush")
