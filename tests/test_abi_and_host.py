"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares,
and the host-side mirror keeps the reference's module structure, names and init."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from pyramidconvblock_amd import _lib

    header = open(os.path.join(ROOT, "include", "pdw.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(pdw_\w+)\s*\(", header))
    assert len(declared) >= 13
    L = _lib.lib()  # loads libpdw.so (built in-tree); no compute call is made here
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(raw, name), f"libpdw.so does not export {name}"
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    assert L.pdw_version() >= 1
    assert L.pdw_conv_out_size(56, 13, 1, 6, 1) == 56
    assert L.pdw_conv_out_size(5, 9, 1, 0, 1) == 0
    assert L.pdw_conv_out_size(32, 7, 2, 3, 1) == 16


def test_argument_validation_without_gpu():
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    # invalid arguments are rejected before any HIP call
    assert L.pdw_dwconv_fwd(None, None, None, 1, 4, 4, 8, 3, 3, 1, 1, 1, 1, 1, 1, 7, None) != 0
    assert b"dtype" in L.pdw_last_error()
    assert L.pdw_dwconv_fwd(None, None, None, 1, 4, 4, 8, 3, 3, 0, 1, 1, 1, 1, 1, 0, None) != 0
    assert b"stride" in L.pdw_last_error()
    assert L.pdw_gate_fwd(None, None, 4, 7, 0, 0, None) != 0
    assert L.pdw_dwconv_wgrad_workspace_bytes(2, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 0) > 0
    assert L.pdw_dwconv_wgrad(1, 1, 1, None, 0, 2, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 0, None) != 0
    assert b"workspace" in L.pdw_last_error()


def test_single_call_block_host_logic_without_gpu():
    """pdw_convblock_*: which shapes are covered, workspace sizes, and rejection before any HIP call."""
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    BF16, F16, F32 = 2, 1, 0
    assert L.pdw_convblock_supported(32, 56, 56, 128, 64, 13, BF16) == 1
    assert L.pdw_convblock_supported(1, 4, 8, 128, 64, 3, F16) == 1
    assert L.pdw_convblock_supported(2, 32, 32, 64, 32, 7, BF16) == 1
    assert L.pdw_convblock_supported(8, 112, 112, 96, 48, 17, F16) == 1
    for bad in ((32, 56, 56, 128, 64, 13, F32),    # 16-bit types only
                (32, 57, 56, 128, 64, 13, BF16),   # odd extent: the pooled scale is not an exact half
                (32, 56, 56, 128, 64, 12, BF16),   # even filter
                (32, 56, 56, 160, 80, 13, BF16),   # widths beyond the dense kernels (128)
                (0, 56, 56, 128, 64, 13, BF16),
                (2, 6, 6, 128, 64, 3, BF16)):      # 36 rows per image: not whole row tiles
        assert L.pdw_convblock_supported(*bad) == 0, bad
        assert L.pdw_convblock_fwd_workspace_bytes(*bad) == 0 and L.pdw_convblock_bwd_workspace_bytes(*bad) == 0
    shape = (32, 56, 56, 128, 64, 13, BF16)
    fwd, bwd = L.pdw_convblock_fwd_workspace_bytes(*shape), L.pdw_convblock_bwd_workspace_bytes(*shape)
    n = 32 * 56 * 56
    assert fwd >= n // L.pdw_dense_colsum_rows() * 128 * 4 + 32 * 128 * 4
    assert bwd >= 3 * n * 64 * 2 + L.pdw_dense_wgrad_workspace_bytes(n, 128, 64) * 2
    assert L.pdw_convblock_fwd(*([None] * 16), 0, *shape, None) != 0 and b"null" in L.pdw_last_error()
    assert L.pdw_convblock_fwd(*([1] * 16), 16, *shape, None) != 0 and b"workspace" in L.pdw_last_error()
    assert L.pdw_convblock_bwd(*([1] * 22), 16, *shape, None) != 0 and b"workspace" in L.pdw_last_error()
    assert L.pdw_convblock_bwd(*([1] * 22), 1 << 40, 32, 57, 56, 128, 64, 13, BF16, None) != 0
    assert b"not covered" in L.pdw_last_error()


@pytest.mark.parametrize("shape", [(128, 2, 64, 64, 3), (128, 4, 64, 64, 3), (128, 6, 64, 64, 13), (96, 2, 34, 16, 5),
                                   (512, 6, 40, 128, 17), (32, 56, 56, 64, 13), (8, 56, 56, 64, 13), (1, 8, 36, 16, 9),
                                   (8, 112, 112, 48, 17), (128, 56, 56, 64, 13)])
def test_bwd3_planner_strip_shaped_inputs(shape):
    """The planner of the backward's three-problem launch (host code, no device touched): images of fewer than four
    rows at the half scale, with batch x channels large enough that only whole-image bands are tried, must still get
    a plan with at least one band per problem (a plan of zero bands is a division by zero in the launcher)."""
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    bands = (ctypes.c_int * 3)(-1, -1, -1)
    rc = L.pdw_dwconv_bwd3_plan(*shape, _lib.dtype_code(torch.bfloat16), ctypes.addressof(bands))
    assert rc == 0, L.pdw_last_error()
    B, H, W, C, K = shape
    assert 1 <= bands[0] <= H and 1 <= bands[1] <= H and 1 <= bands[2] <= max(1, H // 2), list(bands)
    # not covered: fp32, odd extents, narrow images
    assert L.pdw_dwconv_bwd3_plan(*shape, _lib.dtype_code(torch.float32), ctypes.addressof(bands)) == 3
    assert L.pdw_dwconv_bwd3_plan(B, H, 16, C, K, 2, ctypes.addressof(bands)) == 3
    assert L.pdw_dwconv_bwd3_plan(B, H + 1, W, C, K, 2, ctypes.addressof(bands)) == 1
    assert L.pdw_dwconv_bwd3_plan(B, H, W, C, K, 2, None) == 1


def test_module_structure_and_seeded_init_match_reference_recipe():
    import pyramid_dwconv
    from oracle import torch_path

    torch.manual_seed(0)
    m = pyramid_dwconv.ConvBlock(dim=64, kernel_size=7)
    torch.manual_seed(0)
    P = torch_path.default_params(64, 7)
    sd = m.state_dict()
    assert list(sd.keys()) == list(P.keys())
    for k in P:
        assert sd[k].dtype == P[k].dtype and torch.equal(sd[k], P[k]), k
    assert tuple(sd["gates.1.conv_spatial.weight"].shape) == (7, 7, 32)
    assert sd["gates.0.conv_spatial.weight"].dtype == torch.float16
    assert m.gates[1].scale_factor == 0.5 and abs(m.gates[0].scale - 16 ** -0.5) < 1e-12
    mb = m.to(torch.bfloat16)
    assert all(v.dtype == torch.bfloat16 for v in mb.state_dict().values())


def test_no_cpu_path():
    import pyramidconvblock_amd as P

    conv = P.OptimizedDepthwiseConv2d(8, 3, padding=1, dtype=torch.float32)
    assert conv.weight.dtype == torch.float16  # dtype argument ignored, as in the reference
    with pytest.raises(RuntimeError, match="HIP device"):
        conv(torch.zeros(1, 4, 4, 8, dtype=torch.float16))
    with pytest.raises(AssertionError):
        conv(torch.zeros(1, 4, 4, 9))
    with pytest.raises(RuntimeError, match="HIP device"):
        P.ConvBlock(8, kernel_size=3)(torch.zeros(1, 4, 4, 8))
