"""CPU-side checks of the boundary: the library loads and exports every symbol
the header declares; descriptor structs have the C layout."""
import ctypes
import os
import re

from fusilli_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "fusilli_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fhip_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_all_bound_and_exported():
    lib = ctypes.CDLL(capi.library_path())
    declared = _declared_symbols()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), f"{name} declared but not exported"
        assert name in capi.SYMBOLS, f"{name} has no ctypes signature"
    assert sorted(capi.SYMBOLS) == declared


def test_abi_version_and_struct_sizes():
    lib = capi.load()
    assert lib.fhip_abi_version() == 1
    assert ctypes.sizeof(capi.TensorDesc) == 8 + 8 * 8 * 2
    assert ctypes.sizeof(capi.EpilogueOp) == 40 + ctypes.sizeof(capi.TensorDesc)
    assert ctypes.sizeof(capi.PointwiseParams) == 16


def test_supported_queries_need_no_gpu():
    lib = capi.load()
    d = capi.NormDesc()
    d.x = capi.TensorDesc.make([8192, 4096], [4096, 1], capi.BFLOAT16)
    d.scale = capi.TensorDesc.make([1, 4096], [4096, 1], capi.BFLOAT16)
    d.y = capi.TensorDesc.make([8192, 4096], [4096, 1], capi.FLOAT)
    d.out = capi.TensorDesc.make([8192, 4096], [4096, 1], capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.epsilon = 1e-6
    d.epilogue = capi.make_epilogue(
        [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=2.0)])
    assert lib.fhip_norm_fwd_supported(d) == 2  # tuned row kernel
    d.x = capi.TensorDesc.make([8192, 4096], [1, 8192], capi.BFLOAT16)
    assert lib.fhip_norm_fwd_supported(d) == 1  # generic strided kernel
    d.out = capi.TensorDesc.make([8192, 4095], [4095, 1], capi.BFLOAT16)
    assert lib.fhip_norm_fwd_supported(d) == 0  # dims disagree


def test_gradient_and_batchnorm_queries_need_no_gpu():
    lib = capi.load()
    cl = lambda d: [d[1] * d[2] * d[3], 1, d[3] * d[1], d[1]]
    xd, wd, yd = [32, 64, 56, 56], [128, 64, 3, 3], [32, 128, 56, 56]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.BFLOAT16)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 1, 1
    d.epilogue = capi.make_epilogue([])
    assert lib.fhip_conv_dgrad_supported(d) == 2  # forward MFMA kernel, mirrored filter
    assert lib.fhip_conv_wgrad_supported(d) == 2  # the kernel that reads X and DY in place
    n = ctypes.c_size_t(0)
    assert lib.fhip_conv_dgrad_workspace_size(d, ctypes.byref(n)) == 0
    assert n.value == 128 * 64 * 9 * 2
    assert lib.fhip_conv_wgrad_workspace_size(d, ctypes.byref(n)) == 0
    assert n.value == 256 * 9 * 1024 * 4  # 256 workgroups' partial sums, 36 KB each
    for i in range(2):
        d.stride[i] = 2
    d.y = capi.TensorDesc.make([32, 128, 28, 28], cl([32, 128, 28, 28]), capi.BFLOAT16)
    assert lib.fhip_conv_dgrad_supported(d) == 2  # DY spread over a zero grid
    assert lib.fhip_conv_wgrad_supported(d) == 2  # batched GEMMs, B rows two pixels apart
    assert lib.fhip_conv_wgrad_workspace_size(d, ctypes.byref(n)) == 0
    assert n.value > 32 * 58 * 64 * 64 * 2  # zero-padded copies of X and DY
    d.y = capi.TensorDesc.make([32, 128, 28, 27], cl([32, 128, 28, 27]), capi.BFLOAT16)
    assert lib.fhip_conv_dgrad_supported(d) == 0  # DY extent disagrees

    b = capi.BatchNormDesc()
    b.x = b.y = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    b.running_dtype = b.stats_dtype = b.scale_dtype = b.bias_dtype = capi.FLOAT
    b.epsilon = 1e-5
    assert lib.fhip_batchnorm_fwd_supported(b) == 2  # dense channels-last: the column kernels
    b.y = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    assert lib.fhip_batchnorm_fwd_supported(b) == 0
