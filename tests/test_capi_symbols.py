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
