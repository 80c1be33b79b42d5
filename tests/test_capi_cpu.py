"""CPU-only checks of the C ABI: the library loads, exports every symbol the header declares,
and rejects bad arguments before touching the device."""

import ctypes
import os
import re

import pytest

from tilefusion_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "tilefusion_c.h")).read()
    return sorted(set(re.findall(r"TF_API\s+[\w\s\*]+?\b(tf_\w+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared_symbols()
    assert len(names) >= 7
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in tilefusion_c.h but not exported"
        assert n in _capi.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_capi.SIGNATURES) == names


def test_version_and_error_string():
    lib = _capi.load()
    assert b"gfx950" in lib.tf_version()
    assert isinstance(lib.tf_last_error(), bytes)


def test_gemm_argument_validation():
    lib = _capi.load()
    p = 0x1000  # never dereferenced: validation fails first
    assert lib.tf_gemm_f16(None, p, p, 0, 128, 128, 128, 64, 64, 64, 1, 0, None) == _capi.TF_ERR_INVALID_ARG
    assert b"null" in lib.tf_last_error()
    assert lib.tf_gemm_f16(p, p, p, 0, 0, 128, 128, 64, 64, 64, 1, 0, None) == _capi.TF_ERR_INVALID_ARG
    assert lib.tf_gemm_f16(p, p, p, 0, 128, 128, 128, 48, 64, 64, 1, 0, None) == _capi.TF_ERR_INVALID_ARG
    assert b"does not divide" in lib.tf_last_error()
    assert lib.tf_gemm_f16(p, p, p, 0, 128, 128, 128, 64, 64, 64, 4, 0, None) == _capi.TF_ERR_INVALID_ARG
    assert lib.tf_gemm_f16(p, p, p, 0, 128, 128, 128, 64, 64, 64, 1, 3, None) == _capi.TF_ERR_INVALID_ARG
    assert lib.tf_gemm_f16(p, p, p, 0, 128, 128, 100, 64, 64, 100, 1, 0, None) == _capi.TF_ERR_UNSUPPORTED
    with pytest.raises(RuntimeError, match="multiple of 8"):
        _capi.check(_capi.TF_ERR_UNSUPPORTED, "tf_gemm_f16")


def test_fused_argument_validation():
    lib = _capi.load()
    p = 0x1000
    assert lib.tf_fused_two_gemms_f16(p, p, p, None, 1, 64, 64, 64, 64, 64, 64, 64, 64, None) == _capi.TF_ERR_INVALID_ARG
    assert lib.tf_fused_two_gemms_f16(p, p, p, p, 1, 64, 64, 64, 64, 48, 64, 64, 64, None) == _capi.TF_ERR_INVALID_ARG
    assert lib.tf_fused_two_gemms_f16(p, p, p, p, 1, 64, 48, 64, 64, 64, 48, 64, 64, None) == _capi.TF_ERR_UNSUPPORTED
    assert lib.tf_fused_two_gemms_f16(p, p, p, p, 0, 64, 64, 64, 64, 64, 64, 64, 64, None) == _capi.TF_ERR_INVALID_ARG


def test_attention_argument_validation():
    lib = _capi.load()
    p = 0x1000
    f = lib.tf_flash_attention_fwd_f16
    assert f(p, p, None, p, 1, 64, 64, 128, 128, 0, 64, 64, 128, 128, 0.1, 0, None) == _capi.TF_ERR_INVALID_ARG
    assert f(p, p, p, p, 1, 64, 64, 80, 80, 0, 64, 64, 80, 80, 0.1, 0, None) == _capi.TF_ERR_UNSUPPORTED
    assert f(p, p, p, p, 1, 64, 64, 128, 128, 0, 48, 64, 128, 128, 0.1, 0, None) == _capi.TF_ERR_INVALID_ARG
    assert f(p, p, p, p, 1, 64, 60, 128, 128, 1, 64, 60, 128, 128, 0.1, 0, None) == _capi.TF_ERR_UNSUPPORTED
    assert f(p, p, p, p, 1, 64, 64, 128, 128, 0, 64, 64, 128, 128, float("nan"), 0, None) == _capi.TF_ERR_INVALID_ARG


def test_decode_argument_validation_and_workspace():
    lib = _capi.load()
    p = 0x1000
    assert lib.tf_flash_decode_workspace_bytes(512, 128, 64) == 512 * 64 * 130 * 4
    assert lib.tf_flash_decode_workspace_bytes(0, 128, 64) == 0
    f = lib.tf_flash_decode_f16
    assert f(p, p, p, p, None, 0, 4, 128, 128, 4, 0.1, None) == _capi.TF_ERR_INVALID_ARG
    assert f(p, p, p, p, p, 16, 4, 128, 128, 4, 0.1, None) == _capi.TF_ERR_INVALID_ARG
    assert b"workspace" in lib.tf_last_error()
    assert f(p, p, p, p, p, 1 << 20, 4, 128, 96, 4, 0.1, None) == _capi.TF_ERR_UNSUPPORTED   # 128 and 64 only
    assert f(p, p, p, p, p, 1 << 20, 4, 0, 128, 4, 0.1, None) == _capi.TF_ERR_INVALID_ARG


def test_python_wrappers_validate_like_the_reference():
    # python/ops/fused_two_gemms.py:33-38: ValueError for a CPU tensor, TypeError for dtype
    import torch
    from tilefusion_amd import ops
    t = torch.zeros(64, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="must be a cuda tensor"):
        ops.fused_two_gemms(t, t, t, t)
    # CPU tensors never reach a kernel: the op exists only for the CUDA dispatch key
    with pytest.raises((NotImplementedError, RuntimeError)):
        ops.gemm(t, t, torch.zeros(64, 64), 64, 64, 64, 1, 0)
    assert sorted(ops.__all__) == ["FlashAttention", "flash_attention", "flash_decode", "fused_two_gemms", "gemm", "scatter_nd"]


def test_op_schemas_match_the_reference():
    # include/kernels/kernel_list.hpp:15-30
    import torch
    import tilefusion_amd  # noqa: F401
    want = {
        "scatter_nd": "tilefusion::scatter_nd(Tensor data, Tensor(a!) updates, Tensor indices) -> ()",
        "gemm": "tilefusion::gemm(Tensor A, Tensor B, Tensor(a!) C, int m, int n, int k, int num_stages, int pipeline_level) -> ()",
        "fused_two_gemms": "tilefusion::fused_two_gemms(Tensor A, Tensor B, Tensor C, Tensor(a!) D, int tm, int tn, int tk, int tp) -> ()",
        "flash_attention": "tilefusion::flash_attention(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, int tile_length_q, int tile_length_kv, int tile_hidden_qk, int tile_hidden_v, float softmax_scale, bool causal) -> ()",
    }
    for name, schema in want.items():
        op = getattr(torch.ops.tilefusion, name).default
        assert str(op._schema) == schema


def test_reference_package_name_imports_the_same_modules():
    # callers written against the reference do `import tilefusion` / `from tilefusion.ops import gemm`
    import tilefusion
    import tilefusion_amd
    from tilefusion.ops import flash_attention, fused_two_gemms, gemm
    assert tilefusion.ops is tilefusion_amd.ops
    assert gemm is tilefusion_amd.ops.gemm and fused_two_gemms is tilefusion_amd.ops.fused_two_gemms
    assert flash_attention is tilefusion_amd.ops.flash_attention


def test_torch_binding_exports_the_reference_launcher_names():
    # TILEFUSION_EXPORT (include/kernel_registry.hpp:20-24, include/kernels/ops.hpp:36-58): the four host
    # launchers are C-linkage symbols of libtilefusion.so under the reference's names
    import ctypes
    import os

    import torch  # noqa: F401  (the binding links against libtorch)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ctypes.CDLL(os.path.join(root, "tilefusion_amd", "libtilefusion.so"))
    for name in ("gemm", "fused_two_gemms", "flash_attention", "scatter_nd"):
        assert hasattr(lib, name), name
