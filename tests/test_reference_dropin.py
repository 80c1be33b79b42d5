"""Kernels written against the reference's tile-programming surface drop in: the reference's OWN
kernel sources - examples/101_gemm/01_gemm_global_reg/gemm.hpp, 02_gemm_all_mem/gemm.hpp, the
three macro kernels include/kernels/{gemm,fused_two_gemms,flash_attention}_device.cuh and the kernel
of its copy benchmark, benchmarks/cpp/g2s_copy/tilefusion_copy.cuh - are
compiled, unmodified and where they lie, against this repository's headers (recipe: oracle/Makefile,
drivers: tests/cpp/reference_dropin/*.hip) and run on the GPU against the fp32 oracle.

The compile step needs the reference tree and runs wherever it is present (the CPU test below);
the built library oracle/_ref/libreference_kernels.so is not tracked and travels with the tree to
the GPU box, where the GPU tests load it (they skip when it was never built).  The same idiom
written out in this repository - the README kernel with the reference's tile-count formulas - is
tests/test_gpu_tile_api.py::test_readme_example_gemm and runs unconditionally."""

import ctypes
import os
import subprocess

import pytest
import torch

from oracle import numerics as N

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = "/root/reference"
LIB = os.path.join(ROOT, "oracle", "_ref", "libreference_kernels.so")
SYMBOLS = ["dropin_example_01", "dropin_example_01_shape", "dropin_example_02", "dropin_example_02_shape",
           "dropin_ke_gemm", "dropin_ke_gemm_shape", "dropin_ke_fused", "dropin_ke_flash",
           "dropin_g2s_copy", "dropin_g2s_copy_shape"]
DEV = "cuda:0"
_vp, _i = ctypes.c_void_p, ctypes.c_int


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "include", "kernels")),
                    reason="the reference tree is not present on this machine")
def test_reference_kernel_sources_compile_against_these_headers():
    # a full device compile for gfx950 (not a syntax check): every template the drivers name is instantiated
    if os.path.exists(LIB):
        os.remove(LIB)
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-j3", "_ref/libreference_kernels.so"])
    lib = ctypes.CDLL(LIB)
    for name in SYMBOLS:
        assert hasattr(lib, name), name
    # nothing of the reference's text stays behind in the tree
    assert sorted(os.listdir(os.path.dirname(LIB))) == ["libreference_kernels.so"]


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "examples", "101_gemm")),
                    reason="the reference tree is not present on this machine")
def test_only_the_kernel_files_come_from_the_reference():
    # the drivers must see THIS repository's cell/, types/ and util/ headers: list every file the
    # compiler opens and check that the only ones under the reference are the six kernel sources
    inc = os.path.join(ROOT, "tilefusion_amd", "include")
    drivers = os.path.join(ROOT, "tests", "cpp", "reference_dropin")
    opened = set()
    for src, ref_inc in [("example_01.hip", "examples/101_gemm/01_gemm_global_reg"),
                         ("example_02.hip", "examples/101_gemm/02_gemm_all_mem"), ("device_kernels.hip", "include"),
                         ("g2s_copy.hip", "benchmarks/cpp/g2s_copy")]:
        p = subprocess.run(["/opt/rocm/bin/hipcc", "-std=c++20", "--offload-arch=gfx950", "-fsyntax-only", "-H", "-w",
                            "-I" + inc, "-I" + os.path.join(REFERENCE, ref_inc), "-x", "hip", os.path.join(drivers, src)],
                           capture_output=True, text=True)
        assert p.returncode == 0, p.stderr[-2000:]
        for line in p.stderr.splitlines():
            if line.startswith(".") and REFERENCE in line:
                opened.add(os.path.relpath(line.split()[-1], REFERENCE))
    assert opened == {"examples/101_gemm/01_gemm_global_reg/gemm.hpp", "examples/101_gemm/02_gemm_all_mem/gemm.hpp",
                      "include/kernels/gemm_device.cuh", "include/kernels/fused_two_gemms_device.cuh",
                      "include/kernels/flash_attention_device.cuh", "benchmarks/cpp/g2s_copy/tilefusion_copy.cuh"}


# ---- on the GPU ---------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.skip("oracle/_ref/libreference_kernels.so was not built (it needs the reference tree at build time)")
    lib = ctypes.CDLL(LIB)
    lib.dropin_example_01.argtypes = [_i, _vp, _vp, _vp]
    lib.dropin_example_02.argtypes = [_i, _vp, _vp, _vp]
    lib.dropin_ke_gemm.argtypes = [_i, _vp, _vp, _vp]
    for f in (lib.dropin_example_01_shape, lib.dropin_example_02_shape, lib.dropin_ke_gemm_shape):
        f.argtypes = [_i] + [ctypes.POINTER(_i)] * 3
    lib.dropin_ke_fused.argtypes = [_vp] * 4
    lib.dropin_ke_flash.argtypes = [_i, _vp, _vp, _vp, _vp]
    lib.dropin_g2s_copy.argtypes = [_i, _vp, _vp]
    lib.dropin_g2s_copy_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 2
    return lib


def _gemm_case(run, shape, variant):
    m, n, k = _i(), _i(), _i()
    shape(variant, m, n, k)
    m, n, k = m.value, n.value, k.value
    g = torch.Generator().manual_seed(700 + variant)
    # integer operands: products and sums are exact in fp32, so the comparison is bit-exact
    a = torch.randint(-3, 4, (m, k), generator=g).half()
    b = torch.randint(-3, 4, (n, k), generator=g).half()   # [n, k] buffer = column-major k x n
    c = torch.full((m, n), float("nan"), device=DEV)
    for _ in range(3):
        c.fill_(float("nan"))
        assert run(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
        assert torch.equal(c.cpu(), N.gemm_ref(a, b))
    # and real-valued data against the oracle, to the tolerance of the parity tests
    a = (torch.rand(m, k, generator=g) * 2 - 1).half()
    b = (torch.rand(n, k, generator=g) * 2 - 1).half()
    assert run(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    ok, r, ab = N.check_close(c, N.gemm_ref(a, b))
    assert ok and ab < 1e-3, (r, ab)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", range(3))
def test_reference_example_global_reg_gemm_runs_exact(lib, variant):
    # variant 0 is the README's single tile: A 128 x 256, B 256 x 64 column-major, C 128 x 64 fp32
    _gemm_case(lib.dropin_example_01, lib.dropin_example_01_shape, variant)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", range(2))
def test_reference_example_all_mem_gemm_runs_exact(lib, variant):
    _gemm_case(lib.dropin_example_02, lib.dropin_example_02_shape, variant)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", range(4))
def test_reference_ke_gemm_and_pipelines_run_exact(lib, variant):
    _gemm_case(lib.dropin_ke_gemm, lib.dropin_ke_gemm_shape, variant)


@pytest.mark.gpu
def test_reference_ke_fused_two_gemms_runs(lib):
    g = torch.Generator().manual_seed(710)
    m, n, k, p = 256, 128, 64, 64
    a = (torch.randn(m, k, generator=g) / 8).half()
    b = (torch.randn(n, k, generator=g) / 8).half()
    c = (torch.randn(p, n, generator=g) / 8).half()
    d = torch.full((m, p), float("nan"), dtype=torch.float16, device=DEV)
    assert lib.dropin_ke_fused(a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.to(DEV).data_ptr(), d.data_ptr()) == 0
    ok, r, ab = N.check_close(d, N.fused_two_gemms_ref(a, b, c))
    assert ok, (r, ab)
    # exactly representable data: the fp16 intermediate is exact, so is the result
    a = torch.randint(-2, 3, (m, k), generator=g).half()
    b = torch.randint(-2, 3, (n, k), generator=g).half()
    c = torch.randint(-1, 2, (p, n), generator=g).half()
    assert lib.dropin_ke_fused(a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.to(DEV).data_ptr(), d.data_ptr()) == 0
    ref = N.fused_two_gemms_ref(a, b, c)
    assert float(ref.abs().max()) <= 2048 and torch.equal(d.float().cpu(), ref)


@pytest.mark.gpu
@pytest.mark.parametrize("variant,lq,causal", [(0, 64, False), (1, 128, True)])
def test_reference_ke_flash_attention_runs(lib, variant, lq, causal):
    # the reference's kernel keeps its softmax statistics and its output accumulator in fp16
    # (include/kernels/flash_attention_device.cuh:106,191-199), so it is held to the tolerance of the
    # reference's own test (tests/python/test_flash_attn.py:199: atol = rtol = 1e-2), not to the
    # tighter one of this repository's kernels
    g = torch.Generator().manual_seed(720 + variant)
    q = torch.randn(lq, 128, generator=g).half()
    k = torch.randn(128, 128, generator=g).half()
    v = torch.randn(128, 128, generator=g).half()
    vt = v.t().contiguous()   # V column-major: a [Dv, Lkv] buffer
    o = torch.full((lq, 128), float("nan"), dtype=torch.float16, device=DEV)
    assert lib.dropin_ke_flash(variant, q.to(DEV).data_ptr(), k.to(DEV).data_ptr(), vt.to(DEV).data_ptr(), o.data_ptr()) == 0
    ref = N.attention_ref(q, k, v, causal=causal)
    assert torch.allclose(o.float().cpu(), ref, atol=1e-2, rtol=1e-2), (N.rel_l2(o, ref), N.max_abs(o, ref))


@pytest.mark.gpu
@pytest.mark.parametrize("variant", range(11))
def test_reference_g2s_copy_kernel_moves_every_element(lib, variant):
    # the tiles and wavefront layouts of the reference's sweep (benchmarks/cpp/g2s_copy/main.cu:143-165)
    # with its source pattern (element i holds i % 2048, :116-117): global -> swizzled shared -> global
    rows, cols = _i(), _i()
    lib.dropin_g2s_copy_shape(variant, rows, cols)
    numel = rows.value * cols.value
    src = (torch.arange(numel) % 2048).half().to(DEV)
    dst = torch.full((numel,), float("nan"), dtype=torch.float16, device=DEV)
    assert lib.dropin_g2s_copy(variant, src.data_ptr(), dst.data_ptr()) == 0
    assert torch.equal(dst, src)
