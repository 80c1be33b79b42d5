"""Run-time compiled kernels on the GPU: the reference's JIT'd vector add
(tests/cpp/jit/test_jit.cc:28-133) and the three macro kernels instantiated for tile sizes the
ahead-of-time library has no instance of, each against the fp32 oracle."""

import pytest
import torch

from oracle import numerics as N

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True, scope="module")
def fresh_disk_cache(tmp_path_factory):
    """Compile into an empty directory so that no code object left by an earlier build of the
    library can be picked up."""
    import os
    from tilefusion_amd.jit import JitCompiler
    old = os.environ.get("TILEFUSION_CACHE_DIR")
    os.environ["TILEFUSION_CACHE_DIR"] = str(tmp_path_factory.mktemp("jit_cache"))
    JitCompiler.clear_cache()
    yield
    JitCompiler.clear_cache()
    if old is None:
        os.environ.pop("TILEFUSION_CACHE_DIR", None)
    else:
        os.environ["TILEFUSION_CACHE_DIR"] = old


def test_jit_vector_add():
    from tilefusion_amd.jit import JitCompiler
    from tests.test_jit_cpu import ADD_SRC
    n = 1000
    g = torch.Generator().manual_seed(0)
    a, b = torch.rand(n, generator=g), torch.rand(n, generator=g)
    out = torch.full((n,), -1.0, device=DEV)
    kern = JitCompiler.get_or_compile_kernel("add_kernel_float_1000", ADD_SRC)
    kern.launch(((n + 127) // 128,), (128,), (a.to(DEV), b.to(DEV), out))
    assert torch.allclose(out.cpu(), a + b, atol=1e-5)            # the reference's epsilon
    again = JitCompiler.get_or_compile_kernel("add_kernel_float_1000", ADD_SRC)
    assert again._handle == kern._handle                          # in-process cache


@pytest.mark.parametrize("level,stages", [(0, 1), (1, 2), (2, 3)])
def test_jit_gemm_uses_the_requested_tiles(level, stages):
    from tilefusion_amd import jit
    m, n, k, tm, tn, tk = 192, 320, 160, 96, 160, 32      # 96 x 160 tiles: no ahead-of-time instance
    g = torch.Generator().manual_seed(11 + level)
    a = (torch.randn(m, k, generator=g) / k ** 0.5).half()
    b = (torch.randn(n, k, generator=g) / k ** 0.5).half()
    c = torch.full((m, n), float("nan"), device=DEV)
    jit.gemm_jit(a.to(DEV), b.to(DEV), c, tm, tn, tk, stages, level)
    ok, r, ab = N.check_close(c, N.gemm_ref(a, b))
    assert ok, (r, ab)


def test_jit_fused_two_gemms():
    from tilefusion_amd import jit
    m, n, k, p = 256, 128, 64, 64                          # tests/python/test_fused_two_gemms.py
    g = torch.Generator().manual_seed(21)
    a = (torch.randn(m, k, generator=g) / 8).half()
    b = (torch.randn(n, k, generator=g) / 8).half()
    c = (torch.randn(p, n, generator=g) / 8).half()
    d = torch.full((m, p), float("nan"), dtype=torch.float16, device=DEV)
    jit.fused_two_gemms_jit(a.to(DEV), b.to(DEV), c.to(DEV), d, 64, 64, 64, 64)
    ok, r, ab = N.check_close(d, N.fused_two_gemms_ref(a, b, c))
    assert ok, (r, ab)


def test_jit_flash_attention_causal():
    from tilefusion_amd import jit
    lq, lkv, d = 128, 128, 128                             # tests/python/test_flash_attn.py, causal case
    g = torch.Generator().manual_seed(31)
    q = torch.randn(lq, d, generator=g).half()
    k = torch.randn(lkv, d, generator=g).half()
    v = torch.randn(lkv, d, generator=g).half()
    o = torch.full((lq, d), float("nan"), dtype=torch.float16, device=DEV)
    jit.flash_attention_jit(q.to(DEV), k.to(DEV), v.t().contiguous().to(DEV), o, 64, 128, 128, 128, causal=True)
    ok, r, ab = N.check_close(o, N.attention_ref(q, k, v, causal=True))
    assert ok, (r, ab)
