"""Run-time compiler, the parts that need no GPU: source -> code object with hipcc, the
content-addressed disk cache, and the error path (restating what tests/cpp/jit/test_jit.cc
and src/jit/compiler.cc:141-144 expect of a failed compile)."""

import glob
import os

import pytest
import torch

ADD_SRC = """
template <typename DType, const int kNumel>
__device__ void add_device(const DType* a, const DType* b, DType* out) {
  int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < kNumel) out[idx] = a[idx] + b[idx];
}
extern "C" __global__ void add_kernel_float_1000(const float* a, const float* b, float* out) {
  add_device<float, 1000>(a, b, out);
}
"""


@pytest.fixture()
def cache_dir(tmp_path, monkeypatch):
    monkeypatch.setenv("TILEFUSION_CACHE_DIR", str(tmp_path))
    from tilefusion_amd.jit import JitCompiler
    JitCompiler.clear_cache()
    return tmp_path


def test_failed_compile_reports_the_compiler_output(cache_dir):
    from tilefusion_amd.jit import JitCompiler
    with pytest.raises(RuntimeError, match="Failed to compile or retrieve kernel") as e:
        JitCompiler.get_or_compile_kernel("broken", 'extern "C" __global__ void broken() { this is not C++; }')
    assert "error" in str(e.value)
    assert not glob.glob(os.path.join(str(cache_dir), "*.hsaco"))   # nothing cached for a failure


def test_code_object_is_cached_on_disk_by_content(cache_dir):
    from tilefusion_amd.jit import JitCompiler
    assert JitCompiler.cache_dir() == str(cache_dir)

    def compile_once():
        try:
            return JitCompiler.get_or_compile_kernel("add_kernel_float_1000", ADD_SRC)
        except RuntimeError as e:
            # without a GPU the code object is built and cached, only loading it fails
            assert not torch.cuda.is_available() and "hipModuleLoadData" in str(e)
            return None

    compile_once()
    objs = glob.glob(os.path.join(str(cache_dir), "*.hsaco"))
    assert len(objs) == 1 and os.path.getsize(objs[0]) > 0
    stamp = os.path.getmtime(objs[0])
    compile_once()                                   # second request: no recompilation
    assert glob.glob(os.path.join(str(cache_dir), "*.hsaco")) == objs and os.path.getmtime(objs[0]) == stamp
    assert not glob.glob(os.path.join(str(cache_dir), "*.hip"))   # temporaries are removed


def test_wrappers_validate_before_compiling(cache_dir):
    from tilefusion_amd import jit
    t = torch.zeros(64, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="must be a cuda tensor"):
        jit.gemm_jit(t, t, torch.zeros(64, 64), 64, 64, 64)
    with pytest.raises(ValueError, match="must be a cuda tensor"):
        jit.fused_two_gemms_jit(t, t, t, t)
    assert not glob.glob(os.path.join(str(cache_dir), "*"))
