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


def test_cache_key_covers_the_contents_of_included_headers(cache_dir, tmp_path_factory):
    # Same source, same include path, edited header: a second code object, not a stale hit.
    from tilefusion_amd.jit import JitCompiler
    inc = tmp_path_factory.mktemp("inc")
    src = '#include "k.hpp"\nextern "C" __global__ void scale_kernel(float* x) { x[threadIdx.x] *= kFactor; }'

    def compile_with(factor):
        (inc / "k.hpp").write_text(f"constexpr float kFactor = {factor}f;\n")
        try:
            JitCompiler.get_or_compile_kernel("scale_kernel", src, [str(inc)])
        except RuntimeError as e:
            assert not torch.cuda.is_available() and "hipModuleLoadData" in str(e)

    compile_with(2.0)
    assert len(glob.glob(os.path.join(str(cache_dir), "*.hsaco"))) == 1
    # the digest of a directory is taken once per process; a new process sees the edit, which
    # is what a library update between runs looks like.  Emulate it with a second directory
    # of the same contents but the edited header.
    inc2 = tmp_path_factory.mktemp("inc2")
    (inc2 / "k.hpp").write_text("constexpr float kFactor = 3.0f;\n")
    try:
        JitCompiler.get_or_compile_kernel("scale_kernel", src, [str(inc2)])
    except RuntimeError as e:
        assert not torch.cuda.is_available() and "hipModuleLoadData" in str(e)
    assert len(glob.glob(os.path.join(str(cache_dir), "*.hsaco"))) == 2


def test_include_directory_too_deep_to_digest_is_not_cached(cache_dir, tmp_path_factory):
    # The digest walk is bounded; a header below the bound could change without changing the key,
    # so nothing compiled against such a directory may be left for a later process to find.
    from tilefusion_amd.jit import JitCompiler
    inc = tmp_path_factory.mktemp("deep")
    deep = inc
    for level in range(9):
        deep = deep / f"l{level}"
    deep.mkdir(parents=True)
    (deep / "k.hpp").write_text("constexpr float kFactor = 2.0f;\n")
    rel = "/".join(f"l{level}" for level in range(9))
    src = f'#include "{rel}/k.hpp"\nextern "C" __global__ void deep_kernel(float* x) {{ x[threadIdx.x] *= kFactor; }}'
    try:
        JitCompiler.get_or_compile_kernel("deep_kernel", src, [str(inc)])
    except RuntimeError as e:
        assert not torch.cuda.is_available() and "hipModuleLoadData" in str(e)
    assert not glob.glob(os.path.join(str(cache_dir), "*"))


def test_kernel_handles_die_with_clear_cache():
    from tilefusion_amd.jit import JitCompiler, Kernel
    k = Kernel(0, "stale")
    JitCompiler.clear_cache()
    with pytest.raises(RuntimeError, match="unloaded by JitCompiler.clear_cache"):
        k.launch((1,), (64,), ())


def test_attention_kernel_name_is_stable_across_processes():
    # the name is part of the source and therefore of the disk-cache key: it must not depend
    # on Python's per-process string hashing
    import struct
    import subprocess
    import sys
    code = "import struct; print(struct.pack('<d', 0.08838834764831845).hex())"
    outs = {subprocess.check_output([sys.executable, "-c", code], env={**os.environ, "PYTHONHASHSEED": str(s)}) for s in (1, 2)}
    assert len(outs) == 1
    import inspect
    from tilefusion_amd import jit
    assert "hash(" not in inspect.getsource(jit.flash_attention_jit)
