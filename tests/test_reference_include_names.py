"""A C++ translation unit written against the reference's include names and KVCachePool constructor
(tests/cpp/test_reference_include_names.cpp) compiles against include/ and links libinfer_kv.so and
_C_infer_kv.so; run, it exercises the registry on the host and, where there is a GPU, the pool that owns
its device storage (without one the constructor must throw std::runtime_error, which the program accepts)."""
import os
import subprocess
import sys
import sysconfig

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def build_and_run(tmp_path) -> str:
    exe = tmp_path / "ref_names"
    lib_dir = os.path.join(ROOT, "infer_amd")
    tdir = os.path.dirname(torch.__file__)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-std=c++17", "-O0", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(tdir, "include"),
           "-I", os.path.join(tdir, "include", "torch", "csrc", "api", "include"), "-I", os.path.join(rocm, "include"),
           "-I", sysconfig.get_paths()["include"],
           os.path.join(ROOT, "tests", "cpp", "test_reference_include_names.cpp"), "-o", str(exe),
           "-L", lib_dir, "-l:_C_infer_kv.so", "-linfer_kv", "-L", os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu",
           "-lc10", "-ltorch_python", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
           f"-L{sysconfig.get_config_var('LIBDIR')}", f"-lpython{sys.version_info.major}.{sys.version_info.minor}",
           f"-Wl,-rpath,{lib_dir}", f"-Wl,-rpath,{os.path.join(tdir, 'lib')}", f"-Wl,-rpath,{os.path.join(rocm, 'lib')}"]
    subprocess.run(cmd, check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr
    return out.stdout


def test_translation_unit_with_the_reference_names_builds_and_runs(tmp_path):
    build_and_run(tmp_path)


@pytest.mark.gpu
def test_pool_that_owns_its_device_storage(gpu, tmp_path):
    assert "no device" not in build_and_run(tmp_path)      # the constructor allocated, the views point into it
