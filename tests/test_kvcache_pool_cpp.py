"""Builds and runs the host-only C++ test of infer::KVCachePool (tests/cpp/test_kvcache_pool.cpp)
against libinfer_kv.so."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_kvcache_pool_cpp(tmp_path):
    exe = tmp_path / "test_kvcache_pool"
    lib_dir = os.path.join(ROOT, "infer_amd")
    subprocess.run(["g++", "-std=c++17", "-O1", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "test_kvcache_pool.cpp"), "-o", str(exe),
                    "-L", lib_dir, "-linfer_kv", f"-Wl,-rpath,{lib_dir}", "-Wl,-rpath,/opt/rocm/lib"],
                   check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True)
    assert out.stdout.strip().endswith("ok")
