"""The C++ surface from a caller built by another compiler: tests/cpp/plugin_client.cpp uses only
include/trtamd_nvinfer_api.h (virtual interfaces, no HIP headers), is compiled with g++ and linked against the
library, and must find, create, configure, serialise and re-create plugins through the vtables."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_gxx_client_drives_the_plugins(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("g++ is not installed")
    lib_dir = os.path.join(ROOT, "tensorrt_amd", "lib")
    assert os.path.exists(os.path.join(lib_dir, "libtrtamd_bert_plugins.so")), "build the library first"
    exe = tmp_path / "plugin_client"
    cmd = [gxx, "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cpp", "plugin_client.cpp"), "-o", str(exe), "-L", lib_dir,
           "-ltrtamd_bert_plugins", f"-Wl,-rpath,{lib_dir}"]
    built = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert built.returncode == 0, built.stderr
    ran = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert ran.returncode == 0 and ran.stdout.strip().endswith("ok"), ran.stdout + ran.stderr
