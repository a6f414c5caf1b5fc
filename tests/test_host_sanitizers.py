"""Host code of the plugin library under AddressSanitizer and UndefinedBehaviorSanitizer, on the CPU.

The host sources (registry, plugin hosts, legacy (de)serialisers, flat C view, encoder runner, error unit) are compiled
here with `-Xarch_host -fsanitize=address,undefined` (device code is not instrumented) and linked with the kernel
objects of the regular build into a library of their own in a temporary directory; the two clients under tests/cpp are
built with the same compiler and sanitizers and run against it:
  plugin_client  - the interface walk of test_cpp_client.py;
  plugin_stress  - eight threads creating / cloning / serialising / deserialising plugins at once, and
                   deserializePlugin over ~5000 truncated, corrupted and random streams.
A sanitizer report fails the run (exit code and "ERROR:" in the output)."""
import concurrent.futures
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tensorrt_amd", "csrc")
OBJ = os.path.join(CSRC, "_obj")
SAN = ["-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"]


def _host_sources():
    return (sorted(glob.glob(os.path.join(CSRC, "*.cpp"))) + sorted(glob.glob(os.path.join(CSRC, "plugin", "*.cpp")))
            + sorted(glob.glob(os.path.join(CSRC, "runtime", "*.cpp"))))


@pytest.fixture(scope="module")
def sanitized(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    clang = "/opt/rocm/lib/llvm/bin/clang++"
    if not (os.path.exists(hipcc) and os.path.exists(clang)):
        pytest.skip("hipcc / clang++ of ROCm are not installed")
    kernels = sorted(glob.glob(os.path.join(OBJ, "*.hip.o")))
    assert kernels, "build the library first (python -m tensorrt_amd.build): its kernel objects are linked in here"
    work = tmp_path_factory.mktemp("sanitized")
    flags = ["--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}", f"-I{os.path.join(CSRC, 'plugin')}"]
    for f in SAN:
        flags += ["-Xarch_host", f]

    def compile_one(src):
        obj = str(work / (os.path.relpath(src, CSRC).replace(os.sep, "_") + ".o"))
        res = subprocess.run([hipcc, *flags, "-x", "hip", "-c", src, "-o", obj], capture_output=True, text=True, timeout=600)
        assert res.returncode == 0, res.stderr
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        objs = list(pool.map(compile_one, _host_sources()))
    lib = str(work / "libtrtamd_bert_plugins.so")
    # the sanitizer runtime comes from the executables below (clang links it statically into them)
    res = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs, *kernels, "-ldl", "-lpthread"],
                         capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stderr
    exes = {}
    for name in ("plugin_client", "plugin_stress"):
        exe = str(work / name)
        res = subprocess.run([clang, "-std=c++17", "-O1", "-g", *SAN, "-I", os.path.join(ROOT, "include"),
                              os.path.join(ROOT, "tests", "cpp", name + ".cpp"), "-o", exe, "-L", str(work),
                              "-ltrtamd_bert_plugins", f"-Wl,-rpath,{work}", "-lpthread"],
                             capture_output=True, text=True, timeout=600)
        assert res.returncode == 0, res.stderr
        exes[name] = exe
    return exes


def _run(exe, *args):
    # leak checking is off: the HIP runtime the library loads keeps allocations of its own until exit, which the leak
    # checker cannot tell from the library's; every other check (overruns, use after free, undefined behaviour) is on
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0:halt_on_error=1",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    ran = subprocess.run([exe, *args], capture_output=True, text=True, timeout=600, env=env)
    out = ran.stdout + ran.stderr
    assert ran.returncode == 0 and "ERROR: AddressSanitizer" not in out and "runtime error:" not in out, out[-4000:]
    assert ran.stdout.strip().endswith("ok"), out[-2000:]
    return out


def test_interface_walk_under_sanitizers(sanitized):
    _run(sanitized["plugin_client"])


def test_eight_threads_create_and_deserialize_under_sanitizers(sanitized):
    _run(sanitized["plugin_stress"], "threads")


def test_corrupted_legacy_streams_under_sanitizers(sanitized):
    out = _run(sanitized["plugin_stress"], "fuzz")
    assert "fuzz:" in out
