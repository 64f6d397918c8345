"""The host side of the C ABI (argument checks, kernel selection, size arithmetic) under
AddressSanitizer and UndefinedBehaviorSanitizer.

`cascmm_api.hip` is compiled once more with the sanitizers on its host pass only (the device code
is left alone), linked with the library's other objects and a small driver
(`host_sanitizer_driver.cpp`) that walks the selection and size functions over a grid of shapes up
to 2**40 and calls the launching entry points with arguments they must refuse before any HIP call.
A second build, under ThreadSanitizer, is driven by `host_threads_driver.cpp`: eight threads ask for
kernels and sizes at once (the selection keeps a table of earlier answers behind a lock) and must get
what one thread gets.  Nothing here needs a GPU.
"""
import glob
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "basedxl_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def test_host_layer_is_clean_under_asan_and_ubsan(tmp_path):
    objs = [o for o in glob.glob(os.path.join(CSRC, "build", "*.o")) if not o.endswith("cascmm_api.o")]
    if not os.path.exists(HIPCC) or shutil.which("g++") is None or len(objs) < 5:
        pytest.skip("needs hipcc, g++ and the library's object files (python -m basedxl_amd.build)")
    api, drv, exe = str(tmp_path / "api_san.o"), str(tmp_path / "driver.o"), str(tmp_path / "driver")
    flags = ["-O1", "-g", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host", "-fno-sanitize-recover=undefined"]
    r = subprocess.run([HIPCC, *flags, *san, "-c", os.path.join(CSRC, "cascmm_api.hip"), "-o", api], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-I", os.path.join(ROOT, "include"), "-c",
                        os.path.join(HERE, "host_sanitizer_driver.cpp"), "-o", drv], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-fsanitize=address", "-fsanitize=undefined", "-fno-gpu-sanitize", "-rdynamic", "-o", exe, drv, api,
                        *objs], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    # (-rdynamic: the library finds its kernels' names among its exported symbols, which an executable only has with it)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    r = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and "OK (0 failures)" in r.stdout, (r.stdout[-1500:], r.stderr[-1500:])


def test_concurrent_callers_are_clean_under_tsan_and_agree(tmp_path):
    objs = [o for o in glob.glob(os.path.join(CSRC, "build", "*.o")) if not o.endswith("cascmm_api.o")]
    if not os.path.exists(HIPCC) or shutil.which("g++") is None or len(objs) < 5:
        pytest.skip("needs hipcc, g++ and the library's object files (python -m basedxl_amd.build)")
    api, drv, exe = str(tmp_path / "api_tsan.o"), str(tmp_path / "driver.o"), str(tmp_path / "driver")
    flags = ["-O1", "-g", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]
    r = subprocess.run([HIPCC, *flags, "-Xarch_host", "-fsanitize=thread", "-c", os.path.join(CSRC, "cascmm_api.hip"), "-o", api],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=thread", "-I", os.path.join(ROOT, "include"), "-c",
                        os.path.join(HERE, "host_threads_driver.cpp"), "-o", drv], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-fsanitize=thread", "-fno-gpu-sanitize", "-o", exe, drv, api, *objs],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    # every GPU is hidden from the driver: it walks the launch entry point with pointers that must never
    # reach a kernel, and the launchers must give up at their device query
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0 and "OK (0 failures" in r.stdout and "ThreadSanitizer" not in r.stderr, (r.stdout[-1500:], r.stderr[-1500:])
