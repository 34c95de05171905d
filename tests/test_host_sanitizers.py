"""Host code of the path under AddressSanitizer and UndefinedBehaviorSanitizer (no GPU): the plan
arithmetic (`csrc/decode_plan.h`) with a serial restatement of the plan kernel's chunk-table writes,
the host index producers (`torch_shim/host_index.h`) and the argument checks of the libtorch
operators (`torch_shim/ops_api.cpp`), compiled with g++ into one executable and run once."""
import os
import subprocess

import pytest

from xllm_wxh_amd import build as xbuild

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(REPO, "xllm_wxh_amd", "csrc")


def test_host_code_runs_clean_under_asan_and_ubsan(tmp_path):
    import torch
    from torch.utils import cpp_extension as ce

    if not os.path.exists(xbuild.LIB_PATH):
        xbuild.build_library(verbose=False)
    exe = str(tmp_path / "host_sanitizer_harness")
    cmd = ["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-static-libasan", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-Wno-deprecated-declarations",
           "-I", CSRC]
    for inc in ce.include_paths() + [os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "include")]:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(REPO, "tests", "host_sanitizer_harness.cpp"), os.path.join(CSRC, "torch_shim", "ops_api.cpp")]
    # (ops_api.cpp calls the HIP runtime itself: events and pinned memory of the host-side plan's staging buffers)
    lib_dirs = ce.library_paths() + [xbuild.PKG_DIR, os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")]
    for d in lib_dirs:
        cmd += ["-L" + d, "-Wl,-rpath," + d]
    cmd += ["-l:" + xbuild.LIB_NAME, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-lamdhip64", "-o", exe]
    build = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert build.returncode == 0, build.stdout[-4000:]
    # libtorch keeps a few allocations for the life of the process; leak checking is not the point here
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=600)
    assert run.returncode == 0, run.stdout[-4000:]
    assert "sanitizer harness ok" in run.stdout
