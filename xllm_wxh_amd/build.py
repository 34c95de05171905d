"""Build recipe of the gfx950 shared library behind the C ABI.

`build_library()` compiles the HIP sources in `csrc/` with explicit hipcc lines
and leaves `libxllm_hip_paged_kv.so` beside this file, where the loader in
`_lib.py` looks for it.  Intermediate files go to `<repo>/build/`.
"""
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libxllm_hip_paged_kv.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

HIP_SOURCES = ["kv_write.hip", "block_move.hip", "gather_from_cache.hip", "rope_kv_write.hip", "paged_decode.hip", "c_abi_misc.hip"]

# -packed-fp32-ops is switched off: the compiler then never forms v_pk_*_f32.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


def _run(cmd, verbose):
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that is expected.
    lines = [l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l]
    if proc.returncode != 0:
        raise RuntimeError("%s failed:\n%s" % (cmd[0], "\n".join(lines)))
    if verbose and lines:
        print("\n".join(lines))


def build_library(verbose=True, save_temps=False, extra_flags=()):
    """Compile every HIP source for gfx950 (one hipcc process per source, side by side) and link
    them into LIB_PATH; raises on failure."""
    from concurrent.futures import ThreadPoolExecutor

    build_dir = os.path.join(REPO_DIR, "build")
    os.makedirs(build_dir, exist_ok=True)
    tmp_out = os.path.join(build_dir, LIB_NAME)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"] + list(extra_flags)
    if save_temps:
        compile_flags.append("-save-temps=obj")
    objects = [os.path.join(build_dir, os.path.splitext(s)[0] + ".o") for s in HIP_SOURCES]
    jobs = [[hipcc_path()] + compile_flags + ["-c", os.path.join(CSRC_DIR, s), "-o", o]
            for s, o in zip(HIP_SOURCES, objects)]
    with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
        for fut in [pool.submit(_run, cmd, verbose) for cmd in jobs]:
            fut.result()
    _run([hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC"] + objects + ["-o", tmp_out], verbose)
    os.replace(tmp_out, LIB_PATH)
    return LIB_PATH


TORCH_SHIM_NAME = "_xllm_hip_torch.so"
TORCH_SHIM_PATH = os.path.join(PKG_DIR, TORCH_SHIM_NAME)
TORCH_SHIM_SOURCES = ["ops_api.cpp", "attention.cpp", "pybind.cpp"]


def build_torch_shim(verbose=True):
    """Compile the libtorch host side (xllm::kernel / xllm::layer mirrors + pybind module) with g++.
    Host code only: it reaches the GPU through the C ABI of LIB_PATH, which must exist."""
    import sysconfig

    import pybind11
    import torch
    from torch.utils import cpp_extension as ce

    if not os.path.exists(LIB_PATH):
        build_library(verbose=verbose)
    build_dir = os.path.join(REPO_DIR, "build")
    os.makedirs(build_dir, exist_ok=True)
    shim_dir = os.path.join(CSRC_DIR, "torch_shim")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    tmp_out = os.path.join(build_dir, TORCH_SHIM_NAME)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=_xllm_hip_torch",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-Wno-deprecated-declarations"]
    for inc in ce.include_paths() + [pybind11.get_include(), sysconfig.get_paths()["include"],
                                      os.path.join(rocm, "include")]:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(shim_dir, s) for s in TORCH_SHIM_SOURCES]
    for lib_dir in ce.library_paths():
        cmd += ["-L" + lib_dir, "-Wl,-rpath," + lib_dir]
    cmd += ["-L" + PKG_DIR, "-Wl,-rpath,$ORIGIN", "-l:" + LIB_NAME, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch",
            "-ltorch_python", "-o", tmp_out]
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("g++ failed:\n" + proc.stdout)
    os.replace(tmp_out, TORCH_SHIM_PATH)
    return TORCH_SHIM_PATH


if __name__ == "__main__":
    build_library(save_temps="--save-temps" in sys.argv)
    print(LIB_PATH)
    if "--no-shim" not in sys.argv:
        print(build_torch_shim())
