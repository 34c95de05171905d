"""Build recipe of the gfx950 shared library behind the C ABI.

`build_library()` runs one explicit hipcc line over the HIP sources in `csrc/`
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

HIP_SOURCES = ["kv_write.hip", "paged_decode.hip", "c_abi_misc.hip"]

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


def build_library(verbose=True, save_temps=False):
    """Compile every HIP source for gfx950 into LIB_PATH; raises on failure."""
    build_dir = os.path.join(REPO_DIR, "build")
    os.makedirs(build_dir, exist_ok=True)
    tmp_out = os.path.join(build_dir, LIB_NAME)
    cmd = [hipcc_path()] + HIPCC_FLAGS
    if save_temps:
        cmd.append("-save-temps=obj")
    cmd += [os.path.join(CSRC_DIR, s) for s in HIP_SOURCES] + ["-o", tmp_out]
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that is expected.
    lines = [l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l]
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + "\n".join(lines))
    if verbose and lines:
        print("\n".join(lines))
    os.replace(tmp_out, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build_library(save_temps="--save-temps" in sys.argv)
    print(LIB_PATH)
