"""No kernel of the library uses scratch memory (register spills or stack arrays): every HIP source is
compiled for gfx950 with -Rpass-analysis=kernel-resource-usage and the remarks are read back.  A
spill inside the token loop of an attention kernel costs memory round trips on the critical path, and
a kernel with a scratch segment makes the runtime reserve scratch memory for its queue."""
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

from xllm_wxh_amd import build as xbuild


def _remarks(source):
    flags = [f for f in xbuild.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [xbuild.hipcc_path()] + flags + ["--cuda-device-only", "-c", os.path.join(xbuild.CSRC_DIR, source),
                                           "-o", os.devnull, "-Rpass-analysis=kernel-resource-usage"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-3000:]
    return proc.stdout


def test_no_kernel_uses_scratch_memory():
    with ThreadPoolExecutor(max_workers=4) as pool:
        outputs = list(pool.map(_remarks, xbuild.HIP_SOURCES))
    kernels = {}
    for text in outputs:
        name = None
        for line in text.splitlines():
            m = re.search(r"Function Name: (\S+)", line)
            if m:
                name = m.group(1)
            m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
            if m and name:
                kernels[name] = int(m.group(1))
    # the decode kernels alone are 58 instantiations
    assert len(kernels) >= 70, len(kernels)
    assert any("decode_mfma_d128_rows32_kernel" in k for k in kernels)
    spilling = {k: v for k, v in kernels.items() if v != 0}
    assert not spilling, spilling
