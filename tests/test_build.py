"""What the compiler makes of the kernels, where the kernels' correctness hangs on it."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_product_for_65_to_128_rows_spills_no_register(tmp_path):
    """gemm_mid.hip fills registers by load instructions that the compiler does not see, and waits
    for them by count.  A register that the compiler spilled to memory before its load arrived
    would be saved with its old contents: no form of the kernel may spill."""
    from libllm_amd.hip import build
    hipcc = build._hipcc()
    if hipcc is None:
        pytest.skip("hipcc not found")
    src = os.path.join(build.CSRC, "gemm_mid.hip")
    proc = subprocess.run([hipcc] + build.FLAGS + ["-I", build.CSRC, "-c", src, "-o", str(tmp_path / "m.o"),
                                                    "-Rpass-analysis=kernel-resource-usage"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0 and build.OPTIONAL_FLAGS[-1].split("=")[0].lstrip("-") in proc.stdout:
        pytest.skip("this hipcc does not know %s" % build.OPTIONAL_FLAGS[-1])
    assert proc.returncode == 0, proc.stdout[-2000:]
    names = re.findall(r"Function Name: (\S+)", proc.stdout)
    spills = [int(n) for n in re.findall(r"VGPRs Spill: (\d+)", proc.stdout)]
    kernels = [n for n in names if "gemm_mid_kernel" in n]
    assert len(kernels) >= 12 and len(spills) == len(names)
    assert all(s == 0 for n, s in zip(names, spills) if "gemm_mid_kernel" in n), list(zip(names, spills))
