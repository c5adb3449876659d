"""What the compiler makes of the kernels, where the kernels' correctness hangs on it."""
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

REPORT = """
remark: x.hip:1:0: Function Name: _Z15gemm_mid_kernelILi0ELi2EEvPKv [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     SGPRs: 40 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0: Function Name: _Z15gemm_mid_kernelILi1ELi2EEvPKv [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     ScratchSize [bytes/lane]: 24 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     VGPRs Spill: 6 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0: Function Name: _Z11other_thingv [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     ScratchSize [bytes/lane]: 8 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     VGPRs Spill: 2 [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0: Function Name: _Z15gemm_mid_kernelILi2ELi2EEvPKv [-Rpass-analysis=kernel-resource-usage]
remark: x.hip:1:0:     VGPRs: 99 [-Rpass-analysis=kernel-resource-usage]
"""


def test_the_report_of_spills_is_read():
    """A form that spills, one that does not, a kernel of another name, and a form whose report
    lacks the figures (counted as spilling)."""
    from libllm_amd.hip import build
    kernels, bad = build.spills_in_report(REPORT, "gemm_mid_kernel")
    assert kernels == 3
    assert bad == ["_Z15gemm_mid_kernelILi1ELi2EEvPKv", "_Z15gemm_mid_kernelILi2ELi2EEvPKv"]
    assert build.spills_in_report("", "gemm_mid_kernel") == (0, [])


def test_the_build_records_that_the_product_for_33_to_128_rows_spills_no_register(tmp_path):
    """gemm_mid.hip fills registers by load instructions that the compiler does not see, and waits
    for them by count.  A register that the compiler spilled to memory before its load arrived
    would be saved with its old contents.  The build itself reads the compiler's report, with the
    flags it really used, and records what it found beside the library; the host does not use the
    kernel if any form spills.  Here: the record of the build that the tests load names all forms
    and no spill (with this image's compiler), and a record with a spill switches the kernel off."""
    from libllm_amd.hip import build
    if build._hipcc() is None and not any(build._current(d, build.source_hash()) for d in build._lib_dirs()):
        pytest.skip("neither a current build nor hipcc")
    path = build.build(force=False)
    found = build.info(path)
    assert found["hash"] == build.source_hash()
    mid = found["no_spill"]["gemm_mid.hip"]
    assert mid["kernels"] >= 12 and mid["spilling"] == []
    assert build.trusted("gemm_mid.hip", path)
    # a build whose compiler spilled one form
    import json
    import shutil
    other = tmp_path / "lib"
    other.mkdir()
    shutil.copy(os.path.join(os.path.dirname(path), build.INFO_NAME), other / build.INFO_NAME)
    found["no_spill"]["gemm_mid.hip"]["spilling"] = ["_Z15gemm_mid_kernelILi1ELi2EEvPKv"]
    (other / build.INFO_NAME).write_text(json.dumps(found))
    assert not build.trusted("gemm_mid.hip", str(other / build.LIB_NAME))
    found["no_spill"] = {}
    (other / build.INFO_NAME).write_text(json.dumps(found))
    assert not build.trusted("gemm_mid.hip", str(other / build.LIB_NAME))


def test_two_processes_that_find_nothing_built_build_once(tmp_path, monkeypatch):
    """Two callers that find no library at the same moment (two programs started together in a
    fresh checkout): one compiles, the other waits for it and takes what it built, instead of
    both writing the same object files."""
    import json
    import threading
    import time
    from libllm_amd.hip import build
    target = str(tmp_path / "lib")
    calls = []

    def slow_build(folder, hipcc, want, verbose):
        calls.append(folder)
        time.sleep(0.4)
        for name, text in ((build.LIB_NAME, ""), (build.INFO_NAME, json.dumps({"hash": want})),
                           (build.LIB_NAME + ".hash", want)):
            with open(os.path.join(folder, name), "w") as f:
                f.write(text)
        return os.path.join(folder, build.LIB_NAME)

    monkeypatch.setattr(build, "_lib_dirs", lambda: [target])
    monkeypatch.setattr(build, "_hipcc", lambda: "/bin/true")
    monkeypatch.setattr(build, "_build_into", slow_build)
    got = []
    threads = [threading.Thread(target=lambda: got.append(build.build(force=False, verbose=False))) for _ in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert got == [os.path.join(target, build.LIB_NAME)] * 2 and len(calls) == 1
    assert build.build(force=False, verbose=False) == got[0] and len(calls) == 1      # and it stays built
