"""Building and loading the HIP kernels: one shared library, compiled with hipcc for gfx950.

The library lives beside the sources (``libllm_amd/_lib``); if that folder cannot be written, a
per-user folder under the system's temporary directory is used.  A stored hash of the sources
decides whether what is built is current.  Nothing here falls back to another implementation: if
the library cannot be loaded or built, KernelError says why.
"""
import ctypes
import fcntl
import hashlib
import json
import os
import re
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

from ..errors import KernelError

ARCH = "gfx950"
_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
LIB_NAME = "libllm_amd_hip.so"
# Packed FP32 instructions stay switched off for every kernel of this library.  The sums of the
# matrix cores stay in ordinary vector registers (gfx950 has one register file for both kinds):
# left to itself the compiler keeps them in accumulation registers and moves them out and back
# for every other instruction that touches them, two moves a value and page in the attention
# kernels, where instruction issue is what bounds the time.
OPTIONAL_FLAGS = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]    # left out for a compiler that does not know the switch
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"] + OPTIONAL_FLAGS
# Every source is compiled with the compiler's report of what each kernel uses.  It is read for
# the kernels that are only right if the compiler spills none of their registers (they fill
# registers by load instructions that the compiler does not see and wait for them by count: a
# register saved to memory before its load arrived would be saved with its old contents).  What
# is found goes into a file beside the library, and the host switches such a kernel off if any
# of its forms spills: the property belongs to the build that runs, whichever flags it took.
REPORT_FLAGS = ["-Rpass-analysis=kernel-resource-usage"]
NO_SPILL_KERNELS = {"gemm_mid.hip": "gemm_mid_kernel"}     # source -> name that its kernels' symbols contain
INFO_NAME = "libllm_amd_hip.so.json"
_FORMAT = "build-info-1"                                   # part of the hash: a build without the file is not current

_lib: Optional[ctypes.CDLL] = None


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    for path in sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC)
                       if f.endswith((".hip", ".h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS + REPORT_FLAGS + [_FORMAT]).encode())
    return h.hexdigest()[:20]


def spills_in_report(report: str, name_part: str):
    """From the compiler's resource report: (number of kernels whose symbol contains
    ``name_part``, the symbols among them that spill a vector or scalar register or use scratch
    memory).  A report that does not give a kernel's spills counts that kernel as spilling."""
    kernels, bad = 0, []
    for block in report.split("Function Name: ")[1:]:
        name = block.split()[0]
        if name_part not in name:
            continue
        kernels += 1
        found = {key: re.search(key + r"[^:\n]*: (\d+)", block) for key in ("VGPRs Spill", "SGPRs Spill", "ScratchSize")}
        if any(m is None or int(m.group(1)) != 0 for m in found.values()):
            bad.append(name)
    return kernels, bad


def _say(msg: str) -> None:
    print("[libllm_amd] " + msg, file=sys.stderr, flush=True)


def _hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"),
                 os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if cand and os.path.isfile(cand):
            return cand
    return None


def _lib_dirs() -> List[str]:
    in_tree = os.path.join(os.path.dirname(_HERE), "_lib")
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [in_tree, os.path.join(tempfile.gettempdir(), "libllm_amd-%d" % uid)]


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, ".probe-%d" % os.getpid())
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _current(d: str, want: str) -> bool:
    so, stamp = os.path.join(d, LIB_NAME), os.path.join(d, LIB_NAME + ".hash")
    if not (os.path.isfile(so) and os.path.isfile(stamp) and os.path.isfile(os.path.join(d, INFO_NAME))):
        return False
    with open(stamp, "r") as f:
        return f.read().strip() == want


def build(force: bool = True, verbose: bool = True) -> str:
    """Compiles every kernel source and links the library; returns its path."""
    want = source_hash()
    if not force:
        for d in _lib_dirs():
            if _current(d, want):
                return os.path.join(d, LIB_NAME)
    hipcc = _hipcc()
    if hipcc is None:
        raise KernelError("the HIP kernels are not built and hipcc was not found (looked at $HIPCC, "
                          "PATH and $ROCM_PATH/bin)")
    target = next((d for d in _lib_dirs() if _writable(d)), None)
    if target is None:
        raise KernelError("no writable folder for the kernel library (tried %s)" % ", ".join(_lib_dirs()))
    # one build at a time in a folder: a second process waits, and takes what the first has built
    with open(os.path.join(target, ".build.lock"), "w") as lock:
        try:
            fcntl.flock(lock, fcntl.LOCK_EX | fcntl.LOCK_NB)
        except OSError:
            if verbose:
                _say("another process is building the kernels in %s: waiting for it" % target)
            fcntl.flock(lock, fcntl.LOCK_EX)
        if not force and _current(target, want):
            return os.path.join(target, LIB_NAME)
        return _build_into(target, hipcc, want, verbose)


def _build_into(target: str, hipcc: str, want: str, verbose: bool) -> str:
    objdir = os.path.join(target, "obj")
    os.makedirs(objdir, exist_ok=True)
    srcs = sources()
    t0 = time.time()
    if verbose:
        _say("compiling %d HIP sources for %s into %s" % (len(srcs), ARCH, target))

    info = {"hash": want, "optional_flags": True, "no_spill": {}}

    def compile_one(src):
        base = os.path.basename(src)
        obj = os.path.join(objdir, base[:-4] + ".o")
        cmd = [hipcc] + FLAGS + REPORT_FLAGS + ["-I", CSRC, "-c", src, "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0 and OPTIONAL_FLAGS[-1].split("=")[0].lstrip("-") in proc.stdout:
            if verbose:
                _say("  this hipcc does not know %s: compiling %s without it (the attention kernels "
                     "run somewhat slower)" % (OPTIONAL_FLAGS[-1], base))
            info["optional_flags"] = False
            cmd = [hipcc] + FLAGS[:-len(OPTIONAL_FLAGS)] + REPORT_FLAGS + ["-I", CSRC, "-c", src, "-o", obj]
            proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise KernelError("hipcc failed on %s:\n%s" % (base, proc.stdout[-4000:]))
        if base in NO_SPILL_KERNELS:
            kernels, bad = spills_in_report(proc.stdout, NO_SPILL_KERNELS[base])
            info["no_spill"][base] = {"kernels": kernels, "spilling": bad}
            if verbose and (bad or not kernels):
                _say("  %s: %s; the host will not use these kernels"
                     % (base, "%d of %d forms spill registers" % (len(bad), kernels) if kernels
                        else "the compiler's report names no kernel"))
        if verbose:
            _say("  compiled %s (%.0f s since start)" % (base, time.time() - t0))
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp_so = os.path.join(target, LIB_NAME + ".tmp-%d" % os.getpid())
    cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp_so] + objs
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise KernelError("linking the kernel library failed:\n%s" % proc.stdout[-4000:])
    os.replace(tmp_so, os.path.join(target, LIB_NAME))
    with open(os.path.join(target, INFO_NAME), "w") as f:
        json.dump(info, f, indent=1)
    with open(os.path.join(target, LIB_NAME + ".hash"), "w") as f:
        f.write(want)
    if verbose:
        _say("built %s in %.0f s" % (LIB_NAME, time.time() - t0))
    return os.path.join(target, LIB_NAME)


def info(path: Optional[str] = None) -> dict:
    """What the build that made the library at ``path`` (default: the one ``load`` takes) found."""
    path = path or build(force=False)
    with open(os.path.join(os.path.dirname(path), INFO_NAME), "r") as f:
        return json.load(f)


def trusted(source: str, path: Optional[str] = None) -> bool:
    """Whether the kernels of ``source`` (a key of NO_SPILL_KERNELS) may run: the build found
    them, and none of their forms spills."""
    found = info(path).get("no_spill", {}).get(source)
    return bool(found) and found["kernels"] > 0 and not found["spilling"]


CAPI_NAME = "libllm.so"
CLI_NAME = "llm"                 # the command line over the C API, beside the library


def build_capi(force: bool = True, verbose: bool = True) -> str:
    """Compiles the C API (csrc/capi: host code only, against this interpreter's headers and
    library) and the ``llm`` program over it; returns the path of libllm.so (the program lies
    beside it)."""
    import sysconfig
    src = os.path.join(CSRC, "capi", "llm_capi.cc")
    h = hashlib.sha256()
    main_src = os.path.join(CSRC, "capi", "llm_main.cc")
    for path in (src, os.path.join(CSRC, "capi", "llm.h"), main_src):
        with open(path, "rb") as f:
            h.update(f.read())
    want = h.hexdigest()[:20]
    for d in _lib_dirs():
        so, stamp = os.path.join(d, CAPI_NAME), os.path.join(d, CAPI_NAME + ".hash")
        if (not force and os.path.isfile(so) and os.path.isfile(os.path.join(d, CLI_NAME))
                and os.path.isfile(stamp) and open(stamp).read().strip() == want):
            return so
    cxx = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++") or _hipcc()
    if cxx is None:
        raise KernelError("the C API is not built and no C++ compiler was found")
    target = next((d for d in _lib_dirs() if _writable(d)), None)
    if target is None:
        raise KernelError("no writable folder for the C API library (tried %s)" % ", ".join(_lib_dirs()))
    root = os.path.dirname(os.path.dirname(_HERE))
    libdir = sysconfig.get_config_var("LIBDIR") or "/usr/lib"
    pylib = "python" + sysconfig.get_config_var("LDVERSION")
    tmp_so = os.path.join(target, CAPI_NAME + ".tmp-%d" % os.getpid())
    cmd = [cxx, "-O2", "-fPIC", "-shared", "-std=c++17", "-I", sysconfig.get_paths()["include"],
           "-DLIBLLM_AMD_ROOT=\"%s\"" % root, src, "-o", tmp_so,
           "-L", libdir, "-Wl,-rpath," + libdir, "-l" + pylib, "-ldl"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise KernelError("compiling the C API failed:\n%s" % proc.stdout[-4000:])
    os.replace(tmp_so, os.path.join(target, CAPI_NAME))
    tmp_exe = os.path.join(target, CLI_NAME + ".tmp-%d" % os.getpid())
    cmd = [cxx, "-O2", "-std=c++17", "-I", os.path.join(CSRC, "capi"), main_src, "-o", tmp_exe,
           os.path.join(target, CAPI_NAME), "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + libdir]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise KernelError("compiling the llm program failed:\n%s" % proc.stdout[-4000:])
    os.replace(tmp_exe, os.path.join(target, CLI_NAME))
    with open(os.path.join(target, CAPI_NAME + ".hash"), "w") as f:
        f.write(want)
    if verbose:
        _say("built %s" % CAPI_NAME)
    return os.path.join(target, CAPI_NAME)


def load() -> ctypes.CDLL:
    """The kernel library; built first if no current build exists."""
    global _lib
    if _lib is None:
        path = build(force=False)
        try:
            _lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError("cannot load %s: %s" % (path, e))
    return _lib
