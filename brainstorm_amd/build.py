"""Builds libbship.so (the HIP kernels and their C ABI) for gfx950 with hipcc.

The library is built in-tree, next to this file, so that a built copy travels
with the source tree. Run ``python -m brainstorm_amd.build`` or call
:func:`build_lib`.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libbship.so")

ARCH = "gfx950"

# -ffp-contract=off: NumPy rounds every temporary to float32, so a*b+c must not
#   become a fused multiply-add.
# -packed-fp32-ops is switched off: hipcc must not form v_pk_*_f32 instructions.
HIPCC_FLAGS = [
    "--offload-arch=" + ARCH,
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]
LINK_LIBS = ["-lhipblaslt"]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile_one(hipcc: str, src: str, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    extra = os.environ.get("BSHIP_EXTRA_HIPCC_FLAGS", "").split()   # e.g. -DNAME=VALUE for experiments
    cmd = [hipcc] + HIPCC_FLAGS + extra + ["-c", src, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(
        line for line in (res.stdout + res.stderr).splitlines()
        # the host pass does not know the device-only target feature; harmless
        if "packed-fp32-ops" not in line
    )
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    if out.strip() and verbose:
        print(out, flush=True)
    return obj


def build_lib(verbose: bool = False, jobs: int | None = None) -> str:
    """Compiles every csrc/*.hip for gfx950 and links libbship.so. Always recompiles."""
    hipcc = hipcc_path()
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(8, os.cpu_count() or 1)))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile_one(hipcc, s, verbose), srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs + LINK_LIBS
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("linking libbship.so failed:\n" + res.stdout + res.stderr)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def fastcall_path() -> str:
    import sysconfig
    return os.path.join(HERE, "_fastcall" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_fastcall(verbose: bool = False) -> str:
    """Compiles csrc/fastcall.c, the CPython extension through which the handler calls the hottest
    entry points of the C ABI without ctypes' per-argument conversions (plain C, gcc)."""
    import sysconfig
    out = fastcall_path()
    cc = os.environ.get("CC") or shutil.which("gcc") or shutil.which("cc")
    if not cc:
        raise RuntimeError("no C compiler found for brainstorm_amd/csrc/fastcall.c")
    cmd = [cc, "-O2", "-Wall", "-shared", "-fPIC", "-I" + sysconfig.get_paths()["include"],
           os.path.join(CSRC, "fastcall.c"), "-o", out + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building the _fastcall extension failed:\n" + res.stdout + res.stderr)
    os.replace(out + ".tmp", out)
    return out


if __name__ == "__main__":
    path = build_lib(verbose="-v" in sys.argv)
    print("built", path)
    print("built", build_fastcall(verbose="-v" in sys.argv))
