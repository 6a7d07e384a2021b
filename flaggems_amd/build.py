"""Build recipe for libflaggems_amd.so (hipcc, gfx950 only).

    python -m flaggems_amd.build          # compile every .hip under csrc/ and link

The shared library is written next to this file (flaggems_amd/libflaggems_amd.so) so that it is
found in-tree; nothing is installed.  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libflaggems_amd.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep the compiler from forming packed-fp32 VALU instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results land in architectural VGPRs, where the scale FMAs can read them directly
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wall",
    # the global->LDS loads are written in assembly and name m0, which the compiler reports on every expansion
    "-Wno-inline-asm",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines() if "packed-fp32-ops" not in line and line.strip()
    )
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out and "warning" in out:
        print(out, flush=True)
    return out


FASTCALL_SRC = os.path.join(CSRC, "fastcall.c")


def fastcall_path() -> str:
    import sysconfig

    return os.path.join(HERE, "_fg_fastcall" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_fastcall(verbose: bool = True) -> str:
    """Compile the CPython argument-marshalling module (csrc/fastcall.c) with the host C compiler.  It links nothing
    of libflaggems_amd.so: the Python host hands it function addresses."""
    import sysconfig

    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        raise RuntimeError("no host C compiler (gcc / cc) for csrc/fastcall.c")
    out = fastcall_path()
    tmp = out + ".tmp"
    _run([cc, "-O2", "-shared", "-fPIC", "-Wall", "-I" + sysconfig.get_paths()["include"], FASTCALL_SRC, "-o", tmp])
    os.replace(tmp, out)
    if verbose:
        print("[flaggems_amd.build] built", out, flush=True)
    return out


def build(verbose: bool = True, jobs: int = 4) -> str:
    """Compile every HIP source for gfx950 and link the shared library.  Always recompiles."""
    hipcc = _hipcc()
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        out = _run([hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj])
        if verbose:
            print("[flaggems_amd.build] compiled", os.path.basename(src), flush=True)
        return out

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("[flaggems_amd.build] linked", LIB_PATH, flush=True)
    build_fastcall(verbose)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
