"""Build libyvex_rocm.so: gfx950 HIP kernels + the C11 host layer, in-tree.

    python -m yvex_amd.build            # compile everything, link yvex_amd/libyvex_rocm.so

hipcc cross-compiles for gfx950 without a GPU. The C11 host sources are compiled with the
system C compiler and never include a HIP header; they reach the device only through the
launch-level C ABI in include/yvex_rocm_kernels.h.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libyvex_rocm.so")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
CC = os.environ.get("CC") or shutil.which("gcc") or "cc"

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fno-fast-math", "-Wall", "-Wno-unused-function",
    # keep the compiler from forming packed-FP32 instructions on its own
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
C_FLAGS = ["-std=c11", "-O2", "-fPIC", "-Wall", "-Wextra", "-ffp-contract=off", "-pthread",
           "-D_POSIX_C_SOURCE=200809L", f"-I{os.path.join(ROOT, 'include')}"]


def _sources():
    hip_dir, host_dir = os.path.join(CSRC, "hip"), os.path.join(CSRC, "host")
    hip = sorted(os.path.join(hip_dir, f) for f in os.listdir(hip_dir) if f.endswith(".hip"))
    host = sorted(os.path.join(host_dir, f) for f in os.listdir(host_dir) if f.endswith(".c")) \
        if os.path.isdir(host_dir) else []
    return hip, host


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + proc.stdout + proc.stderr)
    noise = "is not a recognized feature for this target"
    return "\n".join(l for l in proc.stderr.splitlines() if l.strip() and noise not in l)


def write_exports_map() -> str:
    """csrc/exports.map lists exactly the entry points the two public headers declare."""
    import re
    names = set()
    for header in ("yvex_rocm.h", "yvex_rocm_kernels.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(yvex_[a-z0-9_]+)\s*\(", text))
    lines = ["/* Everything libyvex_rocm.so exports: the entry points include/yvex_rocm.h (yvex_rocm_*)",
             " * and include/yvex_rocm_kernels.h (yvex_hip_*) declare. No name of the reference's own",
             " * libyvex is defined here, so both can live in one process or one link. */", "{", "  global:"]
    row = "   "
    for name in sorted(names):
        if len(row) + len(name) + 2 > 100:
            lines.append(row)
            row = "   "
        row += " " + name + ";"
    lines += [row, "  local: *;", "};", ""]
    path = os.path.join(CSRC, "exports.map")
    text = "\n".join(lines)
    if not os.path.exists(path) or open(path).read() != text:
        open(path, "w").write(text)
    return path


def build(verbose: bool = False, jobs: int | None = None) -> str:
    os.makedirs(OBJ, exist_ok=True)
    exports = write_exports_map()
    hip, host = _sources()
    tasks = []
    for src in hip:
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        tasks.append((obj, [HIPCC, *HIP_FLAGS, "-c", src, "-o", obj]))
    for src in host:
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        tasks.append((obj, [CC, *C_FLAGS, "-c", src, "-o", obj]))
    jobs = jobs or min(8, os.cpu_count() or 1, max(1, len(tasks)))
    with concurrent.futures.ThreadPoolExecutor(jobs) as pool:
        for warnings in pool.map(lambda t: _run(t[1]), tasks):
            if verbose and warnings:
                print(warnings, file=sys.stderr)
    objs = [t[0] for t in tasks]
    # only the declared entry points leave the library, and its own calls bind inside it
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-lm", "-lpthread",
          f"-Wl,--version-script={exports}", "-Wl,-Bsymbolic"])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
