"""Builds oracle/libdlgrad_cpu_ref.so from dlgrad_cpu_kernels.c (test infrastructure).

Flags and compiler choice are the reference's (dlgrad/runtime/cpu.py:30-41):
clang if on PATH else gcc, -shared -fPIC -O3 -march=native -ffast-math -Werror,
-lm -lmvec.  Because of -march=native the library is tied to the CPU it was built
on: a sidecar file records that CPU's model and feature flags, and `ensure()`
rebuilds when the library is missing or was built for a different CPU.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "dlgrad_cpu_kernels.c")
LIB = os.path.join(HERE, "libdlgrad_cpu_ref.so")
STAMP = LIB + ".cpu"
CFLAGS = ["-shared", "-fPIC", "-O3", "-march=native", "-ffast-math", "-Werror"]
EXTRA_LIBS = ["-lm", "-lmvec"]


def compiler() -> str:
    cc = shutil.which("clang") or shutil.which("gcc")
    if cc is None:
        raise RuntimeError("Clang or GCC not found")
    return cc


def cpu_signature() -> str:
    model, flags = "", ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name") and not model:
                    model = line.split(":", 1)[1].strip()
                elif line.startswith("flags") and not flags:
                    flags = line.split(":", 1)[1].strip()
                if model and flags:
                    break
    except OSError:
        pass
    src = hashlib.sha256(open(SRC, "rb").read()).hexdigest()[:16]
    return f"{model}|{hashlib.sha256(flags.encode()).hexdigest()[:16]}|{os.path.basename(compiler())}|{src}"


def build() -> str:
    cmd = [compiler(), *CFLAGS, "-o", LIB, SRC, *EXTRA_LIBS]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"Compilation failed:\n{res.stderr}")
    with open(STAMP, "w") as f:
        f.write(cpu_signature())
    return LIB


def ensure() -> str:
    """Path of a library that matches this CPU and this source, building if needed."""
    try:
        ok = os.path.exists(LIB) and open(STAMP).read() == cpu_signature()
    except OSError:
        ok = False
    return LIB if ok else build()


if __name__ == "__main__":
    print(build())
