"""Build librswa.so (HIP, gfx950 only) in-tree with hipcc.

Usage: ``python build.py [--force]``.  Objects go to ``build/``, the shared
library to ``lib/librswa.so`` next to this file.  hipcc cross-compiles, so no
GPU is needed to build.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import re
import shutil
import subprocess
import sys
from typing import List

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "librswa.so")
# the same library with every MFMA issued through the compiler builtin (hazards padded by the
# compiler): the cross-check of the hand-kept hazard distance of the inline-assembly MFMAs
LIB_BUILTIN_MFMA = os.path.join(LIBDIR, "librswa_builtin_mfma.so")
ASM_MFMA_SOURCES = ("attn_bwd.hip",)  # sources that issue MFMAs as inline assembly

ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-attributes",
    # packed fp32 VALU forms are kept out of generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # per-kernel register / scratch report on stderr (checked below)
    "-Rpass-analysis=kernel-resource-usage",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> List[str]:
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(os.path.dirname(HERE), "include", "rswa.h"))
    return hs


def _stale(target: str, deps: List[str]) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src: str, force: bool, builtin_mfma: bool = False) -> str:
    stem = os.path.basename(src)[:-4]
    obj = os.path.join(OBJ, stem + (".builtin_mfma.o" if builtin_mfma else ".o"))
    if force or _stale(obj, [src] + _headers()):
        extra = ["-DRSWA_MFMA_BUILTIN_ONLY"] if builtin_mfma else []
        cmd = [_hipcc(), *FLAGS, *extra, "-c", src, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
        if not builtin_mfma:  # the cross-check build may spill: it is never timed
            _check_no_scratch(src, r.stderr)
            warn = _real_warnings(r.stderr)
            if warn:
                sys.stderr.write(warn + "\n")
    return obj


def _real_warnings(stderr: str) -> str:
    """Compiler output minus the resource-usage remarks (each followed by a source line and
    a caret line) and the host pass's note about the device-only target feature."""
    out, skip = [], 0
    for line in stderr.splitlines():
        if skip:
            skip -= 1
            continue
        if "-Rpass-analysis=kernel-resource-usage" in line:
            skip = 2 if "Function Name" in line else 0
            continue
        if "packed-fp32-ops" in line or not line.strip():
            continue
        out.append(line)
    return "\n".join(out)


def _check_no_scratch(src: str, stderr: str) -> None:
    """No kernel may use scratch memory: a register spilled inside a tile loop comes back
    through a load whose wait also waits for every tile load in flight."""
    name, bad = None, []
    for line in stderr.splitlines():
        m = re.search(r"remark:\s+(.*?): (.*?) \[-Rpass-analysis=kernel-resource-usage\]", line)
        if not m:
            continue
        key, val = m.group(1).strip(), m.group(2).strip()
        if key == "Function Name":
            name = val
        elif key.startswith("ScratchSize") and val != "0":
            bad.append(f"{name}: {val} bytes of scratch per lane")
    if bad:
        raise RuntimeError(f"{src}: kernels spill registers to scratch memory:\n  " + "\n  ".join(bad))


def build(force: bool = False, jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = sources()
    asm_srcs = [s for s in srcs if os.path.basename(s) in ASM_MFMA_SOURCES]
    with cf.ThreadPoolExecutor(max_workers=min(jobs, len(srcs) + len(asm_srcs))) as ex:
        futs = [ex.submit(_compile, s, force) for s in srcs]
        alt_futs = {s: ex.submit(_compile, s, force, True) for s in asm_srcs}
        objs = [f.result() for f in futs]
        alt = {s: f.result() for s, f in alt_futs.items()}
    alt_objs = [alt.get(s, o) for s, o in zip(srcs, objs)]
    for lib, members in ((LIB, objs), (LIB_BUILTIN_MFMA, alt_objs)):
        if force or _stale(lib, members):
            cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", lib, *members]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
