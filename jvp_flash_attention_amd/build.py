"""Build ``libjvpfa.so`` (HIP kernels + C ABI) in-tree for gfx950 with hipcc.

``python -m jvp_flash_attention_amd.build`` compiles every translation unit (one per element
type x head dim for the forward and for the backward, plus the C ABI files) in parallel and
links them into ``jvp_flash_attention_amd/libjvpfa.so``.  hipcc cross-compiles, so no GPU is
needed to build.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libjvpfa.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wno-unused-value",
    # keep hipcc from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

TYPES = {"bf16": "__bf16", "fp16": "_Float16", "fp32": "float"}
DIMS = (32, 64, 128, 256)


def units():
    """(object name, source, extra defines) for every translation unit."""
    out = []
    for kind in ("fwd", "bwd"):
        src = os.path.join(CSRC, f"{kind}_inst.hip")
        if not os.path.exists(src):
            continue
        for tag, ctype in TYPES.items():
            for d in DIMS:
                name = f"{kind}_{tag}_{d}"
                out.append((name, src, [f"-DJVPFA_T={ctype}", f"-DJVPFA_D={d}", f"-DJVPFA_NAME={name}"]))
    for api in ("api_fwd", "api_bwd", "mask_tiles"):
        src = os.path.join(CSRC, f"{api}.hip")
        if os.path.exists(src):
            out.append((api, src, []))
    return out


def isa_path(name: str, objdir: str = OBJ) -> str:
    """Where ``build()`` leaves the device ISA text of a translation unit."""
    return os.path.join(objdir, name, name + ".s")


def _compile(unit):
    name, src, defs, objdir, extra = unit
    # a directory per unit: the compiler names its intermediate files after the source, and several
    # units share one source
    udir = os.path.join(objdir, name)
    os.makedirs(udir, exist_ok=True)
    obj = os.path.join(udir, name + ".o")
    cmd = [HIPCC, *FLAGS, *extra, *defs, "-save-temps=obj", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {name}:\n{' '.join(cmd)}\n{r.stderr[-4000:]}")
    # of the intermediate files keep the device ISA text (the asm lint reads it)
    isa = isa_path(name, objdir)
    for f in os.listdir(udir):
        if f.endswith(".s") and "-hip-amdgcn-" in f:
            os.replace(os.path.join(udir, f), isa)
    for f in os.listdir(udir):
        path = os.path.join(udir, f)
        if path not in (obj, isa):
            os.remove(path)
    return obj


def build(jobs: int | None = None, verbose: bool = True, extra_flags=(), lib: str = LIB, objdir: str = OBJ) -> str:
    """Compile and link.  ``extra_flags`` / ``lib`` / ``objdir`` build a variant next to the default
    library (e.g. a build with an extra ``-D`` flag, to compare two versions of a kernel on the same box)."""
    os.makedirs(objdir, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    us = [(*u, objdir, list(extra_flags)) for u in units()]

    # the units that take longest (the 16-bit backward kernels, most template variants) start first, so that the
    # build ends with short ones filling the remaining cores; the link order stays that of units()
    def cost(u):
        name = u[0]
        return -(4 * name.startswith("bwd_") + 2 * ("fp32" not in name) + ("256" not in name))

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        done = dict(zip((u[0] for u in sorted(us, key=cost)), ex.map(_compile, sorted(us, key=cost))))
    objs = [done[u[0]] for u in us]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", lib]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {lib} from {len(objs)} objects", flush=True)
    # the inline-asm matrix instructions of every kernel unit must carry the idle issue slots the
    # compiler cannot add for them (see asm_lint.py); a finding fails the build
    from . import asm_lint

    findings = []
    for name, _src, _defs, *_ in us:
        if name.startswith(("fwd_", "bwd_")):
            with open(isa_path(name, objdir)) as f:
                findings += asm_lint.scan(f.read(), name)
    if findings:
        raise RuntimeError("asm lint:\n" + "\n".join(findings))
    if verbose:
        print("asm lint: clean", flush=True)
    if lib == LIB:
        build_host_check(verbose)
    return lib


HOST_CHECK_SRC = os.path.join(os.path.dirname(HERE), "tests", "cabi_host", "host_check.cpp")
HOST_CHECK_BIN = os.path.join(os.path.dirname(HERE), "tests", "cabi_host", "host_check")


def build_host_check(verbose: bool = True) -> str | None:
    """The plain C++ caller of the C ABI used by the GPU tests (no Python, no torch in the process):
    compiled against ``include/jvpfa.h`` and linked with the library just built."""
    if not os.path.exists(HOST_CHECK_SRC):
        return None
    cmd = [HIPCC, "-O2", "-std=c++17", "-x", "hip", "--offload-arch=gfx950", "-I", os.path.join(os.path.dirname(HERE), "include"),
           HOST_CHECK_SRC, "-o", HOST_CHECK_BIN, "-L", HERE, "-ljvpfa", "-Wl,-rpath,$ORIGIN/../../jvp_flash_attention_amd"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for the host check:\n{' '.join(cmd)}\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {HOST_CHECK_BIN}", flush=True)
    return HOST_CHECK_BIN


if __name__ == "__main__":
    build()
    sys.exit(0)
