"""Build libmi355gq.so (gfx950 code only) with hipcc, in tree.

    python mlc-llm_amd/build.py            # compile every csrc/*.hip and link lib/libmi355gq.so

The TVM-FFI adapter (csrc/tvm_ffi_adapter.cc) is compiled in only when the
`tvm_ffi` Python package (which ships tvm/ffi/c_api.h) is importable.
"""

from __future__ import annotations

import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "libmi355gq.so")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-fno-fast-math",
    # no implicit a*b+c fusion: fp16 rounding points are part of the contract (explicit fma where wanted)
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # packed-FP32 VALU forms are kept out of every code object
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the leading scalar arguments of a kernel (up to 14 dwords on gfx950) arrive in SGPRs with the wave instead of
    # through a memory read at its start; firmware without the feature enters a prologue that loads them
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-attributes",
]


def _tvm_ffi_include() -> str | None:
    try:
        import tvm_ffi  # type: ignore

        inc = os.path.join(os.path.dirname(tvm_ffi.__file__), "include")
        return inc if os.path.exists(os.path.join(inc, "tvm", "ffi", "c_api.h")) else None
    except Exception:
        return None


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    extra: list[str] = []
    link_extra: list[str] = []
    ffi_inc = _tvm_ffi_include()
    adapter = os.path.join(CSRC, "tvm_ffi_adapter.cc")
    jobs = [(s, extra) for s in srcs]
    if ffi_inc and os.path.exists(adapter):
        jobs.append((adapter, ["-x", "hip", f"-I{ffi_inc}"]))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        objs = list(ex.map(lambda a: _compile(*a), jobs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, *link_extra]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(objs)} objects" + (" (+tvm_ffi adapter)" if ffi_inc else ""))
    return LIB


if __name__ == "__main__":
    build()
