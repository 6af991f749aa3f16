"""Builds libgla_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m gla_jax_amd.build            # compile every csrc/*.hip and link
"""
from __future__ import annotations

import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libgla_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU ops are switched off for all device code (some of their forms have produced
# silently wrong results on the target machines)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(HERE, "..", "include")]


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, "build", os.path.basename(src) + ".o")
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    r = subprocess.run([HIPCC, *FLAGS, "-c", src, "-o", obj], capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError("no HIP sources found")
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


def jaxlib_include():
    """Directory holding xla/ffi/api/ffi.h (shipped inside jaxlib), or None."""
    try:
        import jaxlib
    except ImportError:
        return None
    inc = os.path.join(os.path.dirname(jaxlib.__file__), "include")
    return inc if os.path.exists(os.path.join(inc, "xla", "ffi", "api", "ffi.h")) else None


def build_xla_ffi(verbose: bool = True):
    """Compiles the XLA FFI handlers (xla_ffi/gla_xla_ffi.cc) against jaxlib's headers and links them with
    libgla_hip.so.  Returns the path, or None when jaxlib's headers are not installed (then nothing is built:
    the torch front-end does not need them)."""
    inc = jaxlib_include()
    if inc is None:
        if verbose:
            print("xla/ffi/api/ffi.h not found (no jaxlib): the XLA FFI handlers are not built")
        return None
    src = os.path.join(HERE, "xla_ffi", "gla_xla_ffi.cc")
    out = os.path.join(HERE, "xla_ffi", "libgla_xla_ffi.so")
    cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared", "-I", inc, "-I",
           os.path.join(HERE, "..", "include"), src, "-o", out, "-L", HERE, "-lgla_hip", "-Wl,-rpath,$ORIGIN/.."]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("XLA FFI handlers failed to build:\n" + r.stderr)
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    build()
    build_xla_ffi()
