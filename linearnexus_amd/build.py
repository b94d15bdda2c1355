"""Builds liblinearnexus_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: ``python -m linearnexus_amd.build``.  The library is written next to this file so
that it travels with the source tree; nothing is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblinearnexus_hip.so")
SOURCES = ["c_api.hip", "recurrent.hip", "chunk_fwd.hip", "chunk_bwd.hip", "chunk_direct.hip", "conv1d.hip", "dplr.hip", "rmsnorm_gated.hip", "kda_gate.hip", "gdn_gate.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffast-math", "-fno-finite-math-only",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",  # m0 on an asm clobber list (the LDS-direct loads set it) is reported as a reserved register
]


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = ["hipcc", *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(4, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print(f"built {LIB} from {', '.join(srcs)}")
    build_c_abi_smoke(verbose)
    build_xla_ffi(verbose)
    return LIB


def xla_ffi_include_dir():
    """Directory that holds ``xla/ffi/api/ffi.h``: ``XLA_FFI_INCLUDE_DIR`` if set, else what an installed JAX reports
    (``jax.ffi.include_dir()``; ``jax.extend.ffi`` in older releases); None when neither is there."""
    cands = [os.environ.get("XLA_FFI_INCLUDE_DIR")]
    try:
        import jax  # noqa: F401
        try:
            from jax import ffi as jffi
        except ImportError:
            from jax.extend import ffi as jffi
        cands.append(jffi.include_dir())
    except Exception:
        pass
    for d in cands:
        if d and os.path.exists(os.path.join(d, "xla", "ffi", "api", "ffi.h")):
            return d
    return None


def build_xla_ffi(verbose: bool = True) -> str:
    """Compiles csrc/lnx_xla_ffi.cc (the XLA FFI handlers a JAX caller registers) into liblinearnexus_xla_ffi.so next to
    the main library, where the XLA FFI headers exist; skipped with a message otherwise."""
    inc = xla_ffi_include_dir()
    if inc is None:
        if verbose:
            print("XLA FFI headers not found (no JAX installed, XLA_FFI_INCLUDE_DIR unset): csrc/lnx_xla_ffi.cc not built")
        return ""
    out = os.path.join(HERE, "liblinearnexus_xla_ffi.so")
    cmd = ["hipcc", "-O2", "-std=c++17", "-fPIC", "-shared", f"-I{inc}", os.path.join(CSRC, "lnx_xla_ffi.cc"), "-o", out,
           f"-L{HERE}", "-llinearnexus_hip", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the XLA FFI handlers failed:\n" + r.stderr)
    if verbose:
        print(f"built {out}")
    return out


def build_c_abi_smoke(verbose: bool = True) -> str:
    """Compiles tests/c_abi/abi_smoke.c (plain C, gcc) against the library just built; the GPU test
    tests/test_c_abi_gpu.py runs the binary."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "c_abi", "abi_smoke.c")
    exe = os.path.join(root, "tests", "c_abi", "abi_smoke")
    if not os.path.exists(src):
        return ""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-O2", "-D__HIP_PLATFORM_AMD__", f"-I{rocm}/include", src, "-o", exe, f"-L{rocm}/lib", "-lamdhip64",
           f"-L{HERE}", "-llinearnexus_hip", "-lm", "-Wl,-rpath,$ORIGIN/../../linearnexus_amd", f"-Wl,-rpath,{rocm}/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the C-ABI smoke program failed:\n" + r.stderr)
    if verbose:
        print(f"built {exe}")
    return exe


if __name__ == "__main__":
    build()
