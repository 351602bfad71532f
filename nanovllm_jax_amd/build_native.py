"""Compile the HIP kernels and their C ABI into one shared library for gfx950.

``hipcc`` cross-compiles without a GPU.  The library is built in-tree
(``nanovllm_jax_amd/_native/libnvj_paged_attn.so``) so that it travels with the
source tree; nothing here runs at import time of the package.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
NATIVE_DIR = os.path.join(PKG_DIR, "_native")
LIB_NAME = "libnvj_paged_attn.so"
LIB_PATH = os.path.join(NATIVE_DIR, LIB_NAME)

SOURCES = ("store_kvcache.hip", "paged_decode.hip", "qk_norm_rope_store.hip",
           "decode_metadata.hip", "prefill_attention.hip", "layer_glue.hip")

HIPCC_FLAGS = (
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or put /opt/rocm/bin on PATH)")


def build(verbose: bool = True, extra_flags: tuple[str, ...] = ()) -> str:
    """Compile every HIP source into ``LIB_PATH`` (always recompiles)."""
    os.makedirs(NATIVE_DIR, exist_ok=True)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags,
           "-I", os.path.join(REPO_DIR, "include"),
           *[os.path.join(CSRC_DIR, s) for s in SOURCES], "-o", tmp]
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out, flush=True)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def xla_ffi_include_dir() -> str | None:
    """Directory of the XLA FFI headers (they ship inside jaxlib), or None."""
    try:
        import jax.ffi  # noqa: F401  (absent from images without JAX)
        return jax.ffi.include_dir()
    except Exception:
        return None


def build_xla_ffi(verbose: bool = True) -> str | None:
    """Compile the XLA FFI handlers next to the C-ABI library when the XLA FFI
    headers can be found; otherwise say so and return None."""
    inc = xla_ffi_include_dir()
    if inc is None:
        if verbose:
            print("[build] XLA FFI headers not found (jax is not installed): "
                  "csrc/xla_ffi/nvj_xla_ffi.cc skipped", flush=True)
        return None
    out = os.path.join(NATIVE_DIR, "libnvj_xla_ffi.so")
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared",
           "-I", inc, "-I", os.path.join(REPO_DIR, "include"),
           os.path.join(CSRC_DIR, "xla_ffi", "nvj_xla_ffi.cc"),
           "-L", NATIVE_DIR, "-lnvj_paged_attn", "-Wl,-rpath,$ORIGIN", "-o", out]
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    # this source has never met a compiler where it was written: a failure here
    # must not take the rest of the build (and every test behind it) down
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        print(f"[build] XLA FFI handlers did NOT compile (exit {proc.returncode}); the C-ABI "
              f"library is unaffected:\n{proc.stdout}", flush=True)
        return None
    return out


def build_c_caller(verbose: bool = True) -> str:
    """Compile the plain-C caller of the C ABI (csrc/c_caller) with the host C
    compiler against the library just built; the GPU tests run it as a child
    process to show the ABI needs neither C++ nor torch on the calling side."""
    out = os.path.join(NATIVE_DIR, "nvj_c_caller")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [os.environ.get("CC", "gcc"), "-std=c11", "-O2", "-Wall", "-Wextra",
           "-I", os.path.join(REPO_DIR, "include"), "-I", os.path.join(rocm, "include"),
           os.path.join(CSRC_DIR, "c_caller", "nvj_c_caller.c"),
           "-L", NATIVE_DIR, "-lnvj_paged_attn", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib"), "-o", out]
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    print(build(extra_flags=tuple(sys.argv[1:])))
