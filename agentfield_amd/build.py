"""Build driver for the in-tree native libraries.

Two artifacts, both built in-tree so they travel with the repo snapshot:
  * agentfield_amd/libafops.so   — pure-HIP gfx950 kernel library (ctypes C API)
  * agentfield_amd/_native*.so   — CPU-side C++ (pybind11): scheduler/allocator,
                                   Ed25519 via libcrypto (built by native/setup)

hipcc cross-compiles gfx950 without a GPU, so this runs in CPU-only CI too.
"""
from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB = PKG_DIR / "libafops.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = os.environ.get("AF_OFFLOAD_ARCH", "gfx950")

HIP_SOURCES = [
    "rmsnorm.hip",
    "rope.hip",
    "activation.hip",
    "cache.hip",
    "attn_decode.hip",
    "attn_prefill.hip",
    "gemm.hip",
    "gemm_ring.hip",
    "gemm_q8.hip",
    "gemm_mxfp8.hip",
    "allreduce.hip",
    "gemm_skinny.hip",
    "sampling.hip",
    "probe.hip",
]

# Kernel groups that build into their own small libraries, so a process that
# serves only one model family compiles (and loads) only what it runs
# (ops/seqmix.py resolves each entry point to its group):
#   glue    row-wise glue shared by the hybrid families (embedding to an fp32
#           residual, norms, gated units, routers)
#   seq     masked softmax attention + decayed linear recurrences
#   ssm     selective state-space scan + sigmoid attention
#   hyper   multi-stream residual mixing, input convolutions, latent-attention
#           row steps
#   conv    short depthwise causal convolution with carried inputs
#   delta   gated delta-rule recurrence, per-head q/k norm with rotary
#           positions, norm after the residual sum
MIX_GROUPS = {
    "glue": (PKG_DIR / "libafglue.so", ["mix_glue.hip"]),
    "seq": (PKG_DIR / "libafmix.so", ["mix_seq.hip", "mix_attn_mfma.hip"]),
    "ssm": (PKG_DIR / "libafssm.so", ["mix_ssm.hip", "mix_sigattn.hip",
                                       "mix_sigattn_mfma.hip"]),
    "hyper": (PKG_DIR / "libafhyper.so", ["mix_hyper.hip"]),
    "delta": (PKG_DIR / "libafdelta.so", ["mix_delta.hip"]),
    "conv": (PKG_DIR / "libafconv.so", ["mix_conv.hip"]),
}
MIX_SOURCES = [s for _lib, srcs in MIX_GROUPS.values() for s in srcs]
MIX_LIB = MIX_GROUPS["seq"][0]

# hipcc -O3 may otherwise fuse scalar float code into packed-fp32 VALU ops
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _needs_build(lib: Path = LIB, sources=None) -> bool:
    if not lib.exists():
        return True
    lib_m = lib.stat().st_mtime
    deps = [CSRC / s for s in (sources or HIP_SOURCES)] + \
        [CSRC / "common.h", CSRC / "mix_attn.h", Path(__file__)]
    return any(d.stat().st_mtime > lib_m for d in deps)


def build_mix(force: bool = False, verbose: bool = True,
              group: str | None = None):
    """Compile the sequence-mixer kernel groups for gfx950 (one group, or
    all of them); returns the library path(s)."""
    if group is not None:
        lib, srcs = MIX_GROUPS[group]
        return _build_lib(lib, srcs, force, verbose)
    return [_build_lib(lib, srcs, force, verbose)
            for lib, srcs in MIX_GROUPS.values()]


def build_afops(force: bool = False, verbose: bool = True) -> Path:
    """Compile the HIP kernel library for gfx950 (incremental per-object)."""
    return _build_lib(LIB, HIP_SOURCES, force, verbose)


def _run(cmd, verbose: bool) -> None:
    if verbose:
        print("[afops]", " ".join(cmd), file=sys.stderr)
        subprocess.run(cmd, check=True)
        return
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout)
        raise subprocess.CalledProcessError(r.returncode, cmd)


def _build_lib(lib: Path, sources, force: bool, verbose: bool) -> Path:
    if not force and not _needs_build(lib, sources):
        return lib
    import tempfile
    objdir = CSRC / ".obj"
    objdir.mkdir(exist_ok=True)
    objs = []
    for src in sources:
        sp = CSRC / src
        op = objdir / (src + ".o")
        objs.append(op)
        if (not force and op.exists()
                and op.stat().st_mtime > sp.stat().st_mtime
                and op.stat().st_mtime > (CSRC / "common.h").stat().st_mtime):
            continue
        cmd = [
            HIPCC, f"--offload-arch={ARCH}", *HIP_FLAGS,
            "-c", str(sp), "-o", str(op),
        ]
        _run(cmd, verbose)
    # link to a temporary name and rename: a concurrent process never maps a
    # half-written library
    fd, tmp = tempfile.mkstemp(dir=str(lib.parent), prefix=lib.name + ".")
    os.close(fd)
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC",
           *[str(o) for o in objs], "-o", tmp]
    try:
        _run(cmd, verbose)
        os.chmod(tmp, 0o755)
        os.replace(tmp, lib)
    finally:
        if os.path.exists(tmp):
            os.unlink(tmp)
    return lib


def build_native(force: bool = False, verbose: bool = True):
    """Build the CPU-side pybind11 extension (scheduler, allocator, crypto)."""
    import sys as _sys
    _sys.path.insert(0, str(PKG_DIR.parent))
    from agentfield_amd.native_build import build as _build  # lazy import
    return _build(force=force, verbose=verbose)


def build_all(force: bool = False):
    build_afops(force=force)
    build_mix(force=force)
    build_native(force=force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
