"""ctypes loader for the in-tree HIP kernel library (libafops.so).

The kernels are pure HIP (no torch headers); tensors cross the boundary as raw
device pointers + the current HIP stream.  On a GPU box the library MUST load
— ops raise instead of silently falling back to eager torch (the reference
framework has no model math to fall back to; ours must run the native path).
"""
from __future__ import annotations

import ctypes
import functools
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).resolve().parent.parent / "libafops.so"


class AfOpsError(RuntimeError):
    pass


@functools.lru_cache(maxsize=1)
def lib() -> ctypes.CDLL:
    if not _LIB_PATH.exists():
        if torch.cuda.is_available():
            raise AfOpsError(
                f"libafops.so not built at {_LIB_PATH}; run "
                "`python -m agentfield_amd.build` (GPU path never falls back)")
        # CPU-only environment: try to build (hipcc cross-compiles w/o GPU)
        from agentfield_amd.build import build_afops
        build_afops()
    cdll = ctypes.CDLL(str(_LIB_PATH))
    _declare(cdll)
    return cdll


def _declare(l: ctypes.CDLL) -> None:
    p = ctypes.c_void_p
    i = ctypes.c_int
    i64 = ctypes.c_int64
    f = ctypes.c_float
    u32 = ctypes.c_uint32
    l.af_rmsnorm.argtypes = [p, p, p, p, p, f, i, i, p]
    l.af_rope_cache.argtypes = [p, p, p, p, p, p, p, p, p, f, f,
                                i, i, i, i, i64, i64, i64, i, p]
    l.af_silu_mul.argtypes = [p, p, p, f, f, i64, i64, p]
    l.af_add.argtypes = [p, p, p, i64, p]
    l.af_reshape_and_cache.argtypes = [p, p, p, p, p, i, i, i, i, p]
    l.af_embedding.argtypes = [p, p, p, p, i, i, p]
    l.af_attn_decode.argtypes = [p, p, p, p, p, p, p, p, f, i, i, i, i, i, i, i,
                                 i64, i, p]
    l.af_attn_prefill.argtypes = [p, p, p, p, p, p, p, p, p, f,
                                  i, i, i, i, i64, i, i, i, p]
    l.af_gemm_bf16.argtypes = [p, p, p, i, i, i, p]
    l.af_gemm_bf16_ring.argtypes = [p, p, p, i, i, i, p]
    l.af_gemm_mxfp8.argtypes = [p, p, p, p, p, i, i, i, p]
    l.af_gemm_bf16_q8.argtypes = [p, p, p, i, i, i, p]
    l.af_ipc_get_handle.argtypes = [p, p]
    l.af_ipc_open_handle.argtypes = [p, p]
    l.af_ipc_close_handle.argtypes = [p]
    l.af_oneshot_allreduce.argtypes = [p, p, p, i, i, ctypes.c_long,
                                       ctypes.c_long, ctypes.c_ulonglong, p]
    l.af_gemm_skinny.argtypes = [p, p, p, p, p, i, i, i, i, i,
                                 p, f, p, p]
    l.af_sample.argtypes = [p, p, p, p, p, p, u32, i, i, p]
    l.af_sample_topkp.argtypes = [p, p, p, p, p, p, p, p, p, p, p, p,
                                  u32, i, i, p]
    l.af_gather_rows.argtypes = [p, p, p, i, i, p]
    l.af_mfma_probe.argtypes = [p, p, p, p]
    l.af_mfma_mx_probe.argtypes = [p, p, p, p, p, p]
    l.af_lds_stride_probe.argtypes = [p, p, i, p]
    l.af_mfma_mx32_probe.argtypes = [p, p, p, p, p, i, p]
    l.af_axpy.argtypes = [p, p, f, i, p]
    l.af_device_sync.argtypes = []
    for fn in ("af_rmsnorm", "af_rope_cache", "af_silu_mul", "af_add",
               "af_reshape_and_cache", "af_embedding", "af_attn_decode",
               "af_attn_prefill", "af_gemm_bf16", "af_gemm_bf16_ring", "af_gemm_bf16_q8", "af_gemm_mxfp8", "af_oneshot_allreduce",
               "af_gemm_skinny", "af_sample",
               "af_sample_topkp", "af_gather_rows", "af_mfma_probe", "af_mfma_mx_probe", "af_lds_stride_probe", "af_mfma_mx32_probe", "af_axpy",
               "af_device_sync"):
        getattr(l, fn).restype = ctypes.c_int


@functools.lru_cache(maxsize=None)
def mixgroup(group: str) -> ctypes.CDLL:
    """One sequence-mixer kernel group (build.MIX_GROUPS).  Unlike the main
    library a group is compiled on first use when missing or older than its
    sources - on a GPU box too - so a fresh checkout serving a hybrid model
    builds exactly the groups that model calls and nothing else."""
    from agentfield_amd.build import MIX_GROUPS, build_mix
    path = MIX_GROUPS[group][0]
    try:
        build_mix(verbose=False, group=group)
    except Exception as e:
        if not path.exists():
            raise AfOpsError(f"{path.name} could not be built: {e}") from e
    cdll = ctypes.CDLL(str(path))
    for name, args in _MIX_SIGS[group].items():
        fn = getattr(cdll, name)
        fn.argtypes = args
        fn.restype = ctypes.c_int
    return cdll


class _MixLib:
    """Resolves an afm_* entry point to its kernel group on first use."""

    def __getattr__(self, name):
        for group, sigs in _MIX_SIGS.items():
            if name in sigs:
                fn = getattr(mixgroup(group), name)
                setattr(self, name, fn)
                return fn
        raise AttributeError(name)


_MIXLIB = _MixLib()


def mixlib() -> _MixLib:
    return _MIXLIB


def _mix_sigs() -> dict:
    p, i, i64, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
    return {
        "glue": {
            "afm_embed": [p, p, p, p, f, i, i, i, p],
            "afm_add_rows": [p, p, p, i, i, p],
            "afm_dual_norm_shift": [p, p, p, p, p, p, p, p, p, p, p, p, p, f,
                                    i, i, i, p],
            "afm_scatter_state": [p, p, p, p, i, i, p],
            "afm_norm_rows": [p, p, p, p, f, i, i, i, i, p],
            "afm_headnorm_gate": [p, p, p, p, f, i, i, i, i64, i, i, p],
            "afm_polynorm": [p, p, p, f, i, i, i64, i, p],
            "afm_gated_residual": [p, p, f, p, f, p, i64, p, p, p, i64, p,
                                   i, i, i, p],
            "afm_softcap": [p, p, f, i64, i, p],
            "afm_cast_rows": [p, p, i64, i, p],
            "afm_norm_residual": [p, p, p, i64, i, p, p, f, i, i, i, p],
            "afm_glu": [p, i64, i64, p, p, i64, i64, i, p, p, p, i64, i, i,
                        f, i, p],
            "afm_moe_route": [p, p, p, p, p, i, i, i, i, i, f, i, i, p],
            "afm_moe_combine": [p, p, p, p, p, i, i, i, i, p],
        },
        "seq": {
            "afm_qk_norm_cache": [p, p, p, p, p, p, p, p, p, f, i, i, i, i, i,
                                  i, i, i, i64, i64, i64, i, p],
            "afm_masked_attention": [p, p, p, p, p, p, p, f, i, i, i, i, i, i,
                                     i, i, i, i64, i, p, p, p, f, p, p, i64,
                                     i, i, p],
            "afm_attn_prefill_mfma": [p, p, p, p, p, p, p, p, p, f, i, i, i, i,
                                      i, i, i, i, i, i64, p, f, p, p, i64, i,
                                      p],
            "afm_attn_heads_mfma": [p, p, p, p, p, p, p, f, i, i, i, i, i, i,
                                    i, i, i, i64, i, p, p, p, f, p, p, i64, i,
                                    p],
            "afm_attn_split_combine": [p, p, p, i, i, i, i, p],
            "afm_linear_scan": [p, p, p, p, p, p, p, p, p, p, p, p, p, f, f, f,
                                i, i, i, i, i, i64, i64, i64, i64, i, p],
        },
        "conv": {
            "afm_causal_conv": [p, p, i64, p, p, p, p, p, p, p, i, i, i, i, i,
                                i, p],
        },
        "ssm": {
            "afm_selective_scan": [p, p, p, p, p, p, i64, p, i64, p, p, p, p,
                                   p, i, i, i, i, p],
            "afm_qk_unit_cache": [p, p, i64, p, i64, p, i64, p, i64, f, p, p,
                                  p, p, f, f, i, i, i, i, i, i, i, i, p],
            "afm_sigattn_prefill_mfma": [p, p, p, p, p, p, p, p, p, p, p, i, i,
                                         p, p, p, i64, f, i, i, i, i, i, i, i,
                                         p],
            "afm_sigmoid_attention": [p, p, p, p, p, p, p, p, p, p, i, i, p, p,
                                      p, i64, f, i, i, i, i, i, i, i, i, i, i,
                                      p],
        },
        "hyper": {
            "afm_embed_streams": [p, p, p, i, i, i, i, p],
            "afm_hyper_step": [p, p, i64, p, p, p, p, f, p, i, i, i, i, p, p,
                               p, p, i, p, i, p],
            "afm_canon_conv": [p, p, p, p, p, p, p, p, i, i, i, i, i, p],
            "afm_latent_prep": [p, p, p, i64, p, i64, p, p, p, p, f, i, i,
                                i, i, i, i, i, p],
            "afm_gate_heads": [p, p, p, i64, i, i, i, i, p],
            "afm_relu2": [p, p, i64, i, i, i, p],
        },
        "delta": {
            "afm_delta_scan": [p, p, p, i64, p, i64, p, i64, p, i64, p, i64,
                               p, p, p, p, p, i, i, i, i, i, i, f, i, i, p],
            "afm_rotary_table": [p, p, p, i, i, p],
            "afm_qk_rope_cache": [p, p, i64, p, i64, p, i64, p, p, p, p, p,
                                  p, i, p, p, p, f, i, i, i, i, i, i, i, p],
            "afm_postnorm_sum": [p, p, p, i64, i, p, i64, p, p, p, f, f, i,
                                 i, i, p],
            "afm_gate_gather": [p, p, i64, p, i64, i, p, i, i, i, p],
        },
    }


_MIX_SIGS = _mix_sigs()


def cur_stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t: torch.Tensor | None) -> ctypes.c_void_p:
    if t is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(t.data_ptr())


def check(rc: int, name: str) -> None:
    if rc != 0:
        raise AfOpsError(f"{name} failed with code {rc} (hipError or 9xxx arg check)")


def main_lib_ready() -> bool:
    """True when libafops.so is on disk (never triggers a build)."""
    return _LIB_PATH.exists()


def native_loaded() -> bool:
    try:
        lib()
        return True
    except Exception:
        return False
