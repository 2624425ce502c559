"""ctypes binding of libksana_sage_hip.so (declared in include/ksana_sage_hip.h).

The library is loaded once, from this package directory only (never from site-packages), and a
missing or stale library is an error that names the build command - there is no CPU fallback.
"""

from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libksana_sage_hip.so"
ABI_VERSION = 20

BF16, FP16 = 0, 1
OK, EINVAL, ENOTSUP, EHIP = 0, -1, -2, -3
FLAG_PWL_EXP2 = 1
FLAG_SMOOTH_V = 2
FLAG_WG_4_WAVES = 4
FLAG_WG_8_WAVES = 8
FLAG_TILE_SKIP = 16
PREP_WAN, PREP_WAN_COMFY, PREP_QWEN = 0, 1, 2
KEEP = -(2**63)  # KSANA_SAGE_KEEP

EXPORTS = (
    "ksana_sage_abi_version",
    "ksana_sage_last_error",
    "ksana_sage_configure",
    "ksana_sage_one_read_state",
    "ksana_sage_selftest",
    "ksana_sage_workspace_layout",
    "ksana_sage_quant_q",
    "ksana_sage_quant_k",
    "ksana_sage_quant_k_static",
    "ksana_sage_quant_v",
    "ksana_sage_quant_v_smooth",
    "ksana_sage_attn_fwd",
    "ksana_sage_attn_key_split",
    "ksana_sage_quant_status",
    "ksana_sage_block_means",
    "ksana_sage_quant_qk_pooled",
    "ksana_sage_sla_workspace_bytes",
    "ksana_sage_sla_linear",
    "ksana_sage_sla_block_map",
    "ksana_sage_mfma_probe",
    "ksana_sage_forward",
    "ksana_sage_quant_q_prep",
    "ksana_sage_quant_k_prep",
    "ksana_sage_quant_qk_prep",
    "ksana_sage_forward_prep",
    "ksana_sage_attn_fwd_masked",
    "ksana_sage_attn_fwd_varlen",
    "ksana_sage_forward_masked",
)


class Shape(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("B", "Hq", "Hkv", "Lq", "Lk", "D")]


class WsLayout(C.Structure):
    _fields_ = [
        (n, C.c_uint64)
        for n in (
            "total_bytes", "q_i8", "q_scale", "k_i8", "k_scale", "k_mean",
            "v_fp8", "v_scale", "v_inv", "k_part", "v_part", "q_rms", "k_rms", "v_mean", "split_o", "split_ml",
            "k_sync", "v_sync",
        )
    ] + [(n, C.c_int32) for n in ("lq_pad", "nqb", "nkb", "nch")]


class Prep(C.Structure):
    """``ksana_sage_prep``: the step before attention (RMSNorm over the token row, 3-axis RoPE)."""

    _fields_ = [
        ("q_norm_weight", C.c_void_p),
        ("k_norm_weight", C.c_void_p),
        ("norm_eps", C.c_float),
        ("rope_rows", C.c_int32),
        ("rope_freqs", C.c_void_p),
        ("grid_sizes", C.POINTER(C.c_int32)),
        ("kind", C.c_int32),
        ("txt_len", C.c_int32),
        ("q_norm_weight_txt", C.c_void_p),
        ("k_norm_weight_txt", C.c_void_p),
        ("rope_freqs_txt", C.c_void_p),
        ("rope_freqs_img", C.c_void_p),
        ("rope_matrices", C.c_void_p),
    ]


class SageLibraryError(RuntimeError):
    """The HIP library is missing, stale, or rejected a call."""


Strides = C.c_int64 * 4
_lock = threading.Lock()
_lib = None


def _declare(lib):
    vp, i, f = C.c_void_p, C.c_int, C.c_float
    sp, lp, st = C.POINTER(Shape), C.POINTER(WsLayout), C.POINTER(C.c_int64)
    lib.ksana_sage_abi_version.argtypes, lib.ksana_sage_abi_version.restype = [], i
    lib.ksana_sage_last_error.argtypes, lib.ksana_sage_last_error.restype = [], C.c_char_p
    lib.ksana_sage_workspace_layout.argtypes, lib.ksana_sage_workspace_layout.restype = [sp, lp], i
    lib.ksana_sage_configure.argtypes, lib.ksana_sage_configure.restype = [C.c_char_p, C.c_int64], i
    lib.ksana_sage_one_read_state.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int64), C.POINTER(C.c_int)]
    lib.ksana_sage_one_read_state.restype = i
    lib.ksana_sage_selftest.argtypes, lib.ksana_sage_selftest.restype = [], i
    lib.ksana_sage_quant_q.argtypes, lib.ksana_sage_quant_q.restype = [vp, i, st, sp, f, vp, vp], i
    lib.ksana_sage_quant_k.argtypes, lib.ksana_sage_quant_k.restype = [vp, i, st, sp, i, vp, vp], i
    lib.ksana_sage_quant_k_static.argtypes, lib.ksana_sage_quant_k_static.restype = [vp, i, st, sp, i, vp, vp], i
    lib.ksana_sage_quant_v.argtypes, lib.ksana_sage_quant_v.restype = [vp, i, st, sp, vp, vp], i
    lib.ksana_sage_quant_v_smooth.argtypes, lib.ksana_sage_quant_v_smooth.restype = [vp, i, st, sp, i, vp, vp], i
    lib.ksana_sage_attn_fwd.argtypes, lib.ksana_sage_attn_fwd.restype = [vp, vp, i, st, sp, vp, i, i, vp], i
    ip = C.POINTER(C.c_int)
    lib.ksana_sage_attn_key_split.argtypes, lib.ksana_sage_attn_key_split.restype = [sp, ip, ip], i
    lib.ksana_sage_quant_status.argtypes, lib.ksana_sage_quant_status.restype = [vp, sp, vp, ip, ip], i
    lib.ksana_sage_block_means.argtypes = [vp, i, st, i, i, i, i, vp, vp, vp]
    lib.ksana_sage_block_means.restype = i
    lib.ksana_sage_quant_qk_pooled.argtypes = [vp, vp, i, st, st, sp, f, vp, vp, vp, vp]
    lib.ksana_sage_quant_qk_pooled.restype = i
    lib.ksana_sage_sla_workspace_bytes.argtypes = [i, i, i, C.POINTER(C.c_uint64)]
    lib.ksana_sage_sla_workspace_bytes.restype = i
    lib.ksana_sage_sla_linear.argtypes = [vp, vp, vp, i, st, st, st, i, i, i, vp, vp, vp, st, vp, st, vp, vp]
    lib.ksana_sage_sla_linear.restype = i
    lib.ksana_sage_sla_block_map.argtypes, lib.ksana_sage_sla_block_map.restype = [vp, vp, i, i, i, i, i, i, vp, vp], i
    lib.ksana_sage_mfma_probe.argtypes = [vp, C.c_uint64, i, i, vp, C.POINTER(C.c_double)]
    lib.ksana_sage_mfma_probe.restype = i
    lib.ksana_sage_forward.argtypes = [vp, vp, vp, vp, i, st, st, st, st, sp, vp, f, i, i, i, vp, vp]
    lib.ksana_sage_forward.restype = i
    pp = C.POINTER(Prep)
    lib.ksana_sage_quant_q_prep.argtypes, lib.ksana_sage_quant_q_prep.restype = [vp, i, st, sp, pp, f, vp, vp], i
    lib.ksana_sage_quant_k_prep.argtypes, lib.ksana_sage_quant_k_prep.restype = [vp, i, st, sp, pp, i, vp, vp], i
    lib.ksana_sage_quant_qk_prep.argtypes, lib.ksana_sage_quant_qk_prep.restype = [vp, vp, i, st, st, sp, pp, f, i, vp, vp], i
    lib.ksana_sage_forward_prep.argtypes = [vp, vp, vp, vp, i, st, st, st, st, sp, pp, vp, f, i, i, i, vp, vp]
    lib.ksana_sage_forward_prep.restype = i
    ms = C.POINTER(C.c_int64)
    lib.ksana_sage_attn_fwd_masked.argtypes = [vp, vp, i, st, sp, vp, ms, vp, i, i, vp]
    lib.ksana_sage_attn_fwd_masked.restype = i
    lib.ksana_sage_attn_fwd_varlen.argtypes = [vp, vp, i, st, sp, vp, ms, vp, vp, i, i, vp]
    lib.ksana_sage_attn_fwd_varlen.restype = i
    lib.ksana_sage_forward_masked.argtypes = [vp, vp, vp, vp, i, st, st, st, st, sp, vp, ms, vp, f, i, i, i, vp, vp]
    lib.ksana_sage_forward_masked.restype = i


def library_present() -> bool:
    return LIB_PATH.exists()


def load():
    """Return the loaded library; raise ``SageLibraryError`` when it cannot be used."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise SageLibraryError(
                    f"{LIB_PATH} not found: build it with `python -m ksanadit_amd.build` (needs hipcc)"
                )
            try:
                lib = C.CDLL(str(LIB_PATH))
            except OSError as exc:
                raise SageLibraryError(f"cannot load {LIB_PATH}: {exc}") from exc
            missing = [n for n in EXPORTS if not hasattr(lib, n)]
            if missing:
                raise SageLibraryError(f"{LIB_PATH} lacks symbols {missing}: rebuild it")
            _declare(lib)
            if lib.ksana_sage_abi_version() != ABI_VERSION:
                raise SageLibraryError(
                    f"{LIB_PATH} has ABI {lib.ksana_sage_abi_version()}, this package needs {ABI_VERSION}: rebuild it"
                )
            _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """Map a library return code to the exception the reference's callers expect."""
    if rc == OK:
        return
    msg = f"{what}: {load().ksana_sage_last_error().decode()}"
    if rc == EINVAL:
        raise ValueError(msg)
    if rc == ENOTSUP:
        raise NotImplementedError(msg)
    raise SageLibraryError(msg)


def workspace_layout(B: int, Hq: int, Hkv: int, Lq: int, Lk: int, D: int) -> tuple[Shape, WsLayout]:
    shape, layout = Shape(B, Hq, Hkv, Lq, Lk, D), WsLayout()
    check(load().ksana_sage_workspace_layout(C.byref(shape), C.byref(layout)), "workspace_layout")
    return shape, layout
