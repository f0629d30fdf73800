"""ctypes binding of libqvb8_amd.so: one Python function per C entry point of
include/qvb8_amd.h, taking torch tensors for device memory and the current torch
stream.  A failed call raises RuntimeError with the library's message; a missing
library raises NativeLibraryError.  Nothing here computes anything."""
from __future__ import annotations

import ctypes
import os

import torch

from .common.errors import NativeLibraryError

_LIB = None
EXPECTED_ABI = 7            # QVB8_ABI_VERSION of include/qvb8_amd.h that the argument lists below were written for
F32, F16, BF16 = 0, 1, 2
_DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

# every symbol include/qvb8_amd.h declares
SYMBOLS = ("qvb8_abi_version", "qvb8_last_error", "qvb8_decode", "qvb8_lookup_rows", "qvb8_scatter_escapes", "qvb8_certify",
           "qvb8_sat_half", "qvb8_scale_sat_half", "qvb8_gemv_workspace_bytes", "qvb8_gemv", "qvb8_mma_rowinfo_bytes", "qvb8_mma_prepare", "qvb8_mma_workspace_bytes", "qvb8_mma", "qvb8_launch_probe", "qvb8_mlp_workspace_bytes", "qvb8_mlp_init", "qvb8_mlp",
           "qvb8_moe_workspace_bytes", "qvb8_moe_experts", "qvb8_moe_experts_static",
           "qvb8r_decode", "qvb8r_decode_blocks", "qvb8r_gemv_workspace_bytes", "qvb8r_gemv", "qvb8r_walk_probe", "qvb8r_fix_escapes", "qvb8_attn_fwd", "qvb8_attn_combine")


def lib_path() -> str:
    override = os.environ.get("QVB8_AMD_LIB")          # a differently built library, for experiments
    if override:
        return override
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libqvb8_amd.so")


def load(build_if_missing: bool = True):
    """The loaded library.  Built with hipcc on first use when it is not there."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    own = not os.environ.get("QVB8_AMD_LIB")           # a library named by the caller is taken as it is
    missing = not os.path.exists(path)
    stale = False
    if own and not missing:
        from . import build as _b
        stale = _b.needs_build()                       # a source or the header is newer than the library
    if missing or stale:
        if not build_if_missing or not own:
            raise NativeLibraryError(f"{path} is missing: run `python -m qvb8_amd.build`")
        from . import build as _b
        try:
            _b.build(verbose=False)
        except Exception as ex:                      # noqa: BLE001
            if missing:
                raise NativeLibraryError(f"cannot build {path}: {ex}") from None
            # a box without the compiler (or with read-only sources) cannot refresh a library it did not build: say so and
            # refuse rather than run code that no longer matches its sources
            raise NativeLibraryError(f"{path} is older than its sources and cannot be rebuilt here ({ex}): "
                                     "run `python -m qvb8_amd.build` where hipcc is") from None
    try:
        lib = ctypes.CDLL(path)
    except OSError as ex:
        raise NativeLibraryError(f"cannot load {path}: {ex}") from None
    lib.qvb8_abi_version.restype = ctypes.c_int
    found = lib.qvb8_abi_version()
    if found != EXPECTED_ABI:
        raise NativeLibraryError(f"{path} has ABI version {found}, this binding was written for {EXPECTED_ABI}: "
                                 "rebuild it with `python -m qvb8_amd.build`")
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.qvb8_abi_version.restype = i32
    lib.qvb8_last_error.restype = ctypes.c_char_p
    lib.qvb8_decode.argtypes = [vp, i64, vp, vp, vp, vp, i64, i64, i32, vp, vp]
    lib.qvb8_lookup_rows.argtypes = [vp, i64, vp, i64, vp, vp, vp, vp, i64, i64, vp, vp, i64, i32, vp, vp]
    lib.qvb8_scatter_escapes.argtypes = [vp, i32, i64, vp, vp, i64, vp]
    lib.qvb8_certify.argtypes = [vp, i32, vp, i32, i64, ctypes.c_float, vp, vp]
    lib.qvb8_sat_half.argtypes = [vp, i32, i64, vp, vp]
    lib.qvb8_scale_sat_half.argtypes = [vp, i32, i64, ctypes.c_float, vp, vp]
    lib.qvb8_gemv_workspace_bytes.argtypes = [i64, i64, i64]
    lib.qvb8_gemv_workspace_bytes.restype = i64
    lib.qvb8_gemv.argtypes = [vp, i32, i64, vp, i64, vp, vp, vp, vp, i64, i64, vp, vp, i64, vp, vp, i64, vp]
    lib.qvb8_mma_workspace_bytes.argtypes = [i64, i64, i64]
    lib.qvb8_mma_workspace_bytes.restype = i64
    lib.qvb8_mma_rowinfo_bytes.argtypes = [i64]
    lib.qvb8_mma_rowinfo_bytes.restype = i64
    lib.qvb8_mma_prepare.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, vp, vp]
    lib.qvb8_mma.argtypes = [vp, i32, i64, vp, i64, vp, vp, vp, vp, i64, i64, vp, vp, i64, vp, vp, vp, i32, vp, vp, i64, vp]
    lib.qvb8_launch_probe.argtypes = [i64, i64, i64, vp]
    lib.qvb8_mlp_workspace_bytes.argtypes = [i64]
    lib.qvb8_mlp_workspace_bytes.restype = i64
    lib.qvb8_mlp_init.argtypes = [i64, i64, i64, vp, i64, vp, vp, vp, i64, vp, vp, vp, i64, vp, vp]
    lib.qvb8_mlp.argtypes = [vp, vp, i32, i64, i32, i32, vp, i32, vp, vp]
    lib.qvb8_moe_workspace_bytes.argtypes = [i64] * 6
    lib.qvb8_moe_workspace_bytes.restype = i64
    lib.qvb8_moe_experts.argtypes = ([vp, i32, i64, vp, vp, i64, i64] + [vp, i64, vp, vp, vp, vp, i64, i64] * 2
                                     + [i32, vp, i32, vp, i64, vp])
    lib.qvb8_moe_experts_static.argtypes = ([vp, i32, i64, vp, vp, i64, i64] + [vp, i64, vp, vp, vp, vp, i64, i64] * 2
                                            + [i32, vp, i32, vp])
    lib.qvb8r_decode.argtypes = [vp, i64, i32, i64, i64, i64, vp, i64, vp]
    lib.qvb8r_decode_blocks.argtypes = [vp, i64, i32, vp, i64, vp, i64, vp]
    lib.qvb8r_gemv_workspace_bytes.argtypes = [i64, i64]
    lib.qvb8r_gemv_workspace_bytes.restype = i64
    lib.qvb8r_gemv.argtypes = [vp, i32, i64, vp, i64, vp, vp, i64, vp]
    lib.qvb8r_walk_probe.argtypes = [vp, i64, vp, vp]
    lib.qvb8r_fix_escapes.argtypes = [vp, i32, i64, vp, vp, vp, vp, i64, vp, i64, i64, vp]
    lib.qvb8_attn_fwd.argtypes = ([vp, i64, i64, vp, vp, i32, i64, i64] + [vp] * 9 + [i64, vp, vp, vp] + [i64] * 6
                                  + [ctypes.c_double, i64, vp])
    lib.qvb8_attn_combine.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, vp, vp, vp]
    for name in SYMBOLS:
        getattr(lib, name)                           # every declared symbol must be exported
    _LIB = lib
    return lib


MMA_MAX_CLASSES = 3


class MmaLayout(ctypes.Structure):
    """qvb8_mma_layout of include/qvb8_amd.h."""
    _fields_ = [("n_classes", ctypes.c_int32), ("first_pos", ctypes.c_int32 * (MMA_MAX_CLASSES + 1)),
                ("nbits", ctypes.c_int32 * MMA_MAX_CLASSES)]


class MlpPlan(ctypes.Structure):
    """qvb8_mlp_plan of include/qvb8_amd.h."""
    _fields_ = [("hidden", ctypes.c_int64), ("inter", ctypes.c_int64), ("out_features", ctypes.c_int64), ("magic", ctypes.c_int64)]


class RCore(ctypes.Structure):
    """qvb8r_core of include/qvb8_amd.h."""
    _fields_ = [("words", ctypes.c_void_p), ("n_words", ctypes.c_int64), ("tile_off", ctypes.c_void_p),
                ("states", ctypes.c_void_p), ("tiles", ctypes.c_void_p), ("n_tiles", ctypes.c_int64),
                ("blocks", ctypes.c_void_p), ("n_blocks", ctypes.c_int64), ("tab", ctypes.c_void_p),
                ("n_classes", ctypes.c_int64), ("perm", ctypes.c_void_p), ("min_s", ctypes.c_void_p),
                ("tau_s", ctypes.c_void_p), ("drow", ctypes.c_void_p), ("Q", ctypes.c_int64), ("P", ctypes.c_int64)]


def _check(rc: int, lib):
    if rc != 0:
        msg = lib.qvb8_last_error()
        raise RuntimeError((msg.decode() if msg else f"qvb8 native call failed ({rc})"))


def dtype_code(dt) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise RuntimeError(f"qvb8: unsupported dtype {dt}") from None


def ptr(t) -> int | None:
    return None if t is None or t.numel() == 0 else t.data_ptr()


def stream_of(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def require_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("qvb8: inputs must be GPU tensors (there is no CPU path)")
