"""ctypes binding of ``libjigsaw_hip.so``.

The library is plain C ABI (pointers, sizes, a ``hipStream_t``); torch is used
here only to obtain device pointers and the current stream. ``torch`` is imported
first so that the library binds to the HIP runtime torch already loaded.
"""

from __future__ import annotations

import ctypes
import threading
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).resolve().parent / "lib" / "libjigsaw_hip.so"
_lock = threading.Lock()
_lib: ctypes.CDLL | None = None

JG_F32, JG_BF16, JG_F16 = 0, 1, 2
_DTYPES = {torch.float32: JG_F32, torch.bfloat16: JG_BF16, torch.float16: JG_F16}


class LibraryMissing(RuntimeError):
    """``libjigsaw_hip.so`` is not built; there is no fallback path."""


class KernelError(RuntimeError):
    """A C-ABI call returned a negative status."""


class HaloGeom(ctypes.Structure):
    """``jg_halo_geom`` of ``include/jigsaw_hip.h``."""

    _fields_ = [
        ("planes", c_int64),
        ("size", c_int32 * 3),
        ("lo", c_int32 * 3),
        ("hi", c_int32 * 3),
    ]


class AxisSegment(ctypes.Structure):
    """``jg_axis_segment`` of include/jigsaw_hip.h."""

    _fields_ = [
        ("src", ctypes.c_void_p),
        ("src_rows", ctypes.c_int64),
        ("src_start", ctypes.c_int64),
        ("dst_start", ctypes.c_int64),
        ("count", ctypes.c_int64),
    ]


class ConvDesc(ctypes.Structure):
    """``jg_conv_desc`` of ``include/jigsaw_hip.h``."""

    _fields_ = [
        ("n_spatial", c_int32),
        ("groups", c_int32),
        ("batch", c_int64),
        ("c_in", c_int32),
        ("c_out", c_int32),
        ("in_size", c_int32 * 3),
        ("kernel", c_int32 * 3),
        ("stride", c_int32 * 3),
        ("padding", c_int32 * 3),
        ("dilation", c_int32 * 3),
    ]


VoidP27 = c_void_p * 27
VoidP9 = c_void_p * 9

# name -> (restype, argtypes); kept next to include/jigsaw_hip.h by test_abi.py
SIGNATURES: dict[str, tuple] = {
    "jg_last_error": (c_char_p, []),
    "jg_abi_version": (c_int, []),
    "jg_halo_assemble_3d": (c_int, [c_void_p, POINTER(c_void_p), POINTER(HaloGeom), c_int, c_void_p]),
    "jg_halo_assemble_frame_3d": (
        c_int,
        [c_void_p, POINTER(c_void_p), POINTER(HaloGeom), POINTER(c_int32), POINTER(c_int32), c_int, c_void_p],
    ),
    "jg_halo_assemble_2d": (
        c_int,
        [c_void_p, POINTER(c_void_p), c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "jg_halo_pack_3d": (c_int, [POINTER(c_void_p), c_void_p, POINTER(HaloGeom), c_int, c_int, c_void_p]),
    "jg_halo_pack_2d": (
        c_int,
        [POINTER(c_void_p), c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "jg_halo_fold_3d": (c_int, [c_void_p, c_void_p, POINTER(c_void_p), POINTER(HaloGeom), c_int, c_void_p]),
    "jg_halo_fold_border_3d": (c_int, [c_void_p, POINTER(c_void_p), POINTER(HaloGeom), c_int, c_void_p]),
    "jg_halo_fold_2d": (
        c_int,
        [c_void_p, c_void_p, POINTER(c_void_p), c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "jg_halo_axis_gather": (c_int, [c_void_p, c_int64, c_int64, c_int64, POINTER(AxisSegment), c_int, c_int, c_void_p]),
    "jg_halo_axis_scatter_add": (c_int, [c_void_p, c_int64, c_int64, c_int64, POINTER(AxisSegment), c_int, c_int, c_void_p]),
    "jg_roll": (c_int, [c_void_p, c_void_p, c_int, POINTER(c_int64), POINTER(c_int64), c_int, c_void_p]),
    "jg_roll_pack": (c_int, [c_void_p, c_void_p, c_int, POINTER(c_int64), c_int, c_int64, c_int, c_void_p]),
    "jg_roll_pack_fused": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int, POINTER(c_int64), POINTER(c_int64), c_int, c_int64, c_int,
         c_void_p],
    ),
    "jg_roll_unpack_pack": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int64, c_void_p, c_void_p, c_int, c_int64, c_int, POINTER(c_int64), c_int,
         c_void_p],
    ),
    "jg_roll_unpack": (c_int, [c_void_p, c_void_p, c_int, POINTER(c_int64), c_int, c_int64, c_int, c_void_p]),
    "jg_ln_partial_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "jg_ln_apply": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float,
         c_int, c_int, c_void_p],
    ),
    "jg_ln_bwd_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "jg_ln_partial_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p,
         c_size_t, c_void_p],
    ),
    "jg_ln_partial_bwd_static": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p],
    ),
    "jg_ln_bwd_apply": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int,
         c_void_p],
    ),
    "jg_ln_plain_supported": (c_int, [c_int64]),
    "jg_ln_plain_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
    ),
    "jg_ln_plain_bwd_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "jg_ln_plain_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int,
         c_void_p, c_size_t, c_void_p],
    ),
    "jg_ln_plain_bwd_add": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int,
         c_void_p, c_size_t, c_void_p, c_void_p],
    ),
    "jg_gn_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "jg_gn_partial_sum": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_gn_partial_sqdev": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_gn_apply": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
         c_int, c_void_p],
    ),
    "jg_gn_partial_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
         c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_gn_bwd_apply": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
         c_int64, c_int, c_void_p],
    ),
    "jg_proj_nt_fused": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_void_p],
    ),
    "jg_proj_nt": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_void_p],
    ),
    "jg_proj_tn_workspace": (c_size_t, [c_int64, c_int, c_int]),
    "jg_proj_tn": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_conv_workspace_bytes": (c_size_t, [POINTER(ConvDesc), c_int, c_int]),
    "jg_conv_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, POINTER(ConvDesc), c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_conv_dgrad": (c_int, [c_void_p, c_void_p, c_void_p, POINTER(ConvDesc), c_int, c_void_p, c_size_t, c_void_p]),
    "jg_conv_dgrad_fold": (
        c_int,
        [c_void_p, POINTER(c_void_p), c_void_p, c_void_p, POINTER(ConvDesc), POINTER(HaloGeom), c_int, c_void_p, c_size_t,
         c_void_p],
    ),
    "jg_conv_wgrad": (c_int, [c_void_p, c_void_p, c_void_p, POINTER(ConvDesc), c_int, c_void_p, c_size_t, c_void_p]),
    "jg_conv_frame_bands": (c_int, [POINTER(ConvDesc), POINTER(HaloGeom), c_int, POINTER(c_int32), POINTER(c_int32)]),
    "jg_conv_fwd_framed": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(ConvDesc), POINTER(HaloGeom), c_int, c_void_p,
         c_size_t, c_void_p],
    ),
    "jg_conv_wgrad_framed": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(ConvDesc), POINTER(HaloGeom), c_int, c_void_p,
         c_size_t, c_void_p],
    ),
    "jg_conv_wgrad_bias": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, POINTER(ConvDesc), c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_bias_grad_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "jg_bias_grad": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p]),
    "jg_attn_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float, c_void_p,
         c_int64, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "jg_attn_bwd_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "jg_attn_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
         c_int64, c_int64, c_float, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_attn_bwd_chunks": (
        c_int,
        [c_void_p, POINTER(c_void_p), POINTER(c_void_p), c_void_p, c_void_p, POINTER(c_void_p), POINTER(c_void_p), c_int64,
         c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_attn_swin_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
         c_int64, c_float, c_int, c_void_p],
    ),
    "jg_attn_swin_bwd_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "jg_attn_swin_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "jg_lse_merge": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int,
         c_void_p],
    ),
}


def lib_path() -> Path:
    """Path the built library is expected at."""
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load the library once and declare every entry point's signature."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not _LIB_PATH.exists():
            raise LibraryMissing(
                f"{_LIB_PATH} is not built. Run `python -m jigsaw_amd.build` "
                "(needs hipcc); there is no CPU or PyTorch fallback for these operators."
            )
        lib = ctypes.CDLL(str(_LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def abi_version() -> int:
    return int(load().jg_abi_version())


def check(rc: int, what: str = "") -> None:
    """Raise on a negative status, with the library's own message."""
    if rc == 0:
        return
    msg = load().jg_last_error().decode("utf-8", "replace")
    exc = {-1: ValueError, -2: NotImplementedError}.get(rc, KernelError)
    raise exc(f"{what or 'libjigsaw_hip'}: {msg} (status {rc})")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise NotImplementedError(f"dtype {dtype} is not supported by the HIP kernels") from None


def require_gpu(*tensors: torch.Tensor) -> None:
    """Operators only run on HIP device tensors; say so instead of falling back."""
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "jigsaw_amd operators run on the GPU only (got a tensor on "
                f"{t.device}); there is no CPU path in this package."
            )


def ptr(t: torch.Tensor | None) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device | None = None) -> c_void_p:
    """The current stream of ``device`` as the raw handle the C entry points take. Asked of torch's
    C layer directly where it offers that (a tenth of the time of building a ``torch.cuda.Stream``
    object for every launch, which adds up in steps of 40 launches)."""
    if _raw_stream is not None:
        index = device.index if device is not None and device.index is not None else torch.cuda.current_device()
        return c_void_p(_raw_stream(index))
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def i64_array(values) -> ctypes.Array:
    vals = [int(v) for v in values]
    return (c_int64 * len(vals))(*vals)


__all__ = [
    "ConvDesc",
    "HaloGeom",
    "KernelError",
    "LibraryMissing",
    "SIGNATURES",
    "VoidP27",
    "VoidP9",
    "abi_version",
    "check",
    "dtype_code",
    "i64_array",
    "lib_path",
    "load",
    "ptr",
    "require_gpu",
    "stream_ptr",
    "c_float",
    "c_double",
    "c_size_t",
]
