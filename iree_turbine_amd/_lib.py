"""ctypes binding of libturbine_mi355.so (the C ABI declared in include/turbine_mi355.h).

The library is the only implementation of the kernels: when it is missing or a call fails,
this module raises; nothing falls back to a CPU or eager-PyTorch path.

The reference reaches HIP the same way, through ctypes on libamdhip64
(iree/turbine/runtime/device.py:86-150).
"""

from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

import torch  # noqa: F401  (must be imported first: it loads the HIP runtime this library links to)

LIB_PATH = Path(__file__).resolve().parent / "csrc" / "libturbine_mi355.so"

F32, F16, BF16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

_lock = threading.Lock()
_lib = None

_PROTOS = {
    "mi355_abi_version": (c_int, []),
    "mi355_last_error": (c_char_p, []),
    "mi355_build_flags": (c_char_p, []),
    "mi355_variant_count": (c_int, [c_char_p]),
    "mi355_variant_name": (c_char_p, [c_char_p, c_int]),
    "mi355_gemm_f16_nt": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p]),
    "mi355_gemm_bf16_nt": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p]),
    "mi355_gemm_nt_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64]),
    "mi355_gemm_f16_nt_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_int64, c_void_p]),
    "mi355_gemm_bf16_nt_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_int64, c_void_p]),
    "mi355_flash_attn_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
    ),
    "mi355_flash_attn_fwd_strided": (
        c_int,
        [c_void_p] * 4 + [c_int64] * 6 + [ctypes.POINTER(c_int64)] * 4 + [c_float, c_int, c_int, c_void_p],
    ),
    "mi355_flash_attn_fwd_bf16": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
    ),
    "mi355_flash_attn_fwd_strided_bf16": (
        c_int,
        [c_void_p] * 4 + [c_int64] * 6 + [ctypes.POINTER(c_int64)] * 4 + [c_float, c_int, c_int, c_void_p],
    ),
    "mi355_paged_decode_phase0": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
        + [c_int64] * 8
        + [c_float, c_void_p],
    ),
    "mi355_paged_decode_phase1": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "mi355_paged_decode_phase0_bf16": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
        + [c_int64] * 8
        + [c_float, c_void_p],
    ),
    "mi355_paged_decode_phase1_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "mi355_paged_decode_attn": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
        + [c_int64] * 8
        + [c_float, c_void_p],
    ),
    "mi355_paged_decode_attn_fused": (c_int, [c_void_p] * 9 + [c_int64] * 8 + [c_float, c_int64, c_int, c_void_p]),
    "mi355_paged_decode_attn_static": (c_int, [c_void_p] * 6 + [c_int64] * 8 + [c_float, c_void_p]),
    "mi355_paged_decode_attn_window": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
        + [c_int64] * 8
        + [c_float, c_int64, c_void_p],
    ),
    "mi355_paged_decode_attn_window_bf16": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
        + [c_int64] * 8
        + [c_float, c_int64, c_void_p],
    ),
    "mi355_kv_cache_append": (c_int, [c_void_p] * 6 + [c_int64] * 7 + [c_void_p]),
    "mi355_paged_prefill_attn": (c_int, [c_void_p] * 6 + [c_int64] * 8 + [c_float, c_void_p]),
    "mi355_paged_prefill_attn_bf16": (c_int, [c_void_p] * 6 + [c_int64] * 8 + [c_float, c_void_p]),
    "mi355_mxfp4_gemm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p],
    ),
    "mi355_mxfp8_gemm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p],
    ),
    "mi355_mxfp6_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "mi355_fp8_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p]),
    "mi355_calibrate_mfma": (c_int, [c_int, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, ctypes.POINTER(ctypes.c_double), c_void_p]),
    "mi355_calibrate_fa_issue": (c_int, [c_int, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, ctypes.POINTER(ctypes.c_double), c_void_p]),
    "mi355_mxfp4_dequant": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "mi355_mxfp4_quantize": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p]),
    "mi355_mxfp6_quantize": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p]),
    "mi355_mxfp8_quantize": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_PROTOS)


class KernelLibraryError(RuntimeError):
    """Raised when the kernel library is missing, or a kernel call reports an error."""


def load():
    """Loads the shared library once per process (under a lock, like op registration in the
    reference, iree/turbine/runtime/op_reg/base.py:63)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise KernelLibraryError(
                f"{LIB_PATH} is missing: build it with `python -m iree_turbine_amd.build` "
                "(there is no fallback implementation)"
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in _PROTOS.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.mi355_abi_version() != 1:
            raise KernelLibraryError(f"ABI version mismatch: library reports {lib.mi355_abi_version()}, binding expects 1")
        _lib = lib
    return _lib


def build_flags() -> str:
    """The timing-only ablation switches the loaded library was built with ("" for the product build)."""
    return (load().mi355_build_flags() or b"").decode().strip()


def last_error() -> str:
    msg = load().mi355_last_error()
    return msg.decode() if msg else ""


def check(rc: int, what: str) -> None:
    if rc == 0:
        return
    kind = "contract violation" if rc < 0 else "HIP error"
    exc = ValueError if rc < 0 else KernelLibraryError
    raise exc(f"{what}: {kind} {rc}: {last_error()}")


def variants(family: str) -> list[str]:
    lib = load()
    fam = family.encode()
    return [lib.mi355_variant_name(fam, i).decode() for i in range(lib.mi355_variant_count(fam))]


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"unsupported output dtype {dtype}") from None


def current_stream_ptr(device: torch.device) -> int:
    """The raw hipStream_t of torch's current stream on `device`: every launch is ordered on it
    (the reference orders its launches on the same stream, iree/turbine/runtime/device.py:336-361)."""
    return torch.cuda.current_stream(device).cuda_stream
