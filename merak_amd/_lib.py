"""ctypes binding of ``libmerak_tp_gfx950.so`` (the C ABI in
``include/merak_tp_gfx950.h``).

The library is the only compute path of this package: there is no CPU or
eager-PyTorch fallback.  ``lib()`` raises if the shared object has not been
built, and every wrapper raises ``RuntimeError`` with the library's own message
when an entry point reports an error.  ctypes releases the GIL for the
duration of each call, so forward (main thread) and backward (autograd
thread) launches never block each other on the interpreter lock.
"""
from __future__ import annotations

import ctypes as C
import os
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libmerak_tp_gfx950.so"

MTP_F32, MTP_BF16, MTP_F16 = 0, 1, 2
EPI_NONE, EPI_BIAS, EPI_BIAS_GELU, EPI_SWIGLU, EPI_GELU = 0, 1, 2, 3, 4
ABI_VERSION = 12

_i64, _int, _vp = C.c_int64, C.c_int, C.c_void_p

# name -> (restype, argtypes); mirrors include/merak_tp_gfx950.h one to one
SIGNATURES = {
    "mtp_abi_version": (_int, []),
    "mtp_last_error": (C.c_char_p, []),
    "mtp_device_arch": (_int, [C.c_char_p, _int]),
    "mtp_linear_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    "mtp_linear_dgrad": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "mtp_linear_wgrad": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "mtp_linear_bias_grad": (_int, [_vp, _vp, _i64, _i64, _int, _int, _int, _vp]),
    "mtp_linear_workspace_bytes": (_i64, []),
    "mtp_linear_workspace_need": (_i64, [_int, _i64, _i64, _i64, _int]),
    "mtp_linear_fwd_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "mtp_linear_dgrad_ws": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "mtp_linear_wgrad_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "mtp_linear_bwd_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "mtp_activation_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "mtp_embedding_gather": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "mtp_embedding_bwd_workspace_bytes": (_i64, [_i64, _i64]),
    "mtp_embedding_bwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _i64, _i64, _vp]),
    "mtp_vocab_ce_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "mtp_vocab_ce_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "mtp_vocab_ce_fwd_bwd": (_int, [_vp, _vp, _vp, C.c_float, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "mtp_vocab_ce_fwd_bwd_max_vocab": (_i64, [_int]),
    "mtp_vocab_ce_rescale": (_int, [_vp, _vp, C.c_float, _i64, _i64, _int, _vp]),
    "mtp_gemv": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    "mtp_gemv_argmax_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "mtp_gemv_argmax": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "mtp_gemv_argmax_noalloc_max_bytes": (_i64, []),
    "mtp_gemv_argmax_noalloc": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "mtp_argmax_rows": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "mtp_sample_workspace_bytes": (_i64, [_i64]),
    "mtp_sample_top_k_top_p": (_int, [_vp, _int, _i64, _i64, C.c_float, _int, C.c_float, _vp, _vp, _vp, _vp, _i64, _vp]),
    "mtp_gemv_workspace_bytes": (_i64, [_i64, _i64, _i64, _int]),
    "mtp_gemv_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "mtp_gemv_norm_fits": (_int, [_i64, _i64]),
    "mtp_gemv_pair": (_int, [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _int, _vp]),
    "mtp_gemv_fused": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, C.c_float, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int,
                              _int, _vp]),
    "mtp_rmsnorm": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, C.c_float, _int, _vp]),
    "mtp_rope_kv_append": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _int, _i64, _i64, _int, _vp]),
    "mtp_attn_decode_workspace_bytes": (_i64, [_i64, _int, _int, _i64]),
    "mtp_attn_decode": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _int, _i64, _i64, C.c_float, _int, _vp]),
    "mtp_attn_decode_append": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _int, _i64, _i64, _i64,
                                      C.c_float, _int, _vp]),
    "mtp_reload_tuning": (None, []),
    "mtp_stream_copy": (_int, [_vp, _vp, _i64, _vp]),
    "mtp_mfma_peak": (_int, [_vp, _i64, _i64, _int, _vp]),
    "mtp_mfma_peak_gemm_loop": (_int, [_vp, _i64, _i64, _int, _vp]),
}

_lock = threading.Lock()
_lib = None


class KernelLibraryMissing(RuntimeError):
    pass


def lib() -> C.CDLL:
    """Load the kernel library once.  Never builds: run ``python -m merak_amd.build``."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = Path(os.environ.get("MERAK_AMD_LIB", LIB_PATH))
        if not path.exists():
            raise KernelLibraryMissing(
                f"{path} is missing: the gfx950 kernels are the only compute path of merak_amd "
                "(no CPU/eager fallback). Build them with `python -m merak_amd.build`."
            )
        handle = C.CDLL(str(path))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError here = header and library disagree
            fn.restype = res
            fn.argtypes = args
        got = handle.mtp_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{path}: ABI version {got}, this package expects {ABI_VERSION}")
        _lib = handle
        return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().mtp_last_error().decode(errors="replace")
        raise RuntimeError(f"{what} failed ({rc}): {msg}")


def device_arch() -> str:
    buf = C.create_string_buffer(64)
    check(lib().mtp_device_arch(buf, 64), "mtp_device_arch")
    return buf.value.decode()
