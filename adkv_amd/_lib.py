"""ctypes binding of libadkv_hip.so (C ABI: include/adkv_hip.h).

There is deliberately no fallback: if the library is absent or a symbol is missing, importing the
kernels raises.  torch must be imported before the library is opened so that the HIP runtime torch
already loaded (same soname) is the one the kernels register with.
"""
from __future__ import annotations

import ctypes as C
import os

import torch  # noqa: F401  (loads libamdhip64 first)

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "libadkv_hip.so")
ABI_VERSION = 16

_vp, _i, _f = C.c_void_p, C.c_int, C.c_float

# name -> (restype, argtypes); must list every symbol include/adkv_hip.h declares
PROTOTYPES = {
    "adkv_abi_version": (_i, []),
    "adkv_set_mha_kernel": (None, [_i]),
    "adkv_set_fused_step": (None, [_i]),
    "adkv_decode_step_is_fused": (_i, [_i] * 9),
    "adkv_strerror": (C.c_char_p, [_i]),
    "adkv_last_hip_error": (_i, []),
    "adkv_encode_kv": (_i, [_vp] * 7 + [_i] * 5 + [_f, _f, _vp, _vp]),
    "adkv_forward_qk": (_i, [_vp] * 9 + [_i] * 5 + [_f, _f, _vp, _vp]),
    "adkv_forward_ov": (_i, [_vp] * 9 + [_i] * 5 + [_f, _f, _vp, _vp]),
    "adkv_softmax": (_i, [_vp] * 3 + [_i] * 3 + [_f, _vp]),
    "adkv_softmax_workspace_bytes": (C.c_int64, [_i, _i]),
    "adkv_row_pitch": (C.c_int64, [_i]),
    "adkv_softmax_ex": (_i, [_vp] * 3 + [_i, _i, C.c_int64, _i, _f, _vp, C.c_int64, _vp]),
    "adkv_encode_kv_ex": (_i, [_vp] * 7 + [_i] * 5 + [_vp, _vp, _i, _i, _vp]),
    "adkv_append_kv": (_i, [_vp] * 7 + [_i] * 7 + [_vp, _vp, _i, _i, _vp]),
    "adkv_append_kv_pair": (_i, [_vp] * 4 + [_i, _vp, _vp] + [_vp] * 2 + [_i] * 7 + [_vp] * 4 + [_i, _i, _vp]),
    "adkv_forward_qk_ex": (_i, [_vp] * 9 + [_i] * 5 + [_vp, _vp, _i, _i, _vp]),
    "adkv_forward_ov_workspace_bytes": (C.c_int64, [_i] * 6),
    "adkv_forward_ov_ex": (_i, [_vp] * 9 + [_i] * 5 + [_vp, _vp, _i, _i, _vp, C.c_int64, _vp]),
    "adkv_forward_qk_gqa": (_i, [_vp] * 9 + [_i] * 7 + [C.c_int64, _vp, _vp, _i, _i, _vp]),
    "adkv_forward_ov_gqa_workspace_bytes": (C.c_int64, [_i] * 7),
    "adkv_forward_ov_gqa": (_i, [_vp] * 9 + [_i] * 7 + [C.c_int64, _vp, _vp, _i, _i, _vp, C.c_int64, _vp]),
    "adkv_init": (_i, []),
    "adkv_static_scratch_bytes": (C.c_int64, []),
    "adkv_forward_ov_noalloc": (_i, [_vp] * 9 + [_i] * 7 + [C.c_int64, _vp, _vp, _i, _i, _vp]),
    "adkv_decode_step_workspace_bytes": (C.c_int64, [_i] * 7),
    "adkv_decode_step": (_i, [_vp] * 8 + [_i, _f, _vp, _vp, C.c_int64] + [_i] * 8 + [_vp, _vp, _i, _i, _vp,
                                                                            C.c_int64, _vp]),
    "adkv_set_stage_events": (None, [_vp]),
    "adkv_decode_kernel_name": (C.c_char_p, [_i] * 8),
    "adkv_decode_segments": (_i, [_i] * 8 + [_vp, _i, _vp]),
    "adkv_rope_qk": (_i, [_vp] * 6 + [_i] * 5 + [C.c_int64] * 8 + [_i, _vp]),
    "adkv_quant_f32": (_i, [_vp] * 12 + [_i] * 3 + [C.c_int64, C.c_int64] + [_i] * 3 + [_f, _f, _vp]),
    "adkv_fp16_decode_workspace_bytes": (C.c_int64, [_i] * 3),
    "adkv_fp16_decode": (_i, [_vp] * 5 + [C.c_int64] + [_i] * 4 + [_f, _vp]),
}

_lib = None


class ADKVLibraryError(RuntimeError):
    pass


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ADKVLibraryError(
                f"{LIB_PATH} is missing: build it with `python -m adkv_amd.build` "
                "(hipcc --offload-arch=gfx950). There is no CPU fallback.")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            try:
                fn = getattr(L, name)
            except AttributeError as e:
                raise ADKVLibraryError(f"{LIB_PATH} does not export {name}") from e
            fn.restype, fn.argtypes = res, args
        v = L.adkv_abi_version()
        if v != ABI_VERSION:
            raise ADKVLibraryError(f"libadkv_hip ABI {v} != expected {ABI_VERSION}; rebuild")
        _lib = L
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        L = lib()
        msg = L.adkv_strerror(rc).decode()
        if rc == -100:
            msg += f" (hipError {L.adkv_last_hip_error()})"
        raise RuntimeError(f"{what}: {msg}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_ptr(device) -> int:
    """The device's current stream as a ``hipStream_t`` value."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)          # one C call instead of building a Stream object
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device):
    """Context that makes ``device`` current for a launch; free when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)
