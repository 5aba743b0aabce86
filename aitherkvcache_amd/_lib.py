"""ctypes binding of libaitherkv_hip.so (the C ABI declared in include/aitherkv.h).

There is no CPU path behind these functions: if the shared library is missing or a
tensor is not on a HIP device the call raises.  Build the library with
`make -C aitherkvcache_amd/csrc` (or `python -c "import __graft_entry__ as g; g.build()"`).
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libaitherkv_hip.so")

AKV_OK, AKV_ERR_INVALID, AKV_ERR_UNSUPPORTED, AKV_ERR_WORKSPACE, AKV_ERR_HIP = range(5)
AKV_F16, AKV_BF16, AKV_F32 = 0, 1, 2
AKV_I32, AKV_I64 = 0, 1
HYB_TABLE_FLOATS = 288

_DTYPE = {torch.float16: AKV_F16, torch.bfloat16: AKV_BF16, torch.float32: AKV_F32}
_ITYPE = {torch.int32: AKV_I32, torch.int64: AKV_I64}

_p, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float

# name -> (restype, argtypes); must list every symbol include/aitherkv.h declares
SIGNATURES = {
    "akv_version": (C.c_char_p, []),
    "akv_last_error": (C.c_char_p, []),
    "akv_device_cu_count": (_i, [C.POINTER(C.c_int)]),
    "akv_profile_enable": (_i, [_i]),
    "akv_profile_last_ms": (_i, [C.POINTER(C.c_float)]),
    "akv_profile_mean_ms": (_i, [C.POINTER(C.c_float), C.POINTER(C.c_int)]),
    "akv_rotation_prepared_bytes": (_sz, [_i]),
    "akv_rotation_prepare": (_i, [_p, _i, _p, _sz, _p]),
    "akv_quantize_pack": (_i, [_p, _i64, _i, _i64, _p, _i, _p, _i64, _p]),
    "akv_unpack_lookup": (_i, [_p, _i64, _i, _i64, _p, _i, _p, _i64, _p]),
    "akv_encode": (_i, [_p, _i, _i64, _i, _i64, _p, _p, _i, _p, _i64, _p, _p]),
    "akv_encode_paged": (_i, [_p, _i, _i64, _i, _i, _i64, _i64, _p, _i, _p, _p, _i,
                              _p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _i, _i64, _p]),
    "akv_encode_paged_kv": (_i, [_p, _p, _i, _i64, _i, _i, _i64, _i64, _p, _i, _p, _p, _i,
                                 _p, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64, _i, _i64, _p]),
    "akv_decode": (_i, [_p, _i64, _p, _i64, _i, _p, _p, _i, _p, _i, _i64, _p]),
    "akv_decode_blocks": (_i, [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _i, _i64, _i64,
                               _i, _i, _i, _p, _p, _i, _p, _i, _i64, _i64, _i64, _p]),
    "akv_paged_attn_workspace_bytes": (_sz, [_i, _i, _i]),
    "akv_paged_attn": (_i, [_p, _i, _i64, _i64,
                            _p, _i64, _i64, _i64, _p, _i64, _i64, _i64,
                            _p, _i64, _i64, _i64, _p, _i64, _i64, _i64,
                            _p, _i, _i64, _p, _i,
                            _p, _p, _i,
                            _p, _i, _i64, _i64,
                            _i, _i, _i, _i, _i, _i64, _i64, _f,
                            _p, _sz, _p]),
    "akv_paged_attn_static_scratch_bytes": (_sz, []),
    "akv_paged_attn_static": (_i, [_p, _i, _i64, _i64,
                                   _p, _i64, _i64, _i64, _p, _i64, _i64, _i64,
                                   _p, _i64, _i64, _i64, _p, _i64, _i64, _i64,
                                   _p, _i, _i64, _p, _i,
                                   _p, _p, _i,
                                   _p, _i, _i64, _i64,
                                   _i, _i, _i, _i, _i, _i64, _i64, _f,
                                   _p]),
    "akv_paged_attn_status": (_i, [_p, C.POINTER(C.c_int), _p]),
    "akv_debug_set_handoff_spin_limit": (_i, [_i]),
    "akv_debug_read_probe": (_i, [_p, _sz, _p, _p]),
    "akv_hybrid_encode": (_i, [_p, _i, _i64, _i64, _p, _p, _i64, _p]),
    "akv_hybrid_encode_paged": (_i, [_p, _i, _i64, _i, _i64, _i64, _p, _i, _p,
                                     _p, _i64, _i64, _i64, _i, _i64, _p]),
    "akv_hybrid_encode_paged_kv": (_i, [_p, _p, _i, _i64, _i, _i64, _i64, _p, _i, _p,
                                        _p, _p, _i64, _i64, _i64, _i, _i64, _p]),
    "akv_hybrid_decode": (_i, [_p, _i64, _i64, _p, _p, _i64, _p]),
    "akv_hybrid_paged_attn_workspace_bytes": (_sz, [_i, _i]),
    "akv_hybrid_paged_attn": (_i, [_p, _i, _i64, _i64,
                                   _p, _i64, _i64, _i64, _p, _i64, _i64, _i64,
                                   _p, _i, _i64, _p, _i, _p,
                                   _p, _i, _i64, _i64,
                                   _i, _i, _i, _i, _i64, _i64, _f,
                                   _p, _sz, _p]),
    "akv_hybrid25_encode": (_i, [_p, _i, _i64, _i64, _p, _p, _i64, _p]),
    "akv_hybrid25_encode_paged": (_i, [_p, _i, _i64, _i, _i64, _i64, _p, _i, _p,
                                       _p, _i64, _i64, _i64, _i, _i64, _p]),
    "akv_hybrid25_encode_paged_kv": (_i, [_p, _p, _i, _i64, _i, _i64, _i64, _p, _i, _p,
                                          _p, _p, _i64, _i64, _i64, _i, _i64, _p]),
    "akv_hybrid25_decode": (_i, [_p, _i64, _i64, _p, _p, _i64, _p]),
    "akv_hybrid25_paged_attn": (_i, [_p, _i, _i64, _i64,
                                     _p, _i64, _i64, _i64, _p, _i64, _i64, _i64,
                                     _p, _i, _i64, _p, _i, _p,
                                     _p, _i, _i64, _i64,
                                     _i, _i, _i, _i, _i64, _i64, _f,
                                     _p, _sz, _p]),
    "akv_block_rep_update": (_i, [_p, _i, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _p, _p, _p, _i64, _i, _i, _p]),
    "akv_block_rep_finalize": (_i, [_p, _i, _i64, _p, _p, _p, _p, _p, _i64, _i, _i, _p]),
    "akv_block_scores": (_i, [_p, _p, _p, _p, _p, _i, _i64, _p, _i, _i, _i, _i, _i, _i64, _i, _i64, _p, _p]),
    "akv_block_select": (_i, [_p, _p, _i, _i64, _p, _i, _i, _i64, _i, _i, _i, _i, _p, _p, _p]),
    "akv_tri_encode": (_i, [_p, _i, _i64, _i, _i64, _i, _i, _p, _p, _p, _p]),
    "akv_tri_encode_paged": (_i, [_p, _i, _i64, _i, _i, _i64, _i64, _i, _p, _i, _i64, _p, _p, _p, _p]),
    "akv_tri_decode_workspace_bytes": (_sz, [_i, _i, _i]),
    "akv_tri_scores": (_i, [_p, _i, _p, _p, _p, _p, _p, _i, _p, _i, _p, _i, _i64, _i, _i, _i, _i, _i, _i, _p]),
    "akv_tri_decode_step": (_i, [_p, _i, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i,
                                 _p, _i, _i64, _i, _i, _i, _i, _i, _i, _p, _sz, _p]),
    "akv_tri_decode_paged": (_i, [_p, _i, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i64, _p, _i,
                                  _p, _i, _i64, _i, _i64, _i, _i, _i, _i, _i, _p, _sz, _p]),
}

_lib: Optional[C.CDLL] = None


def available() -> bool:
    """True when the shared library has been built (says nothing about a GPU being present)."""
    return os.path.exists(LIB_PATH)


def lib() -> C.CDLL:
    """Load (once) and return the library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} not found: the HIP extension is not built and there is no CPU "
                "fallback. Run `make -C aitherkvcache_amd/csrc`.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


class AkvError(RuntimeError):
    pass


def check(rc: int) -> None:
    """Map an akv_status to the exception the reference API raises in that situation."""
    if rc == AKV_OK:
        return
    msg = lib().akv_last_error().decode("utf-8", "replace")
    if rc == AKV_ERR_INVALID:
        raise ValueError(msg)
    if rc == AKV_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise AkvError(f"akv status {rc}: {msg}")


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported floating dtype {t.dtype}; use float16, bfloat16 or float32")


def itype_code(t: torch.Tensor) -> int:
    try:
        return _ITYPE[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported index dtype {t.dtype}; use int32 or int64")


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    """All tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "aitherkvcache_amd runs on MI355X HIP devices only: got a tensor on "
                f"'{t.device}'. There is no CPU implementation in this package.")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError(f"tensors on different devices: {dev} and {t.device}")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device) -> int:
    """Handle of torch's current stream on `device` (what the kernels are launched on)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def attn_status(workspace: Optional[torch.Tensor]) -> int:
    """Status word of the most recent attention call on `workspace` (0 = clean)."""
    if workspace is None:
        return 0
    flags = C.c_int(0)
    check(lib().akv_paged_attn_status(workspace.data_ptr(), C.byref(flags), stream_ptr(workspace.device)))
    return flags.value


def attn_status_static(device) -> int:
    """Status word of the most recent akv_paged_attn_static call on `device` (the built-in scratch array)."""
    flags = C.c_int(0)
    with torch.cuda.device(device):
        check(lib().akv_paged_attn_status(None, C.byref(flags), stream_ptr(device)))
    return flags.value


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()
