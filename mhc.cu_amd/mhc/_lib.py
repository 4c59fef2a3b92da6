"""ctypes binding of libmhc_hip.so (the C ABI declared in include/mhc_hip.h).

PyTorch is used for device memory and streams only: tensors are passed as raw device pointers,
work is enqueued on torch's current HIP stream, and the scratch workspace is a cached torch
byte tensor per (device, stream).  There is no CPU or PyTorch fallback: if the library is
missing, importing this module raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MHC_HIP_LIBRARY") or os.path.join(_HERE, "libmhc_hip.so")

MHC_F32, MHC_BF16, MHC_F32_AS_BF16 = 0, 1, 2
MHC_MAX_N = 32
ABI_VERSION = 2

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} not found. Build the HIP library first:\n    python mhc.cu_amd/build.py"
    )

lib = ctypes.CDLL(LIB_PATH)

_P, _I, _F, _Z = c_void_p, c_int, c_float, c_size_t

_SIGNATURES = {
    "mhc_abi_version": (c_int, []),
    "mhc_status_string": (c_char_p, [_I]),
    "mhc_max_sinkhorn_iters": (c_int, [_I]),
    "mhc_layer_dynamic_accepts_f32_as_bf16": (c_int, [_I, _I, _I, _I]),
    "mhc_layer_dynamic_workspace_bytes": (_Z, [_I, _I, _I]),
    "mhc_layer_sinkhorn_state_floats": (_Z, [_I, _I, _I]),
    "mhc_layer_fwd_dynamic": (c_int, [_P, _I, _P, _I, _P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P,
                                      _P, _P, _I, _I, _I, _I, _F, _P, _Z, _P]),
    "mhc_layer_bwd_dynamic": (c_int, [_P, _I, _P, _I, _P, _I, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P,
                                      _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _P, _Z, _P]),
    "mhc_pack_dynamic_params": (c_int, [_P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P]),
    "mhc_static_scratch_capacity": (_Z, []),
    "mhc_layer_fwd_dynamic_scratch_bytes": (_Z, [_I, _I, _I]),
    "mhc_static_scratch_init": (c_int, []),
    "mhc_layer_fwd_dynamic_static_scratch": (c_int, [_P, _I, _P, _I, _P, _I, _P, _P, _P, _P, _I, _P, _P, _P,
                                                     _P, _P, _P, _P, _I, _I, _I, _I, _F, _P]),
    "mhc_layer_static_workspace_bytes": (_Z, [_I, _I, _I]),
    "mhc_layer_fwd": (c_int, [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I,
                              _F, _P, _Z, _P]),
    "mhc_layer_bwd": (c_int, [_P, _I, _P, _I, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P,
                              _P, _P, _I, _I, _I, _I, _F, _P, _Z, _P]),
    "mhc_sinkhorn_knopp_fwd": (c_int, [_P, _P, _I, _I, _I, _I, _F, _P]),
    "mhc_sinkhorn_knopp_bwd": (c_int, [_P, _P, _P, _I, _I, _I, _I, _F, _P, _Z, _P]),
    "mhc_sinkhorn_knopp_bwd_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "mhc_rmsnorm_fwd": (c_int, [_P, _I, _P, _I, _P, _P, _I, _I, _F, _P]),
    "mhc_rmsnorm_bwd": (c_int, [_P, _P, _I, _P, _I, _P, _P, _P, _I, _I, _P, _Z, _P]),
    "mhc_rmsnorm_bwd_workspace_bytes": (_Z, [_I, _I]),
}

def _bind(handle):
    for _name, (_res, _args) in _SIGNATURES.items():
        _fn = getattr(handle, _name)  # AttributeError here means the library does not match the header
        _fn.restype = _res
        _fn.argtypes = _args
    if handle.mhc_abi_version() != ABI_VERSION:
        raise ImportError(f"{handle._name}: ABI {handle.mhc_abi_version()} != binding ABI {ABI_VERSION}")
    return handle


_bind(lib)

_TUNING_LIB = None


def tuning_lib():
    """The test/experiment build of the same library (libmhc_hip_tuning.so, `build.py --tuning`): the same
    entry points plus mhc_tuning_set / mhc_tuning_get, which override the launch heuristics
    (csrc/tuning.h) for the whole process.  The product library above has no such hooks; tests load
    this one to compare two launch paths on the same inputs."""
    global _TUNING_LIB
    if _TUNING_LIB is None:
        path = os.environ.get("MHC_HIP_TUNING_LIBRARY") or os.path.join(_HERE, "libmhc_hip_tuning.so")
        if not os.path.exists(path):
            raise ImportError(f"{path} not found: python mhc.cu_amd/build.py --tuning")
        handle = _bind(ctypes.CDLL(path))
        handle.mhc_tuning_set.restype = c_int
        handle.mhc_tuning_set.argtypes = [c_int, c_int]
        handle.mhc_tuning_get.restype = c_int
        handle.mhc_tuning_get.argtypes = [c_int]
        _TUNING_LIB = handle
    return _TUNING_LIB


class MHCError(RuntimeError):
    def __init__(self, fn, status):
        self.status = status
        super().__init__(f"{fn} failed: {lib.mhc_status_string(status).decode()} (status {status})")


def check(fn, status):
    if status != 0:
        raise MHCError(fn, status)


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return MHC_F32
    if t.dtype == torch.bfloat16:
        return MHC_BF16
    raise TypeError(f"unsupported dtype {t.dtype}: the HIP library takes float32 or bfloat16")


def ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


def require_gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("mhc: tensors must live on a HIP (cuda) device; there is no CPU path")
        if not t.is_contiguous():
            raise RuntimeError("mhc: tensors must be contiguous")


def stream_ptr(device) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


_WORKSPACES: dict = {}


def workspace(device, nbytes: int) -> torch.Tensor:
    """Scratch buffer of at least nbytes for the current stream of `device` (grown on demand).

    Kernels that use it are ordered on that stream, so reuse across calls is safe.
    """
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = buf
    return buf
