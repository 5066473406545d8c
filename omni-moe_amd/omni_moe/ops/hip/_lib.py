"""ctypes binding of libomni_moe_hip.so (the C ABI declared in include/omni_moe_hip.h).

The library is loaded after ``import torch`` so that its HIP symbols bind to the HIP
runtime torch has already loaded (same soname), which makes torch's streams and device
pointers valid inside it.  There is no fallback: if the library is missing or a call
is made without a GPU, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p

import torch  # noqa: F401  (must precede loading the library)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libomni_moe_hip.so")

OMNI_BF16, OMNI_F16, OMNI_F32 = 0, 1, 2
ALGO_AUTO, ALGO_GATHER, ALGO_SEGMENT, ALGO_SPLIT, ALGO_DENSE = 0, 1, 2, 3, 4
ERR_TOPK, ERR_SHAPE, ERR_UNSUPPORTED = -4, -2, -5

DTYPE_CODE = {torch.bfloat16: OMNI_BF16, torch.float16: OMNI_F16, torch.float32: OMNI_F32}

# name -> (restype, argtypes); mirrors include/omni_moe_hip.h one to one
SIGNATURES = {
    "omni_abi_version": (c_int32, []),
    "omni_error_string": (c_char_p, [c_int32]),
    "omni_init": (c_int32, []),
    "omni_router_select": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "omni_schedule_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int64]),
    "omni_schedule": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int64, c_void_p, c_void_p]),
    "omni_schedule_noalloc": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int64, c_void_p]),
    "omni_expert_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int64, c_int32, c_int32, c_int32]),
    "omni_mlp_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int32, c_int32]),
    "omni_mlp_fwd": (c_int32, [c_void_p] * 6 + [c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "omni_linear_fwd": (c_int32, [c_void_p] * 4 + [c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "omni_swiglu_linear_fwd": (c_int32, [c_void_p] * 4 + [c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "omni_swiglu_linear_fwd_shared": (c_int32, [c_void_p] * 4 + [c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "omni_swiglu_linear_save_fwd": (c_int32, [c_void_p] * 6 + [c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "omni_moe_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int32, c_int64, c_int32, c_int32, c_int32]),
    "omni_moe_fwd": (c_int32, [c_void_p] * 15 + [c_int64, c_int32, c_int32, c_int64, c_int32, c_int32, c_int32, c_int32,
                               c_int32, c_float, c_float] + [c_void_p] * 5),
    "omni_moe_workspace_bytes_algo": (c_size_t, [c_int64, c_int32, c_int32, c_int64, c_int32, c_int32, c_int32, c_int32]),
    "omni_moe_fwd_algo": (c_int32, [c_void_p] * 15 + [c_int64, c_int32, c_int32, c_int64, c_int32, c_int32, c_int32, c_int32,
                                    c_int32, c_float, c_float] + [c_void_p] * 5 + [c_int32]),
    "omni_probe_mfma": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "omni_probe_mfma16": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "omni_add_inplace": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    "omni_linear2_fwd": (c_int32, [c_void_p] * 4 + [c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "omni_router_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int32]),
    "omni_router_fwd": (c_int32, [c_void_p] * 9 + [c_int32, c_float, c_float, c_void_p, c_void_p, c_void_p,
                                  c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "omni_expert_fwd": (c_int32, [c_void_p] * 6 + [c_int64, c_int32, c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "omni_router_bwd": (c_int32, [c_void_p] * 4 + [c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "omni_expert_bwd_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int64, c_int32, c_int32]),
    "omni_expert_bwd": (c_int32, [c_void_p] * 10 + [c_int64, c_int32, c_int64, c_int32, c_int32, c_void_p, c_void_p]),
    "omni_swiglu_fwd": (c_int32, [c_void_p] * 3 + [c_int64, c_int32, c_void_p]),
    "omni_swiglu_bwd": (c_int32, [c_void_p] * 5 + [c_int64, c_int32, c_void_p]),
    "omni_router_workspace_stats_offset": (c_size_t, [c_int64, c_int32, c_int32]),
    "omni_router_norm_bwd_workspace_bytes": (c_size_t, [c_int64, c_int32]),
    "omni_router_norm_bwd": (c_int32, [c_void_p] * 6 + [c_int64, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
}

_lib = None


class OmniHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Loads the library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OmniHipError(
                f"{LIB_PATH} is missing: build it with `python -m omni_moe.ops.hip.build` "
                "(there is no non-HIP fallback for this path)")
        lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_LOCAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    if code == 0:
        return
    msg = load().omni_error_string(code).decode()
    if code == ERR_TOPK:
        raise AssertionError(f"{what}: {msg}")          # the reference asserts (utils.py:81-104)
    if code < 0:
        raise ValueError(f"{what}: {msg} (code {code})")
    raise OmniHipError(f"{what}: {msg} (code {code})")


_prepared_devices = set()


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise OmniHipError("omni_moe HIP ops need tensors on an AMD GPU (device type 'cuda' under ROCm); got %s" % dev)
    for t in tensors:
        if t.device != dev:
            raise ValueError("all tensors must be on the same device")
    if dev.index not in _prepared_devices:
        # kernel attributes and the device scratch, once per device and before any launch, so that none of it
        # can fall inside a later stream capture
        with torch.cuda.device(dev):
            check(load().omni_init(), "omni_init")
        _prepared_devices.add(dev.index)
    return dev


def ptr(t) -> int:
    return 0 if t is None or t.numel() == 0 else t.data_ptr()


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream
