"""ctypes binding of libparoatten_hip.so (the C ABI declared in include/paroatten.h).

The library is the only compute path of this package: if it is missing or cannot be loaded the
import of any operator raises, there is no fallback.  Error codes of the C ABI map back to the
exception types the reference's extension raises (csrc/utils.cuh:20-38 -> RuntimeError;
csrc/dispatch_utils.h:23-112 -> ValueError).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

import torch

PARO_OK = 0
PARO_ERR_INVALID_VALUE = -1
PARO_ERR_RUNTIME = -2
PARO_ERR_UNSUPPORTED = -3
PARO_ERR_HIP = -4
PARO_ATTN_EXACT_EXP = 1
PARO_ATTN_PACED = 2
PARO_ATTN_UNPACED = 4
PARO_ATTN_TWO_WAVES = 8
PARO_ATTN_PV_F16 = 16
PARO_ATTN_QK_PER_THREAD = 32

DTYPE_CODE = {torch.float16: 0, torch.bfloat16: 1}

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libparoatten_hip.so"

_I, _L, _F, _P = c_int, c_int64, c_float, c_void_p

# name -> (restype, argtypes); kept next to the header so that the loader can verify every export
SIGNATURES = {
    "paro_abi_version": (c_int, []),
    "paro_last_error": (c_char_p, []),
    "paro_build_arch": (c_char_p, []),
    "paro_quant_int8": (c_int, [_P, _I, _P, _P, _P, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                                _I, _I, _I, _F, _P]),
    "paro_quant_int8_per_thread": (c_int, [_P, _I, _P, _P, _P, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _L, _L,
                                           _I, _P]),
    "paro_v_fp8_bytes": (c_int64, [_I, _I, _I, _I]),
    "paro_v_fp8_partial_floats": (c_int64, [_I, _I, _I, _I]),
    "paro_v_fp8_pack": (c_int, [_P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _L, _L, _L, _I, _P]),
    "paro_attn_sparse_fwd": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _I, _P, _P,
                                     _I, _I, _I, _I, _I, _I,
                                     _L, _L, _L, _L, _L, _L, _L, _L, _L, _F, _I, _I, _P]),
    "paro_attn_sparse_unpermute_fwd": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _I, _P,
                                               _I, _I, _I, _I, _I, _I,
                                               _L, _L, _L, _L, _L, _L, _L, _L, _L, _F, _I, _I,
                                               _P, _I, _I, _I, _I, _P]),
    "paro_attn_workspace_bytes": (c_int64, [_I, _I, _I, _I]),
    "paro_attn_workspace_bytes_for": (c_int64, [_I, _I, _I, _I, _I]),
    "paro_v_f16_bytes": (c_int64, [_I, _I, _I, _I]),
    "paro_v_f16_pack": (c_int, [_P, _I, _P, _I, _I, _I, _I, _L, _L, _L, _P]),
    "paro_qk_int8_sv_f16_attn": (c_int, [_P, _P, _P, _I, _P, _I, _P, _P, _P, _L, _P, _P, _L,
                                         _I, _I, _I, _I, _I, _I,
                                         _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                                         _I, _I, _I, _F, _I, _I, _P]),
    "paro_rope_permute_fwd": (c_int, [_P, _P, _P, _P, _P, _P, _I, _P, _P, _P,
                                      _I, _I, _I, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _P]),
    "paro_permute_inv": (c_int, [_P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _P]),
    "paro_permute_index_map": (c_int, [_P, _P, _I, _I, _I, _I, _P]),
    "paro_prep_workspace_bytes": (c_int64, [_I, _I, _I, _I]),
    "paro_rope_permute_quant_fwd": (c_int, [_P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L,
                                            _I, _I, _I, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                                            _L, _L, _I, _P]),
    "paro_prep_smooth_workspace_bytes": (c_int64, [_I, _I, _I, _I]),
    "paro_rope_k_mean_permute_quant_fwd": (c_int, [_P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L,
                                                   _I, _I, _I, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                                                   _L, _L, _I, _P]),
    "paro_rope_k_mean": (c_int, [_P, _I, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _I, _I,
                                 _L, _L, _L, _L, _L, _P]),
    "paro_rope_k_mean_static": (c_int, [_P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I,
                                        _L, _L, _L, _L, _L, _P]),
    "paro_mask_bits_bytes": (c_int64, [_L]),
    "paro_mask_pack": (c_int, [_P, _P, _L, _P]),
    "paro_mask_unpack": (c_int, [_P, _P, _L, _P]),
    "paro_transpose_pad_permute": (c_int, [_P, _P, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _P]),
    "paro_channel_quant_fp8": (c_int, [_P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F,
                                       _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _P]),
    "paro_sub_mean": (c_int, [_P, _I, _P, _P, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _L, _L, _P]),
}

_lib = None


def load():
    """Load the shared library once; raise loudly if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    path = Path(os.environ.get("PAROATTEN_LIB", LIB_PATH))
    if not path.exists():
        raise ImportError(
            f"{path} is not built: run `python paroatten_amd/build.py` (hipcc, gfx950). "
            "paroatten_amd has no fallback path."
        )
    lib = ctypes.CDLL(str(path))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the export is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int):
    if rc == PARO_OK:
        return
    msg = load().paro_last_error().decode()
    if rc == PARO_ERR_INVALID_VALUE:
        raise ValueError(msg)
    if rc == PARO_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)


def ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def stream_of(t: torch.Tensor):
    """Current HIP stream of the tensor's device, as void*."""
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def require_gpu(t: torch.Tensor, name: str):
    # same wording as CHECK_CUDA of the reference (csrc/utils.cuh:20-21)
    if not t.is_cuda:
        raise RuntimeError(f"Tensor {name} must be a CUDA tensor")


class _OnDevice:
    """`on(t).paro_xxx(args)`: the C ABI launches on the CURRENT device, so the call runs under a
    device guard for the tensor's device (the reference works around the missing guard with
    torch.cuda.set_device, paroattention/core.py:168-174) and its return code goes through check()."""

    def __init__(self, t):
        self._device = t.device

    def __getattr__(self, name):
        fn = getattr(load(), name)

        def call(*args):
            with torch.cuda.device(self._device):
                check(fn(*args))
        return call


def on(t: torch.Tensor) -> _OnDevice:
    return _OnDevice(t)
