"""ctypes binding of librwkv_wkv_hip.so (the C ABI declared in include/rwkv_wkv_hip.h).

The library is prebuilt in-tree by ``make -C rwkv-infctx-trainer_amd/csrc`` (or
``__graft_entry__.build()``).  There is no fallback: if it is missing, loading
raises."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_size_t, c_uint, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("RWKV_WKV_LIB", os.path.join(_HERE, "librwkv_wkv_hip.so"))

WKV_F32, WKV_BF16, WKV_F16 = 0, 1, 2
FLOOR_DECAY = 1
CHECKPOINTS_VALID = 2
W_BF16 = 4          # WKV6, chunked algorithm: w and gw are bf16
ALGO_AUTO, ALGO_RECURRENT, ALGO_CHUNKED = 0, 1, 2
TUNE_SEGMENTS = 1
TUNE_PIECE_STEPS = 2

_P = c_void_p
_I = c_int

# name -> (restype, argtypes); the one list the symbol-export test walks
SIGNATURES = {
    "wkv_strerror": (c_char_p, [_I]),
    "wkv_abi_version": (_I, []),
    "wkv_init": (_I, []),
    "wkv_tune": (_I, [_I, _I]),
    "wkv_profile_begin": (_I, [_I, _I]),
    "wkv_profile_end": (_I, [_P, _I]),
    "wkv6_forward_workspace": (c_size_t, [_I] * 6),
    "wkv6_forward": (_I, [_P, _I, _I, _I, _I, _I, c_uint, _I] + [_P] * 8 + [_P, c_size_t]),
    "wkv6_forward_noalloc": (_I, [_P, _I, _I, _I, _I, _I, c_uint] + [_P] * 8),
    "wkv6_backward_workspace": (c_size_t, [_I] * 6),
    "wkv6_backward": (_I, [_P, _I, _I, _I, _I, _I, c_uint, _I] + [_P] * 14 + [_P, c_size_t]),
    "wkv5_forward_workspace": (c_size_t, [_I] * 6),
    "wkv5_forward": (_I, [_P, _I, _I, _I, _I, _I, c_uint, _I] + [_P] * 8 + [_P, c_size_t]),
    "wkv5_backward_workspace": (c_size_t, [_I] * 6),
    "wkv5_backward": (_I, [_P, _I, _I, _I, _I, _I, c_uint, _I] + [_P] * 14 + [_P, c_size_t]),
    "wkv4_checkpoint_bytes": (c_size_t, [_I] * 3),
    "wkv4_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 8),
    "wkv4_backward_workspace": (c_size_t, [_I] * 4),
    "wkv4_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 13 + [_P, c_size_t]),
    "wkv_cumsum_decay": (_I, [_P, _I, _I, _I, _I, _I] + [_P] * 6),
    "wkv_cumsum_decay_factors": (_I, [_P, _I, _I, _I, _I, _I, _I] + [_P] * 11),
    "wkv_shift_mix_forward": (_I, [_P, _I, _I, _I, _I, _I, _I] + [_P] * 5),
    "wkv_shift_mix_backward_workspace": (c_size_t, [_I] * 4),
    "wkv_shift_mix_backward": (_I, [_P, _I, _I, _I, _I, _I, _I] + [_P] * 9 + [_P, c_size_t]),
    "wkv_lora_mix_forward": (_I, [_P, _I, _I, _I] + [_P] * 6),
    "wkv_lora_mix_backward_workspace": (c_size_t, [_I] * 3),
    "wkv_lora_mix_backward": (_I, [_P, _I, _I, _I] + [_P] * 10 + [_P, c_size_t]),
    "wkv_ln_gate_forward": (_I, [_P, _I, _I, _I, c_float, c_float] + [_P] * 5),
    "wkv_ln_gate_backward_workspace": (c_size_t, [_I] * 2),
    "wkv_ln_gate_backward": (_I, [_P, _I, _I, _I, c_float, c_float] + [_P] * 8 + [_P, c_size_t]),
    "wkv_relu_square_forward": (_I, [_P, c_size_t, _I, _P, _P]),
    "wkv_relu_square_backward": (_I, [_P, c_size_t, _I, _P, _P, _P]),
    "wkv_sigmoid_mul_forward": (_I, [_P, c_size_t, _I, _P, _P, _P]),
    "wkv_sigmoid_mul_backward": (_I, [_P, c_size_t, _I] + [_P] * 5),
    "wkv_l2wrap_backward": (_I, [_P, _I, _I, _I, c_float, _P, _P, _P]),
}

_lib = None


class WKVError(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise WKVError(
                f"{LIB_PATH} is missing: build the HIP library first "
                "(make -C rwkv-infctx-trainer_amd/csrc).  There is no CPU fallback.")
        import torch  # noqa: F401  (first, so that both share one HIP runtime)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
        try:
            import torch
            if torch.cuda.is_available():
                L.wkv_init()         # so that no operator call has set-up left to do (e.g. inside a graph capture)
        except Exception:            # noqa: BLE001 - set-up then happens on the first call
            pass
    return _lib


def check(status: int, what: str):
    if status != 0:
        msg = lib().wkv_strerror(status).decode()
        if status in (-1, -3):
            raise ValueError(f"{what}: {msg}")
        raise WKVError(f"{what}: {msg} (status {status})")
