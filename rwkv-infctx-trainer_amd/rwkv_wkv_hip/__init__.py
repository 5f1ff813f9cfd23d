"""MI355X-native WKV time-mix operators (RWKV v4 / v5 / v6) behind the
reference trainer's autograd call signatures.  See ops.py."""
from ._lib import WKVError, LIB_PATH
from .ops import (WKV_5, WKV_6, RUN_WKV5_CUDA, RUN_WKV6STATE_CUDA, wkv_op, cumsum_decay, set_algo, RecomputeCache,
                  recompute_cache, call_key, stats)

from . import blocks  # noqa: E402,F401  (token shift + mixing, ln_x * gate, channel-mix activations, L2Wrap)

# the reference's class names, same in-place calling convention as its RUN_* wrappers
class WKV5_CUDA:
    apply = staticmethod(RUN_WKV5_CUDA)


class WKV6STATE_CUDA:
    apply = staticmethod(RUN_WKV6STATE_CUDA)


__all__ = ["WKV_5", "WKV_6", "WKV5_CUDA", "WKV6STATE_CUDA", "RUN_WKV5_CUDA", "RUN_WKV6STATE_CUDA", "wkv_op",
           "cumsum_decay", "blocks", "set_algo", "RecomputeCache", "recompute_cache", "call_key", "stats", "WKVError", "LIB_PATH"]
