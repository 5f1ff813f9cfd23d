"""No-GPU checks of the C ABI: the library loads, exports every function the
header declares, and rejects bad arguments before touching the GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rwkv_wkv_hip.h")


@pytest.fixture(scope="module")
def L():
    from rwkv_wkv_hip import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return _lib.lib()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wkv[0-9a-z_]*)\s*\(", text)))


def test_header_symbols_exported(L):
    from rwkv_wkv_hip import _lib
    names = declared_functions()
    assert len(names) >= 15
    for n in names:
        assert hasattr(L, n), f"{n} declared in the header but not exported"
    assert set(names) == set(_lib.SIGNATURES), "python binding and header disagree"


def test_version_and_messages(L):
    assert L.wkv_abi_version() == 2
    assert L.wkv_strerror(0) == b"ok"
    for code in range(-8, 0):
        assert L.wkv_strerror(code) not in (b"ok", b"unknown status")


def test_argument_checks_return_before_any_launch(L):
    null = None
    one = ctypes.c_void_p(16)        # never dereferenced: the checks fail first
    # C != H*64
    assert L.wkv6_forward(null, 1, 8, 100, 2, 1, 0, 0, one, one, one, one, one, one, one, one, null, 0) == -1
    # non-positive T
    assert L.wkv5_forward(null, 1, 0, 64, 1, 1, 0, 0, one, one, one, one, one, one, one, one, null, 0) == -1
    # a sequence too long for 32-bit byte offsets (T*C = 2^30)
    assert L.wkv6_forward(null, 1, 1 << 18, 4096, 64, 1, 0, 0, one, one, one, one, one, one, one, one, null, 0) == -1
    # dtype out of range
    assert L.wkv6_forward(null, 1, 8, 64, 1, 7, 0, 0, one, one, one, one, one, one, one, one, null, 0) == -3
    # NULL r
    assert L.wkv6_forward(null, 1, 8, 64, 1, 1, 0, 0, null, one, one, one, one, one, one, one, null, 0) == -2
    # misaligned pointer
    odd = ctypes.c_void_p(24)
    assert L.wkv6_forward(null, 1, 8, 64, 1, 1, 0, 0, odd, one, one, one, one, one, one, one, null, 0) == -4
    # state_out overlapping state_in
    assert L.wkv6_forward(null, 1, 8, 64, 1, 1, 0, 0, one, one, one, one, one, ctypes.c_void_p(4096), one,
                          ctypes.c_void_p(4096 + 64), null, 0) == -8
    # backward: workspace too small
    need = L.wkv6_backward_workspace(1, 8, 64, 1, 1, 0)
    assert need > 0
    args = [one] * 14
    assert L.wkv6_backward(null, 1, 8, 64, 1, 1, 1, 0, *args, one, need - 1) == -5   # flags = WKV_FLOOR_DECAY
    # gstate_in overlapping gstate_out (arguments 8 and 14 of the 14 pointers), for either algorithm
    assert L.wkv6_backward(null, 1, 8, 64, 1, 1, 1, 0, *args, one, need) == -8
    assert L.wkv5_backward(null, 1, 8, 64, 1, 0, 1, 0, *args, one, L.wkv5_backward_workspace(1, 8, 64, 1, 0, 0)) == -8
    assert L.wkv4_forward(null, 0, 8, 64, 0, one, one, one, one, null, one, null, null) == -1
    assert L.wkv4_backward(null, 1, 8, 64, 0, *([one] * 13), one, 0) == -5
    assert L.wkv_cumsum_decay(null, 1, 100, 64, 16, 1, one, null, null, null, null, null) == -1
    # the element-wise passes around the operator
    outs = (ctypes.c_void_p * 2)(16, 16)
    assert L.wkv_shift_mix_forward(null, 1, 8, 100, 1, 2, 1, one, one, one, null, outs) == -1        # C % 8
    assert L.wkv_shift_mix_forward(null, 1, 8, 64, 1, 6, 1, one, one, one, null, outs) == -1         # more than 5 mixes
    assert L.wkv_shift_mix_forward(null, 1, 8, 64, 1, 2, 1, one, null, one, null, outs) == -2
    assert L.wkv_shift_mix_forward(null, 1, 8, 64, 1, 2, 1, one, one, one, null, (ctypes.c_void_p * 2)(16, 24)) == -4
    need = L.wkv_shift_mix_backward_workspace(1, 8, 64, 2)
    assert need == 1 * 1 * 2 * 64 * 4
    assert L.wkv_shift_mix_backward(null, 1, 8, 64, 1, 2, 1, one, one, one, null, outs, one, one, one, null, one, need - 1) == -5
    assert L.wkv_shift_mix_backward(null, 1, 8, 64, 1, 2, 0, one, one, one, one, outs, one, one, one, null, one, need) == -2  # dyn, no gdyn
    assert L.wkv_ln_gate_forward(null, 4, 96, 1, 1.0, 1e-5, one, one, one, one, one) == -1           # C % 64
    assert L.wkv_ln_gate_backward(null, 4, 64, 1, 1.0, 1e-5, one, one, one, one, one, one, null, one, one, 1 << 20) == -2
    assert L.wkv_ln_gate_backward(null, 4, 64, 1, 1.0, 1e-5, one, one, one, one, one, one, one, one, one, 8) == -5
    assert L.wkv_relu_square_forward(null, 12, 1, one, one) == -1                                    # n % 8
    assert L.wkv_sigmoid_mul_backward(null, 16, 9, one, one, one, one, one) == -3
    assert L.wkv_l2wrap_backward(null, 0, 8, 1, 1.0, one, null, one) == -1


def test_python_front_end_rejects_cpu_tensors():
    import torch
    import rwkv_wkv_hip as W
    B, T, C, H = 1, 4, 64, 1
    z = lambda *s: torch.zeros(*s)
    with pytest.raises(W.WKVError):
        W.WKV_6.apply(B, T, C, H, z(B, T, C), z(B, T, C), z(B, T, C), z(B, T, C), z(H, 64), z(B, H, 64, 64))
    with pytest.raises(ValueError):
        W.WKV_5.apply(B, T, C, H, z(B, H, 64, 64), z(B, T, C).double(), z(B, T, C).double(), z(B, T, C).double(),
                      z(H, 64), z(H, 64))
