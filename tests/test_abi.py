"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

from xlstm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "xlstm_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xs_[a-z_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    lib = _lib.load()
    syms = _declared_symbols()
    assert set(syms) == set(_lib.EXPORTS)
    for name in syms:
        assert getattr(lib, name) is not None


def test_abi_version_and_struct_mirror():
    lib = _lib.load()
    assert lib.xs_abi_version() == _lib.ABI_VERSION
    # xs_slstm_args: 6 int32, pointers/int64 after -> 8-byte aligned, 15 more 8-byte fields
    assert ctypes.sizeof(_lib.SlstmArgs) == 24 + 15 * 8
    assert ctypes.sizeof(_lib.SlstmStatus) == 64


def test_argument_errors_without_touching_the_gpu():
    lib = _lib.load()
    assert lib.xs_slstm_forward(None) == -1 and b"NULL" in lib.xs_last_error()
    a = _lib.SlstmArgs()
    a.B, a.T, a.NH, a.dh = 1, 1, 0, 8
    assert lib.xs_slstm_forward(ctypes.byref(a)) == -2  # bad dims
    a.NH = 1
    a.wx_dtype = 7
    assert lib.xs_slstm_forward(ctypes.byref(a)) == -3  # bad dtype
    a.wx_dtype, a.r_dtype = _lib.XS_F32, _lib.XS_BF16
    assert lib.xs_slstm_forward(ctypes.byref(a)) == -3  # fp32 wx needs fp32 R
    a.r_dtype = _lib.XS_F32
    assert lib.xs_slstm_forward(ctypes.byref(a)) == -1  # r / bias / s_out missing
    a.T = 2
    assert lib.xs_slstm_step(ctypes.byref(a)) == -2  # step needs T == 1
    assert b"T == 1" in lib.xs_last_error()
    # s_out may not overlap s0 anywhere (fake, never dereferenced addresses: validation comes before any launch)
    a.T = 1
    a.r, a.bias = 0x10000, 0x20000
    a.s0, a.s_out = 0x100000, 0x100000 + 64  # 16 * B * NH * dh = 128 bytes each
    assert lib.xs_slstm_step(ctypes.byref(a)) == -2 and b"overlap" in lib.xs_last_error()
    a.s_out = 0x100000 - 64
    assert lib.xs_slstm_step(ctypes.byref(a)) == -2 and b"overlap" in lib.xs_last_error()
    a.s_out = 0x100000 + 128  # adjacent is fine: the next complaint is about wx / h_out
    assert lib.xs_slstm_step(ctypes.byref(a)) == -1


def test_workspace_bytes_is_bounded_and_monotone():
    lib = _lib.load()
    w = lib.xs_slstm_workspace_bytes
    assert w(16, 2048, 4, 256) == w(16, 1, 4, 256)  # independent of T: a ring, not a per-step buffer
    assert w(16, 2048, 4, 256) < 16 << 20
    assert w(64, 4096, 4, 1024) >= w(16, 4096, 4, 1024)
    assert w(1, 1, 1, 8) % 256 == 0
