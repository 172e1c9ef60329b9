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
    assert ctypes.sizeof(_lib.SlstmArgs) == 24 + 17 * 8
    assert ctypes.sizeof(_lib.SlstmStatus) == 64
    # xs_conv_args: 5 int32 (+4 padding), then 12 8-byte fields; xs_gates_args: 4 int32, then 11 8-byte fields
    assert ctypes.sizeof(_lib.ConvArgs) == 24 + 12 * 8
    assert ctypes.sizeof(_lib.GatesArgs) == 16 + 11 * 8
    assert ctypes.sizeof(_lib.NormArgs) == 24 + 7 * 8  # 5 int32 + float, then 7 8-byte fields
    # 5 int32 (+4), 17 8-byte fields, int32 (+4), 3 more, int32 + float, 4 pointers
    assert ctypes.sizeof(_lib.SlstmBwdArgs) == 24 + 17 * 8 + 8 + 3 * 8 + 8 + 4 * 8 + 8


def test_backward_argument_errors_without_touching_the_gpu():
    lib = _lib.load()
    assert lib.xs_slstm_backward(None) == -1 and lib.xs_slstm_backward_prepare(None) == -1
    a = _lib.SlstmBwdArgs()
    a.B, a.T, a.NH, a.dh, a.dtype = 2, 3, 2, 48, _lib.XS_F32
    assert lib.xs_slstm_backward(ctypes.byref(a)) == -5 and b"head dim 48" in lib.xs_last_error()
    a.dh = 64
    assert lib.xs_slstm_backward_prepare(ctypes.byref(a)) == -1  # coef missing
    a.dtype = 5
    assert lib.xs_slstm_backward(ctypes.byref(a)) == -3
    # d_wx in bf16 goes with bf16 operands
    a.dtype, a.d_wx_dtype = _lib.XS_F32, _lib.XS_BF16
    assert lib.xs_slstm_backward(ctypes.byref(a)) == -3 and lib.xs_slstm_backward_params(ctypes.byref(a)) in (-1, -3)
    # the tiling of R for the reverse kernels
    assert lib.xs_slstm_backward_tile_r(None) == -1
    t = _lib.SlstmBwdArgs()
    t.NH, t.dh, t.dtype, t.split = 2, 64, _lib.XS_F32, 0
    assert lib.xs_slstm_backward_tile_r(ctypes.byref(t)) == -1 and b"r and r_t" in lib.xs_last_error()
    buf = (ctypes.c_char * 64)()
    t.r = t.r_t = ctypes.addressof(buf)
    t.split = 2
    assert lib.xs_slstm_backward_tile_r(ctypes.byref(t)) == -5  # row tiles of 4 rows: bf16
    t.split, t.dh = 3, 96
    assert lib.xs_slstm_backward_tile_r(ctypes.byref(t)) == -5  # (not a multiple of 64)
    t.split = 7
    assert lib.xs_slstm_backward_tile_r(ctypes.byref(t)) == -5


def test_backward_alignment_errors_without_touching_the_gpu():
    """What the backward kernels fetch in pieces of 16 bytes (W.x, R.h, the coefficients, d_h) or write in pairs of
    floats (d_wx) must be aligned for it: XS_ERR_ALIGN before anything is launched (fake addresses, never used)."""
    lib = _lib.load()
    a = _lib.SlstmBwdArgs()
    a.B, a.T, a.NH, a.dh, a.dtype = 2, 3, 2, 64, _lib.XS_BF16
    H = 128
    a.coef, a.wx, a.r, a.bias, a.h_out = 0x100000, 0x200000, 0x300000, 0x400000, 0x900000
    a.wx_stride_b, a.wx_stride_t = 3 * 4 * H, 4 * H
    for field, bad in (("wx", 0x200002), ("wx_stride_t", 4 * H + 1), ("wx_stride_b", 3 * 4 * H + 4), ("r", 0x300008),
                       ("h_out", 0x900004), ("coef", 0x100004)):
        keep = getattr(a, field)
        setattr(a, field, bad)
        assert lib.xs_slstm_backward_prepare(ctypes.byref(a)) == -4, field
        assert b"aligned" in lib.xs_last_error()
        setattr(a, field, keep)
    a.d_h, a.r_t, a.d_wx, a.d_s0 = 0x500000, 0x600000, 0x700000, 0x800000
    a.d_wx_stride_b, a.d_wx_stride_t = 3 * 4 * H, 4 * H
    for field, bad in (("d_h", 0x500002), ("r_t", 0x600008), ("d_wx", 0x700004), ("d_wx_stride_t", 4 * H + 1), ("coef", 0x100008)):
        keep = getattr(a, field)
        setattr(a, field, bad)
        assert lib.xs_slstm_backward(ctypes.byref(a)) == -4, field
        setattr(a, field, keep)
    a.d_r, a.d_bias = 0xA00000, 0xB00000
    for field, bad in (("d_wx", 0x700004), ("d_wx_stride_t", 4 * H + 2), ("h_out", 0x900008)):
        keep = getattr(a, field)
        setattr(a, field, bad)
        assert lib.xs_slstm_backward_params(ctypes.byref(a)) == -4, field
        setattr(a, field, keep)


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


def test_layer_op_argument_errors_without_touching_the_gpu():
    lib = _lib.load()
    assert lib.xs_causal_conv_silu(None) == -1 and lib.xs_headwise_gates(None) == -1
    c = _lib.ConvArgs()
    c.B, c.T, c.D, c.K, c.dtype = 1, 4, 16, 4, _lib.XS_F32
    assert lib.xs_causal_conv_silu(ctypes.byref(c)) == -3  # bf16 only
    c.dtype, c.K = _lib.XS_BF16, 5
    assert lib.xs_causal_conv_silu(ctypes.byref(c)) == -5 and b"taps" in lib.xs_last_error()
    c.K, c.D = 4, 12
    assert lib.xs_causal_conv_silu(ctypes.byref(c)) == -5  # D not a multiple of 8
    c.D = 16
    assert lib.xs_causal_conv_silu(ctypes.byref(c)) == -1  # x / weight / out missing
    c.x, c.weight, c.out, c.x_stride_b, c.x_stride_t = 0x1000, 0x2000, 0x3008, 64, 16
    assert lib.xs_causal_conv_silu(ctypes.byref(c)) == -4  # out not 16-byte aligned
    c.T = 0
    assert lib.xs_causal_conv_silu(ctypes.byref(c)) == 0  # nothing to do, nothing launched
    g = _lib.GatesArgs()
    g.M, g.NH, g.dh, g.dtype = 4, 2, 32, _lib.XS_BF16
    assert lib.xs_headwise_gates(ctypes.byref(g)) == -5 and b"multiple of 64" in lib.xs_last_error()
    g.dh = 64
    assert lib.xs_headwise_gates(ctypes.byref(g)) == -1
    g.x, g.x_conv, g.out = 0x1000, 0x2000, 0x3000
    for i in range(4):
        g.w[i] = 0x4000
    g.x_stride_row, g.x_conv_stride_row, g.out_stride_row = 128, 128, 128
    assert lib.xs_headwise_gates(ctypes.byref(g)) == -2  # out rows overlap
    g.M = 0
    assert lib.xs_headwise_gates(ctypes.byref(g)) == 0
    assert lib.xs_headwise_group_norm(None) == -1
    n = _lib.NormArgs()
    n.B, n.T, n.NH, n.dh, n.dtype = 2, 3, 4, 6, _lib.XS_BF16
    assert lib.xs_headwise_group_norm(ctypes.byref(n)) == -5  # head dim not a multiple of 4
    n.dh = 2048
    assert lib.xs_headwise_group_norm(ctypes.byref(n)) == -5
    n.dh = 64
    assert lib.xs_headwise_group_norm(ctypes.byref(n)) == -1  # x / out missing
    n.x, n.out, n.x_stride_b, n.x_stride_t, n.x_stride_h = 0x1000, 0x2000, 256, 514, 64
    assert lib.xs_headwise_group_norm(ctypes.byref(n)) == -4  # stride not 8-byte aligned
    n.B = 0
    assert lib.xs_headwise_group_norm(ctypes.byref(n)) == 0


def test_workspace_bytes_is_bounded_and_monotone():
    lib = _lib.load()
    w = lib.xs_slstm_workspace_bytes
    assert w(16, 2048, 4, 256) == w(16, 1, 4, 256)  # independent of T: a ring, not a per-step buffer
    assert w(16, 2048, 4, 256) < 16 << 20
    assert w(64, 4096, 4, 1024) >= w(16, 4096, 4, 1024)
    assert w(1, 1, 1, 8) % 256 == 0
