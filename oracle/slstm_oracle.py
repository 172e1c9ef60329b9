"""ctypes front-end of the C restatement in ``slstm_oracle.c``.

TEST INFRASTRUCTURE ONLY (see the header of ``slstm_oracle.c``).  The shared
object is built by ``make -C oracle`` (``__graft_entry__.build()`` does that);
if it is missing this module builds it with the same recipe.

Reference lines restated: ``xlstm/blocks/slstm/src/vanilla/__init__.py:17-74``
(time loop) and ``xlstm/blocks/slstm/src/vanilla/slstm.py:8-37`` (pointwise).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libslstm_oracle.so")
_LIB = None

N0_PER_ELEMENT = 0  # native-kernel rule, slstm_pointwise.cu:79
N0_WHOLE_TENSOR = 1  # vanilla rule, vanilla/slstm.py:25


def build(force: bool = False) -> str:
    """Compile the oracle with gcc; returns the path of the shared object."""
    srcs = [os.path.join(_HERE, f) for f in ("slstm_oracle.c", "slstm_oracle_backward.c")]
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < max(os.path.getmtime(f) for f in srcs):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return _SO


def _lib():
    global _LIB
    if _LIB is None:
        build()  # (no-op when the library is newer than its sources)
        lib = ctypes.CDLL(_SO)
        for name in ("slstm_oracle_forward_f64", "slstm_oracle_forward_f32"):
            fn = getattr(lib, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.c_void_p] * 7 + [ctypes.c_int] * 5
        if hasattr(lib, "slstm_oracle_backward_f64"):  # (a library built before the backward oracle existed has none)
            lib.slstm_oracle_backward_f64.restype = ctypes.c_int
            lib.slstm_oracle_backward_f64.argtypes = [ctypes.c_void_p] * 11 + [ctypes.c_int] * 6 + [ctypes.c_double]
        _LIB = lib
    return _LIB


def slstm_forward(
    wx: np.ndarray,  # [B, T, 4*H]  external order (gate, head, unit)
    r_ext: np.ndarray,  # [NH, dh, 4, dh]
    b_ext: np.ndarray,  # [NH, 4, dh]
    s0: Optional[np.ndarray] = None,  # [4, B, H]
    reset: Optional[np.ndarray] = None,  # [B, T] bool / uint8
    n0_rule: int = N0_PER_ELEMENT,
    dtype=np.float64,
) -> Tuple[np.ndarray, np.ndarray]:
    """Returns ``(h[T,B,H], state[4,B,H])`` computed in ``dtype`` arithmetic."""
    dtype = np.dtype(dtype)
    assert dtype in (np.dtype(np.float64), np.dtype(np.float32))
    NH, dh = int(r_ext.shape[0]), int(r_ext.shape[1])
    assert r_ext.shape == (NH, dh, 4, dh), r_ext.shape
    assert b_ext.shape == (NH, 4, dh), b_ext.shape
    H = NH * dh
    B, T = int(wx.shape[0]), int(wx.shape[1])
    assert wx.shape == (B, T, 4 * H), wx.shape
    wx_c = np.ascontiguousarray(wx, dtype=dtype)
    r_c = np.ascontiguousarray(r_ext, dtype=dtype)
    b_c = np.ascontiguousarray(b_ext, dtype=dtype)
    s0_c = None
    if s0 is not None:
        assert s0.shape == (4, B, H), s0.shape
        s0_c = np.ascontiguousarray(s0, dtype=dtype)
    reset_c = None
    if reset is not None:
        assert reset.shape == (B, T), reset.shape
        reset_c = np.ascontiguousarray(reset != 0, dtype=np.uint8)
    h = np.empty((T, B, H), dtype=dtype)
    s = np.empty((4, B, H), dtype=dtype)
    fn = _lib().slstm_oracle_forward_f64 if dtype == np.float64 else _lib().slstm_oracle_forward_f32
    rc = fn(
        wx_c.ctypes.data, r_c.ctypes.data, b_c.ctypes.data,
        s0_c.ctypes.data if s0_c is not None else None,
        reset_c.ctypes.data if reset_c is not None else None,
        h.ctypes.data, s.ctypes.data, B, T, NH, dh, int(n0_rule),
    )
    if rc != 0:
        raise MemoryError("slstm oracle: allocation failed")
    return h, s


def slstm_forward_per_document(wx, r_ext, b_ext, reset, dtype=np.float64):
    """Definition of the reset semantics: every document of every row is run
    ALONE from a zero state and the results are concatenated.  Deliberately a
    separate code path from the ``reset`` argument of :func:`slstm_forward`."""
    B, T = wx.shape[0], wx.shape[1]
    H = r_ext.shape[0] * r_ext.shape[1]
    h = np.zeros((T, B, H), dtype=dtype)
    s = np.zeros((4, B, H), dtype=dtype)
    for b in range(B):
        starts = [t for t in range(T) if reset[b, t]]
        if not starts or starts[0] != 0:
            raise ValueError("per-document oracle needs a document start at t=0 in every row")
        bounds = starts + [T]
        for lo, hi in zip(bounds[:-1], bounds[1:]):
            hd, sd = slstm_forward(wx[b:b + 1, lo:hi], r_ext, b_ext, None, None, dtype=dtype)
            h[lo:hi, b] = hd[:, 0]
            s[:, b] = sd[:, 0]
    return h, s


def slstm_backward(wx, r_ext, b_ext, s0, reset, d_h, d_s_final=None, n0_rule=N0_PER_ELEMENT, recurrent_cut=False,
                   recurrent_clipval=None):
    """Gradients of a loss with d loss / d h_out = ``d_h`` [T,B,H] (and d loss / d final state = ``d_s_final`` [4,B,H])
    with respect to W.x [B,T,4H], R_ext [NH,dh,4,dh], b_ext [NH,4,dh] and the initial state [4,B,H], in float64, by
    the rule of the reference's native kernel: the stabiliser m is a constant (slstm_pointwise.cu:118-196).
    ``recurrent_cut`` leaves out the gradient from a step to the y it started from (slstm_backward_cut.cu:265-312),
    ``recurrent_clipval`` clips that gradient to +-clipval before d_h is added (slstm_pointwise.cu:136-143)."""
    lib = _lib()
    B, T = wx.shape[0], wx.shape[1]
    NH, dh = r_ext.shape[0], r_ext.shape[1]
    H = NH * dh
    f64 = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.float64)
    wx_, r_, b_, s0_, dh_, dsf_ = f64(wx), f64(r_ext), f64(b_ext), f64(s0), f64(d_h), f64(d_s_final)
    rs_ = None if reset is None else np.ascontiguousarray(reset, dtype=np.uint8)
    assert wx_.shape == (B, T, 4 * H) and dh_.shape == (T, B, H)
    d_wx = np.zeros((B, T, 4 * H)); d_r = np.zeros((NH, dh, 4, dh)); d_b = np.zeros((NH, 4, dh)); d_s0 = np.zeros((4, B, H))
    ptr = lambda a: None if a is None else a.ctypes.data_as(ctypes.c_void_p)
    rc = lib.slstm_oracle_backward_f64(ptr(wx_), ptr(r_), ptr(b_), ptr(s0_), ptr(rs_), ptr(dh_), ptr(dsf_), ptr(d_wx),
                                       ptr(d_r), ptr(d_b), ptr(d_s0), B, T, NH, dh, n0_rule, int(bool(recurrent_cut)),
                                       float(recurrent_clipval) if recurrent_clipval is not None else 0.0)
    if rc != 0:
        raise MemoryError("slstm_oracle_backward_f64 failed")
    return d_wx, d_r, d_b, d_s0
