"""xs_slstm_forward_static (the entry point that allocates nothing and brings its own scratch) against
xs_slstm_forward, called through the C ABI with ctypes: same bits, two calls in a row, the second one smaller."""
import ctypes

import pytest
import torch

from tests._util import geometric_reset_mask, make_problem, r_ext_to_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _args(wx, r, bias, s0, mask, h_out, s_out, ws):
    from xlstm_amd import _lib

    B, T = int(wx.shape[0]), int(wx.shape[1])
    NH, dh = int(r.shape[0]), int(r.shape[2])
    a = _lib.SlstmArgs()
    a.B, a.T, a.NH, a.dh = B, T, NH, dh
    a.wx_dtype = _lib.XS_BF16 if wx.dtype == torch.bfloat16 else _lib.XS_F32
    a.r_dtype = _lib.XS_BF16 if r.dtype == torch.bfloat16 else _lib.XS_F32
    a.wx, a.wx_stride_b, a.wx_stride_t = wx.data_ptr(), wx.stride(0), wx.stride(1)
    a.r, a.bias = r.data_ptr(), bias.data_ptr()
    a.s0 = s0.data_ptr() if s0 is not None else None
    a.reset = mask.data_ptr() if mask is not None else None
    a.reset_stride_b = mask.stride(0) if mask is not None else 0
    a.h_out, a.s_out = h_out.data_ptr(), s_out.data_ptr()
    a.workspace = ws.data_ptr() if ws is not None else None
    a.workspace_bytes = ws.numel() if ws is not None else 0
    a.stream = torch.cuda.current_stream().cuda_stream
    a.spin_limit = 0
    a.h_prev = None
    return a


def _both(B, T, NH, dh, bf16, seed, with_state, resets, r_bf16=False):
    """Runs one problem through both entry points and compares every output bit."""
    from xlstm_amd import _lib
    from xlstm_amd import functional as F

    lib = _lib.load()
    print("case static scratch", B, T, NH, dh, bf16, with_state, resets, flush=True)
    wx, r, b, s0 = make_problem(seed, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=with_state)
    wx_t = torch.from_numpy(wx).to(DEV)
    wx_t = wx_t.bfloat16() if bf16 else wx_t
    r_t = r_ext_to_kernel(torch.from_numpy(r)).to(DEV)
    r_t = r_t.bfloat16() if r_bf16 else r_t
    b_t = torch.from_numpy(b).to(DEV)
    s0_t = torch.from_numpy(s0).to(DEV) if with_state else None
    m_t = torch.from_numpy(geometric_reset_mask(seed, B, T, max(2, T // 3))).to(DEV) if resets else None
    H = NH * dh
    outs = []
    for static in (False, True):
        h = torch.full((T, B, H), 7.0, dtype=wx_t.dtype, device=DEV)
        s = torch.full((4, B, H), 7.0, dtype=torch.float32, device=DEV)
        ws = None if static else F.workspace_for(B, T, NH, dh, DEV)
        a = _args(wx_t, r_t, b_t, s0_t, m_t, h, s, ws)
        rc = (lib.xs_slstm_forward_static if static else lib.xs_slstm_forward)(ctypes.byref(a))
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        if not static:
            assert F.read_status(ws)["aborted"] == 0
        outs.append((h, s))
    (h0, s0_), (h1, s1) = outs
    assert bool(torch.isfinite(s1).all()) and bool(torch.isfinite(h1.float()).all())
    assert torch.equal(h0, h1) and torch.equal(s0_, s1)


def test_static_scratch_entry_point_matches_the_workspace_entry_point():
    # two calls in a row on the same scratch array, the second with a smaller input (fewer rows, fewer steps,
    # a smaller head): whatever the first left behind must not leak into the second
    _both(16, 96, 4, 256, True, 51, False, True)    # BASELINE config 2's kernel variant
    _both(5, 17, 2, 64, True, 52, True, True)
    # other variants: float32, four row tiles over two XCDs, a single token (the step kernel), empty calls
    _both(40, 9, 4, 128, False, 53, True, False)
    _both(70, 6, 4, 1024, True, 54, False, False)
    _both(64, 1, 2, 128, True, 55, True, False, r_bf16=True)
    _both(3, 0, 2, 32, False, 56, True, False)
    _both(16, 40, 4, 256, True, 57, True, True)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    """float32, four row tiles on every compute unit: an 8 MiB exchange ring, more than the static array holds.
    The refusal comes before anything is launched."""
    from xlstm_amd import _lib

    lib = _lib.load()
    B, T, NH, dh = 256, 2, 4, 512
    wx = torch.zeros(B, T, 4 * NH * dh, device=DEV)
    r = torch.zeros(NH, 4 * dh, dh, device=DEV)
    bias = torch.zeros(NH, 4, dh, device=DEV)
    h = torch.full((T, B, NH * dh), 7.0, device=DEV)
    s = torch.full((4, B, NH * dh), 7.0, device=DEV)
    a = _args(wx, r, bias, None, None, h, s, None)
    rc = lib.xs_slstm_forward_static(ctypes.byref(a))
    assert rc == -6 and "static array holds" in _lib.last_error(), (rc, _lib.last_error())
    torch.cuda.synchronize()
    assert float(h.min()) == 7.0 and float(s.min()) == 7.0  # nothing ran
