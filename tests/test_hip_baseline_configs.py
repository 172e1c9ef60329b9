"""The five BASELINE configurations on the GPU.

Configs 1, 2 and the cell of config 4 are checked against the float64 oracle at
FULL size (the oracle needs a few seconds for them).  Configs 3 and 5 are checked
at full width against the oracle on a slice it can afford (a few batch rows, the
first steps) and at full size through properties that do not depend on the size:
step-by-step == sequence, chunked == whole, |h| <= 1, n >= 1.
"""
import numpy as np
import pytest
import torch

from oracle import slstm_oracle as so
from tests._util import geometric_reset_mask, make_problem, max_err, r_ext_to_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _hip(wx_t, r_t, b_t, s0=None, mask=None, **kw):
    from xlstm_amd import functional as F

    ws = F.workspace_for(wx_t.shape[0], wx_t.shape[1], r_t.shape[0], r_t.shape[2], wx_t.device)
    h, s = F.slstm_forward(wx_t, r_t, b_t, s0, mask, workspace=ws, **kw)
    torch.cuda.synchronize()
    st = F.read_status(ws)
    assert st["aborted"] == 0, st
    return h, s


def _params(r_ext, b_ext):
    return r_ext_to_kernel(torch.from_numpy(r_ext)).to(DEV), torch.from_numpy(b_ext).to(DEV)


def test_config1_fp32_full_size():
    """B=4, T=256, D=512 (4 x 128), fp32, reference init (zeros and 'standard' R), small_init bias, zero state."""
    B, T, NH, dh = 4, 256, 4, 128
    for rscale in (0.0, 1.0):
        print("config 1, R scale", rscale, flush=True)
        wx, r, b, _ = make_problem(101, B, T, NH, dh, rscale=rscale)
        h_ref, s_ref = so.slstm_forward(wx, r, b)
        r_t, b_t = _params(r, b)
        h, s = _hip(torch.from_numpy(wx).to(DEV), r_t, b_t)
        assert max_err(h.cpu().numpy(), h_ref) <= 1e-5
        assert max_err(s.cpu().numpy(), s_ref) <= 1e-5


@pytest.mark.parametrize("B,mean_len,name", [(16, 512, "config 2"), (8, 768, "config 4 cell")])
def test_config2_and_config4_cell_packed_documents_full_size(B, mean_len, name):
    """T=2048, D=1024 (4 x 256), bf16 W.x, packed geometric documents with a reset mask."""
    T, NH, dh = 2048, 4, 256
    print(name, "full size", flush=True)
    wx, r, b, _ = make_problem(102, B, T, NH, dh, bf16=True)
    mask = geometric_reset_mask(102, B, T, mean_len)
    h_ref, s_ref = so.slstm_forward(wx, r, b, None, mask)
    r_t, b_t = _params(r, b)
    wx_t = torch.from_numpy(wx).to(DEV).bfloat16()
    mask_t = torch.from_numpy(mask).to(DEV)
    h, s = _hip(wx_t, r_t, b_t, None, mask_t)
    eh, es = max_err(h.float().cpu().numpy(), h_ref), max_err(s.cpu().numpy(), s_ref)
    print(name, "max err h %.2e state %.2e" % (eh, es), flush=True)
    assert eh <= 2e-2 and es <= 2e-2
    # bit-exact resets: the longest document of row 0, run alone from a zero state
    starts = list(np.flatnonzero(mask[0])) + [T]
    lo, hi = max(zip(starts[:-1], starts[1:]), key=lambda p: p[1] - p[0])
    hd, sd = _hip(wx_t[0:1, lo:hi], r_t, b_t)
    assert torch.equal(hd[:, 0], h[lo:hi, 0])
    if hi == T:
        assert torch.equal(sd[:, 0], s[:, 0])


def test_config3_decode_full_width():
    """B=256, D=2048 (8 x 256), bf16: 128-token prefill, then 1024 consecutive T=1 steps carrying the state,
    as BASELINE states it, driven the way the benchmark's decode leg drives them: a ``StepPlan`` whose every step
    gets the h of the step before as its bf16 operand.  That is the pipelined step kernel, and the status block must
    say so; the first 64 steps are run a second time without the operand hint (the tile kernel)."""
    B, NH, dh, PRE, STEPS = 256, 8, 256, 128, 1024
    H = NH * dh
    print("config 3: building inputs on the device", flush=True)
    g = torch.Generator(device=DEV).manual_seed(103)
    wx_t = torch.empty(B, PRE + STEPS, 4 * H, dtype=torch.bfloat16, device=DEV)
    for row in range(B):
        wx_t[row] = torch.randn(PRE + STEPS, 4 * H, generator=g, device=DEV).bfloat16()
    _, r, b, _ = make_problem(103, 1, 1, NH, dh)
    r_t, b_t = _params(r, b)
    r_step = r_t.bfloat16()
    print("config 3: prefill + 1024 steps", flush=True)
    h_pre, s = _hip(wx_t[:, :PRE], r_t, b_t)
    from xlstm_amd import functional as F

    ws = F.workspace_for(B, 1, NH, dh, wx_t.device)
    plan = F.StepPlan(B, r_t, b_t, wx_dtype=torch.bfloat16, workspace=ws)
    h_dec = torch.empty(STEPS, B, H, dtype=torch.bfloat16, device=DEV)
    s_a, s_b = s.clone(), torch.empty_like(s)
    wx_steps = wx_t[:, PRE:].transpose(0, 1).contiguous()  # [STEPS, B, 4H]: a step's W.x as the layer hands it over
    for t in range(STEPS):
        plan(wx_steps[t], s_a, s_b, h_dec[t], h_prev=h_dec[t - 1] if t else h_pre[PRE - 1])
        s_a, s_b = s_b, s_a
    torch.cuda.synchronize()
    st = F.read_status(ws)
    print("config 3: status after the last step", st, flush=True)
    assert st["step_kernel"] == 1 and st["pipelined_step"] == 1 and st["aborted"] == 0
    # property at full size: decoding step by step == one sequence call, bit for bit
    print("config 3: one sequence call over all 1152 tokens", flush=True)
    h_all, s_all = _hip(wx_t, r_t, b_t)
    assert torch.equal(h_all[:PRE], h_pre) and torch.equal(h_all[PRE:], h_dec) and torch.equal(s_all, s_a)
    # the same steps without the operand hint: the tile kernel, the same bits
    s_a, s_b = s.clone(), torch.empty_like(s)
    h_tile = torch.empty(64, B, H, dtype=torch.bfloat16, device=DEV)
    for t in range(64):
        F.slstm_forward(wx_t[:, PRE + t:PRE + t + 1], r_step, b_t, s_a, None, step=True, workspace=ws,
                        h_out=h_tile[t:t + 1], s_out=s_b)
        s_a, s_b = s_b, s_a
    torch.cuda.synchronize()
    st = F.read_status(ws)
    assert st["step_kernel"] == 1 and st["pipelined_step"] == 0
    assert torch.equal(h_tile, h_dec[:64])
    # oracle on a few rows (rows are independent)
    rows = [0, 17, 255]
    h_ref, s_ref = so.slstm_forward(wx_t[rows].float().cpu().numpy(), r, b)
    assert max_err(h_all[:, rows].float().cpu().numpy(), h_ref) <= 2e-2
    assert max_err(s_all[:, rows].cpu().numpy(), s_ref) <= 2e-2
    assert tuple(h_all.shape) == (PRE + STEPS, B, H)


def test_pipelined_step_whose_waves_give_up_on_each_other_says_so():
    """Host-forced: with a spin limit of one look the waves of a workgroup of the pipelined step kernel give up on
    each other at once (every wave still runs to its end).  Either some workgroup gave up - then the status block says
    so and that workgroup's tile of the outputs is NaN - or every wait happened to be satisfied at the first look and
    the step is the usual one.  The test prints which of the two it saw."""
    from xlstm_amd import _lib
    from xlstm_amd import functional as F
    import ctypes

    B, NH, dh = 256, 8, 256
    H = NH * dh
    g = torch.Generator(device=DEV).manual_seed(104)
    wx = torch.randn(B, 1, 4 * H, generator=g, device=DEV).bfloat16()
    _, r, b, _ = make_problem(104, 1, 1, NH, dh)
    r_t, b_t = _params(r, b)
    s0 = torch.randn(4, B, H, generator=g, device=DEV)
    s0[2] = s0[2].abs() + 1.0
    s0[0] = s0[0].bfloat16().float()
    h_prev = s0[0].bfloat16()
    ws = F.workspace_for(B, 1, NH, dh, wx.device)
    good_h, good_s = F.slstm_forward(wx, r_t.bfloat16(), b_t, s0, None, step=True, workspace=ws, h_prev=h_prev)
    torch.cuda.synchronize()
    assert F.read_status(ws)["pipelined_step"] == 1
    h, s = F.slstm_forward(wx, r_t.bfloat16(), b_t, s0, None, step=True, workspace=ws, h_prev=h_prev, spin_limit=1)
    torch.cuda.synchronize()
    st = F.read_status(ws)
    if st["aborted"]:
        print("pipelined step, spin limit 1: gave up (workgroup %d); NaN tiles" % st["abort_wg"], flush=True)
        assert not bool(torch.isfinite(h.float()).all()) and not bool(torch.isfinite(s).all())
        # a tile is all NaN or untouched by the give-up: what is finite is the usual result
        ok = torch.isfinite(h.float())
        assert torch.equal(h[ok], good_h[ok])
    else:
        print("pipelined step, spin limit 1: every wait was satisfied at the first look", flush=True)
        assert torch.equal(h, good_h) and torch.equal(s, good_s)


def test_config5_large_heads_full_size():
    """B=64, T=4096, D=4096 (4 x 1024), bf16: a head spans 64 compute units on all XCDs."""
    B, T, NH, dh = 64, 4096, 4, 1024
    H = NH * dh
    print("config 5: building 8.6 GB of inputs on the device", flush=True)
    g = torch.Generator(device=DEV).manual_seed(105)
    wx_t = torch.empty(B, T, 4 * H, dtype=torch.bfloat16, device=DEV)
    for row in range(B):  # row by row: no 34 GB fp32 temporary
        wx_t[row] = torch.randn(T, 4 * H, generator=g, device=DEV).bfloat16()
    _, r, b, _ = make_problem(105, 1, 1, NH, dh)
    r_t, b_t = _params(r, b)
    print("config 5: full-size launch", flush=True)
    h, s = _hip(wx_t, r_t, b_t)
    assert bool(torch.isfinite(s).all())
    assert float(h.float().abs().max()) <= 1.0 + 1e-2  # |y| <= 1 up to bf16 rounding
    assert float(s[2].min()) >= 1.0 - 1e-5             # n >= 1 after the first step
    # chunked == whole at full size (state carried through the C ABI), bit for bit
    print("config 5: two half-length launches", flush=True)
    ha, sa = _hip(wx_t[:, : T // 2], r_t, b_t)
    assert torch.equal(ha, h[: T // 2])
    hb, sb = _hip(wx_t[:, T // 2:], r_t, b_t, sa)
    assert torch.equal(hb, h[T // 2:]) and torch.equal(sb, s)
    del ha, hb
    # oracle on a slice: 3 rows, first 96 steps
    rows, Ts = [0, 31, 63], 96
    print("config 5: oracle on a slice", flush=True)
    wx_s = wx_t[rows, :Ts].float().cpu().numpy()
    h_ref, _ = so.slstm_forward(wx_s, r, b)
    assert max_err(h[:Ts, rows].float().cpu().numpy(), h_ref) <= 2e-2
