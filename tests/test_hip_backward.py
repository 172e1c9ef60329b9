"""GPU parity of the backward pass (xs_slstm_backward_prepare + xs_slstm_backward, through ``functional.slstm_backward``
and through the cell's autograd) against the float64 backward oracle, which the reference's own autograd gradients pin
(tests/test_oracle_backward.py).  Tolerances: float32 1e-5, bfloat16 2e-2, relative to the largest entry of a gradient
(at least 1), the bars of the forward tests."""
import numpy as np
import pytest
import torch

from oracle import slstm_oracle as so
from tests._util import geometric_reset_mask, make_problem, r_ext_to_kernel

pytestmark = pytest.mark.gpu


def _rel(a, g):
    return float(np.abs(a - g).max() / max(1.0, np.abs(g).max()))


CASES = [
    # bf16, B, T, NH, dh, masked + state
    (False, 3, 7, 2, 64, False),
    (False, 5, 9, 2, 64, True),
    (False, 20, 6, 2, 128, True),     # two row tiles, the second ragged
    (False, 4, 12, 4, 256, True),
    (False, 1, 1, 1, 64, False),      # one step
    (False, 33, 40, 2, 128, True),
    (True, 5, 9, 2, 64, True),
    (True, 16, 10, 4, 256, True),     # config 2's cell, a few steps
    (True, 40, 33, 8, 128, True),
    (True, 8, 64, 4, 256, False),
]


# what the kernel that spreads a head over dh / 64 compute units adds: head dim 512 (bf16), many row tiles
def test_a_batch_with_more_row_tiles_than_the_device_holds_runs_in_slices_of_rows():
    """B = 500 at head dim 256 with two heads is 32 row tiles x 2 heads x 4 compute units = 256 workgroups, more than
    the device holds beside the prefetching ones: two launches of the split kernel over slices of rows, against the
    oracle."""
    from xlstm_amd import functional as F

    B, T, NH, dh = 500, 3, 2, 256
    H = NH * dh
    wx, r, b, s0 = make_problem(93, B, T, NH, dh, rscale=2.0, bf16=True, with_state=True)
    reset = geometric_reset_mask(8, B, T, 2)
    d_h = torch.from_numpy(np.random.default_rng(94).standard_normal((T, B, H)).astype(np.float32)).bfloat16().float().numpy()
    r = torch.from_numpy(r).bfloat16().float().numpy()
    dev = torch.device("cuda:0")
    wx_t, r_t, b_t = torch.from_numpy(wx).to(dev).bfloat16(), r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev)
    s0_t, m_t = torch.from_numpy(s0).to(dev), torch.from_numpy(reset).to(dev)
    h, _ = F.slstm_forward(wx_t, r_t, b_t, s0_t, m_t)
    d_wx, d_r, d_b, d_s0 = F.slstm_backward(wx_t, r_t, b_t, s0_t, m_t, h, torch.from_numpy(d_h).to(dev))
    torch.cuda.synchronize()
    o_wx, o_r, o_b, o_s0 = so.slstm_backward(wx, r, b, s0, reset, d_h)
    errs = dict(d_wx=_rel(d_wx.cpu().numpy(), o_wx), d_r=_rel(d_r.cpu().numpy(), r_ext_to_kernel(torch.from_numpy(o_r)).numpy()),
                d_b=_rel(d_b.cpu().numpy(), o_b), d_s0=_rel(d_s0.cpu().numpy(), o_s0))
    assert all(np.isfinite(v) and v <= 2e-2 for v in errs.values()), errs


PADDED_CASES = [
    # head dims between the kernels' sizes: run as the next size up with zero units
    (False, 3, 6, 2, 16, True),
    (True, 5, 7, 3, 96, True),
    (False, 18, 4, 2, 192, True),
    (True, 4, 5, 2, 384, True),
]

SPLIT_CASES = [
    (False, 3, 1, 2, 128, False),     # one step: the feeders' first slot only
    (True, 17, 2, 2, 256, True),      # two steps, two row tiles
    (True, 9, 7, 2, 512, True),
    (True, 100, 5, 2, 256, True),
    (False, 50, 6, 4, 128, True),
]


def _row_tile_of(kernel):
    """``kernel``: "one-unit" (one workgroup per head), "split" (a head over dh/64 compute units, row tiles of 16 rows),
    "quad" (the same in row tiles of 4 rows: bf16, head dims up to 256).  Returns (split_override, row_tile_override)."""
    return kernel != "one-unit", {"one-unit": None, "split": 16, "quad": 4}[kernel]


def _kernels_of(bf16, dh):
    """The reverse kernels that cover a case: head dim 512 (and what is padded up to it) has the split kernel only, row
    tiles of 4 rows go with bf16 and head dims up to 256."""
    dh_k = (dh + 63) // 64 * 64
    return (["one-unit"] if dh_k <= 256 else []) + ["split"] + (["quad"] if bf16 and dh_k <= 256 else [])


QUAD_CASES = [
    (True, 1, 1, 1, 64, False),       # one row, one step
    (True, 2, 3, 1, 128, True),       # fewer steps than the feeder wave runs ahead
    (True, 7, 4, 3, 256, True),       # a ragged second row tile, as many steps as feeder slots
    (True, 6, 5, 2, 64, True),
    (True, 16, 300, 16, 64, True),    # 64 groups, eight per XCD, long enough for the prefetching workgroups to follow and skip
    (True, 64, 6, 4, 256, True),      # 256 workgroups: the whole device, no room for prefetching workgroups
]


@pytest.mark.parametrize("bf16,B,T,NH,dh,masked,kernel", [c + (k,) for c in CASES + SPLIT_CASES + PADDED_CASES + QUAD_CASES
                                                          for k in _kernels_of(c[0], c[4])])
def test_backward_against_the_oracle(bf16, B, T, NH, dh, masked, kernel):
    from xlstm_amd import functional as F

    split, row_tile = _row_tile_of(kernel)
    print("case backward", bf16, B, T, NH, dh, masked, kernel, flush=True)
    H = NH * dh
    wx, r, b, s0 = make_problem(91, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=masked)
    reset = geometric_reset_mask(7, B, T, max(2, T // 2)) if masked else None
    if reset is not None:
        reset[0, 0] = 0  # one row that uses the supplied state
    rng = np.random.default_rng(92)
    d_h = rng.standard_normal((T, B, H)).astype(np.float32)
    d_sf = rng.standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    dev = torch.device("cuda:0")
    wx_t = torch.from_numpy(wx).to(dev)
    if bf16:
        wx_t = wx_t.bfloat16()
        d_h = torch.from_numpy(d_h).bfloat16().float().numpy()
        r = torch.from_numpy(r).bfloat16().float().numpy()  # the forward rounds R to bf16; give the oracle the same R
    r_t = r_ext_to_kernel(torch.from_numpy(r)).to(dev)
    b_t = torch.from_numpy(b).to(dev)
    s0_t = torch.from_numpy(s0).to(dev) if s0 is not None else None
    m_t = torch.from_numpy(reset).to(dev) if reset is not None else None
    h, _ = F.slstm_forward(wx_t, r_t, b_t, s0_t, m_t)
    d_wx, d_r, d_b, d_s0 = F.slstm_backward(wx_t, r_t, b_t, s0_t, m_t, h, torch.from_numpy(d_h).to(dev), torch.from_numpy(d_sf).to(dev),
                                            split_override=split, row_tile_override=row_tile)
    torch.cuda.synchronize()
    o_wx, o_r, o_b, o_s0 = so.slstm_backward(wx, r, b, s0, reset, d_h, d_sf)
    o_r_k = r_ext_to_kernel(torch.from_numpy(o_r)).numpy()
    tol = 2e-2 if bf16 else 1e-5
    errs = dict(d_wx=_rel(d_wx.cpu().numpy(), o_wx), d_r=_rel(d_r.cpu().numpy(), o_r_k), d_b=_rel(d_b.cpu().numpy(), o_b),
                d_s0=_rel(d_s0.cpu().numpy(), o_s0))
    print(errs, flush=True)
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs


def test_packed_rows_have_the_gradients_of_their_documents():
    """A reset cuts the recurrence: the gradients of a packed batch are those of the two halves run alone."""
    from xlstm_amd import functional as F

    B, T, NH, dh, cut = 6, 11, 2, 64, 5
    H = NH * dh
    wx, r, b, _ = make_problem(93, B, T, NH, dh, rscale=2.0)
    dev = torch.device("cuda:0")
    wx_t, r_t, b_t = torch.from_numpy(wx).to(dev), r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev)
    mask = torch.zeros(B, T, dtype=torch.uint8, device=dev)
    mask[:, 0] = 1
    mask[:, cut] = 1
    d_h = torch.randn(T, B, H, generator=torch.Generator().manual_seed(5)).to(dev)
    h, _ = F.slstm_forward(wx_t, r_t, b_t, None, mask)
    whole = F.slstm_backward(wx_t, r_t, b_t, None, mask, h, d_h)
    parts = []
    for lo, hi in ((0, cut), (cut, T)):
        hp, _ = F.slstm_forward(wx_t[:, lo:hi], r_t, b_t)
        parts.append(F.slstm_backward(wx_t[:, lo:hi], r_t, b_t, None, None, hp, d_h[lo:hi].contiguous()))
    assert torch.equal(whole[0][:, :cut], parts[0][0]) and torch.equal(whole[0][:, cut:], parts[1][0])
    torch.testing.assert_close(whole[1], parts[0][1] + parts[1][1], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(whole[2], parts[0][2] + parts[1][2], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
def test_cell_autograd_matches_the_oracle(dtype, tol):
    """loss.backward() through ``sLSTMCell(backend="hip")``: gradients of the input, the parameters (in the reference's
    external views) and the initial state for a loss that is a linear form of the output in its public BNSH layout."""
    from tests.test_hip_cell import _cell_from

    B, T, NH, dh = 3, 8, 2, 64
    H = NH * dh
    bf16 = dtype == "bfloat16"
    wx, r, b, s0 = make_problem(94, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=True)
    if bf16:
        r = torch.from_numpy(r).bfloat16().float().numpy()
        s0 = torch.from_numpy(s0).bfloat16().float().numpy()
    cell = _cell_from(r, b, dtype=dtype).train()
    tdt = torch.bfloat16 if bf16 else torch.float32
    x = torch.from_numpy(wx).cuda().to(tdt).requires_grad_(True)
    st = torch.from_numpy(s0).cuda().to(tdt).requires_grad_(True)
    out, _ = cell(x, st)                                   # [B, NH, T, dh]
    w = torch.randn(out.shape, generator=torch.Generator().manual_seed(6)).cuda()
    if bf16:
        w = w.bfloat16().float()
    (out.float() * w).sum().backward()
    d_h = w.permute(2, 0, 1, 3).reshape(T, B, H).cpu().numpy()
    o_wx, o_r, o_b, o_s0 = so.slstm_backward(wx, r, b, s0, None, d_h, None)
    d_r_ext = cell._recurrent_kernel_int2ext(cell._recurrent_kernel_.grad).float().cpu().numpy()
    d_b_ext = cell._bias_int2ext(cell._bias_.grad).float().cpu().numpy()
    errs = dict(d_wx=_rel(x.grad.float().cpu().numpy(), o_wx), d_r=_rel(d_r_ext, o_r), d_b=_rel(d_b_ext, o_b),
                d_s0=_rel(st.grad.float().cpu().numpy()[:3], o_s0[:3]))
    print(errs, flush=True)
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs


@pytest.mark.parametrize("row_tile", [16, 4])
def test_a_wait_between_compute_units_that_runs_out_is_reported(row_tile):
    """Host-forced: a negative spin limit makes every wait between the workgroups of a head give up at its first look
    (every kernel still exits normally).  The call must raise, the gradient of the initial state must be NaN, and the
    next call must be the usual one.  (A bound of one look does not do it: the peers' deltas are always there by the
    second look, as five calls in a row showed.)"""
    import ctypes

    from xlstm_amd import _lib
    from xlstm_amd import functional as F

    B, T, NH, dh = 16, 12, 4, 256
    wx, r, b, _ = make_problem(95, B, T, NH, dh, rscale=2.0, bf16=True)
    dev = torch.device("cuda:0")
    wx_t = torch.from_numpy(wx).to(dev).bfloat16()
    r_t, b_t = r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev)
    d_h = torch.randn(T, B, NH * dh, generator=torch.Generator().manual_seed(7)).to(dev).bfloat16()
    h, _ = F.slstm_forward(wx_t, r_t, b_t)
    print("case backward give-up, row tile", row_tile, flush=True)
    kw = dict(split_override=True, row_tile_override=row_tile)
    good = F.slstm_backward(wx_t, r_t, b_t, None, None, h, d_h, **kw)
    with pytest.raises(F.EngineError, match="ran out"):
        F.slstm_backward(wx_t, r_t, b_t, None, None, h, d_h, spin_limit=-1, **kw)
    # the same call with the synchronisation left to the caller (timings asked for): nothing raises, d_s0 is NaN
    t = {}
    got = F.slstm_backward(wx_t, r_t, b_t, None, None, h, d_h, spin_limit=-1, timings=t, **kw)
    torch.cuda.synchronize()
    assert bool(torch.isnan(got[3][:3]).all())
    again = F.slstm_backward(wx_t, r_t, b_t, None, None, h, d_h, **kw)  # the next call is unaffected
    assert torch.equal(again[0], good[0]) and torch.equal(again[3], good[3])
    # the way the cell's autograd function calls it: the abort word goes to the cell's status ring, nothing
    # synchronises or raises in the call, the cell reports it afterwards
    from tests.test_hip_cell import _cell_from

    cell = _cell_from(r, b, dtype="bfloat16")
    got = F.slstm_backward(wx_t, r_t, b_t, None, None, h, d_h, spin_limit=-1, abort_sink=cell._watch_word, **kw)
    with pytest.raises(F.EngineError, match="gave up"):
        cell.check_status()
    assert bool(torch.isnan(got[3][:3]).all())
    F.slstm_backward(wx_t, r_t, b_t, None, None, h, d_h, abort_sink=cell._watch_word, **kw)
    cell.check_status()  # (a good call leaves nothing to report)


_ORACLE_RESULTS = {}


def _kernel_kw(split):
    """False: one workgroup per head; True: a head over dh/64 compute units in row tiles of 16 rows; 4: in row tiles of 4."""
    return dict(split_override=bool(split), row_tile_override=None if split is False else (4 if split == 4 and split is not True else 16))


def _run_both(bf16, B, T, NH, dh, seed, masked, with_state, mean_len=None, d_sf=None, **opts):
    """The engine's backward and the oracle's on one seeded problem; returns the four relative errors."""
    from xlstm_amd import functional as F

    H = NH * dh
    wx, r, b, s0 = make_problem(seed, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=with_state)
    reset = geometric_reset_mask(seed + 1, B, T, mean_len or max(2, T // 2)) if masked else None
    if reset is not None and with_state:
        reset[0, 0] = 0
    d_h = np.random.default_rng(seed + 2).standard_normal((T, B, H)).astype(np.float32)
    dev = torch.device("cuda:0")
    wx_t = torch.from_numpy(wx).to(dev)
    if bf16:
        wx_t = wx_t.bfloat16()
        d_h = torch.from_numpy(d_h).bfloat16().float().numpy()
        r = torch.from_numpy(r).bfloat16().float().numpy()
    r_t, b_t = r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev)
    s0_t = torch.from_numpy(s0).to(dev) if s0 is not None else None
    m_t = torch.from_numpy(reset).to(dev) if reset is not None else None
    dsf_t = torch.from_numpy(d_sf).to(dev) if d_sf is not None else None
    h, _ = F.slstm_forward(wx_t, r_t, b_t, s0_t, m_t)
    kw = {k: v for k, v in opts.items() if k in ("recurrent_cut", "recurrent_clipval", "split_override", "row_tile_override", "stepwise_override", "d_wx_dtype")}
    d_wx, d_r, d_b, d_s0 = F.slstm_backward(wx_t, r_t, b_t, s0_t, m_t, h, torch.from_numpy(d_h).to(dev), dsf_t, **kw)
    torch.cuda.synchronize()
    okw = {k: v for k, v in opts.items() if k in ("recurrent_cut", "recurrent_clipval")}
    key = (bf16, B, T, NH, dh, seed, masked, with_state, mean_len, None if d_sf is None else d_sf.tobytes(), tuple(sorted(okw.items())))
    if key not in _ORACLE_RESULTS:  # (the same problem through several kernels: the oracle runs once)
        _ORACLE_RESULTS[key] = so.slstm_backward(wx, r, b, s0, reset, d_h, d_sf, **okw)
    o_wx, o_r, o_b, o_s0 = _ORACLE_RESULTS[key]
    errs = dict(d_wx=_rel(d_wx.float().cpu().numpy(), o_wx), d_r=_rel(d_r.cpu().numpy(), r_ext_to_kernel(torch.from_numpy(o_r)).numpy()),
                d_b=_rel(d_b.cpu().numpy(), o_b), d_s0=_rel(d_s0.cpu().numpy(), o_s0))
    return errs, (d_wx, d_r, d_b, d_s0), (o_wx, o_r, o_b, o_s0)


@pytest.mark.parametrize("row_tile", [4, 16])
def test_backward_over_2048_steps_bf16_packed_documents(row_tile):
    """The length of BASELINE config 2 (T = 2048, 4 heads of 256, bf16, packed geometric documents) on a few batch
    rows (rows are independent; the oracle affords three of them): what 2048 reverse steps on bf16 operands do to the
    error, against the float64 oracle, in both row tilings of the kernel that spreads a head over four compute units
    (4 rows: what config 2 itself runs).  Tolerance 2e-2."""
    print("case backward T=2048 bf16 B=3 row tile", row_tile, flush=True)
    errs, _, _ = _run_both(True, 3, 2048, 4, 256, 301, masked=True, with_state=False, mean_len=512, row_tile_override=row_tile)
    print("backward, T = 2048, bf16:", errs, flush=True)
    assert all(np.isfinite(v) and v <= 2e-2 for v in errs.values()), errs


def test_backward_config1_shape_fp32_full_size():
    """BASELINE config 1 at full size (B 4, T 256, 4 heads of 128, float32, zero state): 1e-5 against the oracle."""
    print("case backward config 1 fp32", flush=True)
    errs, _, _ = _run_both(False, 4, 256, 4, 128, 302, masked=False, with_state=False)
    print("backward, config 1:", errs, flush=True)
    assert all(np.isfinite(v) and v <= 1e-5 for v in errs.values()), errs


@pytest.mark.parametrize("bf16,B,T,NH,dh,split", [(False, 5, 11, 2, 64, True), (False, 20, 9, 2, 128, True), (True, 16, 12, 4, 256, True),
                                                  (False, 4, 10, 2, 128, False), (True, 9, 8, 2, 512, True),
                                                  (True, 16, 12, 4, 256, 4), (True, 7, 10, 2, 128, 4)])
def test_the_gradient_of_the_final_state_by_the_chain_rule(bf16, B, T, NH, dh, split):
    """``d_s_final`` on the GPU, pinned the way the oracle's is: the gradients of a sequence are those of its second
    part, started from the state after step k - 1, and of its first part with the second part's ``d_s0`` as the
    gradient of its final state.  d_wx and d_s0 of the two calls reproduce the whole call's (float32: to rounding;
    bf16: the hand-over itself is exact, the deltas then differ by the rounding of the operands), and the y, c and n
    planes all carry something."""
    from xlstm_amd import functional as F

    k = T // 2
    H = NH * dh
    wx, r, b, s0 = make_problem(310, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=True)
    dev = torch.device("cuda:0")
    wx_t = torch.from_numpy(wx).to(dev)
    if bf16:
        wx_t = wx_t.bfloat16()
    r_t, b_t = r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev)
    s0_t = torch.from_numpy(s0).to(dev)
    d_h = torch.randn(T, B, H, generator=torch.Generator().manual_seed(311)).to(dev).to(wx_t.dtype)
    h, _ = F.slstm_forward(wx_t, r_t, b_t, s0_t)
    whole = F.slstm_backward(wx_t, r_t, b_t, s0_t, None, h, d_h, **_kernel_kw(split))
    h_a, s_k = F.slstm_forward(wx_t[:, :k], r_t, b_t, s0_t)
    h_b, _ = F.slstm_forward(wx_t[:, k:], r_t, b_t, s_k)
    assert torch.equal(torch.cat([h_a, h_b]), h)
    tail = F.slstm_backward(wx_t[:, k:], r_t, b_t, s_k, None, h_b, d_h[k:].contiguous(), **_kernel_kw(split))
    assert all(float(tail[3][i].abs().max()) > 0 for i in range(3)) and not bool(tail[3][3].any())
    head = F.slstm_backward(wx_t[:, :k], r_t, b_t, s0_t, None, h_a, d_h[:k].contiguous(), tail[3], **_kernel_kw(split))
    torch.cuda.synchronize()
    tol = 2e-2 if bf16 else 1e-5

    def rel(a, g):
        return float((a - g).abs().max() / max(1.0, float(g.abs().max())))

    errs = dict(d_wx=rel(torch.cat([head[0], tail[0]], 1), whole[0]), d_r=rel(head[1] + tail[1], whole[1]),
                d_b=rel(head[2] + tail[2], whole[2]), d_s0=rel(head[3], whole[3]))
    print("chain rule", bf16, B, T, NH, dh, split, errs, flush=True)
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs
    # not vacuous: without the hand-over the first part's gradients are not the whole call's
    plain = F.slstm_backward(wx_t[:, :k], r_t, b_t, s0_t, None, h_a, d_h[:k].contiguous(), **_kernel_kw(split))
    assert rel(plain[0], whole[0][:, :k]) > 10 * tol
    # and against the oracle, d_s_final given
    d_sf = tail[3].cpu().numpy()
    o = so.slstm_backward(wx[:, :k], torch.from_numpy(r).to(wx_t.dtype).float().numpy(), b, s0, None,
                          d_h[:k].float().cpu().numpy(), d_sf)
    assert _rel(head[0].cpu().numpy(), o[0]) <= tol and _rel(head[3].cpu().numpy(), o[3]) <= tol


@pytest.mark.parametrize("bf16,B,T,NH,dh,split", [(False, 5, 9, 2, 64, True), (False, 20, 7, 2, 128, True), (True, 16, 10, 4, 256, True),
                                                  (False, 4, 12, 4, 256, False), (True, 9, 7, 2, 512, True), (True, 6, 9, 2, 128, False),
                                                  (False, 7, 6, 2, 256, True), (True, 16, 10, 4, 256, 4), (True, 5, 9, 2, 64, 4)])
@pytest.mark.parametrize("opts", [dict(recurrent_cut=True), dict(recurrent_clipval=0.05), dict(recurrent_clipval=1.0),
                                  dict(recurrent_cut=True, recurrent_clipval=0.05)],
                         ids=["cut", "clip0.05", "clip1", "cut+clip"])
def test_recurrent_cut_and_clipval_against_the_oracle(bf16, B, T, NH, dh, split, opts):
    """``gradient_recurrent_cut`` / ``gradient_recurrent_clipval`` of the reference's native backward pass
    (slstm_backward_cut.cu:265-312, slstm_pointwise.cu:136-143) in both reverse kernels, with a mask, a state and a
    gradient of the final state, against the oracle's flags (pinned in tests/test_oracle_backward.py)."""
    H = NH * dh
    d_sf = np.random.default_rng(320).standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    print("case cut/clip", bf16, B, T, NH, dh, split, opts, flush=True)
    errs, got, want = _run_both(bf16, B, T, NH, dh, 321, masked=True, with_state=True, d_sf=d_sf, **_kernel_kw(split), **opts)
    print(errs, flush=True)
    tol = 2e-2 if bf16 else 1e-5
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs
    if opts.get("recurrent_cut"):
        assert not bool(got[3][0].any())  # nothing reaches the y of the initial state
    # the option bites: the plain gradient of the same problem is something else
    if opts.get("recurrent_cut") or opts.get("recurrent_clipval", 1.0) < 1.0:
        _, got_plain, _ = _run_both(bf16, B, T, NH, dh, 321, masked=True, with_state=True, d_sf=d_sf, **_kernel_kw(split))
        assert float((got_plain[0] - got[0]).abs().max()) > 1e-3


def test_cell_config_gradient_recurrent_cut_and_clipval():
    """The cell hands ``gradient_recurrent_cut`` / ``gradient_recurrent_clipval`` of its config to the backward pass
    (cell.py:84-87, 580-583 of the reference); a clip value below 1 would also clip the reference's forward
    (cell.py:200-210) and is refused at construction."""
    from tests.test_hip_cell import _cell_from
    from xlstm_amd.cell import sLSTMCell, sLSTMCellConfig

    B, T, NH, dh = 3, 8, 2, 64
    H = NH * dh
    wx, r, b, s0 = make_problem(330, B, T, NH, dh, rscale=2.0, with_state=True)
    w = np.random.default_rng(331).standard_normal((T, B, H)).astype(np.float32) * 4.0
    for kw in (dict(gradient_recurrent_cut=True), dict(gradient_recurrent_clipval=1.0)):
        cell = _cell_from(r, b, dtype="float32", **kw).train()
        x = torch.from_numpy(wx).cuda().requires_grad_(True)
        st = torch.from_numpy(s0).cuda().requires_grad_(True)
        out, _ = cell(x, st)                               # [B, NH, T, dh]
        (out * torch.from_numpy(w).cuda().view(T, B, NH, dh).permute(1, 2, 0, 3)).sum().backward()
        o = so.slstm_backward(wx, r, b, s0, None, w, None, recurrent_cut=kw.get("gradient_recurrent_cut", False),
                              recurrent_clipval=kw.get("gradient_recurrent_clipval"))
        plain = so.slstm_backward(wx, r, b, s0, None, w, None)
        assert np.abs(plain[0] - o[0]).max() > 1e-3, "the option does not bite in this problem"
        d_r_ext = cell._recurrent_kernel_int2ext(cell._recurrent_kernel_.grad).cpu().numpy()
        errs = dict(d_wx=_rel(x.grad.cpu().numpy(), o[0]), d_r=_rel(d_r_ext, o[1]),
                    d_s0=_rel(st.grad.cpu().numpy()[:3], o[3][:3]))
        print(kw, errs, flush=True)
        assert all(v <= 1e-5 for v in errs.values()), errs
    with pytest.raises(NotImplementedError, match="gradient_recurrent_clipval"):
        sLSTMCell(sLSTMCellConfig(hidden_size=H, num_heads=NH, backend="hip", gradient_recurrent_clipval=0.5))


@pytest.mark.parametrize("bf16,B,T,NH,dh,split", [(False, 5, 9, 2, 64, True), (True, 16, 12, 4, 256, True), (False, 4, 10, 2, 128, False),
                                                  (True, 14, 12, 4, 256, 4), (True, 3, 6, 1, 1024, "step"), (False, 66, 3, 1, 512, "step")])
def test_all_four_gradients_through_the_c_abi(bf16, B, T, NH, dh, split):
    """A caller without torch arithmetic - the binding a maintainer would put in place of the reference's
    ``sLSTMFunc.backward`` (slstm.cc:137-221, which returns {dx, ds0, dR, db} from one native call): forward, then the
    three backward entry points, through ctypes with buffers the caller owns; the recurrent matrix is brought into the
    reverse kernel's operand order with numpy on the host or by ``xs_slstm_backward_tile_r``.  All four gradients against
    the oracle."""
    import ctypes

    from xlstm_amd import _lib
    from xlstm_amd import functional as F

    lib = _lib.load()
    H = NH * dh
    wx, r, b, s0 = make_problem(340, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=True)
    reset = geometric_reset_mask(341, B, T, max(2, T // 2))
    reset[0, 0] = 0
    rng = np.random.default_rng(342)
    d_h = rng.standard_normal((T, B, H)).astype(np.float32)
    d_sf = rng.standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    tdt = torch.bfloat16 if bf16 else torch.float32
    dev = torch.device("cuda:0")
    if bf16:
        d_h = torch.from_numpy(d_h).bfloat16().float().numpy()
        r = torch.from_numpy(r).bfloat16().float().numpy()
    r_k = r_ext_to_kernel(torch.from_numpy(r)).numpy()                       # [NH, 4 dh, dh], the forward's layout
    # R transposed in the reverse kernel's operand order (include/xlstm_amd.h), by numpy
    epc = 8 if bf16 else 4
    tile_rows = 4 if split == 4 and split is not True else 16  # (split: False, True = row tiles of 16 rows, 4 = of 4 rows)
    stepwise = split == "step"                                 # ("step": one launch per step, the largest head dims)
    if stepwise:
        ks = 128 if bf16 else 64                                              # R transposed in slabs of 256 bytes of K
        r_t = r_k.transpose(0, 2, 1).reshape(NH, dh // 32, 32, 4 * dh // ks, ks).transpose(0, 1, 3, 2, 4)
    elif tile_rows == 4:
        S, ksteps = dh // 64, 4 * dh // 8 // 32                               # K ordered (unit, gate)
        r_t = (r_k.reshape(NH, 4, dh, dh).transpose(0, 2, 1, 3).reshape(NH, 4 * dh, dh)
               .reshape(NH, 8, ksteps, 4, 8, S, 4, 16).transpose(0, 5, 1, 2, 6, 3, 7, 4))
    elif split:
        S, ksteps = dh // 64, 4 * dh // 8 // (4 * epc)
        r_t = (r_k.reshape(NH, 4, S, 64, dh).transpose(0, 2, 1, 3, 4).reshape(NH, 4 * dh, dh)
               .reshape(NH, 8, ksteps, 4, epc, S, 4, 16).transpose(0, 5, 1, 2, 6, 3, 7, 4))
    else:
        r_t = r_k.transpose(0, 2, 1).reshape(NH, dh // 16, 16, 4 * dh // (4 * epc), 4, epc).transpose(0, 1, 3, 4, 2, 5)
    dev_t = lambda a, dt=torch.float32: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dt)
    wx_t, r_fwd, rt_t, b_t, s0_t = dev_t(wx, tdt), dev_t(r_k, tdt), dev_t(r_t, tdt), dev_t(b), dev_t(s0)
    m_t = torch.from_numpy(reset).to(dev)
    dh_t, dsf_t = dev_t(d_h, tdt), dev_t(d_sf)
    h, _ = F.slstm_forward(wx_t, r_fwd if bf16 else dev_t(r_k), b_t, s0_t, m_t)
    groups = NH * ((B + tile_rows - 1) // tile_rows)
    rows = (B + tile_rows - 1) // tile_rows * tile_rows if split and not stepwise else ((B + 63) // 64 * 64 if stepwise else B)
    coef = torch.empty(T * rows * 9 * H, dtype=torch.float32, device=dev)
    d_wx = torch.empty(B, T, 4 * H, dtype=torch.float32, device=dev)
    d_s0 = torch.empty(4, B, H, dtype=torch.float32, device=dev)
    d_r = torch.empty(NH, 4 * dh, dh, dtype=torch.float32, device=dev)
    d_b = torch.empty(NH, 4, dh, dtype=torch.float32, device=dev)
    exchange = torch.empty(4 * groups * tile_rows * 4 * dh, dtype=tdt, device=dev)
    counters = torch.empty(1 + 2 * groups, dtype=torch.int32, device=dev)
    if stepwise:  # (states and deltas from launch to launch; no counters: nothing waits)
        esz = 2 if bf16 else 4
        exchange = torch.empty(max(16 * B * H + 4 * NH * dh * dh * esz, 8 * ((B + 63) // 64 * 64) * H * esz), dtype=torch.uint8, device=dev)
    a = _lib.SlstmBwdArgs()
    a.B, a.T, a.NH, a.dh, a.dtype = B, T, NH, dh, _lib.XS_BF16 if bf16 else _lib.XS_F32
    a.wx, a.wx_stride_b, a.wx_stride_t = wx_t.data_ptr(), wx_t.stride(0), wx_t.stride(1)
    a.r, a.h_out, a.bias, a.s0 = r_fwd.data_ptr(), h.data_ptr(), b_t.data_ptr(), s0_t.data_ptr()
    a.reset, a.reset_stride_b = m_t.data_ptr(), m_t.stride(0)
    a.coef, a.d_h, a.d_s_final, a.r_t = coef.data_ptr(), dh_t.data_ptr(), dsf_t.data_ptr(), rt_t.data_ptr()
    a.d_wx, a.d_wx_stride_b, a.d_wx_stride_t, a.d_s0 = d_wx.data_ptr(), d_wx.stride(0), d_wx.stride(1), d_s0.data_ptr()
    a.d_r, a.d_bias = d_r.data_ptr(), d_b.data_ptr()
    a.stream = torch.cuda.current_stream().cuda_stream
    a.split = 3 if stepwise else ((2 if tile_rows == 4 else 1) if split else 0)
    a.exchange, a.counters = (exchange.data_ptr(), counters.data_ptr()) if split else (None, None)
    if stepwise:
        a.counters = None
    if stepwise or tile_rows == 4:  # (these cases let the library bring R into the reverse kernel's order)
        rt_lib = torch.empty(r_fwd.numel(), dtype=tdt, device=dev)
        a.r_t = rt_lib.data_ptr()
        assert lib.xs_slstm_backward_tile_r(ctypes.byref(a)) == 0, _lib.last_error()
    for fn in (lib.xs_slstm_backward_prepare, lib.xs_slstm_backward, lib.xs_slstm_backward_params):
        rc = fn(ctypes.byref(a))
        assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    if split and not stepwise:
        assert int(counters[0]) == 0
    o_wx, o_r, o_b, o_s0 = so.slstm_backward(wx, r, b, s0, reset, d_h, d_sf)
    tol = 2e-2 if bf16 else 1e-5
    errs = dict(d_wx=_rel(d_wx.cpu().numpy(), o_wx), d_r=_rel(d_r.cpu().numpy(), r_ext_to_kernel(torch.from_numpy(o_r)).numpy()),
                d_b=_rel(d_b.cpu().numpy(), o_b), d_s0=_rel(d_s0.cpu().numpy(), o_s0))
    print("C ABI backward", bf16, B, T, NH, dh, split, errs, flush=True)
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs


@pytest.mark.parametrize("B,T,NH,dh,masked", [(16, 12, 4, 256, True), (6, 9, 2, 128, True), (4, 2, 2, 128, False), (9, 33, 1, 256, True)])
def test_a_training_forward_leaves_the_coefficients_of_the_backward_pass(B, T, NH, dh, masked):
    """``slstm_forward(..., coef_out=)`` (the forward's kernel for row tiles of 4 rows with the gate values kept): h and
    the state are bit for bit those of the plain call, and the backward pass that takes the coefficients instead of
    walking forward itself returns the gradients of the one that does (the same formulas compiled into two kernels: last
    bits of a coefficient differ, and a gate delta that the compute units exchange in bf16 then rounds the other way:
    2e-3 of the largest entry) and the oracle's (2e-2)."""
    from xlstm_amd import functional as F

    H = NH * dh
    print("case forward coefficients", B, T, NH, dh, masked, flush=True)
    wx, r, b, s0 = make_problem(350, B, T, NH, dh, rscale=2.0, bf16=True, with_state=masked)
    reset = geometric_reset_mask(351, B, T, max(2, T // 2)) if masked else None
    if reset is not None:
        reset[0, 0] = 0
    rng = np.random.default_rng(352)
    d_h = torch.from_numpy(rng.standard_normal((T, B, H)).astype(np.float32)).bfloat16().float().numpy()
    d_sf = rng.standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    r = torch.from_numpy(r).bfloat16().float().numpy()
    dev = torch.device("cuda:0")
    wx_t = torch.from_numpy(wx).to(dev).bfloat16()
    r_t, b_t = r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev)
    s0_t = torch.from_numpy(s0).to(dev) if s0 is not None else None
    m_t = torch.from_numpy(reset).to(dev) if reset is not None else None
    dh_t, dsf_t = torch.from_numpy(d_h).to(dev), torch.from_numpy(d_sf).to(dev)
    coef = F.backward_coefficients_buffer(wx_t, NH)
    assert coef is not None and tuple(coef.shape) == (T, (B + 3) // 4 * 4, 9, H)
    coef.fill_(float("nan"))
    h_plain, s_plain = F.slstm_forward(wx_t, r_t, b_t, s0_t, m_t)
    h, s = F.slstm_forward(wx_t, r_t, b_t, s0_t, m_t, coef_out=coef)
    torch.cuda.synchronize()
    assert torch.equal(h, h_plain) and torch.equal(s, s_plain)
    # every coefficient of a row that exists has been written
    tiles = coef.view(T, (B + 3) // 4, NH, dh // 64, 4, 9, 64)
    rows_there = torch.arange((B + 3) // 4 * 4, device=dev).view(-1, 4) < B
    assert bool(torch.isfinite(tiles.permute(1, 4, 0, 2, 3, 5, 6)[rows_there]).all())
    got = F.slstm_backward(wx_t, r_t, b_t, s0_t, m_t, h, dh_t, dsf_t, coef=coef)
    ref = F.slstm_backward(wx_t, r_t, b_t, s0_t, m_t, h, dh_t, dsf_t, row_tile_override=4)
    torch.cuda.synchronize()
    for name, a, g in zip(("d_wx", "d_r", "d_b", "d_s0"), got, ref):
        assert _rel(a.cpu().numpy(), g.cpu().numpy()) <= 2e-3, name
    o_wx, o_r, o_b, o_s0 = so.slstm_backward(wx, r, b, s0, reset, d_h, d_sf)
    errs = dict(d_wx=_rel(got[0].cpu().numpy(), o_wx), d_r=_rel(got[1].cpu().numpy(), r_ext_to_kernel(torch.from_numpy(o_r)).numpy()),
                d_b=_rel(got[2].cpu().numpy(), o_b), d_s0=_rel(got[3].cpu().numpy(), o_s0))
    print(errs, flush=True)
    assert all(np.isfinite(v) and v <= 2e-2 for v in errs.values()), errs


def test_calls_that_cannot_leave_coefficients_say_so_before_anything_runs():
    """float32 inputs, head dims other than 128 and 256, batches whose row tiles of 4 rows do not fit the device: no
    buffer is offered, and a call that is handed one all the same raises ``CoefficientsUnsupported``."""
    from xlstm_amd import functional as F

    dev = torch.device("cuda:0")
    assert F.backward_coefficients_buffer(torch.zeros(4, 8, 4 * 256, device=dev), 2) is None                             # float32
    assert F.backward_coefficients_buffer(torch.zeros(4, 8, 4 * 128, device=dev, dtype=torch.bfloat16), 2) is None        # head dim 64
    assert F.backward_coefficients_buffer(torch.zeros(300, 8, 4 * 1024, device=dev, dtype=torch.bfloat16), 4) is None     # too many rows
    B, T, NH, dh = 300, 3, 4, 256
    H = NH * dh
    wx = torch.randn(B, T, 4 * H, device=dev).bfloat16()
    r = torch.randn(NH, 4 * dh, dh, device=dev) * 0.05
    b = torch.zeros(NH, 4, dh, device=dev)
    coef = torch.empty(T, (B + 3) // 4 * 4, 9, H, device=dev)
    with pytest.raises(F.CoefficientsUnsupported):
        F.slstm_forward(wx, r, b, coef_out=coef)
    h, _ = F.slstm_forward(wx, r, b)  # the plain call is the usual one
    assert bool(torch.isfinite(h.float()).all())


def test_cell_that_keeps_the_backward_coefficients_has_the_same_gradients(monkeypatch):
    """The cell's default (a training forward leaves the coefficients, the backward call skips its forward walk) against
    ``keep_backward_coefficients = False``; the backward calls are watched to see that each ran the way it was meant to."""
    from tests.test_hip_cell import _cell_from
    from xlstm_amd import cell as cell_module
    from xlstm_amd import functional as F

    assert cell_module.sLSTMCell_hip.keep_backward_coefficients is True
    seen = []
    plain_backward = F.slstm_backward

    def watched(*a, **kw):
        seen.append(kw.get("coef") is not None)
        return plain_backward(*a, **kw)

    monkeypatch.setattr(cell_module.F_hip, "slstm_backward", watched)

    B, T, NH, dh = 8, 16, 2, 128
    wx, r, b, s0 = make_problem(360, B, T, NH, dh, rscale=2.0, bf16=True, with_state=True)
    r = torch.from_numpy(r).bfloat16().float().numpy()
    mask = torch.from_numpy(geometric_reset_mask(361, B, T, 6)).cuda()
    w = torch.randn(B, NH, T, dh, generator=torch.Generator().manual_seed(9)).cuda()
    grads = []
    for keep in (False, True):
        cell = _cell_from(r, b, dtype="bfloat16").train()
        cell.keep_backward_coefficients = keep
        x = torch.from_numpy(wx).cuda().bfloat16().requires_grad_(True)
        st = torch.from_numpy(s0).cuda().bfloat16().requires_grad_(True)
        out, _ = cell(x, st, reset_mask=mask)
        (out.float() * w).sum().backward()
        grads.append((x.grad.float(), cell._recurrent_kernel_.grad.float(), cell._bias_.grad.float(), st.grad.float()))
    assert seen == [False, True]
    for a, g in zip(grads[1], grads[0]):
        assert float((a - g).abs().max()) <= 2e-3 * max(1.0, float(g.abs().max()))


@pytest.mark.parametrize("bf16,NH,dh,split", [(True, 2, 256, 0), (False, 2, 128, 0), (True, 2, 512, 1), (False, 3, 256, 1), (True, 4, 256, 2),
                                              (True, 1, 64, 2), (True, 2, 1024, 3), (True, 1, 640, 3), (False, 2, 512, 3), (False, 1, 320, 3)])
def test_the_library_tiles_r_as_the_header_describes(bf16, NH, dh, split):
    """``xs_slstm_backward_tile_r`` against the layouts of ``r_t`` in ``include/xlstm_amd.h`` written out with numpy, for
    every reverse kernel (``split`` 0 to 3), bit for bit."""
    import ctypes

    from xlstm_amd import _lib

    lib = _lib.load()
    rng = np.random.default_rng(370)
    r_k = rng.standard_normal((NH, 4 * dh, dh)).astype(np.float32)          # [NH, k = g dh + a, d]
    epc = 8 if bf16 else 4
    if split == 0:
        want = r_k.transpose(0, 2, 1).reshape(NH, dh // 16, 16, 4 * dh // (4 * epc), 4, epc).transpose(0, 1, 3, 4, 2, 5)
    elif split == 3:
        ks = 128 if bf16 else 64
        want = r_k.transpose(0, 2, 1).reshape(NH, dh // 32, 32, 4 * dh // ks, ks).transpose(0, 1, 3, 2, 4)
    else:
        S, ksteps = dh // 64, 4 * dh // 8 // (4 * epc)
        if split == 2:                                                       # K ordered (unit, gate)
            rp = r_k.reshape(NH, 4, dh, dh).transpose(0, 2, 1, 3).reshape(NH, 4 * dh, dh)
        else:                                                                # K ordered (owner slice, gate, unit % 64)
            rp = r_k.reshape(NH, 4, S, 64, dh).transpose(0, 2, 1, 3, 4).reshape(NH, 4 * dh, dh)
        want = rp.reshape(NH, 8, ksteps, 4, epc, S, 4, 16).transpose(0, 5, 1, 2, 6, 3, 7, 4)
    tdt = torch.bfloat16 if bf16 else torch.float32
    r_dev = torch.from_numpy(r_k).cuda().to(tdt)
    out = torch.empty(r_dev.numel(), dtype=tdt, device="cuda")
    a = _lib.SlstmBwdArgs()
    a.NH, a.dh, a.dtype, a.split = NH, dh, _lib.XS_BF16 if bf16 else _lib.XS_F32, split
    a.r, a.r_t = r_dev.data_ptr(), out.data_ptr()
    a.stream = torch.cuda.current_stream().cuda_stream
    assert lib.xs_slstm_backward_tile_r(ctypes.byref(a)) == 0, _lib.last_error()
    torch.cuda.synchronize()
    want_t = torch.from_numpy(np.ascontiguousarray(want)).to(tdt).reshape(-1)
    assert torch.equal(out.cpu(), want_t)


@pytest.mark.parametrize("B,T,NH,dh,kernel", [(6, 9, 2, 128, "one-unit"), (20, 7, 2, 256, "split"), (9, 6, 2, 512, "split"),
                                              (16, 12, 4, 256, "quad"), (7, 5, 3, 64, "quad"), (5, 6, 1, 1024, "step"), (70, 3, 2, 640, "step")])
def test_gate_deltas_in_bfloat16(B, T, NH, dh, kernel):
    """``d_wx_dtype = XS_BF16``: every reverse kernel writes the gate deltas rounded to bf16 - exactly the float32 ones
    rounded - and the parameter kernel reads them in that type: all four gradients against the oracle as before."""
    print("case d_wx in bf16", B, T, NH, dh, kernel, flush=True)
    H = NH * dh
    d_sf = np.random.default_rng(381).standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    if kernel == "step":
        kw = {}
    else:
        split, row_tile = _row_tile_of(kernel)
        kw = dict(split_override=split, row_tile_override=row_tile)
    errs, got, _ = _run_both(True, B, T, NH, dh, 380, masked=True, with_state=True, d_sf=d_sf, d_wx_dtype=torch.bfloat16, **kw)
    print(errs, flush=True)
    assert got[0].dtype == torch.bfloat16
    assert all(np.isfinite(v) and v <= 2e-2 for v in errs.values()), errs
    _, ref, _ = _run_both(True, B, T, NH, dh, 380, masked=True, with_state=True, d_sf=d_sf, **kw)
    assert torch.equal(got[0], ref[0].bfloat16())
    assert torch.equal(got[3], ref[3])
