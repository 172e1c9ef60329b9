"""GPU parity tests: the HIP engine (through the C ABI) against the CPU oracle.

Tolerances (|a - ref| <= tol * max(1, |ref|)):
  float32 path : 1e-5 against the float64 oracle
  bfloat16 path: 2e-2 against the float64 oracle run on the bf16-rounded inputs
  resets / chunking / step-by-step: bit-exact against the engine itself
"""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import slstm_oracle as so
from tests._util import geometric_reset_mask, make_problem, max_err, r_ext_to_kernel

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
TOL_F32 = 1e-5
TOL_BF16 = 2e-2


def _run_hip(wx, r_ext, b_ext, s0=None, reset=None, bf16=False, **kw):
    from xlstm_amd import functional as F

    dev = torch.device("cuda:0")
    wx_t = torch.from_numpy(wx).to(dev)
    if bf16:
        wx_t = wx_t.bfloat16()
    r_t = r_ext_to_kernel(torch.from_numpy(r_ext)).to(dev)
    b_t = torch.from_numpy(b_ext).to(dev)
    s0_t = torch.from_numpy(s0).to(dev) if s0 is not None else None
    m_t = torch.from_numpy(reset).to(dev) if reset is not None else None
    ws = F.workspace_for(wx.shape[0], wx.shape[1], r_ext.shape[0], r_ext.shape[1], dev)
    h, s = F.slstm_forward(wx_t, r_t, b_t, s0_t, m_t, workspace=ws, **kw)
    torch.cuda.synchronize()
    status = F.read_status(ws)
    return h.float().cpu().numpy(), s.cpu().numpy(), status


def _check(h, s, h_ref, s_ref, tol, status):
    assert status["aborted"] == 0, status
    assert np.isfinite(h).all() and np.isfinite(s).all()
    eh, es = max_err(h, h_ref), max_err(s, s_ref)
    assert eh <= tol, f"h error {eh:.3e} > {tol}"
    assert es <= tol, f"state error {es:.3e} > {tol}"


@pytest.mark.parametrize("path", sorted(p for p in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(p).startswith(("layer_", "ckpt_", "bwd_"))), ids=lambda p: os.path.basename(p)[:-4])
def test_reference_golden_vectors_f32(path):
    """The reference's own vanilla outputs (written by tests/golden/make_golden.py)."""
    z = np.load(path)
    if "mixed_n" in path:
        pytest.skip("vanilla's whole-tensor n==0 rule; the engine uses the native per-element rule")
    s0 = z["s0"] if z["s0"].size else None
    NH = z["r_ext"].shape[0]
    print("case", os.path.basename(path), z["wx"].shape, flush=True)
    h, s, status = _run_hip(z["wx"], z["r_ext"], z["b_ext"], s0)
    T, B, H = h.shape
    out = h.reshape(T, B, NH, H // NH).transpose(1, 2, 0, 3)
    _check(out, s, z["out_bnsh"], z["state"], TOL_F32, status)


def test_mixed_n_golden_matches_per_element_oracle():
    z = np.load(os.path.join(GOLDEN, "seq_mixed_n.npz"))
    h_ref, s_ref = so.slstm_forward(z["wx"], z["r_ext"], z["b_ext"], z["s0"], None, n0_rule=so.N0_PER_ELEMENT)
    h, s, status = _run_hip(z["wx"], z["r_ext"], z["b_ext"], z["s0"])
    _check(h, s, h_ref, s_ref, TOL_F32, status)


F32_CASES = [
    # B, T, NH, dh, with_state, resets
    (4, 256, 4, 128, False, False),   # BASELINE config 1
    (1, 1, 4, 16, True, False),       # the reference test's shape
    (3, 40, 2, 64, True, True),
    (5, 33, 3, 24, False, True),      # head dim not a multiple of 16
    (17, 20, 2, 32, True, True),      # batch not a multiple of 16 -> two tiles
    (40, 12, 1, 256, False, False),
    (2, 64, 2, 512, True, True),      # largest fp32 head
    (70, 6, 4, 512, False, True),     # four row tiles per workgroup (ragged), the drainer wave publishes
    (50, 9, 8, 256, True, True),      # two row tiles (ragged): W.x is fetched in bursts of four iterations
    (64, 1, 16, 128, False, False),   # two full row tiles, a single step: fewer iterations than one burst
    (70, 5, 4, 128, True, True),      # one row tile of 16 rows (ragged batch): bursts with one tile
]


@pytest.mark.parametrize("B,T,NH,dh,with_state,resets", F32_CASES)
def test_f32_against_f64_oracle(B, T, NH, dh, with_state, resets):
    print("case f32", B, T, NH, dh, with_state, resets, flush=True)
    wx, r, b, s0 = make_problem(11, B, T, NH, dh, rscale=4.0, with_state=with_state)
    reset = geometric_reset_mask(5, B, T, max(2, T // 3)) if resets else None
    if reset is not None and with_state:
        reset[:, 0] = 0  # let the supplied state matter
    h_ref, s_ref = so.slstm_forward(wx, r, b, s0, reset)
    h, s, status = _run_hip(wx, r, b, s0, reset)
    _check(h, s, h_ref, s_ref, TOL_F32, status)


BF16_CASES = [
    (16, 128, 4, 256, False, True),   # BASELINE config 2 shape, short T
    (4, 50, 2, 128, True, True),
    (3, 30, 4, 16, True, False),
    (20, 16, 2, 64, False, True),
    (64, 8, 1, 1024, False, False),   # config 5 head size, one head
    (33, 10, 8, 256, True, True),     # config 3 prefill shape, short
    (50, 12, 4, 1024, True, True),    # config 5 shape, ragged batch: four row tiles, groups over two XCDs
    (100, 6, 8, 256, True, True),     # four row tiles inside one XCD, two row groups, ragged
    (40, 8, 4, 768, True, False),     # 48 members per head: 24 + 24 on an XCD pair
    (24, 8, 3, 1000, False, True),    # odd member count (spread placement), partial last member, two row tiles
    (40, 21, 8, 256, True, True),     # two row tiles (ragged), W.x in bursts of eight iterations, 42 iterations
    (64, 37, 8, 256, False, True),    # two full row tiles, bursts, 74 iterations
    (64, 3, 4, 512, True, False),     # two full row tiles of a 512-wide head, fewer iterations than one burst
    (32, 21, 4, 256, True, True),     # one row tile of 8 rows: prefetch waves and bursts together, 21 iterations
    (50, 9, 4, 256, False, True),     # one row tile of 16 rows, ragged batch, bursts
]


@pytest.mark.parametrize("B,T,NH,dh,with_state,resets", BF16_CASES)
def test_bf16_against_f64_oracle(B, T, NH, dh, with_state, resets):
    print("case bf16", B, T, NH, dh, with_state, resets, flush=True)
    wx, r, b, s0 = make_problem(12, B, T, NH, dh, rscale=1.0, bf16=True, with_state=with_state)
    reset = geometric_reset_mask(6, B, T, max(2, T // 3)) if resets else None
    if reset is not None and with_state:
        reset[:, 0] = 0
    h_ref, s_ref = so.slstm_forward(wx, r, b, s0, reset)
    h, s, status = _run_hip(wx, r, b, s0, reset, bf16=True)
    _check(h, s, h_ref, s_ref, TOL_BF16, status)


@pytest.mark.parametrize("bf16", [False, True])
def test_packed_documents_equal_documents_run_alone_bit_exact(bf16):
    B, T, NH, dh = 6, 48, 2, 64
    wx, r, b, _ = make_problem(13, B, T, NH, dh, rscale=4.0, bf16=bf16)
    reset = geometric_reset_mask(7, B, T, 12)
    h, s, status = _run_hip(wx, r, b, None, reset, bf16=bf16)
    assert status["aborted"] == 0
    for row in range(B):
        starts = list(np.flatnonzero(reset[row])) + [T]
        for lo, hi in zip(starts[:-1], starts[1:]):
            hd, sd, st = _run_hip(wx[row:row + 1, lo:hi], r, b, None, None, bf16=bf16)
            assert st["aborted"] == 0
            np.testing.assert_array_equal(hd[:, 0], h[lo:hi, row])
            if hi == T:
                np.testing.assert_array_equal(sd[:, 0], s[:, row])


@pytest.mark.parametrize("bf16", [False, True])
def test_chunked_and_stepwise_equal_whole_bit_exact(bf16):
    B, T, NH, dh = 5, 24, 2, 128
    wx, r, b, s0 = make_problem(14, B, T, NH, dh, rscale=4.0, bf16=bf16, with_state=True)
    h, s, _ = _run_hip(wx, r, b, s0, bf16=bf16)
    ha, sa, _ = _run_hip(wx[:, :10], r, b, s0, bf16=bf16)
    hb, sb, _ = _run_hip(wx[:, 10:], r, b, sa, bf16=bf16)
    np.testing.assert_array_equal(np.concatenate([ha, hb]), h)
    np.testing.assert_array_equal(sb, s)
    st = s0
    for t in range(T):
        ht, st, status = _run_hip(wx[:, t:t + 1], r, b, st, bf16=bf16, step=True)
        assert status["aborted"] == 0
        np.testing.assert_array_equal(ht[0], h[t])
    np.testing.assert_array_equal(st, s)


def test_empty_sequence_returns_initial_state():
    wx, r, b, s0 = make_problem(15, 3, 0, 2, 32, with_state=True)
    h, s, _ = _run_hip(wx, r, b, s0)
    assert h.shape == (0, 3, 64)
    np.testing.assert_array_equal(s, s0)
    h, s, _ = _run_hip(wx, r, b, None)
    np.testing.assert_array_equal(s, np.zeros_like(s0))


def _assert_flagged_or_right(h, s, status, h_ref, s_ref):
    """A call whose bounded wait ran out says so twice: in the status block and by NaN in every output a workgroup
    wrote after the give-up (at least the final state of the workgroup that gave up).  A call that never had to
    wait longer than the bound is simply right."""
    if status["aborted"]:
        assert not np.isfinite(s).all(), "aborted call left a plausible final state"
        assert not np.isfinite(h).all(), "aborted call left a plausible h"
    else:
        assert max_err(h, h_ref) <= TOL_BF16 and max_err(s, s_ref) <= TOL_BF16


def test_spin_limit_runs_out_is_reported_not_hung():
    """Error path forced from the host: a one-iteration bound on the waits
    between compute units.  The kernel must finish, flag the call and poison its outputs."""
    wx, r, b, _ = make_problem(16, 16, 64, 4, 256, bf16=True)
    h_ref, s_ref = so.slstm_forward(wx, r, b, None, None)
    # (256 workgroups that look for their 15 peers exactly once: some peer is always a moment late.  Should every look
    # ever succeed the call is simply right, so the call is made up to five times until the give-up path has run.)
    seen = []
    for _ in range(5):
        h, s, status = _run_hip(wx, r, b, bf16=True, spin_limit=1)
        assert status["aborted"] in (0, 1)
        seen.append(status["aborted"])
        if status["aborted"]:
            assert status["abort_step"] >= 1
        _assert_flagged_or_right(h, s, status, h_ref, s_ref)
        if status["aborted"]:
            break
    print("one row tile, spin limit 1: aborted flags of the calls made:", seen, flush=True)
    assert seen[-1] == 1, "the give-up path never ran"
    # four row tiles per workgroup: the drainer wave's wait for the compute waves is bounded the same way
    wx, r, b, _ = make_problem(17, 64, 6, 4, 1024, bf16=True)
    h_ref, s_ref = so.slstm_forward(wx, r, b, None, None)
    seen = []
    for _ in range(5):
        h, s, status = _run_hip(wx, r, b, bf16=True, spin_limit=1)
        assert status["aborted"] in (0, 1)
        seen.append(status["aborted"])
        _assert_flagged_or_right(h, s, status, h_ref, s_ref)
        if status["aborted"]:
            break
    print("four row tiles, spin limit 1: aborted flags of the calls made:", seen, flush=True)
    assert seen[-1] == 1, "the give-up path never ran"
    # and the next call on the same device is unaffected
    h2, s2, status2 = _run_hip(wx, r, b, bf16=True)
    assert status2["aborted"] == 0
    assert max_err(h2, h_ref) <= TOL_BF16


def test_cell_raises_for_an_aborted_call_at_the_next_host_contact():
    """The cell copies the status word of every sequence call to pinned memory behind the kernel; a call that gave
    up surfaces as EngineError from check_status() (or from the cell's next call)."""
    from xlstm_amd import functional as F
    from xlstm_amd.cell import sLSTMCell, sLSTMCellConfig

    wx, r, b, _ = make_problem(16, 16, 64, 4, 256, bf16=True)
    cell = sLSTMCell(sLSTMCellConfig(hidden_size=1024, num_heads=4, backend="hip", output_shape="SBH"))
    cell.recurrent_kernel[:] = torch.from_numpy(r)
    cell.bias[:] = torch.from_numpy(b)
    cell = cell.to("cuda:0").eval()
    x = torch.from_numpy(wx).cuda().bfloat16()
    with torch.no_grad():
        out, st = cell(x)
        cell.check_status()  # a normal call: nothing to report
        assert cell.last_status()["aborted"] == 0 and bool(torch.isfinite(st.float()).all())
        # the same call with a one-poll bound, through the cell's own workspace and watch
        ws = cell._workspace(16, x.device)
        h, s = F.slstm_forward(x, cell._recurrent_kernel_.detach(), cell._bias_.detach().view(4, 4, 256), None, None,
                               workspace=ws, spin_limit=1)
        cell._watch(ws)
        torch.cuda.synchronize()
        gave_up = bool(F.read_status(ws)["aborted"])
        print("cell watch, spin limit 1: the call gave up:", gave_up, flush=True)
        assert gave_up, "256 workgroups looking for their peers exactly once all found them"
        assert not bool(torch.isfinite(s).all())
        with pytest.raises(F.EngineError, match="gave up waiting"):
            cell.check_status()
        out2, st2 = cell(x)  # the cell keeps working
        cell.check_status()
        assert torch.equal(out2, out) and torch.equal(st2, st)


MASKED_START_CASES = [
    # bf16, B, T, NH, dh: a supplied state AND a mask whose first column is mixed 0 / 1
    (False, 6, 9, 2, 64),      # one row tile of 4 rows ... 8 rows
    (False, 40, 5, 4, 128),    # 16-row tiles, ragged
    (False, 70, 4, 4, 512),    # four row tiles (the drainer publishes), fp32
    (True, 16, 12, 4, 256),    # BASELINE config 2's variant
    (True, 50, 6, 8, 256),     # two row tiles
    (True, 70, 5, 4, 1024),    # four row tiles, groups over two XCDs
    (True, 5, 7, 3, 40),       # K tail
]


@pytest.mark.parametrize("bf16,B,T,NH,dh", MASKED_START_CASES)
def test_mask_at_the_first_step_overrides_the_supplied_state(bf16, B, T, NH, dh):
    """mask[b, 0] = 1 makes row b ignore the state it was given (the row starts a document), rows with
    mask[b, 0] = 0 continue from it: sequence kernel and step kernel against the oracle, and the masked rows
    bit for bit against the same call without a state."""
    print("case masked start", bf16, B, T, NH, dh, flush=True)
    wx, r, b, s0 = make_problem(31, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=True)
    reset = geometric_reset_mask(9, B, T, max(2, T // 2))
    reset[:, 0] = (np.arange(B) % 3 != 1).astype(np.uint8)  # rows 1, 4, 7, ... continue from s0
    tol = TOL_BF16 if bf16 else TOL_F32
    h_ref, s_ref = so.slstm_forward(wx, r, b, s0, reset)
    h, s, status = _run_hip(wx, r, b, s0, reset, bf16=bf16)
    _check(h, s, h_ref, s_ref, tol, status)
    # the state really matters for the rows that keep it, and not at all for the others
    h_z, s_z, _ = _run_hip(wx, r, b, None, reset, bf16=bf16)
    fresh = reset[:, 0] != 0
    np.testing.assert_array_equal(h[:, fresh], h_z[:, fresh])
    np.testing.assert_array_equal(s[:, fresh], s_z[:, fresh])
    assert np.abs(h[0][~fresh] - h_z[0][~fresh]).max() > 1e-3
    # the step kernel, one token at a time, with the same first-column mask
    st = s0
    for t in range(min(T, 3)):
        ht, st, status = _run_hip(wx[:, t:t + 1], r, b, st, reset[:, t:t + 1], bf16=bf16, step=True)
        assert status["step_kernel"] == 1
        np.testing.assert_array_equal(ht[0], h[t])
    h1_ref, s1_ref = so.slstm_forward(wx[:, :1], r, b, s0, reset[:, :1])
    h1, s1, _ = _run_hip(wx[:, :1], r, b, s0, reset[:, :1], bf16=bf16, step=True)
    assert max_err(h1, h1_ref) <= tol and max_err(s1, s1_ref) <= tol


def test_head_groups_are_sized_per_xcd():
    """24 workgroups per head group (dh 384): an XCD of 32 compute units holds ONE such group, so 10 heads go in
    two launches of at most 8 groups.  Sized per device (256 / 24 = 10 groups) two XCDs would get 48 workgroups
    and the late group's members would spin until the early ones finish.  A few hundred steps, no long waits."""
    B, T, NH, dh = 4, 300, 10, 384
    print("case per-XCD sizing", B, T, NH, dh, flush=True)
    wx, r, b, _ = make_problem(41, B, T, NH, dh, bf16=True)
    h_ref, s_ref = so.slstm_forward(wx, r, b, None, None)
    h, s, status = _run_hip(wx, r, b, bf16=True)
    _check(h, s, h_ref, s_ref, TOL_BF16, status)
    assert status["launches"] == 2, status
    assert status["max_spins"] < 20000, status  # (a starved group would need millions of polls per step)


def test_status_reports_the_number_of_launches():
    """A batch that does not fit the compute units at once runs as several launches of row chunks."""
    from xlstm_amd import functional as F

    dev = torch.device("cuda:0")
    torch.manual_seed(9)
    for B, NH, dh, want in ((16, 4, 256, 1), (256, 8, 256, 2)):
        H = NH * dh
        wx = torch.randn(B, 3, 4 * H, device=dev).bfloat16()
        r = (torch.rand(NH, 4 * dh, dh, device=dev) - 0.5) * 0.1
        bias = torch.zeros(NH, 4, dh, device=dev)
        ws = F.workspace_for(B, 3, NH, dh, dev)
        F.slstm_forward(wx, r, bias, None, None, workspace=ws)
        torch.cuda.synchronize()
        st = F.read_status(ws)
        assert st["aborted"] == 0 and st["launches"] == want, st


def test_fresh_rows_among_continued_rows_match_vanilla_rule_up_to_the_stabiliser():
    """A supplied state whose rows are partly fresh (all zero) and partly
    carried: vanilla's whole-tensor test (vanilla/slstm.py:24-28) then takes
    m' = max(i, m + logsigmoid(f)) also for the fresh rows, the per-element
    rule (slstm_pointwise.cu:79) m' = i.  That only moves the stabiliser:
    h, c / n and m + log(n) are the same, and those are what is compared."""
    B, T, NH, dh = 6, 24, 2, 32
    wx, r_ext, b_ext, s0 = make_problem(77, B, T, NH, dh, with_state=True)
    s0[:, ::2] = 0.0  # rows 0, 2, 4 start fresh
    h_ref, s_ref = so.slstm_forward(wx, r_ext, b_ext, s0, None, n0_rule=so.N0_WHOLE_TENSOR)
    print("case fresh-among-continued", wx.shape, flush=True)
    h, s, status = _run_hip(wx, r_ext, b_ext, s0)
    assert status["aborted"] == 0, status
    assert max_err(h, h_ref) <= TOL_F32
    assert max_err(s[0], s_ref[0]) <= TOL_F32
    assert max_err(s[1] / s[2], s_ref[1] / s_ref[2]) <= TOL_F32
    assert max_err(s[3] + np.log(s[2]), s_ref[3] + np.log(s_ref[2])) <= TOL_F32
    # the rules do differ here: the stabiliser of a fresh row is not the vanilla one
    h1, s1 = so.slstm_forward(wx[:, :1], r_ext, b_ext, s0, None, n0_rule=so.N0_WHOLE_TENSOR)
    h2, s2 = so.slstm_forward(wx[:, :1], r_ext, b_ext, s0, None, n0_rule=so.N0_PER_ELEMENT)
    assert np.abs(s1[3, ::2] - s2[3, ::2]).max() > 1e-3
    assert max_err(h1, h2) <= 1e-12
