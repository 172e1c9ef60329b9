"""Pins the CPU oracle: reference golden vectors, closed forms, brute force,
invariants.  Each check is chosen so that a plausible mistake (gate order,
transposed R, wrong stabiliser, dropped bias, wrong state order) fails it."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import slstm_oracle as so
from oracle import vanilla_port as vp

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _cases():
    return sorted(p for p in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(p).startswith(("layer_", "ckpt_", "bwd_")))


def _bnsh(h, NH):
    T, B, H = h.shape
    return h.reshape(T, B, NH, H // NH).transpose(1, 2, 0, 3)


def test_golden_files_present():
    assert len(_cases()) >= 7


@pytest.mark.parametrize("path", _cases(), ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_matches_reference_vanilla_golden(path):
    z = np.load(path)
    s0 = z["s0"] if z["s0"].size else None
    NH = z["r_ext"].shape[0]
    for dtype, tol in ((np.float64, 2e-6), (np.float32, 5e-6)):
        h, s = so.slstm_forward(z["wx"], z["r_ext"], z["b_ext"], s0, None,
                                n0_rule=so.N0_WHOLE_TENSOR, dtype=dtype)
        np.testing.assert_allclose(_bnsh(h, NH), z["out_bnsh"], rtol=tol, atol=tol)
        np.testing.assert_allclose(s, z["state"], rtol=tol, atol=tol)


@pytest.mark.parametrize("path", _cases(), ids=lambda p: os.path.basename(p)[:-4])
def test_torch_port_matches_reference_vanilla_golden(path):
    z = np.load(path)
    s0 = torch.from_numpy(z["s0"]) if z["s0"].size else None
    NH = z["r_ext"].shape[0]
    h, s = vp.slstm_forward(torch.from_numpy(z["wx"]), torch.from_numpy(z["r_ext"]),
                            torch.from_numpy(z["b_ext"]), s0, None, per_element_n0=False)
    np.testing.assert_allclose(_bnsh(h.numpy(), NH), z["out_bnsh"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(s.numpy(), z["state"], rtol=1e-5, atol=1e-5)


def test_mixed_n_golden_separates_the_two_stabiliser_rules():
    z = np.load(os.path.join(GOLDEN, "seq_mixed_n.npz"))
    h_el, _ = so.slstm_forward(z["wx"], z["r_ext"], z["b_ext"], z["s0"], None, n0_rule=so.N0_PER_ELEMENT)
    h_wh, _ = so.slstm_forward(z["wx"], z["r_ext"], z["b_ext"], z["s0"], None, n0_rule=so.N0_WHOLE_TENSOR)
    # row 1 (n > 0) agrees, row 0 (n == 0, m != 0) carries a different stabiliser m
    np.testing.assert_allclose(h_el[:, 1], h_wh[:, 1], rtol=1e-12, atol=0)
    _, s_el = so.slstm_forward(z["wx"], z["r_ext"], z["b_ext"], z["s0"], None, n0_rule=so.N0_PER_ELEMENT)
    _, s_wh = so.slstm_forward(z["wx"], z["r_ext"], z["b_ext"], z["s0"], None, n0_rule=so.N0_WHOLE_TENSOR)
    assert np.abs(s_el[3, 0] - s_wh[3, 0]).max() > 1e-3


def _rand_problem(rng, B, T, NH, dh, rscale=0.5):
    H = NH * dh
    wx = rng.standard_normal((B, T, 4 * H))
    r = rng.standard_normal((NH, dh, 4, dh)) * rscale / np.sqrt(dh)
    b = rng.standard_normal((NH, 4, dh))
    return wx, r, b


def test_closed_form_first_step_from_zero_state():
    rng = np.random.default_rng(0)
    B, NH, dh = 3, 2, 5
    H = NH * dh
    wx, r, b = _rand_problem(rng, B, 1, NH, dh)
    h, s = so.slstm_forward(wx, r, b)
    raw = wx[:, 0].reshape(B, 4, NH, dh) + b.transpose(1, 0, 2)[None]
    i, f, z, o = (raw[:, g].reshape(B, H) for g in range(4))
    sig = 1.0 / (1.0 + np.exp(-o))
    np.testing.assert_allclose(s[3], i, rtol=1e-14)  # m = raw_i
    np.testing.assert_allclose(s[2], np.ones_like(i), rtol=1e-14)  # n = 1
    np.testing.assert_allclose(s[1], np.tanh(z), rtol=1e-14)  # c = tanh z
    np.testing.assert_allclose(s[0], sig * np.tanh(z), rtol=1e-13)  # y
    np.testing.assert_allclose(h[0], s[0], rtol=0, atol=0)


def test_r_zero_scan_against_unstabilised_float64_recurrence():
    """With R = 0 the cell is an elementwise scan.  The stabiliser m cancels in
    y = o * c / n, so the plain recurrence C_t = sig(f) C + exp(i) tanh z,
    N_t = sig(f) N + exp(i) must reproduce y (a wrong m rule, clamp or gate
    order would not)."""
    rng = np.random.default_rng(1)
    B, T, NH, dh = 2, 40, 2, 3
    H = NH * dh
    wx, r, b = _rand_problem(rng, B, T, NH, dh)
    r[:] = 0
    h, s = so.slstm_forward(wx, r, b)
    C = np.zeros((B, H)); N = np.zeros((B, H))
    bb = b.transpose(1, 0, 2).reshape(4, H)
    for t in range(T):
        raw = wx[:, t].reshape(B, 4, H) + bb[None]
        i, f, z, o = raw[:, 0], raw[:, 1], raw[:, 2], raw[:, 3]
        sf = 1 / (1 + np.exp(-f))
        C = sf * C + np.exp(i) * np.tanh(z)
        N = sf * N + np.exp(i)
        y = (1 / (1 + np.exp(-o))) * C / N
        np.testing.assert_allclose(h[t], y, rtol=1e-10, atol=1e-12)
    # the carried pair (c, n) is the true pair scaled by exp(-m)
    np.testing.assert_allclose(s[1] * np.exp(s[3]), C, rtol=1e-10)
    np.testing.assert_allclose(s[2] * np.exp(s[3]), N, rtol=1e-10)


def test_contraction_against_brute_force_and_einsum():
    rng = np.random.default_rng(2)
    B, NH, dh = 2, 2, 3
    H = NH * dh
    wx, r, b = _rand_problem(rng, B, 2, NH, dh, rscale=2.0)
    h, _ = so.slstm_forward(wx, r, b)
    y0 = h[0]
    # second step by hand, contraction as an explicit loop over (b, h, g, a, d)
    ry = np.zeros((B, 4, NH, dh))
    for bb in range(B):
        for hh in range(NH):
            for g in range(4):
                for a in range(dh):
                    for d in range(dh):
                        ry[bb, g, hh, a] += y0[bb, hh * dh + d] * r[hh, d, g, a]
    np.testing.assert_allclose(ry, np.einsum("bhd,hdga->bgha", y0.reshape(B, NH, dh), r), rtol=1e-13)
    _, s1 = so.slstm_forward(wx[:, :1], r, b)
    # run step 2 with R folded into the input: Wx' = Wx + Ry, R = 0
    wx2 = wx[:, 1:2] + ry.reshape(B, 1, 4 * H)
    h2, _ = so.slstm_forward(wx2, np.zeros_like(r), b, s1)
    np.testing.assert_allclose(h2[0], h[1], rtol=1e-12, atol=1e-14)


def test_chunked_equals_whole_and_steps_equal_sequence():
    rng = np.random.default_rng(3)
    B, T, NH, dh = 2, 17, 2, 4
    wx, r, b = _rand_problem(rng, B, T, NH, dh, rscale=2.0)
    h, s = so.slstm_forward(wx, r, b)
    ha, sa = so.slstm_forward(wx[:, :6], r, b)
    hb, sb = so.slstm_forward(wx[:, 6:], r, b, sa)
    np.testing.assert_array_equal(np.concatenate([ha, hb]), h)
    np.testing.assert_array_equal(sb, s)
    st = None
    for t in range(T):
        ht, st = so.slstm_forward(wx[:, t:t + 1], r, b, st)
        np.testing.assert_array_equal(ht[0], h[t])
    np.testing.assert_array_equal(st, s)


def test_causality_and_row_independence():
    rng = np.random.default_rng(4)
    B, T, NH, dh = 3, 9, 2, 4
    wx, r, b = _rand_problem(rng, B, T, NH, dh, rscale=2.0)
    h, _ = so.slstm_forward(wx, r, b)
    wx2 = wx.copy()
    wx2[1, 5:] += 1.0
    h2, _ = so.slstm_forward(wx2, r, b)
    np.testing.assert_array_equal(h2[:5], h[:5])  # earlier steps untouched
    np.testing.assert_array_equal(h2[:, [0, 2]], h[:, [0, 2]])  # other rows untouched
    assert np.abs(h2[5:, 1] - h[5:, 1]).max() > 1e-3


def test_heads_are_block_diagonal():
    rng = np.random.default_rng(5)
    B, T, NH, dh = 2, 6, 3, 4
    wx, r, b = _rand_problem(rng, B, T, NH, dh, rscale=2.0)
    h, _ = so.slstm_forward(wx, r, b)
    for hh in range(NH):
        sl = slice(hh * dh, (hh + 1) * dh)
        wxh = wx.reshape(B, T, 4, NH, dh)[:, :, :, hh].reshape(B, T, 4 * dh)
        h1, _ = so.slstm_forward(wxh, r[hh:hh + 1], b[hh:hh + 1])
        np.testing.assert_allclose(h1, h[:, :, sl], rtol=1e-13, atol=1e-15)


def test_state_bounds():
    rng = np.random.default_rng(6)
    wx, r, b = _rand_problem(rng, 2, 50, 2, 4, rscale=3.0)
    h, s = so.slstm_forward(wx * 3, r, b)
    assert np.all(np.abs(h) <= 1.0 + 1e-12)
    assert np.all(s[2] >= 1.0 - 1e-12)  # one of i', f' is exactly 1 at every step


def test_reset_equals_per_document_runs_bit_exact():
    rng = np.random.default_rng(7)
    B, T, NH, dh = 3, 30, 2, 4
    wx, r, b = _rand_problem(rng, B, T, NH, dh, rscale=2.0)
    reset = np.zeros((B, T), np.uint8)
    reset[:, 0] = 1
    reset[0, [7, 8, 20]] = 1
    reset[1, [29]] = 1
    for dtype in (np.float64, np.float32):
        h, s = so.slstm_forward(wx, r, b, None, reset, dtype=dtype)
        hd, sd = so.slstm_forward_per_document(wx, r, b, reset, dtype=dtype)
        np.testing.assert_array_equal(h, hd)
        np.testing.assert_array_equal(s, sd)
    # a reset at t=0 makes the supplied initial state irrelevant
    s0 = rng.standard_normal((4, B, NH * dh)); s0[2] = np.abs(s0[2]) + 1
    h0, _ = so.slstm_forward(wx, r, b, s0, reset)
    np.testing.assert_array_equal(h0, h.astype(np.float64) if False else so.slstm_forward(wx, r, b, None, reset)[0])


def test_f32_oracle_and_torch_port_track_f64():
    rng = np.random.default_rng(8)
    B, T, NH, dh = 2, 64, 2, 16
    wx, r, b = _rand_problem(rng, B, T, NH, dh, rscale=1.0)
    reset = np.zeros((B, T), np.uint8); reset[:, 0] = 1; reset[1, 33] = 1
    h64, s64 = so.slstm_forward(wx, r, b, None, reset)
    h32, s32 = so.slstm_forward(wx, r, b, None, reset, dtype=np.float32)
    np.testing.assert_allclose(h32, h64, rtol=1e-5, atol=1e-5)
    ht, st = vp.slstm_forward(torch.from_numpy(wx).float(), torch.from_numpy(r).float(),
                              torch.from_numpy(b).float(), None, torch.from_numpy(reset))
    np.testing.assert_allclose(ht.numpy(), h64, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(st.numpy(), s64, rtol=2e-5, atol=2e-5)
