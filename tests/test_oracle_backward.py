"""The backward oracle (oracle/slstm_oracle_backward.c, float64) against what pins it: the gradients that the reference's
vanilla cell returns through autograd (tests/golden/bwd_*.npz, written by tests/golden/make_golden_backward.py),
central finite differences of the forward oracle, and the reset property (a packed row = its documents alone).

The oracle follows the rule of the reference's native kernel (slstm_pointwise.cu:118-196): the stabiliser m is a constant
of the differentiation.  For a loss on the outputs that is the gradient; the vectors show where it is not."""
import glob
import os

import numpy as np
import pytest

from oracle import slstm_oracle as so

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _rel(a, g):
    return np.abs(a - g).max() / max(1.0, np.abs(g).max())


def _load(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    wx, r, b = z["wx"], z["r_ext"], z["b_ext"]
    s0 = z["s0"] if z["s0"].size else None
    NH, dh = r.shape[0], r.shape[1]
    B, T = wx.shape[:2]
    d_h = z["w_out_bnsh"].transpose(2, 0, 1, 3).reshape(T, B, NH * dh)  # [B,NH,T,dh] -> [T,B,H]
    return z, wx, r, b, s0, d_h


@pytest.mark.parametrize("name", ["bwd_nostate", "bwd_state", "bwd_onehead"])
def test_reference_autograd_vectors_loss_on_the_outputs(name):
    z, wx, r, b, s0, d_h = _load(name)
    assert not z["w_state"].any()
    d_wx, d_r, d_b, d_s0 = so.slstm_backward(wx, r, b, s0, None, d_h, None, n0_rule=so.N0_WHOLE_TENSOR)
    tol = 5e-6  # (the vectors are float32)
    assert _rel(d_wx, z["d_wx"]) <= tol
    assert _rel(d_r, z["d_r_ext"]) <= tol
    assert _rel(d_b, z["d_b_ext"]) <= tol
    if s0 is not None:
        for i in range(3):  # y, c, n
            assert _rel(d_s0[i], z["d_s0"][i]) <= tol
        # the stabiliser: the native rule writes zero; autograd returns the derivative of a shift of m with c and n
        # held, which is c * dc + n * dn (the true state is c e^m, n e^m)
        assert not d_s0[3].any()
        assert _rel(z["d_s0"][3], s0[1] * z["d_s0"][1] + s0[2] * z["d_s0"][2]) <= tol


def test_a_loss_on_the_final_c_n_m_is_where_the_native_rule_is_not_the_gradient():
    z, wx, r, b, s0, d_h = _load("bwd_state_loss")
    d_wx, _, _, _ = so.slstm_backward(wx, r, b, s0, None, d_h, z["w_state"], n0_rule=so.N0_WHOLE_TENSOR)
    assert _rel(d_wx, z["d_wx"]) > 0.1


def _loss(wx, r, b, s0, reset, w):
    h, _ = so.slstm_forward(wx, r, b, s0, reset)
    return float((h * w).sum())


def test_central_finite_differences_of_the_forward_oracle():
    rng = np.random.default_rng(31)
    B, T, NH, dh = 3, 6, 2, 4
    H = NH * dh
    wx = rng.standard_normal((B, T, 4 * H))
    r = rng.uniform(-1, 1, (NH, dh, 4, dh)) * 0.8
    b = rng.standard_normal((NH, 4, dh))
    s0 = rng.standard_normal((4, B, H))
    s0[0] = np.tanh(s0[0])
    s0[2] = np.abs(s0[2]) + 1.0
    reset = np.zeros((B, T), np.uint8)
    reset[1, 3] = 1
    reset[2, 0] = 1  # a row that ignores the supplied state
    w = rng.standard_normal((T, B, H))
    d_wx, d_r, d_b, d_s0 = so.slstm_backward(wx, r, b, s0, reset, w)
    eps = 1e-6

    def fd(arr, idx):
        keep = arr[idx]
        arr[idx] = keep + eps
        up = _loss(wx, r, b, s0, reset, w)
        arr[idx] = keep - eps
        dn = _loss(wx, r, b, s0, reset, w)
        arr[idx] = keep
        return (up - dn) / (2 * eps)

    for _ in range(40):
        idx = tuple(rng.integers(0, n) for n in wx.shape)
        assert abs(fd(wx, idx) - d_wx[idx]) <= 1e-6 * max(1.0, abs(d_wx[idx]))
    for _ in range(40):
        idx = tuple(rng.integers(0, n) for n in r.shape)
        assert abs(fd(r, idx) - d_r[idx]) <= 1e-6 * max(1.0, abs(d_r[idx]))
    for idx in np.ndindex(*b.shape):
        assert abs(fd(b, idx) - d_b[idx]) <= 1e-6 * max(1.0, abs(d_b[idx]))
    for comp in range(3):  # y, c, n (m: see the vectors above)
        for _ in range(20):
            idx = (comp,) + tuple(rng.integers(0, n) for n in s0.shape[1:])
            assert abs(fd(s0, idx) - d_s0[idx]) <= 1e-6 * max(1.0, abs(d_s0[idx]))
    assert not d_s0[:, 2].any()  # the row whose first token starts a document took nothing from the state


def test_gradients_of_a_packed_row_are_those_of_its_documents():
    rng = np.random.default_rng(32)
    B, T, NH, dh, cut = 2, 9, 2, 4, 4
    H = NH * dh
    wx = rng.standard_normal((B, T, 4 * H))
    r = rng.uniform(-1, 1, (NH, dh, 4, dh)) * 0.8
    b = rng.standard_normal((NH, 4, dh))
    w = rng.standard_normal((T, B, H))
    reset = np.zeros((B, T), np.uint8)
    reset[:, 0] = 1
    reset[:, cut] = 1
    d_wx, d_r, d_b, _ = so.slstm_backward(wx, r, b, None, reset, w)
    a = so.slstm_backward(wx[:, :cut], r, b, None, None, w[:cut])
    c = so.slstm_backward(wx[:, cut:], r, b, None, None, w[cut:])
    np.testing.assert_allclose(d_wx[:, :cut], a[0], rtol=0, atol=1e-12)
    np.testing.assert_allclose(d_wx[:, cut:], c[0], rtol=0, atol=1e-12)
    np.testing.assert_allclose(d_r, a[1] + c[1], rtol=0, atol=1e-11)
    np.testing.assert_allclose(d_b, a[2] + c[2], rtol=0, atol=1e-11)


def _small_problem(seed, B=3, T=7, NH=2, dh=4, rscale=0.8):
    rng = np.random.default_rng(seed)
    H = NH * dh
    wx = rng.standard_normal((B, T, 4 * H))
    r = rng.uniform(-1, 1, (NH, dh, 4, dh)) * rscale
    b = rng.standard_normal((NH, 4, dh))
    s0 = rng.standard_normal((4, B, H))
    s0[0] = np.tanh(s0[0])
    s0[2] = np.abs(s0[2]) + 1.0
    w = rng.standard_normal((T, B, H))
    return wx, r, b, s0, w


@pytest.mark.parametrize("k", [1, 3, 6])
def test_d_s_final_by_the_chain_rule(k):
    """Pins the ``d_s_final`` argument (its y, c and n planes): the state after step k - 1 is all that the steps from k
    on see of the steps before, so the gradients of the whole sequence are those of [k:T] (started from that state)
    and of [0:k] with the second part's ``d_s0`` as the gradient of its final state.  A dropped plane, a wrong sign or
    a plane read from the wrong place breaks the first part's gradients."""
    wx, r, b, s0, w = _small_problem(41)
    T = wx.shape[1]
    reset = np.zeros(wx.shape[:2], np.uint8)
    reset[1, 2] = 1
    whole = so.slstm_backward(wx, r, b, s0, reset, w)
    _, s_k = so.slstm_forward(wx[:, :k], r, b, s0, reset[:, :k])
    tail = so.slstm_backward(wx[:, k:], r, b, s_k, reset[:, k:], w[k:])
    assert np.abs(tail[3][:3]).min() > 0  # (all three planes carry something)
    head = so.slstm_backward(wx[:, :k], r, b, s0, reset[:, :k], w[:k], tail[3])
    np.testing.assert_allclose(np.concatenate([head[0], tail[0]], 1), whole[0], rtol=0, atol=1e-12)
    np.testing.assert_allclose(head[1] + tail[1], whole[1], rtol=0, atol=1e-11)
    np.testing.assert_allclose(head[2] + tail[2], whole[2], rtol=0, atol=1e-11)
    np.testing.assert_allclose(head[3], whole[3], rtol=0, atol=1e-12)
    # and it is not vacuous: without the hand-over the first part's gradients are different
    plain = so.slstm_backward(wx[:, :k], r, b, s0, reset[:, :k], w[:k])
    assert np.abs(plain[0] - whole[0][:, :k]).max() > 1e-3


def test_recurrent_cut_is_the_gradient_with_the_recurrent_input_held_constant():
    """``recurrent_cut`` (slstm_backward_cut.cu: no contraction with R transposed) treats the y a step starts from as
    a constant.  The same gate deltas come out of the pinned path (no cut) when the recurrent contribution is moved
    into the inputs: W.x'_t = W.x_t + R y_{t-1} with R = 0 gives the same outputs and lets no gradient through y.  The
    gradient of R is then the sum of the outer products of those deltas with the y the steps started from."""
    wx, r, b, s0, w = _small_problem(42, T=6)
    B, T = wx.shape[:2]
    NH, dh = r.shape[0], r.shape[1]
    H = NH * dh
    reset = np.zeros((B, T), np.uint8)
    reset[2, 3] = 1
    h, _ = so.slstm_forward(wx, r, b, s0, reset)
    y_prev = np.concatenate([s0[0][None], h[:-1]], 0).copy()          # [T,B,H]
    y_prev[reset.T != 0] = 0.0
    ry = np.einsum("tbhd,hdqa->btqha", y_prev.reshape(T, B, NH, dh), r).reshape(B, T, 4 * H)
    h2, _ = so.slstm_forward(wx + ry, np.zeros_like(r), b, s0, reset)
    np.testing.assert_allclose(h2, h, rtol=0, atol=1e-12)
    d_sf = np.random.default_rng(43).standard_normal((4, B, H))
    want = so.slstm_backward(wx + ry, np.zeros_like(r), b, s0, reset, w, d_sf)
    got = so.slstm_backward(wx, r, b, s0, reset, w, d_sf, recurrent_cut=True)
    np.testing.assert_allclose(got[0], want[0], rtol=0, atol=1e-12)
    np.testing.assert_allclose(got[2], want[2], rtol=0, atol=1e-11)
    np.testing.assert_allclose(got[3], want[3], rtol=0, atol=1e-12)  # (the y plane is zero in both)
    assert not got[3][0].any()
    d_r = np.einsum("tbhd,btqha->hdqa", y_prev.reshape(T, B, NH, dh), got[0].reshape(B, T, 4, NH, dh))
    np.testing.assert_allclose(got[1], d_r, rtol=0, atol=1e-11)
    full = so.slstm_backward(wx, r, b, s0, reset, w, d_sf)
    assert np.abs(full[0] - got[0]).max() > 1e-3  # (the cut changes the gradient of this problem)


@pytest.mark.parametrize("clipval", [0.05, 0.5, 1e9])
def test_recurrent_clipval_step_by_step(clipval):
    """``recurrent_clipval`` (slstm_pointwise.cu:136-143): written out as a loop over single steps in numpy.  Step t is
    a one-step call of the pinned oracle on the state it started from, with ``d_h`` = the outside gradient plus the
    CLIPPED gradient that step t + 1 sent back to its y, and the c, n gradients handed over unclipped."""
    wx, r, b, s0, w = _small_problem(44, T=5, rscale=1.5)
    B, T = wx.shape[:2]
    H = wx.shape[2] // 4
    d_sf = np.random.default_rng(45).standard_normal((4, B, H))
    d_sf[3] = 0.0
    states = [s0]
    for t in range(T):
        states.append(so.slstm_forward(wx[:, t:t + 1], r, b, states[-1])[1])
    d_wx = np.zeros_like(wx)
    d_r, d_b = np.zeros_like(r), np.zeros_like(b)
    carry = np.zeros((4, B, H))
    for t in range(T - 1, -1, -1):
        dy = w[t] + np.clip(carry[0], -clipval, clipval)
        d_state = carry.copy()
        d_state[0] = 0.0
        if t == T - 1:                      # what comes from outside at the last step is not clipped
            dy = w[t] + d_sf[0]
            d_state = d_sf.copy()
            d_state[0] = 0.0
        one = so.slstm_backward(wx[:, t:t + 1], r, b, states[t], None, dy[None], d_state)
        d_wx[:, t:t + 1] = one[0]
        d_r += one[1]
        d_b += one[2]
        carry = one[3]
    got = so.slstm_backward(wx, r, b, s0, None, w, d_sf, recurrent_clipval=clipval)
    np.testing.assert_allclose(got[0], d_wx, rtol=0, atol=1e-11)
    np.testing.assert_allclose(got[1], d_r, rtol=0, atol=1e-10)
    np.testing.assert_allclose(got[2], d_b, rtol=0, atol=1e-10)
    np.testing.assert_allclose(got[3], carry, rtol=0, atol=1e-11)
    full = so.slstm_backward(wx, r, b, s0, None, w, d_sf)
    if clipval > 1e6:
        np.testing.assert_allclose(got[0], full[0], rtol=0, atol=1e-12)
    else:
        assert np.abs(full[0] - got[0]).max() > 1e-3  # (the clip bites in this problem)
