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
