"""GPU parity of the backward pass for the head dims that only the kernels of one launch per step cover (``split == 3``
of the C ABI: beyond 512 up to 1024 with bfloat16, beyond 256 up to 512 with float32 - the rest of the forward's range),
against the float64 backward oracle.  Tolerances as everywhere: float32 1e-5, bfloat16 2e-2, relative to the largest
entry of a gradient (at least 1)."""
import numpy as np
import pytest
import torch

from oracle import slstm_oracle as so
from tests._util import make_problem, r_ext_to_kernel
from tests.test_hip_backward import _rel, _run_both

pytestmark = pytest.mark.gpu


CASES = [
    # bf16, B, T, NH, dh, masked + state
    (True, 3, 9, 2, 1024, True),      # config 5's cell, a few rows and steps
    (True, 2, 1, 1, 1024, False),     # one step: the first launch and the one for the initial state only
    (True, 70, 4, 1, 1024, True),     # two row tiles, the second ragged
    (True, 5, 6, 2, 768, True),       # a multiple of 128 between the sizes runs as it is
    (True, 4, 5, 1, 600, True),       # padded up to 640
    (False, 3, 8, 2, 512, True),
    (False, 66, 3, 1, 512, False),
    (False, 4, 6, 2, 320, True),
    (False, 2, 5, 1, 296, True),      # padded up to 320
    (True, 9, 40, 8, 640, True),      # eight heads: one per XCD
    (False, 5, 4, 3, 320, True),      # three heads: tiles dealt out head by head
    (True, 129, 3, 1, 576, True),     # a head dim whose rows of K are no whole number of 256-byte slabs in the walk; three row tiles
    (False, 1, 9, 3, 384, True),      # one batch row
]


@pytest.mark.parametrize("bf16,B,T,NH,dh,masked", CASES)
def test_backward_of_the_largest_head_dims_against_the_oracle(bf16, B, T, NH, dh, masked):
    print("case stepwise backward", bf16, B, T, NH, dh, masked, flush=True)
    H = NH * dh
    d_sf = np.random.default_rng(401).standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    errs, got, _ = _run_both(bf16, B, T, NH, dh, 400, masked=masked, with_state=masked, d_sf=d_sf)
    print(errs, flush=True)
    tol = 2e-2 if bf16 else 1e-5
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs
    assert not bool(got[3][3].any())  # the stabiliser's gradient is zero by the rule


@pytest.mark.parametrize("bf16,B,T,NH,dh", [(True, 9, 12, 2, 512), (False, 7, 10, 2, 256), (True, 130, 5, 4, 512)])
def test_one_launch_per_step_agrees_with_one_launch_per_call(bf16, B, T, NH, dh):
    """Head dim 512 in bfloat16 and 256 in float32 run both ways: the kernels of one launch per step against the oracle
    and against the persistent kernels on the same problem (float32: the same sums in another order; bfloat16: the same
    rounding of the deltas to the operand type)."""
    print("case stepwise against persistent", bf16, B, T, NH, dh, flush=True)
    H = NH * dh
    d_sf = np.random.default_rng(411).standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    tol = 2e-2 if bf16 else 1e-5
    errs, got, _ = _run_both(bf16, B, T, NH, dh, 410, masked=True, with_state=True, d_sf=d_sf, stepwise_override=True)
    print(errs, flush=True)
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs
    _, ref, _ = _run_both(bf16, B, T, NH, dh, 410, masked=True, with_state=True, d_sf=d_sf)
    for a, g, name in zip(got, ref, ("d_wx", "d_r", "d_b", "d_s0")):
        err = float((a - g).abs().max() / max(1.0, float(g.abs().max())))
        assert err <= tol, (name, err)


@pytest.mark.parametrize("bf16,B,T,NH,dh", [(True, 3, 8, 1, 1024), (False, 4, 7, 2, 512)])
@pytest.mark.parametrize("opts", [dict(recurrent_cut=True), dict(recurrent_clipval=0.05), dict(recurrent_cut=True, recurrent_clipval=0.05)],
                         ids=["cut", "clip0.05", "cut+clip"])
def test_recurrent_cut_and_clipval_with_one_launch_per_step(bf16, B, T, NH, dh, opts):
    """``gradient_recurrent_cut`` / ``gradient_recurrent_clipval`` (slstm_backward_cut.cu:265-312,
    slstm_pointwise.cu:136-143) in the kernel of one launch per step, against the oracle's flags."""
    print("case stepwise cut/clip", bf16, B, T, NH, dh, opts, flush=True)
    H = NH * dh
    d_sf = np.random.default_rng(421).standard_normal((4, B, H)).astype(np.float32)
    d_sf[3] = 0.0
    errs, got, _ = _run_both(bf16, B, T, NH, dh, 420, masked=True, with_state=True, d_sf=d_sf, **opts)
    print(errs, flush=True)
    tol = 2e-2 if bf16 else 1e-5
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs
    if opts.get("recurrent_cut"):
        assert not bool(got[3][0].any())
    _, plain, _ = _run_both(bf16, B, T, NH, dh, 420, masked=True, with_state=True, d_sf=d_sf)
    assert float((plain[0] - got[0]).abs().max()) > 1e-3  # the option bites


@pytest.mark.parametrize("bf16,B,T,NH,dh", [(True, 3, 10, 1, 1024), (False, 3, 8, 1, 512)])
def test_the_gradient_of_the_final_state_by_the_chain_rule_with_one_launch_per_step(bf16, B, T, NH, dh):
    """The gradients of a sequence are those of its second part, started from the state after step k - 1, and of its
    first part with the second part's ``d_s0`` as the gradient of its final state."""
    from xlstm_amd import functional as F

    k = T // 2
    H = NH * dh
    wx, r, b, s0 = make_problem(430, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=True)
    dev = torch.device("cuda:0")
    wx_t = torch.from_numpy(wx).to(dev)
    if bf16:
        wx_t = wx_t.bfloat16()
    r_t, b_t = r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev)
    s0_t = torch.from_numpy(s0).to(dev)
    d_h = torch.randn(T, B, H, generator=torch.Generator().manual_seed(431)).to(dev).to(wx_t.dtype)
    h, _ = F.slstm_forward(wx_t, r_t, b_t, s0_t)
    whole = F.slstm_backward(wx_t, r_t, b_t, s0_t, None, h, d_h)
    h_a, s_k = F.slstm_forward(wx_t[:, :k], r_t, b_t, s0_t)
    h_b, _ = F.slstm_forward(wx_t[:, k:], r_t, b_t, s_k)
    tail = F.slstm_backward(wx_t[:, k:], r_t, b_t, s_k, None, h_b, d_h[k:].contiguous())
    assert all(float(tail[3][i].abs().max()) > 0 for i in range(3)) and not bool(tail[3][3].any())
    head = F.slstm_backward(wx_t[:, :k], r_t, b_t, s0_t, None, h_a, d_h[:k].contiguous(), tail[3])
    torch.cuda.synchronize()
    tol = 2e-2 if bf16 else 1e-5

    def rel(a, g):
        return float((a - g).abs().max() / max(1.0, float(g.abs().max())))

    errs = dict(d_wx=rel(torch.cat([head[0], tail[0]], 1), whole[0]), d_r=rel(head[1] + tail[1], whole[1]),
                d_b=rel(head[2] + tail[2], whole[2]), d_s0=rel(head[3], whole[3]))
    print("chain rule, one launch per step", bf16, errs, flush=True)
    assert all(np.isfinite(v) and v <= tol for v in errs.values()), errs
    plain = F.slstm_backward(wx_t[:, :k], r_t, b_t, s0_t, None, h_a, d_h[:k].contiguous())
    assert rel(plain[0], whole[0][:, :k]) > 10 * tol


def test_cell_autograd_at_head_dim_1024():
    """The cell of BASELINE config 5 (4 heads of 1024, bfloat16) trains through the hip backend: the gradients of the
    input, the recurrent matrix and the bias (in the reference's external views) and of the initial state against the
    oracle."""
    from tests.test_hip_cell import _cell_from

    B, T, NH, dh = 3, 6, 4, 1024
    H = NH * dh
    wx, r, b, s0 = make_problem(440, B, T, NH, dh, rscale=2.0, bf16=True, with_state=True)
    r = torch.from_numpy(r).bfloat16().float().numpy()
    s0 = torch.from_numpy(s0).bfloat16().float().numpy()
    cell = _cell_from(r, b, dtype="bfloat16").train()
    x = torch.from_numpy(wx).cuda().bfloat16().requires_grad_(True)
    st = torch.from_numpy(s0).cuda().bfloat16().requires_grad_(True)
    out, _ = cell(x, st)                                   # [B, NH, T, dh]
    w = torch.randn(out.shape, generator=torch.Generator().manual_seed(441)).cuda().bfloat16().float()
    (out.float() * w).sum().backward()
    d_h = w.permute(2, 0, 1, 3).reshape(T, B, H).cpu().numpy()
    o_wx, o_r, o_b, o_s0 = so.slstm_backward(wx, r, b, s0, None, d_h, None)
    d_r_ext = cell._recurrent_kernel_int2ext(cell._recurrent_kernel_.grad).float().cpu().numpy()
    d_b_ext = cell._bias_int2ext(cell._bias_.grad).float().cpu().numpy()
    errs = dict(d_wx=_rel(x.grad.float().cpu().numpy(), o_wx), d_r=_rel(d_r_ext, o_r), d_b=_rel(d_b_ext, o_b),
                d_s0=_rel(st.grad.float().cpu().numpy()[:3], o_s0[:3]))
    print("cell autograd, head dim 1024:", errs, flush=True)
    assert all(np.isfinite(v) and v <= 2e-2 for v in errs.values()), errs
