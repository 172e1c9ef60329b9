"""GPU parity of the sequence kernel for workgroups of four row tiles (MFMA waves + gating waves), variant by variant:
every chunk count of the recurrent matrix per lane, both dtypes, full tiles and ragged ones (missing rows, a K tail),
with and without a mask and an initial state, against the CPU oracle - plus the bit-exact properties (packed ==
per document, step by step == sequence).  The status block says which kernel ran (rows_per_workgroup == 64).

Tolerances as in test_hip_parity.py: float32 1e-5, bfloat16 2e-2 against the float64 oracle."""
import numpy as np
import pytest
import torch

from oracle import slstm_oracle as so
from tests._util import geometric_reset_mask, make_problem
from tests.test_hip_parity import TOL_BF16, TOL_F32, _check, _run_hip

pytestmark = pytest.mark.gpu

# bf16, B, T, NH, dh: shapes whose head groups leave room for only one or two groups per head, so that 64 rows go to
# one workgroup (a head group has dh / 16 workgroups; an XCD of 32 compute units holds 32 / (dh / 16) of them)
CASES = [
    (True, 128, 6, 16, 128),    # 1 chunk per lane, full tiles
    (True, 80, 7, 16, 128),     # ... 5 row tiles: the second workgroup of a head has one
    (True, 80, 5, 16, 104),     # ... and a K tail (dh not a multiple of 16)
    (True, 128, 9, 8, 256),     # 2 chunks
    (True, 128, 6, 4, 512),     # 4 chunks
    (True, 100, 6, 4, 512),     # ... ragged
    (True, 64, 17, 4, 1024),    # 8 chunks, head groups over two XCDs; T not a multiple of the prefetch ring
    (False, 80, 5, 32, 64),     # fp32: 1 chunk, ragged
    (False, 128, 6, 16, 128),   # 2 chunks
    (False, 128, 5, 8, 256),    # 4 chunks
    (False, 128, 5, 4, 512),    # 8 chunks
    (False, 72, 6, 4, 504),     # ... ragged, K tail
]


@pytest.mark.parametrize("bf16,B,T,NH,dh", CASES)
@pytest.mark.parametrize("masked", [False, True], ids=["plain", "mask+state"])
def test_four_row_tiles_against_the_oracle(bf16, B, T, NH, dh, masked):
    print("case four row tiles", bf16, B, T, NH, dh, masked, flush=True)
    wx, r, b, s0 = make_problem(77, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=masked)
    reset = geometric_reset_mask(5, B, T, max(2, T // 2)) if masked else None
    h_ref, s_ref = so.slstm_forward(wx, r, b, s0, reset)
    h, s, status = _run_hip(wx, r, b, s0, reset, bf16=bf16)
    assert status["rows_per_workgroup"] == 64, status
    _check(h, s, h_ref, s_ref, TOL_BF16 if bf16 else TOL_F32, status)
    # the last token as a single step from the state before it: the same bits
    if T >= 2:
        _, s_prev, _ = _run_hip(wx[:, :T - 1], r, b, s0, None if reset is None else reset[:, :T - 1], bf16=bf16)
        h1, s1, st1 = _run_hip(wx[:, T - 1:], r, b, s_prev, None if reset is None else reset[:, T - 1:], bf16=bf16, step=True)
        assert st1["step_kernel"] == 1 and st1["rows_per_workgroup"] == 0
        np.testing.assert_array_equal(h1[0], h[T - 1])
        np.testing.assert_array_equal(s1, s)


@pytest.mark.parametrize("bf16,B,NH,dh", [(True, 128, 4, 512), (False, 80, 16, 128), (True, 64, 4, 1024)])
def test_four_row_tiles_packed_documents_equal_separate_calls(bf16, B, NH, dh):
    """A row that holds two documents gives, bit for bit, what the two documents give as separate calls."""
    T, cut = 9, 4
    print("case four row tiles packed", bf16, B, NH, dh, flush=True)
    wx, r, b, _ = make_problem(78, B, T, NH, dh, rscale=2.0, bf16=bf16)
    reset = np.zeros((B, T), dtype=np.uint8)
    reset[:, cut] = 1
    h, s, status = _run_hip(wx, r, b, None, reset, bf16=bf16)
    assert status["rows_per_workgroup"] == 64 and status["aborted"] == 0
    ha, _, _ = _run_hip(wx[:, :cut], r, b, None, None, bf16=bf16)
    hb, sb, _ = _run_hip(wx[:, cut:], r, b, None, None, bf16=bf16)
    np.testing.assert_array_equal(h[:cut], ha)
    np.testing.assert_array_equal(h[cut:], hb)
    np.testing.assert_array_equal(s, sb)


def test_rows_a_gigabyte_apart_fall_back_to_two_row_tiles():
    """The kernel of four row tiles addresses four rows with 32-bit lane offsets.  A W.x whose rows lie a gigabyte apart
    (a view into a larger buffer) runs through the kernel of two row tiles in more launches instead: same results."""
    from xlstm_amd import functional as F
    from tests._util import r_ext_to_kernel

    bf16, B, T, NH, dh = True, 33, 3, 8, 512
    H = NH * dh
    print("case rows a gigabyte apart", B, T, NH, dh, flush=True)
    wx, r, b, _ = make_problem(79, B, T, NH, dh, rscale=2.0, bf16=bf16)
    h_ref, s_ref = so.slstm_forward(wx, r, b, None, None)
    dev = torch.device("cuda:0")
    stride = 1 << 29  # elements: 1 GiB of bf16 per row
    try:
        buf = torch.empty(B * stride, dtype=torch.bfloat16, device=dev)
    except RuntimeError as e:  # (a box without 33 GiB to spare)
        pytest.skip(f"cannot allocate the spread-out buffer: {e}")
    wx_t = buf.as_strided((B, T, 4 * H), (stride, 4 * H, 1))
    wx_t.copy_(torch.from_numpy(wx).to(dev))
    ws = F.workspace_for(B, T, NH, dh, dev)
    h, s = F.slstm_forward(wx_t, r_ext_to_kernel(torch.from_numpy(r)).to(dev), torch.from_numpy(b).to(dev), None, None, workspace=ws)
    torch.cuda.synchronize()
    status = F.read_status(ws)
    assert status["rows_per_workgroup"] == 32 and status["launches"] == 2, status
    _check(h.float().cpu().numpy(), s.cpu().numpy(), h_ref, s_ref, TOL_BF16, status)
    # and the same call on a contiguous W.x takes the kernel of four row tiles
    _, _, st4 = _run_hip(wx, r, b, None, None, bf16=bf16)
    assert st4["rows_per_workgroup"] == 64, st4
