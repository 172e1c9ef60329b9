"""Seeded sweep over odd shapes: every kernel variant, placement and tile size against the float64 oracle,
and the decode step against the sequence kernel (bit for bit)."""
import numpy as np
import pytest
import torch

from oracle import slstm_oracle as so
from tests._util import geometric_reset_mask, make_problem, max_err, r_ext_to_kernel

pytestmark = pytest.mark.gpu


def _cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        bf16 = bool(rng.integers(0, 2))
        NH = int(rng.choice([1, 2, 3, 4, 5, 8]))
        dh = 8 * int(rng.integers(1, (1024 if bf16 else 512) // 8 + 1))
        if rng.random() < 0.5:
            dh = int(rng.choice([16, 32, 64, 128, 256, 512] + ([1024] if bf16 else [])))
        if NH * ((dh + 15) // 16) > 256:
            continue
        B = int(rng.integers(1, 97))
        T = int(rng.integers(1, 14))
        out.append((bf16, B, T, NH, dh, bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), int(rng.integers(0, 1 << 30))))
    return out


# more heads than the device holds at once (NH * ceil(dh/16) workgroups > 256 compute units): the heads are
# independent, so the engine runs them in several launches
_MANY_HEADS = [
    (True, 5, 6, 32, 256, True, False, 11),    # 512 workgroups: two launches of 16 heads
    (True, 40, 5, 24, 384, False, True, 12),   # 24 workgroups per head: 10 + 10 + 4 heads, three row chunks
    (False, 3, 7, 40, 128, True, True, 13),    # fp32, 320 workgroups: 32 + 8 heads
    (True, 70, 4, 6, 1024, False, False, 14),  # 64 workgroups per head: 4 + 2 heads, two XCDs per head
]


# four row tiles per workgroup with a head dim that fills the K range exactly: the variants that request the tile
# after next behind the gating (with document starts, carried state, a second launch of fewer rows)
_FOUR_TILES = [
    (True, 64, 9, 8, 512, True, True, 21),
    (True, 128, 6, 4, 512, False, True, 22),
    (True, 64, 7, 4, 1024, True, True, 23),
    (False, 64, 5, 16, 256, False, True, 24),
    (True, 96, 5, 8, 512, False, False, 25),
]


@pytest.mark.parametrize("bf16,B,T,NH,dh,with_state,resets,seed", _cases(40, 2024) + _cases(16, 7) + _MANY_HEADS + _FOUR_TILES)
def test_random_shape_against_oracle_and_stepwise(bf16, B, T, NH, dh, with_state, resets, seed):
    from xlstm_amd import functional as F

    print("case", bf16, B, T, NH, dh, with_state, resets, seed, flush=True)
    dev = torch.device("cuda:0")
    wx, r, b, s0 = make_problem(seed % 1000, B, T, NH, dh, rscale=2.0, bf16=bf16, with_state=with_state)
    reset = geometric_reset_mask(seed % 997, B, T, max(2, T // 2)) if resets else None
    if reset is not None and with_state:
        reset[:, 0] = 0
    h_ref, s_ref = so.slstm_forward(wx, r, b, s0, reset)
    wx_t = torch.from_numpy(wx).to(dev)
    if bf16:
        wx_t = wx_t.bfloat16()
    r_t = r_ext_to_kernel(torch.from_numpy(r)).to(dev)
    b_t = torch.from_numpy(b).to(dev)
    s0_t = torch.from_numpy(s0).to(dev) if s0 is not None else None
    m_t = torch.from_numpy(reset).to(dev) if reset is not None else None
    ws = F.workspace_for(B, T, NH, dh, dev)
    h, s = F.slstm_forward(wx_t, r_t, b_t, s0_t, m_t, workspace=ws)
    torch.cuda.synchronize()
    assert F.read_status(ws)["aborted"] == 0
    tol = 2e-2 if bf16 else 1e-5
    assert max_err(h.float().cpu().numpy(), h_ref) <= tol
    assert max_err(s.cpu().numpy(), s_ref) <= tol
    # the same tokens one step at a time (the step kernel wants R in the operand type)
    r_step = r_t.bfloat16() if bf16 else r_t
    st = s0_t
    for t in range(T):
        ht, st = F.slstm_forward(wx_t[:, t:t + 1], r_step, b_t, st, m_t[:, t:t + 1] if m_t is not None else None, step=True)
        # (with a float32 master R the sequence kernel rounds it in registers exactly as .bfloat16() does)
        assert torch.equal(ht[0], h[t]), t
    assert torch.equal(st, s)
