"""PyTorch-CPU restatement of the vanilla sLSTM cell with the SAME structure as
the reference (a Python loop over timesteps; per step one batched matmul for
R·y and the elementwise exponential-gating ops; pre-allocated ``states_all`` and
gate buffers).

TEST INFRASTRUCTURE ONLY.  Two uses: a second, independently written witness
for the C oracle, and the host-CPU baseline timed by ``bench.py``.

Reference lines followed:
  xlstm/blocks/slstm/src/vanilla/__init__.py:17-74  (loop, buffers, matmul)
  xlstm/blocks/slstm/src/vanilla/slstm.py:8-37      (pointwise)
  xlstm/blocks/slstm/cell.py:601-642                (vanilla internal layouts)
  xlstm/blocks/slstm/cell.py:327-374,496-506        (permute in / out)
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def r_ext_to_vanilla(r_ext: torch.Tensor) -> torch.Tensor:
    """[NH, dh_in, 4, dh_out] -> [NH, 4*dh_out, dh_in] (cell.py:601-617)."""
    NH, dh = r_ext.shape[0], r_ext.shape[1]
    return r_ext.permute(0, 2, 3, 1).reshape(NH, 4 * dh, dh)


def b_ext_to_vanilla(b_ext: torch.Tensor) -> torch.Tensor:
    """[NH, 4, dh] -> gate-major flat [4*H] (cell.py:635-642)."""
    return b_ext.permute(1, 0, 2).reshape(-1)


def pointwise(wx, ry, b, states, per_element_n0: bool):
    raw = wx + ry + b
    y, c, n, m = torch.unbind(states, dim=0)
    iraw, fraw, zraw, oraw = torch.unbind(raw.view(raw.shape[0], 4, -1), dim=1)
    logfplusm = m + F.logsigmoid(fraw)
    if per_element_n0:
        mnew = torch.where(n == 0.0, iraw, torch.max(iraw, logfplusm))
    elif torch.all(n == 0.0):
        mnew = iraw
    else:
        mnew = torch.max(iraw, logfplusm)
    ogate = torch.sigmoid(oraw)
    igate = torch.minimum(torch.exp(iraw - mnew), torch.ones_like(iraw))
    fgate = torch.minimum(torch.exp(logfplusm - mnew), torch.ones_like(iraw))
    cnew = fgate * c + igate * torch.tanh(zraw)
    nnew = fgate * n + igate
    ynew = ogate * cnew / nnew
    return torch.stack((ynew, cnew, nnew, mnew), dim=0), torch.stack((igate, fgate, zraw, ogate), dim=0)


def slstm_forward(
    wx: torch.Tensor,  # [B, T, 4H] external (gate, head, unit) order
    r_ext: torch.Tensor,  # [NH, dh, 4, dh]
    b_ext: torch.Tensor,  # [NH, 4, dh]
    s0: Optional[torch.Tensor] = None,  # [4, B, H]
    reset: Optional[torch.Tensor] = None,  # [B, T]
    per_element_n0: bool = True,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns ``(h[T,B,H], state[4,B,H])`` in ``wx.dtype`` arithmetic."""
    NH, dh = r_ext.shape[0], r_ext.shape[1]
    H = NH * dh
    B, T = wx.shape[0], wx.shape[1]
    x = wx.permute(1, 0, 2)  # [T, B, 4H]; the vanilla internal order is gate-major too
    R = r_ext_to_vanilla(r_ext).to(wx.dtype)
    b = b_ext_to_vanilla(b_ext).to(wx.dtype)
    states = torch.zeros(4, B, H, dtype=wx.dtype) if s0 is None else s0.to(wx.dtype).clone()
    g = torch.zeros(T + 1, 4, B, H, dtype=wx.dtype)
    states_all = torch.zeros(4, T + 1, B, H, dtype=wx.dtype)
    states_all[:, 0] = states
    Rt = R.transpose(1, 2).reshape(1, NH, dh, 4 * dh)
    for i, wx_t in enumerate(x.unbind(dim=0)):
        if reset is not None:
            keep = (reset[:, i] == 0).to(wx.dtype).view(1, B, 1)
            states = states * keep
        ry = (
            states[0].reshape(B, NH, 1, dh).matmul(Rt)
            .reshape(B, NH, 4, dh).transpose(1, 2).reshape(B, -1)
        )
        states, gates = pointwise(wx_t, ry, b, states, per_element_n0)
        g[i] = gates
        states_all[:, i + 1] = states
    return states_all[0, 1:], states
