"""Writes gradient vectors (``bwd_*.npz``) in this folder from the reference's VANILLA sLSTM cell and autograd.

Run once, in the build container only (the reference tree never travels):

    python tests/golden/make_golden_backward.py

What they pin for a backward pass of the cell: the reference's conventions for the gradients — with respect to the
``[B,S,4H]`` input (gate order i,f,z,o), the external parameter views ``recurrent_kernel[NH,dh_in,4,dh_out]`` and
``bias[NH,4,dh]``, and the initial state ``[4,B,H]`` — of a loss that is a fixed linear form of the outputs (and, in one
case, of the final state as well).  The loss weights are stored with the vectors.  Everything float32.
"""
import os
import sys

import numpy as np
import torch

REF = "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))


def main():
    sys.path.insert(0, REF)
    from xlstm.blocks.slstm.cell import sLSTMCell, sLSTMCellConfig  # noqa: E402

    cases = [
        # name, hidden, heads, B, T, with state, loss on the final state too, seed
        ("bwd_nostate", 32, 2, 2, 6, False, False, 21),
        ("bwd_state", 32, 2, 3, 5, True, False, 22),
        ("bwd_state_loss", 32, 4, 2, 7, True, True, 23),
        ("bwd_onehead", 16, 1, 2, 4, True, False, 24),
    ]
    for name, hidden, heads, B, T, with_state, state_loss, seed in cases:
        torch.manual_seed(seed)
        cfg = sLSTMCellConfig(hidden_size=hidden, num_heads=heads, backend="vanilla", dtype="float32",
                              recurrent_weight_init="standard", bias_init="standard")
        cell = sLSTMCell(cfg)
        with torch.no_grad():
            cell._recurrent_kernel_.mul_(6.0)  # (a wrong index or transposition must show far above tolerance)
        x = torch.randn(B, T, 4 * hidden, requires_grad=True)
        state = None
        if with_state:
            state = torch.randn(4, B, hidden)
            state[2] = state[2].abs() + 0.5  # a normaliser is positive in any reachable state
            state.requires_grad_(True)
        out, st = cell(x, state)  # out [B, NH, T, dh], st [4, B, H]
        w_out = torch.randn_like(out)
        w_st = torch.randn_like(st) if state_loss else torch.zeros_like(st)
        loss = (out * w_out).sum() + (st * w_st).sum()
        loss.backward()
        np.savez(
            os.path.join(OUT, f"{name}.npz"),
            wx=x.detach().numpy(),
            r_ext=cell.recurrent_kernel[:].detach().contiguous().numpy(),
            b_ext=cell.bias[:].detach().contiguous().numpy(),
            s0=(state.detach().numpy() if state is not None else np.zeros((0,), np.float32)),
            w_out_bnsh=w_out.numpy(),
            w_state=w_st.numpy(),
            loss=np.float32(loss.item()),
            d_wx=x.grad.numpy(),
            d_r_ext=cell._recurrent_kernel_int2ext(cell._recurrent_kernel_.grad).contiguous().numpy(),
            d_b_ext=cell._bias_int2ext(cell._bias_.grad).contiguous().numpy(),
            d_s0=(state.grad.numpy() if state is not None else np.zeros((0,), np.float32)),
        )
        print(name, "loss", float(loss), "|d_wx|", float(x.grad.abs().max()))


if __name__ == "__main__":
    main()
