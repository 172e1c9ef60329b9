"""Writes the golden vectors in this folder from the reference's VANILLA sLSTM cell.

Run once, in the build container only (the reference tree never travels):

    python tests/golden/make_golden.py

What the vectors pin that nothing else can: the reference's conventions — gate
order i,f,z,o inside the ``[B,S,4H]`` input, state order y,c,n,m, the flattening
``(gate, head, unit)`` of the input, the external parameter views
``recurrent_kernel[NH,dh_in,4,dh_out]`` / ``bias[NH,4,dh]``, the ``BNSH`` output
view, and the whole-tensor ``all(n == 0)`` stabiliser rule of the vanilla path.

Parameters are exported through the reference's backend-agnostic external views
(``cell.recurrent_kernel[:]``, ``cell.bias[:]``), so the fixtures do not depend
on any backend-internal layout.  Every case stores inputs and outputs as float32.
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
        # name, hidden, heads, B, T, recurrent init, bias init, with state, seed
        ("ref_test_shape_nostate", 64, 4, 1, 1, "zeros", "powerlaw_blockdependent", False, 42),
        ("ref_test_shape_state", 64, 4, 1, 1, "zeros", "powerlaw_blockdependent", True, 42),
        ("seq_standard_nostate", 64, 4, 3, 12, "standard", "small_init", False, 1),
        ("seq_standard_state", 64, 2, 2, 9, "standard", "standard", True, 2),
        ("seq_onehead", 32, 1, 2, 7, "standard", "powerlaw_blockdependent", True, 3),
        ("seq_dh128", 256, 2, 2, 16, "standard", "small_init", False, 4),
        # row 0 starts with n == 0 but m != 0, row 1 with n > 0: the vanilla path's
        # whole-tensor test `all(n == 0)` is False, so row 0 takes max(i, m + logsig f)
        # where the native per-element rule would take i.
        ("seq_mixed_n", 64, 4, 2, 5, "standard", "small_init", "mixed", 5),
    ]
    for name, hidden, heads, B, T, rinit, binit, with_state, seed in cases:
        torch.manual_seed(seed)
        cfg = sLSTMCellConfig(
            hidden_size=hidden, num_heads=heads, backend="vanilla", dtype="float32",
            recurrent_weight_init=rinit, bias_init=binit,
        )
        cell = sLSTMCell(cfg)
        if rinit == "standard":
            # U(+-1/sqrt(hidden)) keeps R·y tiny; scale up so that a wrong index,
            # transposition or gate order in the contraction is far above tolerance.
            with torch.no_grad():
                cell._recurrent_kernel_.mul_(6.0)
        x = torch.randn(B, T, 4 * hidden)
        state = torch.randn(4, B, hidden) if with_state else None
        if state is not None:
            state[2] = state[2].abs() + 0.5  # a normaliser is positive in any reachable state
            if with_state == "mixed":
                state[2, 0] = 0.0
        with torch.no_grad():
            out, st = cell(x, state)
        assert out.shape == (B, heads, T, hidden // heads)
        np.savez(
            os.path.join(OUT, f"{name}.npz"),
            wx=x.numpy(),
            r_ext=cell.recurrent_kernel[:].contiguous().numpy(),
            b_ext=cell.bias[:].contiguous().numpy(),
            s0=(state.numpy() if state is not None else np.zeros((0,), np.float32)),
            out_bnsh=out.contiguous().numpy(),
            state=st.contiguous().numpy(),
        )
        print(name, "out", tuple(out.shape), "state", tuple(st.shape))

    # ---- sLSTMLayer (caller of the cell): conv1d + SiLU, headwise gate projections, cell, group norm
    from xlstm.blocks.slstm.layer import sLSTMLayer, sLSTMLayerConfig  # noqa: E402

    for name, D, NH, B, T, seed in (("layer_d64", 64, 4, 2, 10, 11), ("layer_d128", 128, 2, 3, 7, 12)):
        torch.manual_seed(seed)
        cfg = sLSTMLayerConfig(embedding_dim=D, num_heads=NH, conv1d_kernel_size=4, backend="vanilla",
                               dtype="float32", recurrent_weight_init="standard", bias_init="small_init")
        layer = sLSTMLayer(cfg)
        layer.reset_parameters()
        with torch.no_grad():
            layer.slstm_cell._recurrent_kernel_.mul_(6.0)
            layer.group_norm.weight.normal_(0.0, 0.3)
            for g in (layer.igate, layer.fgate, layer.zgate, layer.ogate):
                g.weight.mul_(4.0)  # make the gate wiring (which module feeds which slot) matter
        x = torch.randn(B, T, D)
        with torch.no_grad():
            out = layer(x)
        np.savez(
            os.path.join(OUT, f"{name}.npz"),
            x=x.numpy(), out=out.numpy(),
            conv_weight=layer.conv1d.conv.weight.detach().numpy(), conv_bias=layer.conv1d.conv.bias.detach().numpy(),
            fgate=layer.fgate.weight.detach().numpy(), igate=layer.igate.weight.detach().numpy(),
            zgate=layer.zgate.weight.detach().numpy(), ogate=layer.ogate.weight.detach().numpy(),
            r_ext=layer.slstm_cell.recurrent_kernel[:].contiguous().numpy(),
            b_ext=layer.slstm_cell.bias[:].contiguous().numpy(),
            gn_weight=layer.group_norm.weight.detach().numpy(),
            num_heads=np.array(NH),
        )
        print(name, "out", tuple(out.shape))

    write_checkpoint_layouts()

    # Notebook shape fixture (notebooks/xlstm/xLSTM_test_notebook.ipynb, cell 2):
    # zeros[4,4,512] through hidden=128, heads=2 -> out [4,2,4,64], state [4,4,128].
    torch.manual_seed(0)
    cell = sLSTMCell(sLSTMCellConfig(hidden_size=128, num_heads=2, backend="vanilla", dtype="float32"))
    with torch.no_grad():
        out, st = cell(torch.zeros(4, 4, 512))
    print("notebook shapes", tuple(out.shape), tuple(st.shape))
    assert tuple(out.shape) == (4, 2, 4, 64) and tuple(st.shape) == (4, 4, 128)


def write_checkpoint_layouts():
    """The same external parameters as each reference backend stores them (its ``state_dict``
    tensors ``_recurrent_kernel_`` / ``_bias_``): what a checkpoint written with backend
    "vanilla" or "cuda" holds.  The cuda cell is built with ``skip_backend_init=True`` as in
    the reference's own doctests (cell.py:712-716), so nothing is compiled."""
    sys.path.insert(0, REF)
    from xlstm.blocks.slstm.cell import sLSTMCell_cuda, sLSTMCell_vanilla, sLSTMCellConfig  # noqa: E402

    torch.manual_seed(21)
    hidden, heads = 48, 3
    r_ext = torch.randn(heads, hidden // heads, 4, hidden // heads)
    b_ext = torch.randn(heads, 4, hidden // heads)
    out = {"r_ext": r_ext.numpy(), "b_ext": b_ext.numpy(), "num_heads": np.array(heads)}
    for backend, cls in (("vanilla", sLSTMCell_vanilla), ("cuda", sLSTMCell_cuda)):
        cell = cls(sLSTMCellConfig(hidden_size=hidden, num_heads=heads, backend=backend, dtype="float32"),
                   skip_backend_init=True)
        cell.recurrent_kernel[:] = r_ext
        cell.bias[:] = b_ext
        sd = cell.state_dict()
        out[f"r_{backend}"] = sd["_recurrent_kernel_"].contiguous().numpy()
        out[f"b_{backend}"] = sd["_bias_"].contiguous().numpy()
        print("checkpoint layout", backend, out[f"r_{backend}"].shape, out[f"b_{backend}"].shape)
    np.savez(os.path.join(OUT, "ckpt_layouts.npz"), **out)


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "--checkpoint-layouts-only":
        write_checkpoint_layouts()
    else:
        main()
