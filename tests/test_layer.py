"""sLSTMLayer around the hip cell: host logic on the CPU, parity with the reference layer on the GPU."""
import glob
import os

import numpy as np
import pytest
import torch

from tests._util import max_err

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _layer_from(z, **kw):
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    D = z["x"].shape[-1]
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=D, num_heads=int(z["num_heads"]), conv1d_kernel_size=4,
                                        backend="hip", dtype="float32", **kw))
    with torch.no_grad():
        layer.conv1d.conv.weight.copy_(torch.from_numpy(z["conv_weight"]))
        layer.conv1d.conv.bias.copy_(torch.from_numpy(z["conv_bias"]))
        for name in ("fgate", "igate", "zgate", "ogate"):
            getattr(layer, name).weight.copy_(torch.from_numpy(z[name]))
        layer.group_norm.weight.copy_(torch.from_numpy(z["gn_weight"]))
    layer.slstm_cell.recurrent_kernel[:] = torch.from_numpy(z["r_ext"])
    layer.slstm_cell.bias[:] = torch.from_numpy(z["b_ext"])
    return layer


def test_state_dict_names_match_reference_layer():
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=64, num_heads=4))
    assert set(layer.state_dict().keys()) == {
        "conv1d.conv.weight", "conv1d.conv.bias", "fgate.weight", "igate.weight", "zgate.weight", "ogate.weight",
        "slstm_cell._recurrent_kernel_", "slstm_cell._bias_", "group_norm.weight",
    }
    assert layer.config.hidden_size == 64  # sLSTMLayerConfig.__post_init__, layer.py:28-30


def test_masked_causal_conv_equals_per_document_conv():
    from xlstm_amd.layer import CausalConv1d

    torch.manual_seed(0)
    conv = CausalConv1d(6, 4)
    x = torch.randn(2, 12, 6)
    mask = torch.zeros(2, 12, dtype=torch.uint8)
    mask[:, 0] = 1; mask[0, 5] = 1; mask[1, [2, 3, 11]] = 1
    with torch.no_grad():
        y = conv(x, reset_mask=mask)
        np.testing.assert_allclose(conv(x, reset_mask=torch.zeros_like(mask)).numpy(), conv(x).numpy(), rtol=1e-6, atol=1e-6)
        for b in range(2):
            starts = list(torch.nonzero(mask[b]).flatten().tolist()) + [12]
            for lo, hi in zip(starts[:-1], starts[1:]):
                np.testing.assert_allclose(y[b, lo:hi].numpy(), conv(x[b:b + 1, lo:hi])[0].numpy(), rtol=1e-6, atol=1e-6)


def test_conv_step_matches_forward_and_state_handover():
    from xlstm_amd.layer import CausalConv1d

    torch.manual_seed(1)
    conv = CausalConv1d(5, 4)
    x = torch.randn(2, 9, 5)
    with torch.no_grad():
        y = conv(x)
        st = None
        for t in range(9):
            yt, st = conv.step(x[:, t:t + 1], st)
            np.testing.assert_allclose(yt[:, 0].numpy(), y[:, t].numpy(), rtol=1e-5, atol=1e-6)
        ya, cs = conv(x[:, :4], return_last_state=True)
        yb = conv(x[:, 4:], cs)
        np.testing.assert_allclose(torch.cat([ya, yb], 1).numpy(), y.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "layer_*.npz"))), ids=lambda p: os.path.basename(p)[:-4])
def test_layer_reproduces_reference_layer_output(path):
    """x -> conv/SiLU -> gates -> hip cell -> group norm against the reference's vanilla-backend layer."""
    z = np.load(path)
    layer = _layer_from(z).to("cuda:0").eval()
    with torch.no_grad():
        out = layer(torch.from_numpy(z["x"]).cuda())
    assert out.shape == z["out"].shape
    assert max_err(out.cpu().numpy(), z["out"]) <= 2e-5


@pytest.mark.gpu
def test_layer_packed_documents_equal_documents_alone_and_step_equals_forward():
    z = np.load(os.path.join(GOLDEN, "layer_d64.npz"))
    layer = _layer_from(z).to("cuda:0").eval()
    torch.manual_seed(3)
    x = torch.randn(2, 20, 64, device="cuda")
    mask = torch.zeros(2, 20, dtype=torch.uint8, device="cuda")
    mask[:, 0] = 1; mask[0, 7] = 1; mask[1, [4, 15]] = 1
    with torch.no_grad():
        out = layer(x, reset_mask=mask)
        for b in range(2):
            starts = torch.nonzero(mask[b]).flatten().tolist() + [20]
            for lo, hi in zip(starts[:-1], starts[1:]):
                alone = layer(x[b:b + 1, lo:hi])
                assert max_err(alone[0].cpu().numpy(), out[b, lo:hi].cpu().numpy()) <= 1e-5
        # decode: layer.step token by token == layer.forward
        full = layer(x)
        conv_state, cell_state = None, None
        for t in range(20):
            o, st = layer.step(x[:, t:t + 1], conv_state=conv_state, slstm_state=cell_state)
            conv_state, cell_state = st["conv_state"], st["slstm_state"]
            assert max_err(o[:, 0].cpu().numpy(), full[:, t].cpu().numpy()) <= 1e-5


def test_conv_step_accepts_the_state_a_prefill_returns():
    from xlstm_amd.layer import CausalConv1d

    torch.manual_seed(2)
    conv = CausalConv1d(5, 4)
    x = torch.randn(2, 9, 5)
    with torch.no_grad():
        y = conv(x)
        _, cs = conv(x[:, :5], return_last_state=True)  # [B, k-1, D], conv.py:126-127
        st = cs
        for t in range(5, 9):
            yt, st = conv.step(x[:, t:t + 1], st)
            np.testing.assert_allclose(yt[:, 0].numpy(), y[:, t].numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_prefill_then_steps_equals_one_forward(dtype):
    """forward(x[:, :k], return_last_state=True) followed by step() per token = forward(x)."""
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    torch.manual_seed(3)
    dev = torch.device("cuda:0")
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=128, num_heads=4, backend="hip",
                                        recurrent_weight_init="standard")).to(dev).to(dtype)
    layer.slstm_cell.keep_state_fp32 = True
    x = torch.randn(3, 12, 128, device=dev).to(dtype)
    with torch.no_grad():
        whole = layer(x)
        pre, st = layer(x[:, :7], return_last_state=True)
        outs = [pre]
        for t in range(7, 12):
            o, st = layer.step(x[:, t:t + 1], conv_state=st["conv_state"], slstm_state=st["slstm_state"])
            outs.append(o)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert max_err(torch.cat(outs, 1).float().cpu().numpy(), whole.float().cpu().numpy()) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("B,D,NH", [(8, 256, 4), (64, 512, 4), (5, 96, 3), (16, 2048, 4)],
                         ids=["engine-ops", "engine-ops-operand-hint", "torch-ops", "head-dim-512-r-in-slabs"])
def test_graphed_decoder_replays_equal_eager_steps(B, D, NH):
    """Two alternating HIP graphs of layer.step against the eager loop, with host work between replays.
    (64, 512, 4) is a shape where the step kernel takes the previous h as its bf16 operand; (5, 96, 3)
    one where the ops around the cell are PyTorch's; (16, 2048, 4) one where the step kernel reads R in slabs."""
    from xlstm_amd.decode import GraphedLayerDecoder
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    torch.manual_seed(4)
    dev = torch.device("cuda:0")
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=D, num_heads=NH, backend="hip",
                                        recurrent_weight_init="standard")).to(dev).bfloat16()
    layer.slstm_cell.keep_state_fp32 = True
    x = torch.randn(B, 16, D, device=dev).bfloat16()
    with torch.no_grad():
        _, st0 = layer(x[:, :5], return_last_state=True)
        dec = GraphedLayerDecoder(layer, B)
        for trial in range(2):  # the second pass re-uses the graphs after a state reload
            dec.load_state(st0["conv_state"], st0["slstm_state"])
            st = st0
            for t in range(5, 16):
                want, st = layer.step(x[:, t:t + 1], conv_state=st["conv_state"], slstm_state=st["slstm_state"])
                if trial == 0:
                    got = dec.step(x[:, t:t + 1])
                else:  # the producer writes the token into the decoder's input buffer
                    dec.x.copy_(x[:, t:t + 1])
                    got = dec.step()
                torch.cuda.synchronize()
                assert torch.equal(got, want), (trial, t)
                assert torch.equal(dec.state()["slstm_state"], st["slstm_state"]), (trial, t)
