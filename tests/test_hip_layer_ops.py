"""The two HIP kernels in front of the cell (convolution + SiLU, headwise gate projections) against float32
PyTorch restatements of the same operations on the same bf16-rounded operands.  Tolerance 2e-2 on
max |a - d| / max(1, |d|), the bf16 bar of the cell; the outputs are float32 results rounded once to bf16."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests._util import geometric_reset_mask, max_err

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = 2e-2


def conv_silu_reference(x, w, bias, conv_state, mask):
    """float32, per document: silu(causal depthwise conv) with taps cut at document starts."""
    B, T, D = x.shape
    K = w.shape[1]
    x = x.float(); w = w.float()
    prev = torch.zeros(B, K - 1, D) if conv_state is None else conv_state.float()
    xa = torch.cat([prev, x], 1)  # token t sits at t + K - 1
    out = torch.zeros(B, T, D)
    for b in range(B):
        last_start = None
        for t in range(T):
            if mask is not None and mask[b, t]:
                last_start = t
            acc = torch.zeros(D) if bias is None else bias.float().clone()
            for back in range(K):
                ts = t - back
                if last_start is not None and ts < last_start:
                    continue
                acc = acc + w[:, K - 1 - back] * xa[b, ts + K - 1]
            out[b, t] = acc
    return F.silu(out)


@pytest.mark.parametrize("B,T,D,K,with_state,with_mask,with_bias", [
    (2, 19, 64, 4, False, False, True),
    (3, 33, 128, 4, True, True, True),
    (1, 7, 8, 3, True, False, False),
    (2, 40, 24, 2, False, True, True),
    (5, 1, 256, 4, True, False, True),  # a decode step
])
def test_causal_conv_silu_equals_float32_restatement(B, T, D, K, with_state, with_mask, with_bias):
    from xlstm_amd import functional as hipF

    g = torch.Generator().manual_seed(B * 1000 + T)
    x = torch.randn(B, T, D, generator=g).bfloat16()
    w = (torch.randn(D, K, generator=g) * 0.5).bfloat16()
    bias = torch.randn(D, generator=g).bfloat16() if with_bias else None
    state = torch.randn(B, K - 1, D, generator=g).bfloat16() if with_state else None
    mask = None
    if with_mask:
        mask = torch.from_numpy(geometric_reset_mask(T, B, T, 5))
        mask[:, 0] = 0  # the first document continues from conv_state / zero padding
        mask[0, 1] = 1; mask[0, 2] = 1  # documents of one token
    want = conv_silu_reference(x, w, bias, state, mask)
    got = hipF.causal_conv_silu(x.to(DEV), w.view(D, 1, K).to(DEV), None if bias is None else bias.to(DEV),
                                None if state is None else state.to(DEV), None if mask is None else mask.to(DEV))
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (B, T, D)
    assert max_err(got.float().cpu().numpy(), want.numpy()) <= TOL


def test_causal_conv_silu_reads_a_ring_view_and_strided_input():
    """conv_state as the [:, :-1] view of a [B,K,D] ring and x as a slice of a longer sequence: no copies needed."""
    from xlstm_amd import functional as hipF

    g = torch.Generator().manual_seed(5)
    B, D, K = 4, 128, 4
    ring = torch.randn(B, K, D, generator=g).bfloat16()
    w = torch.randn(D, K, generator=g).bfloat16()
    bias = torch.randn(D, generator=g).bfloat16()
    x = ring[:, -1:]
    want = conv_silu_reference(x, w, bias, ring[:, :-1], None)
    ring_d = ring.to(DEV)
    got = hipF.causal_conv_silu(ring_d[:, -1:], w.to(DEV), bias.to(DEV), ring_d[:, :-1])
    assert max_err(got.float().cpu().numpy(), want.numpy()) <= TOL
    long = torch.randn(B, 30, D, generator=g).bfloat16()
    want = conv_silu_reference(long[:, 10:25], w, bias, long[:, 7:10], None)
    long_d = long.to(DEV)
    got = hipF.causal_conv_silu(long_d[:, 10:25], w.to(DEV), bias.to(DEV), long_d[:, 7:10])
    assert max_err(got.float().cpu().numpy(), want.numpy()) <= TOL


def test_causal_conv_silu_step_writes_the_next_ring():
    from xlstm_amd import functional as hipF

    g = torch.Generator().manual_seed(6)
    B, D, K = 3, 64, 4
    ring = torch.randn(B, K, D, generator=g).bfloat16().to(DEV)
    x = torch.randn(B, 1, D, generator=g).bfloat16().to(DEV)
    w = torch.randn(D, K, generator=g).bfloat16().to(DEV)
    new_ring = torch.full((B, K, D), 7.0, dtype=torch.bfloat16, device=DEV)
    got = hipF.causal_conv_silu(x, w, None, ring[:, 1:], ring_out=new_ring)
    want = hipF.causal_conv_silu(x, w, None, ring[:, 1:].contiguous())
    assert torch.equal(got, want)
    assert torch.equal(new_ring, torch.cat([ring[:, 1:], x], 1))
    first = torch.full((B, K, D), 7.0, dtype=torch.bfloat16, device=DEV)  # no state yet: zeros, then x
    hipF.causal_conv_silu(x, w, None, None, ring_out=first)
    assert torch.equal(first, torch.cat([torch.zeros(B, K - 1, D, dtype=torch.bfloat16, device=DEV), x], 1))
    with pytest.raises(hipF.EngineError):
        hipF.causal_conv_silu(x, w, None, ring[:, 1:], ring_out=ring)  # in place is refused


@pytest.mark.parametrize("lead,NH,dh", [
    ((2, 37), 4, 64),      # 64-token x 64-unit tiles, ragged token count
    ((3, 50), 2, 256),     # 64 x 128
    ((4, 1100), 4, 128),   # 128 x 128 (>= 4096 tokens), ragged
    ((4100,), 4, 64),      # 128 x 64, ragged
    ((256, 1), 8, 256),    # the decode shape of BASELINE config 3
    ((1, 1), 1, 192),      # one token, three 64-unit tiles per slot
    ((8, 2048), 4, 256),   # the layer of BASELINE config 4: weights resident, 8 token partitions of 16 tiles
    ((5, 999), 16, 256),   # 128 combinations: two token partitions, no XCD grouping, ragged
    ((3, 1000), 3, 128),   # 12 combinations, 16 partitions of one or two tiles
    ((2, 3), 1, 128),      # fewer token tiles than partitions
])
def test_headwise_gates_equal_float32_einsum(lead, NH, dh):
    from xlstm_amd import functional as hipF

    g = torch.Generator().manual_seed(NH * dh + len(lead))
    H = NH * dh
    x = torch.randn(*lead, H, generator=g).bfloat16()
    xc = torch.randn(*lead, H, generator=g).bfloat16()
    ws = [(torch.randn(NH, dh, dh, generator=g) / np.sqrt(dh)).bfloat16() for _ in range(4)]
    want = torch.cat([torch.einsum("...hd,hod->...ho", (xc if s < 2 else x).float().view(*lead, NH, dh), ws[s].float()).reshape(*lead, H)
                      for s in range(4)], dim=-1)
    got = hipF.headwise_gates(x.to(DEV), xc.to(DEV), [w.to(DEV) for w in ws], NH)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == tuple(lead) + (4 * H,)
    assert max_err(got.float().cpu().numpy(), want.numpy()) <= TOL


def test_headwise_gates_slot_wiring_one_hot():
    """Exact check of the indexing: with one-hot operands every output is a single weight, bit for bit."""
    from xlstm_amd import functional as hipF

    NH, dh = 2, 64
    H = NH * dh
    g = torch.Generator().manual_seed(9)
    ws = [torch.randn(NH, dh, dh, generator=g).bfloat16() for _ in range(4)]
    x = torch.zeros(3, H).bfloat16(); xc = torch.zeros(3, H).bfloat16()
    x[0, 5] = 1; x[1, 64 + 17] = 1; x[2, 63] = 1        # z, o read x
    xc[0, 64 + 3] = 1; xc[1, 9] = 1; xc[2, 127] = 1     # i, f read x_conv
    got = hipF.headwise_gates(x.to(DEV), xc.to(DEV), [w.to(DEV) for w in ws], NH).cpu()
    for m, (cx, cxc) in enumerate([(5, 64 + 3), (64 + 17, 9), (63, 127)]):
        for s in range(4):
            c = cxc if s < 2 else cx
            h, d = divmod(c, dh)
            want = torch.zeros(H).bfloat16()
            want[h * dh:(h + 1) * dh] = ws[s][h, :, d]
            assert torch.equal(got[m, s * H:(s + 1) * H], want), (m, s)


@pytest.mark.parametrize("B,NH,T,dh,with_weight,cell_layout", [
    (3, 4, 17, 64, True, True),
    (2, 2, 5, 256, True, True),
    (2, 3, 9, 36, False, False),    # 9 pieces of 4 units: part of a wave idles
    (1, 1, 4, 1024, True, True),    # four pieces per lane
    (5, 2, 1, 520, True, False),    # three pieces used of four
])
def test_headwise_group_norm_equals_float32_group_norm(B, NH, T, dh, with_weight, cell_layout):
    from xlstm_amd import functional as hipF

    g = torch.Generator().manual_seed(B + NH + T + dh)
    H = NH * dh
    if cell_layout:  # the cell's output: [S,B,H] storage seen as [B,NH,S,DH] (cell.py:354-374)
        y = (torch.randn(T, B, H, generator=g) * 3 + 0.5).bfloat16().view(T, B, NH, dh).permute(1, 2, 0, 3)
    else:
        y = (torch.randn(B, NH, T, dh, generator=g) * 3 + 0.5).bfloat16()
    w = (torch.randn(H, generator=g) * 0.2).bfloat16() if with_weight else None
    want = F.group_norm(y.float().transpose(1, 2).reshape(B * T, H), NH, None if w is None else 1.0 + w.float(), None, 1e-5)
    got = hipF.headwise_group_norm(y.to(DEV), None if w is None else w.to(DEV), 1e-5)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (B, T, H)
    assert max_err(got.float().cpu().numpy(), want.view(B, T, H).numpy()) <= TOL


def test_layer_with_engine_pre_ops_equals_layer_with_torch_pre_ops():
    """sLSTMLayer.forward and .step: the HIP conv / projection kernels against the PyTorch ops they replace."""
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    torch.manual_seed(11)
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=256, num_heads=4, backend="hip",
                                        recurrent_weight_init="standard")).to(DEV).bfloat16().eval()
    layer.slstm_cell.keep_state_fp32 = True
    x = torch.randn(3, 40, 256, device=DEV).bfloat16()
    mask = torch.from_numpy(geometric_reset_mask(2, 3, 40, 9)).to(DEV)
    with torch.no_grad():
        assert layer._fused(x)
        fused, st_f = layer(x, reset_mask=mask, return_last_state=True)
        o_f, st_f2 = layer.step(x[:, :1], conv_state=st_f["conv_state"], slstm_state=st_f["slstm_state"])
        layer.fused_pre_ops = False
        plain, st_p = layer(x, reset_mask=mask, return_last_state=True)
        o_p, st_p2 = layer.step(x[:, :1], conv_state=st_p["conv_state"], slstm_state=st_p["slstm_state"])
        # a forward continues from the ring a step returned (k inputs) and from a shorter state alike
        layer.fused_pre_ops = True
        a1 = layer(x[:, 1:9], conv_state=st_f2["conv_state"])
        a2 = layer(x[:, 1:9], conv_state=st_f2["conv_state"][0][:, -2:])
        layer.fused_pre_ops = False
        b1 = layer(x[:, 1:9], conv_state=st_p2["conv_state"])
        b2 = layer(x[:, 1:9], conv_state=st_p2["conv_state"][0][:, -2:])
        # the same layer in float32 (bf16-rounded parameters, PyTorch ops, float32 cell kernel): the yardstick
        import copy

        ref_layer = copy.deepcopy(layer).float()
        ref_layer.fused_pre_ops = False
        ref32 = ref_layer(x.float(), reset_mask=mask)
    # The engine's layer path against the float32 layer at the bf16 bar.  The PyTorch bf16 path rounds after every op
    # (conv, SiLU, each projection) and is itself up to that far from float32, so the two bf16 pipelines are compared
    # with each other at the sum of the two bars, after the group norm has divided by a head's spread.
    e_fused = max_err(fused.float().cpu().numpy(), ref32.cpu().numpy())
    e_plain = max_err(plain.float().cpu().numpy(), ref32.cpu().numpy())
    print("layer vs float32 layer: engine ops %.3e, torch ops %.3e" % (e_fused, e_plain), flush=True)
    assert e_fused <= 2e-2
    assert max_err(fused.float().cpu().numpy(), plain.float().cpu().numpy()) <= 2e-2 + max(e_plain, 2e-2)
    assert max_err(a1.float().cpu().numpy(), b1.float().cpu().numpy()) <= 5e-2
    assert max_err(a2.float().cpu().numpy(), b2.float().cpu().numpy()) <= 5e-2
    assert torch.equal(st_f["conv_state"], st_p["conv_state"])
    assert max_err(st_f["slstm_state"].cpu().numpy(), st_p["slstm_state"].cpu().numpy()) <= 5e-2
    assert max_err(o_f.float().cpu().numpy(), o_p.float().cpu().numpy()) <= 5e-2
    assert torch.equal(st_f2["conv_state"][0], st_p2["conv_state"][0])


def test_layer_under_autograd_keeps_the_pytorch_ops_and_trains_through_the_cell():
    """The engine's layer kernels record no graph: with grad enabled the layer keeps its PyTorch ops around the cell,
    and the cell's own backward kernels carry the gradient (head dims in between their sizes run padded)."""
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    torch.manual_seed(12)
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=256, num_heads=4, backend="hip")).to(DEV).bfloat16()
    x = torch.randn(2, 6, 256, device=DEV).bfloat16().requires_grad_(True)
    with torch.no_grad():
        assert layer._fused(x)
    assert not layer._fused(x)  # parameters require grad and grad mode is on
    out = layer(x)
    assert out.requires_grad
    out.float().sum().backward()
    grads = [p.grad for p in layer.parameters()]
    assert all(g is not None and torch.isfinite(g.float()).all() for g in grads)
    assert x.grad is not None and torch.isfinite(x.grad.float()).all() and x.grad.float().abs().max() > 0
    small = sLSTMLayer(sLSTMLayerConfig(embedding_dim=256, num_heads=8, backend="hip")).to(DEV).bfloat16()  # head dim 32: padded
    small(x.detach()).float().sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad.float()).all() for p in small.parameters())


def test_layer_ops_accept_empty_inputs():
    from xlstm_amd import functional as hipF

    w = torch.zeros(64, 4, dtype=torch.bfloat16, device=DEV)
    assert tuple(hipF.causal_conv_silu(torch.zeros(2, 0, 64, dtype=torch.bfloat16, device=DEV), w).shape) == (2, 0, 64)
    assert tuple(hipF.causal_conv_silu(torch.zeros(0, 5, 64, dtype=torch.bfloat16, device=DEV), w).shape) == (0, 5, 64)
    ws = [torch.zeros(1, 64, 64, dtype=torch.bfloat16, device=DEV)] * 4
    e = torch.zeros(0, 3, 64, dtype=torch.bfloat16, device=DEV)
    assert tuple(hipF.headwise_gates(e, e, ws, 1).shape) == (0, 3, 256)
    assert tuple(hipF.headwise_group_norm(torch.zeros(2, 1, 0, 64, dtype=torch.bfloat16, device=DEV)).shape) == (2, 0, 64)
    torch.cuda.synchronize()
