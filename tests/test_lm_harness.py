"""Config-4 harness at a small size: runs, stays finite, times its sLSTM cells, and the
document mask reaches them (the second document of a packed row is unaffected by the first
inside the sLSTM layers)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_small_harness_forward_and_cell_timing():
    from xlstm_amd.lm_harness import HarnessConfig, xLSTMLMHarness

    torch.manual_seed(0)
    cfg = HarnessConfig(vocab_size=512, embedding_dim=128, num_blocks=4, slstm_at=[1, 3], num_heads=4, context_length=64)
    model = xLSTMLMHarness(cfg).to("cuda:0").bfloat16().eval()
    idx = torch.randint(0, 512, (2, 64), device="cuda")
    mask = torch.zeros(2, 64, dtype=torch.uint8, device="cuda")
    mask[:, 0] = 1; mask[0, 30] = 1
    with torch.no_grad():
        logits = model(idx, reset_mask=mask, time_cells=True)
    assert logits.shape == (2, 64, 512) and bool(torch.isfinite(logits.float()).all())
    assert len(model.cell_ms) == 2 and all(t > 0 for t in model.cell_ms)
    assert len(model.slstm_cells()) == 2


def test_reset_mask_reaches_the_cells():
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    torch.manual_seed(1)
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=64, num_heads=4, recurrent_weight_init="standard")).cuda().eval()
    with torch.no_grad():
        layer.slstm_cell._recurrent_kernel_.mul_(6.0)
    x = torch.randn(1, 24, 64, device="cuda")
    mask = torch.zeros(1, 24, dtype=torch.uint8, device="cuda")
    mask[0, 0] = 1; mask[0, 10] = 1
    with torch.no_grad():
        a = layer(x, reset_mask=mask)
        x2 = x.clone(); x2[0, :10] += 1.0  # change only the first document
        b = layer(x2, reset_mask=mask)
    assert torch.equal(a[0, 10:], b[0, 10:])
    assert float((a[0, :10] - b[0, :10]).abs().max()) > 1e-3
