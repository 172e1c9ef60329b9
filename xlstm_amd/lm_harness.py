"""Measurement harness for BASELINE config 4: an xLSTM language model with random weights whose
sLSTM cells run on the HIP engine while everything else (mLSTM blocks, norms, projections,
feed-forward, embedding, head) stays in PyTorch-ROCm.

Structure restated from the reference: block stack with sLSTM blocks at ``slstm_at`` and mLSTM
blocks elsewhere (xlstm/xlstm_block_stack.py:40-50,77-124), pre-norm residual blocks with an
optional gated feed-forward (blocks/xlstm_block.py:43-80, components/feedforward.py:46-80),
mLSTM layer with the stabilised parallel form (blocks/mlstm/layer.py:33-120,
blocks/mlstm/cell.py:27-86, blocks/mlstm/backends.py:9-90), embedding and LM head
(xlstm_lm_model.py:22-54).  It exists to time the sLSTM cells inside a realistic forward pass;
it is not a training model (random init, forward only).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional

import torch
import torch.nn.functional as F
from torch import nn

from .layer import CausalConv1d, MultiHeadLayerNorm, sLSTMLayer, sLSTMLayerConfig


def _round_up(x: float, m: int = 64) -> int:
    return int(math.ceil(x / m) * m)


class LayerNorm(nn.Module):
    """Weight-only layer norm with residual weight (components/ln.py:8-47)."""

    def __init__(self, ndim: int, eps: float = 1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(ndim))
        self.ndim, self.eps = ndim, eps

    def forward(self, x):
        return F.layer_norm(x, (self.ndim,), weight=1.0 + self.weight, bias=None, eps=self.eps)


class BlockLinear(nn.Module):
    """Headwise projection with small blocks (components/linear_headwise.py:42-82)."""

    def __init__(self, features: int, blocksize: int):
        super().__init__()
        self.nb = features // blocksize
        self.weight = nn.Parameter(torch.randn(self.nb, blocksize, blocksize) * math.sqrt(2 / 5 / blocksize))

    def forward(self, x):
        shape = x.shape
        return torch.einsum("...hd,hod->...ho", x.view(*shape[:-1], self.nb, -1), self.weight).reshape(shape)


def mlstm_parallel(q, k, v, ig, fg, eps: float = 1e-6):
    """Stabilised parallel mLSTM, [B,NH,S,DH] (blocks/mlstm/backends.py:9-90)."""
    B, NH, S, DH = q.shape
    log_f = F.logsigmoid(fg)  # [B,NH,S,1]
    csum = torch.cat([torch.zeros_like(log_f[:, :, :1]), torch.cumsum(log_f, dim=-2)], dim=-2)  # [B,NH,S+1,1]
    m = csum - csum.transpose(-2, -1)  # [B,NH,S+1,S+1]
    ltr = torch.tril(torch.ones(S, S, dtype=torch.bool, device=q.device))
    log_d = torch.where(ltr, m[:, :, 1:, 1:], torch.full_like(m[:, :, 1:, 1:], -float("inf"))) + ig.transpose(-2, -1)
    max_log_d = log_d.max(dim=-1, keepdim=True).values
    d = torch.exp(log_d - max_log_d)
    c = (q @ (k / math.sqrt(DH)).transpose(-2, -1)) * d
    normalizer = torch.maximum(c.sum(dim=-1, keepdim=True).abs(), torch.exp(-max_log_d))
    return (c / (normalizer + eps)) @ v


class mLSTMLayer(nn.Module):
    def __init__(self, D: int, num_heads: int, proj_factor: float = 2.0, conv_k: int = 4, qkv_blocksize: int = 4):
        super().__init__()
        self.inner = _round_up(proj_factor * D)
        self.num_heads = num_heads
        self.proj_up = nn.Linear(D, 2 * self.inner, bias=False)
        self.q_proj = BlockLinear(self.inner, qkv_blocksize)
        self.k_proj = BlockLinear(self.inner, qkv_blocksize)
        self.v_proj = BlockLinear(self.inner, qkv_blocksize)
        self.conv1d = CausalConv1d(self.inner, conv_k)
        self.igate = nn.Linear(3 * self.inner, num_heads)
        self.fgate = nn.Linear(3 * self.inner, num_heads)
        nn.init.normal_(self.igate.bias, 0.0, 0.1)
        with torch.no_grad():
            self.fgate.bias.copy_(torch.linspace(3.0, 6.0, num_heads))
        self.outnorm = MultiHeadLayerNorm(self.inner)
        self.learnable_skip = nn.Parameter(torch.ones(self.inner))
        self.proj_down = nn.Linear(self.inner, D, bias=False)

    def forward(self, x, **kwargs):
        B, S, _ = x.shape
        x_m, z = self.proj_up(x).split(self.inner, dim=-1)
        x_c = F.silu(self.conv1d(x_m))
        q, k, v = self.q_proj(x_c), self.k_proj(x_c), self.v_proj(x_m)
        gate_in = torch.cat([q, k, v], dim=-1)
        ig = self.igate(gate_in).transpose(-1, -2).unsqueeze(-1)
        fg = self.fgate(gate_in).transpose(-1, -2).unsqueeze(-1)
        heads = lambda t: t.view(B, S, self.num_heads, -1).transpose(1, 2)
        h = mlstm_parallel(heads(q), heads(k), heads(v), ig, fg)
        h = self.outnorm(h).transpose(1, 2).reshape(B, S, -1)
        return self.proj_down((h + self.learnable_skip * x_c) * F.silu(z))


class GatedFeedForward(nn.Module):
    def __init__(self, D: int, proj_factor: float = 1.3):
        super().__init__()
        self.up = _round_up(proj_factor * D)
        self.proj_up = nn.Linear(D, 2 * self.up, bias=False)
        self.proj_down = nn.Linear(self.up, D, bias=False)

    def forward(self, x, **kwargs):
        g, u = self.proj_up(x).split(self.up, dim=-1)
        return self.proj_down(F.gelu(g) * u)


class Block(nn.Module):
    def __init__(self, D: int, layer: nn.Module, ffn: Optional[nn.Module]):
        super().__init__()
        self.xlstm_norm = LayerNorm(D)
        self.xlstm = layer
        self.ffn_norm = LayerNorm(D) if ffn is not None else None
        self.ffn = ffn

    def forward(self, x, **kwargs):
        x = x + self.xlstm(self.xlstm_norm(x), **kwargs)
        if self.ffn is not None:
            x = x + self.ffn(self.ffn_norm(x))
        return x


@dataclass
class HarnessConfig:
    vocab_size: int = 50304
    embedding_dim: int = 1024
    num_blocks: int = 24
    slstm_at: List[int] = field(default_factory=lambda: [3, 11, 19])
    num_heads: int = 4
    context_length: int = 2048
    slstm_backend: str = "hip"


class xLSTMLMHarness(nn.Module):
    def __init__(self, cfg: HarnessConfig):
        super().__init__()
        self.cfg = cfg
        D = cfg.embedding_dim
        self.token_embedding = nn.Embedding(cfg.vocab_size, D)
        blocks = []
        for i in range(cfg.num_blocks):
            if i in cfg.slstm_at:
                lcfg = sLSTMLayerConfig(embedding_dim=D, num_heads=cfg.num_heads, conv1d_kernel_size=4,
                                        backend=cfg.slstm_backend, bias_init="powerlaw_blockdependent",
                                        recurrent_weight_init="standard", _block_idx=i, _num_blocks=cfg.num_blocks)
                blocks.append(Block(D, sLSTMLayer(lcfg), GatedFeedForward(D, 1.3)))
            else:
                blocks.append(Block(D, mLSTMLayer(D, cfg.num_heads), None))
        self.blocks = nn.ModuleList(blocks)
        self.post_blocks_norm = LayerNorm(D)
        self.lm_head = nn.Linear(D, cfg.vocab_size, bias=False)
        self.cell_ms: List[float] = []
        self.layer_ms: List[float] = []

    def slstm_layers(self):
        return [b.xlstm for i, b in enumerate(self.blocks) if i in self.cfg.slstm_at]

    def slstm_cells(self):
        return [b.xlstm.slstm_cell for i, b in enumerate(self.blocks) if i in self.cfg.slstm_at]

    def forward(self, idx: torch.Tensor, reset_mask: Optional[torch.Tensor] = None, time_cells: bool = False):
        """``idx`` [B,S] token ids.  With ``time_cells`` the sLSTM cell calls are bracketed by
        events on the current stream; ``self.cell_ms`` then holds one time per sLSTM block and
        ``self.layer_ms`` the time of the sLSTM layer around it (conv, gate projections, cell, group norm)."""
        events = []
        layer_events = []
        hooks = []
        if time_cells:
            for mods, evs in ((self.slstm_cells(), events), (self.slstm_layers(), layer_events)):
                for mod in mods:
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    evs.append((e0, e1))
                    hooks.append(mod.register_forward_pre_hook(lambda m, a, e=e0: e.record()))
                    hooks.append(mod.register_forward_hook(lambda m, a, o, e=e1: e.record()))
        x = self.token_embedding(idx)
        for i, block in enumerate(self.blocks):
            x = block(x, reset_mask=reset_mask) if i in self.cfg.slstm_at else block(x)
        logits = self.lm_head(self.post_blocks_norm(x))
        for h in hooks:
            h.remove()
        if time_cells:
            torch.cuda.synchronize()
            self.cell_ms = [e0.elapsed_time(e1) for e0, e1 in events]
            self.layer_ms = [e0.elapsed_time(e1) for e0, e1 in layer_events]
        return logits
