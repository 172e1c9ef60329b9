"""sLSTM layer around the hip cell: the caller of the hot path.

Mirrors ``xlstm/blocks/slstm/layer.py`` of NX-AI/xlstm (config :18-30, module
:33-162): causal depthwise conv1d (k = 4) + SiLU on the i/f branch, four
block-diagonal ("headwise") gate projections, ``torch.cat([i, f, z, o])`` into
the cell, dropout, per-head group norm.  Submodule and parameter names are the
reference's (``conv1d.conv``, ``fgate``, ``igate``, ``zgate``, ``ogate``,
``slstm_cell``, ``group_norm``), including its wiring of the module called
``fgate`` to the i slot and ``igate`` to the f slot (layer.py:144-149), so a
reference state dict maps one to one (the cell's two tensors go through the
external views, ``cell.reference_state_dict_to_hip``).

For bfloat16 inputs with a head dim that is a multiple of 64 the ops in front of the cell run
as two HIP kernels of the engine (convolution + SiLU; the four projections written straight into the
cell's input), see ``functional.causal_conv_silu`` / ``functional.headwise_gates``, and so does the
group norm behind it (``functional.headwise_group_norm``); otherwise they are PyTorch-ROCm ops.
New: ``reset_mask[B,S]`` (document starts of packed rows) reaches the cell, and
the causal convolution does not look across a document start either.
"""
from __future__ import annotations

from dataclasses import dataclass
from math import sqrt
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from . import functional as hipF
from .cell import sLSTMCell, sLSTMCellConfig


@dataclass
class sLSTMLayerConfig(sLSTMCellConfig):
    """layer.py:18-30."""

    embedding_dim: int = -1
    num_heads: int = 4
    conv1d_kernel_size: int = 4  # 0 means no convolution included
    group_norm_weight: bool = True
    dropout: float = 0.0

    def __post_init__(self):
        self.hidden_size = self.embedding_dim
        sLSTMCellConfig.__post_init__(self)


class CausalConv1d(nn.Module):
    """Causal depthwise convolution over time, ``components/conv.py:51-157``
    (feature-wise groups, bias, left padding of k-1), parameters under ``conv``."""

    def __init__(self, feature_dim: int, kernel_size: int = 4, bias: bool = True):
        super().__init__()
        self.kernel_size = kernel_size
        self.pad = kernel_size - 1
        self.conv = nn.Conv1d(feature_dim, feature_dim, kernel_size, padding=self.pad, groups=feature_dim, bias=bias)

    def forward(self, x: torch.Tensor, conv_state: Optional[torch.Tensor] = None, return_last_state: bool = False,
                reset_mask: Optional[torch.Tensor] = None):
        """``x`` [B,S,D].  ``conv_state`` [B,k-1,D] holds the inputs before ``x`` (conv.py:113-127).
        With ``reset_mask`` the taps that would reach before the start of a token's document read zero."""
        if conv_state is not None:
            x_all = torch.cat([conv_state, x], dim=1)
        else:
            x_all = x
        if reset_mask is None:
            y = self.conv(x_all.transpose(2, 1))[:, :, : x_all.shape[1]].transpose(2, 1)
        else:
            y = self._masked(x_all, conv_state, reset_mask)
        if conv_state is not None:
            y = y[:, conv_state.shape[1]:]
        if return_last_state:
            return y, x_all[:, -self.pad:]
        return y

    def _masked(self, x_all, conv_state, reset_mask):
        B, S_all, D = x_all.shape
        n_prev = conv_state.shape[1] if conv_state is not None else 0
        starts = torch.zeros(B, S_all, dtype=torch.bool, device=x_all.device)
        starts[:, n_prev:] = reset_mask != 0
        idx = torch.arange(S_all, device=x_all.device).expand(B, S_all)
        last_start = torch.cummax(torch.where(starts, idx, torch.full_like(idx, -S_all - self.pad)), dim=1).values
        since = idx - last_start  # tokens since the document start (huge where no start was seen)
        xp = F.pad(x_all, (0, 0, self.pad, 0))  # [B, S_all + k-1, D]
        w = self.conv.weight[:, 0, :]  # [D, k]; tap j multiplies x[t - (k-1) + j]
        y = torch.zeros_like(x_all)
        for j in range(self.kernel_size):
            back = self.pad - j
            tap = xp[:, j: j + S_all]
            if back > 0:
                tap = tap * (since >= back).unsqueeze(-1).to(tap.dtype)
            y = y + tap * w[:, j]
        if self.conv.bias is not None:
            y = y + self.conv.bias
        return y

    def advance(self, x: torch.Tensor, conv_state=None) -> torch.Tensor:
        """The ring state after one more token: [B,k,D], oldest input first, ``x`` last (conv.py:142-149)."""
        B, S, D = x.shape
        assert S == 1, f"x has sequence length {S} but it should be 1"
        if conv_state is None:
            return torch.cat([torch.zeros(B, self.kernel_size - 1, D, device=x.device, dtype=x.dtype), x], dim=1)
        prev = conv_state[0] if isinstance(conv_state, (tuple, list)) else conv_state
        if prev.shape[1] == self.kernel_size:
            prev = prev[:, 1:]  # the oldest slot is dropped
        assert prev.shape[1] == self.kernel_size - 1, f"conv state holds {prev.shape[1]} inputs, expected {self.kernel_size}"
        return torch.cat([prev.to(x.dtype), x], dim=1)

    def step(self, x: torch.Tensor, conv_state=None):
        """One token, ring state [B,k,D] in a 1-tuple as in conv.py:131-157.  Also accepted: the
        bare [B,k-1,D] tensor that ``forward(..., return_last_state=True)`` hands back
        (conv.py:126-127), so that a prefill can be followed by steps."""
        state = self.advance(x, conv_state)
        y = torch.sum(state * self.conv.weight[:, 0, :].transpose(0, 1), dim=1, keepdim=True)
        if self.conv.bias is not None:
            y = y + self.conv.bias
        return y, (state,)


class LinearHeadwiseExpand(nn.Module):
    """Block-diagonal projection ``...hd,hod->...ho`` (components/linear_headwise.py:42-82), no bias here."""

    def __init__(self, in_features: int, num_heads: int):
        super().__init__()
        self.num_heads = num_heads
        d = in_features // num_heads
        self.weight = nn.Parameter(torch.empty(num_heads, d, d))
        nn.init.normal_(self.weight, mean=0.0, std=sqrt(2 / 5 / d))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        shape = x.shape
        y = torch.einsum("...hd,hod->...ho", x.view(*shape[:-1], self.num_heads, -1), self.weight)
        return y.reshape(*shape[:-1], -1)


class MultiHeadLayerNorm(nn.Module):
    """Per-head group norm of [B,NH,S,DH] with residual weight (components/ln.py:8-68)."""

    def __init__(self, ndim: int, weight: bool = True, eps: float = 1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(ndim)) if weight else None
        self.eps = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        assert x.dim() == 4, "Input must be 4D tensor (B, NH, S, DH)"
        B, NH, S, DH = x.shape
        gn_in = x.transpose(1, 2).reshape(B * S, NH * DH)
        w = None if self.weight is None else 1.0 + self.weight
        out = F.group_norm(gn_in, num_groups=NH, weight=w, bias=None, eps=self.eps)
        return out.view(B, S, NH, DH).transpose(1, 2)


class sLSTMLayer(nn.Module):
    config_class = sLSTMLayerConfig

    def __init__(self, config: sLSTMLayerConfig):
        super().__init__()
        self.config = config
        D, NH = config.embedding_dim, config.num_heads
        if config.conv1d_kernel_size > 0:
            self.conv1d = CausalConv1d(D, config.conv1d_kernel_size)
            self.conv_act_fn = nn.SiLU()
        self.fgate = LinearHeadwiseExpand(D, NH)
        self.igate = LinearHeadwiseExpand(D, NH)
        self.zgate = LinearHeadwiseExpand(D, NH)
        self.ogate = LinearHeadwiseExpand(D, NH)
        self.slstm_cell = sLSTMCell(config)
        self.group_norm = MultiHeadLayerNorm(ndim=D, weight=config.group_norm_weight)
        self.dropout = nn.Dropout(config.dropout)
        self.fused_pre_ops = True  # use the engine's conv and projection kernels where they apply
        self.reset_parameters()

    def reset_parameters(self):
        self.slstm_cell.reset_parameters()
        if self.group_norm.weight is not None:
            nn.init.zeros_(self.group_norm.weight)
        std = sqrt(2 / (5 * self.config.embedding_dim))  # small_init_init_, components/init.py:18-25
        for gate in (self.igate, self.fgate, self.zgate, self.ogate):
            nn.init.normal_(gate.weight, mean=0.0, std=std)

    def _gates(self, x, x_conv):
        # the module named fgate feeds the i slot, igate the f slot (layer.py:144-149)
        if self._fused(x):
            return hipF.headwise_gates(x, x_conv, (self.fgate.weight, self.igate.weight, self.zgate.weight, self.ogate.weight),
                                       self.config.num_heads)
        return torch.cat([self.fgate(x_conv), self.igate(x_conv), self.zgate(x), self.ogate(x)], dim=-1)

    def _norm(self, y, B, S):
        """Group norm per head of the cell output [B,NH,S,DH] -> [B,S,D] (layer.py:159)."""
        if (self._engine_ops_allowed(y) and y.shape[-1] % 4 == 0 and y.shape[-1] <= 1024
                and (self.group_norm.weight is None or self.group_norm.weight.dtype == torch.bfloat16)):
            return hipF.headwise_group_norm(y, self.group_norm.weight, self.group_norm.eps)
        return self.group_norm(y).transpose(1, 2).reshape(B, S, -1)

    def _engine_ops_allowed(self, t) -> bool:
        # the engine's kernels record no autograd graph: under grad mode the PyTorch ops run, and a backward pass
        # reaches the cell, which raises (inference engine)
        return self.fused_pre_ops and t.is_cuda and t.dtype == torch.bfloat16 and not (
            torch.is_grad_enabled() and (t.requires_grad or any(q.requires_grad for q in self.parameters())))

    def _fused(self, x) -> bool:
        return (self._engine_ops_allowed(x) and self.fgate.weight.dtype == torch.bfloat16
                and hipF.fused_layer_ops_supported(x, self.config.num_heads, self.config.conv1d_kernel_size))

    def forward(self, x: torch.Tensor, conv_state: Optional[torch.Tensor] = None,
                slstm_state: Optional[torch.Tensor] = None, return_last_state: bool = False,
                reset_mask: Optional[torch.Tensor] = None, **kwargs):
        B, S, _ = x.shape
        if isinstance(conv_state, (tuple, list)):  # the ring a step returned (conv.py:131-157): oldest input first
            conv_state = conv_state[0]
        if self.config.conv1d_kernel_size > 0 and self._fused(x):
            conv = self.conv1d.conv
            pad = self.conv1d.pad
            taps = conv_state
            if taps is not None and taps.shape[1] != pad:  # only the last k-1 inputs matter; missing ones are zeros
                taps = taps[:, -pad:] if taps.shape[1] > pad else F.pad(taps, (0, 0, pad - taps.shape[1], 0))
            x_conv = hipF.causal_conv_silu(x, conv.weight, conv.bias, taps, reset_mask)
            if return_last_state:  # the last k-1 inputs (conv.py:126-127)
                x_all = x if conv_state is None else torch.cat([conv_state.to(x.dtype), x], dim=1)
                conv_state = x_all[:, -self.conv1d.pad:]
        elif self.config.conv1d_kernel_size > 0:
            if return_last_state:
                x_conv, conv_state = self.conv1d(x, conv_state, return_last_state=True, reset_mask=reset_mask)
            else:
                x_conv = self.conv1d(x, conv_state, reset_mask=reset_mask)
            x_conv = self.conv_act_fn(x_conv)
        else:
            x_conv = x
        y, slstm_state = self.slstm_cell(self._gates(x, x_conv), state=slstm_state, reset_mask=reset_mask)
        out = self._norm(self.dropout(y), B, S)
        if return_last_state:
            return out, {"conv_state": conv_state, "slstm_state": slstm_state}
        return out

    def step(self, x: torch.Tensor, conv_state: Optional[tuple] = None, slstm_state: Optional[torch.Tensor] = None,
             slstm_state_out: Optional[torch.Tensor] = None, conv_state_out: Optional[torch.Tensor] = None,
             h_out: Optional[torch.Tensor] = None, h_prev: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None):
        """One token (layer.py:92-121).  The optional buffers let a decode loop run without allocations:
        ``slstm_state_out`` / ``h_out`` / ``h_prev`` are handed to the cell's ``step``; ``conv_state_out``
        ([B,k,D]) receives the new convolution ring and ``out`` ([B,1,D]) the result - both only on the engine's
        bfloat16 path (``_fused``), elsewhere fresh tensors are returned as usual."""
        B, S, _ = x.shape
        fused = self._fused(x)
        if self.config.conv1d_kernel_size > 0 and fused:
            conv = self.conv1d.conv
            k = self.config.conv1d_kernel_size
            prev = conv_state[0] if isinstance(conv_state, (tuple, list)) else conv_state
            if prev is not None:
                assert prev.shape[1] in (k, k - 1), f"conv state holds {prev.shape[1]} inputs, expected {k} or {k - 1}"
                if prev.shape[1] == k:
                    prev = prev[:, 1:]  # the oldest slot is dropped
            ring = conv_state_out if conv_state_out is not None else torch.empty(B, k, x.shape[2], dtype=x.dtype, device=x.device)
            x_conv = hipF.causal_conv_silu(x, conv.weight, conv.bias, prev, ring_out=ring)
            conv_state = (ring,)
        elif self.config.conv1d_kernel_size > 0:
            x_conv, conv_state = self.conv1d.step(x, conv_state=conv_state)
            x_conv = self.conv_act_fn(x_conv)
        else:
            x_conv = x
        y, slstm_state = self.slstm_cell.step(self._gates(x, x_conv), slstm_state, state_out=slstm_state_out,
                                              h_out=h_out, h_prev=h_prev)
        y = self.dropout(y)
        if fused and out is not None:
            out = hipF.headwise_group_norm(y, self.group_norm.weight, self.group_norm.eps, out=out)
        else:
            out = self._norm(y, B, S)
        return out, {"conv_state": conv_state, "slstm_state": slstm_state}
