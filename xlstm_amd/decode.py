"""Decode loop for one sLSTM layer replayed from HIP graphs.

The reference decodes by calling ``sLSTMLayer.step`` once per token from Python
(``xlstm/blocks/slstm/layer.py:92-121`` via ``xlstm_block_stack.py:126-137``).  One such
step is a dozen small launches, so the host sets the pace.  ``GraphedLayerDecoder`` captures
the step twice - once reading state set 0 and writing set 1, once the other way round -
and replays the two graphs alternately: no allocation, no state copy and no Python between
the launches of a token.

Only kernels are recorded (the engine's entry points enqueue nothing else); the state
buffers are cleared with ``zero_()``, which is a fill kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from .layer import sLSTMLayer


class GraphedLayerDecoder:
    def __init__(self, layer: sLSTMLayer, batch_size: int, dtype: torch.dtype = torch.bfloat16,
                 device: Optional[torch.device] = None):
        cfg = layer.config
        if cfg.conv1d_kernel_size <= 0:
            raise ValueError("GraphedLayerDecoder expects a layer with a causal convolution")
        device = device or next(layer.parameters()).device
        if device.type != "cuda":
            raise RuntimeError("GraphedLayerDecoder needs the layer on a GPU")
        self.layer = layer
        self.cell_keeps_fp32 = layer.slstm_cell.keep_state_fp32
        layer.slstm_cell.keep_state_fp32 = True  # the state stays in the engine's float32 between tokens
        B, D, K = batch_size, cfg.embedding_dim, cfg.conv1d_kernel_size
        self.x = torch.zeros(B, 1, D, dtype=dtype, device=device)
        self.out = torch.zeros(B, 1, D, dtype=dtype, device=device)
        self.conv = [torch.zeros(B, K, D, dtype=dtype, device=device) for _ in range(2)]
        self.slstm = [torch.zeros(4, B, D, dtype=torch.float32, device=device) for _ in range(2)]
        self.h = [torch.zeros(1, B, D, dtype=dtype, device=device) for _ in range(2)]  # hidden state of each set in dtype
        self.cur = 0
        self.graphs = [None, None]
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side), torch.no_grad():
            for k in range(2):  # warm-up outside the capture: lazy initialisation must not be recorded
                self._one_step(k)
            torch.cuda.synchronize(device)
            for k in range(2):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    self._one_step(k)
                self.graphs[k] = g
        torch.cuda.current_stream(device).wait_stream(side)
        torch.cuda.synchronize(device)
        self.reset()

    def _one_step(self, k: int) -> None:
        out, st = self.layer.step(self.x, conv_state=(self.conv[k],), slstm_state=self.slstm[k],
                                  slstm_state_out=self.slstm[1 - k], conv_state_out=self.conv[1 - k],
                                  h_out=self.h[1 - k], h_prev=self.h[k], out=self.out)
        if st["conv_state"][0].data_ptr() != self.conv[1 - k].data_ptr():  # a path that did not use the buffers
            self.conv[1 - k].copy_(st["conv_state"][0])
        if out.data_ptr() != self.out.data_ptr():
            self.out.copy_(out)

    def reset(self) -> None:
        """Zero state: the start of a document."""
        for t in self.conv + self.slstm + self.h:
            t.zero_()
        self.cur = 0

    def load_state(self, conv_state, slstm_state: torch.Tensor) -> None:
        """Continue after a prefill: takes what ``layer(x, return_last_state=True)`` returned."""
        prev = conv_state[0] if isinstance(conv_state, (tuple, list)) else conv_state
        K = self.layer.config.conv1d_kernel_size
        buf = self.conv[self.cur]
        buf.zero_()
        buf[:, K - prev.shape[1]:].copy_(prev)
        self.slstm[self.cur].copy_(slstm_state)
        self.h[self.cur].copy_(self.slstm[self.cur][0:1])  # the step kernel's operand hint: y rounded to dtype

    def step(self, x: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``x`` [B,1,D] -> the layer's output for this token (a buffer that the next call overwrites).
        With ``x=None`` the token is taken from ``self.x``, where its producer has written it: one copy
        kernel (and the gap in front of the graph) less per token."""
        if x is not None and x.data_ptr() != self.x.data_ptr():
            self.x.copy_(x)
        self.graphs[self.cur].replay()
        self.cur ^= 1
        return self.out

    def state(self):
        """Current state in the reference's per-block format (xlstm_block_stack.py:126-137)."""
        return {"conv_state": (self.conv[self.cur],), "slstm_state": self.slstm[self.cur]}
