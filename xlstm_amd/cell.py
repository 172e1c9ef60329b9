"""sLSTM cell with the ``hip`` backend behind the reference's cell interface.

Mirrors ``xlstm/blocks/slstm/cell.py`` of NX-AI/xlstm for the forward /
inference path: the same config dataclass (``backend`` gains ``"hip"``,
cell.py:68), the same external parameter views ``recurrent_kernel
[NH, dh_in, 4, dh_out]`` / ``bias [NH, 4, dh]`` behind ``ParameterProxy``
(cell.py:234-261), the same initialisers (cell.py:376-434), the same call
contract ``cell(input[B,S,4H], state=None) -> (output, state[4,B,H])`` with the
same input / output shape options (cell.py:327-374, 496-506), and the same
backend switch ``sLSTMCell(config)`` (cell.py:777-788).

What differs, on purpose:
  * only the sequence of hidden states and the final state are materialised
    (the reference keeps ``[4, S+1, B, H]`` states and a gate cache);
  * ``reset_mask[B,S]`` marks document starts inside packed rows (not in the
    reference, whose only hook is the unused ``lengths``, cell.py:496);
  * the stabiliser uses the native kernel's per-element ``n == 0`` rule
    (slstm_pointwise.cu:79), which equals the vanilla rule for every state the
    cell itself can produce;
  * training: ``loss.backward()`` runs the engine's backward kernels (``functional.slstm_backward``), with the
    reference's ``gradient_recurrent_cut`` and ``gradient_recurrent_clipval``, for every head dim the forward runs.
    A forward call that is asked for a gradient leaves the backward pass nine coefficients per step and element
    where its kernel can (``keep_backward_coefficients``); otherwise it stores nothing and the backward call
    recomputes them;
  * a call with S == 1 -- what the reference's ``sLSTMLayer.step`` makes for every decoded
    token (layer.py:113-115) -- runs the single-token step kernel, bit-identical to the same
    step inside a longer call.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from math import sqrt
from typing import Callable, Literal, Optional, Sequence, Union

import torch
from torch import nn

from . import functional as F_hip

DTYPE_DICT = {
    "bfloat16": torch.bfloat16,
    "float16": torch.float16,
    "float32": torch.float32,
}
DTYPES = Literal["bfloat16", "float16", "float32"]

rnn_function_registry = {"slstm": {"states": 4}}


class ParameterProxy:
    """Backend-agnostic (external) view of a parameter stored in a backend
    layout; same protocol as ``xlstm/components/util.py:26-74``."""

    def __init__(self, module, parameter_name, internal_to_external: Callable, external_to_internal: Callable):
        self.module = module
        self.parameter_name = parameter_name
        self.internal_to_external = internal_to_external
        self.external_to_internal = external_to_internal

    def _param(self):
        return getattr(self.module, self.parameter_name)

    def __getitem__(self, key):
        return self.internal_to_external(self._param()).detach()[key]

    def __setitem__(self, key, value):
        with torch.no_grad():
            ext = self.internal_to_external(self._param())
            ext[key] = value
            self._param().data = self.external_to_internal(ext).contiguous()

    def clone(self):
        return self.internal_to_external(self._param()).clone()

    @property
    def shape(self):
        return self.internal_to_external(self._param()).shape

    @property
    def ndim(self):
        return self.internal_to_external(self._param()).ndim

    @property
    def grad(self):
        return self.internal_to_external(self._param().grad)

    def __getattr__(self, name: str):
        # (only reached for names the proxy itself lacks; while a copy is being rebuilt it has no fields yet)
        if name in ("module", "parameter_name") or (name.startswith("__") and name.endswith("__")):
            raise AttributeError(name)
        return getattr(getattr(self.module, self.parameter_name), name)


@dataclass
class sLSTMCellConfig:
    """Field-for-field the reference's config (cell.py:61-163); the fields that
    only parameterise its CUDA build (batch_size, constants, the dtype_* of its
    intermediate buffers) are accepted and ignored by the hip backend."""

    hidden_size: int = -1
    num_heads: int = 4
    num_states: int = 4
    backend: Literal["vanilla", "cuda", "hip"] = "hip"
    function: str = "slstm"
    bias_init: Literal["powerlaw_blockdependent", "small_init", "standard", "zeros"] = "powerlaw_blockdependent"
    recurrent_weight_init: Literal["zeros", "standard"] = "zeros"
    _block_idx: int = 0
    _num_blocks: int = 1
    num_gates: int = 4
    gradient_recurrent_cut: bool = False
    gradient_recurrent_clipval: Optional[float] = None
    forward_clipval: Optional[float] = None
    batch_size: int = 8
    input_shape: Literal["BSGNH", "SBGNH"] = "BSGNH"
    internal_input_shape: Literal["SBNGH", "SBGNH", "SBNHG"] = "SBNGH"
    output_shape: Literal["BNSH", "SBH", "BSH", "SBNH"] = "BNSH"
    constants: dict = field(default_factory=dict)
    dtype: DTYPES = "bfloat16"
    dtype_b: Optional[DTYPES] = "float32"
    dtype_r: Optional[DTYPES] = None
    dtype_w: Optional[DTYPES] = None
    dtype_g: Optional[DTYPES] = None
    dtype_s: Optional[DTYPES] = None
    dtype_a: Optional[DTYPES] = None
    enable_automatic_mixed_precision: bool = True
    initial_val: Union[float, Sequence[float]] = 0.0

    @property
    def head_dim(self):
        return self.hidden_size // self.num_heads

    @property
    def input_dim(self):
        return 4 * self.hidden_size

    @property
    def torch_dtype(self) -> torch.dtype:
        return DTYPE_DICT[self.dtype]

    @property
    def torch_dtype_b(self) -> torch.dtype:
        return DTYPE_DICT[self.dtype_b]

    @property
    def torch_dtype_r(self) -> torch.dtype:
        return DTYPE_DICT[self.dtype_r]

    @property
    def torch_dtype_w(self) -> torch.dtype:
        return DTYPE_DICT[self.dtype_w]

    @property
    def torch_dtype_s(self) -> torch.dtype:
        return DTYPE_DICT[self.dtype_s]

    def __post_init__(self):
        if self.num_heads <= 0:
            self.num_heads = 1
        if self.dtype_b is None:
            self.dtype_b = self.dtype
        if self.dtype_a is None:
            self.dtype_a = self.dtype_b
        if self.dtype_r is None:
            self.dtype_r = self.dtype
        if self.dtype_w is None:
            self.dtype_w = self.dtype
        if self.dtype_s is None:
            self.dtype_s = self.dtype_w
        if self.dtype_g is None:
            self.dtype_g = self.dtype_r
        assert self.function in rnn_function_registry, f"RNN function {self.function} not in registry"
        self.num_states = rnn_function_registry[self.function]["states"]


BACKWARD_MAX_HEAD_DIM = {torch.float32: 512, torch.bfloat16: 1024}  # what xs_slstm_backward covers: the forward's range


class _ForwardOnly(torch.autograd.Function):
    """Identity on (h, state) whose backward raises: for the head dims the backward kernels of the hip backend do
    not cover, a backward pass fails loudly instead of silently yielding no gradient."""

    @staticmethod
    def forward(ctx, h, s, *deps):
        return h.view_as(h), s.view_as(s)

    @staticmethod
    def backward(ctx, *grads):
        raise RuntimeError(
            "sLSTMCell backend 'hip' has a backward pass for head dims up to 512 (float32) and 1024 (bfloat16) only; "
            "use the reference's 'cuda' or 'vanilla' backend to train this shape"
        )


class _CellFunction(torch.autograd.Function):
    """Joins the results of a forward call of the engine to the autograd graph.  The backward runs the engine's two
    backward kernels (``functional.slstm_backward``): the gradient by the rule of the reference's native kernel
    (``slstm_pointwise.cu:118-196``; what ``sLSTMFunc.backward`` returns, ``slstm.cc:137-304``).  ``h`` and ``s`` are
    what the forward call returned for ``x, r, bias, state, mask``; nothing else is stored for the backward."""

    @staticmethod
    def forward(ctx, x, r, bias, state, h, s, mask, num_heads, cut, clipval, coef, abort_sink):
        ctx.save_for_backward(x, r, bias, h, *(() if state is None else (state,)))
        ctx.mask, ctx.num_heads, ctx.cut, ctx.clipval = mask, num_heads, cut, clipval
        ctx.coef = coef  # (what a training forward left for the backward pass, or None: see keep_backward_coefficients)
        ctx.abort_sink = abort_sink  # (takes the backward call's abort word: the cell looks at it later, without a synchronisation)
        return h.view_as(h), s.view_as(s)

    @staticmethod
    def backward(ctx, d_h, d_s):
        x, r, bias, h = ctx.saved_tensors[:4]
        state = ctx.saved_tensors[4] if len(ctx.saved_tensors) > 4 else None
        NH, dh = ctx.num_heads, r.shape[2]
        d_wx, d_r, d_bias, d_s0 = F_hip.slstm_backward(
            x.detach(), r.detach(), bias.detach().view(NH, 4, dh), None if state is None else state.detach(), ctx.mask,
            h, d_h, d_s, recurrent_cut=ctx.cut, recurrent_clipval=ctx.clipval, coef=ctx.coef,
            d_wx_dtype=torch.bfloat16 if x.dtype == torch.bfloat16 else None,  # (the input's gradient in the input's type)
            abort_sink=ctx.abort_sink)
        ctx.coef = None
        return (d_wx.to(x.dtype), d_r.to(r.dtype), d_bias.reshape(bias.shape).to(bias.dtype),
                None if state is None else d_s0.to(state.dtype), None, None, None, None, None, None, None, None)


class _Runtime:
    """What a cell keeps between calls and must not travel with it: workspaces, pinned status words and events of
    calls in flight, the cached bf16 copy of R, the decode plan.  A copied or unpickled cell starts with none."""

    def __init__(self):
        self.workspaces = {}
        self.status_ring = None
        self.last_workspace = None
        self.r_bf16 = None
        self.step_plan = None
        self.last_step = None  # (state tensor handed out by the last fast step, its version, h tensor, its version)

    def __deepcopy__(self, memo):
        return _Runtime()

    def __reduce__(self):
        return (_Runtime, ())


class sLSTMCell_hip(nn.Module):
    """The cell on the MI355X engine.

    Internal parameter layouts (what the kernels read, no copy per call):
      ``_recurrent_kernel_`` [NH, 4*dh, dh]  -- r[h, g*dh + a, d] = R_ext[h, d, g, a];
          identical to the reference's vanilla layout (cell.py:601-617), so a
          vanilla checkpoint loads as is.
      ``_bias_`` [4*H] head-major -- b[h*4*dh + g*dh + a] = b_ext[h, g, a];
          identical to the reference's cuda layout (cell.py:726-733).
    """

    config_class = sLSTMCellConfig

    #: Training: let the forward call leave the backward pass its coefficients (36 bytes per step and element, held
    #: until the backward has run) where it can - bfloat16 inputs, head dim 128 or 256, a batch whose row tiles of 4
    #: rows fit the device - instead of having the backward pass recompute them in a forward walk of its own.  The
    #: reference's native forward always keeps its states and gate values when it trains (slstm.cc:79-108); set this to
    #: False to keep nothing (the memory then goes to the backward call alone).  The gradients are the same either way.
    keep_backward_coefficients: bool = True

    def __init__(self, config: sLSTMCellConfig, skip_backend_init: bool = False):
        super().__init__()
        self.config = config
        if self.config.hidden_size % self.config.num_heads != 0:
            raise ValueError(
                f"Hidden Size {self.config.hidden_size} must be divisible by head num {self.config.num_heads}"
            )
        NH, dh = self.config.num_heads, self.head_dim
        # master parameters are float32; the bf16 path converts R once per launch inside the kernel
        self._recurrent_kernel_ = nn.Parameter(torch.zeros(NH, 4 * dh, dh, dtype=torch.float32))
        self.recurrent_kernel = ParameterProxy(
            self, "_recurrent_kernel", self._recurrent_kernel_int2ext, self._recurrent_kernel_ext2int
        )
        self._bias_ = nn.Parameter(torch.zeros(4 * NH * dh, dtype=torch.float32))
        self.bias = ParameterProxy(self, "_bias", self._bias_int2ext, self._bias_ext2int)
        self.config.internal_input_shape = "SBGNH"  # the kernel reads the external (gate, head, unit) order in place
        if self.config.forward_clipval is not None:
            # the reference's native kernel clips y to +-clipval when built with it (slstm_pointwise.cu:107-110);
            # the hip kernels have no such path, and ignoring the setting would change results silently
            raise NotImplementedError("sLSTMCell backend 'hip' does not implement forward_clipval; leave it None")
        clipval = self.config.gradient_recurrent_clipval
        if clipval is not None and not clipval >= 1.0:
            # The reference's cuda build clips y to +-gradient_recurrent_clipval in the FORWARD as well (cell.py:200-210
            # hands that value, not forward_clipval, to SLSTM_FORWARD_CLIPVAL; slstm_pointwise.cu:107-110).  |y| <= 1 for
            # every state the cell reaches from a zero state (y = sigmoid(o) c / n, c / n a weighted mean of tanh values),
            # so a bound of 1 or more leaves the forward as it is and is implemented (the backward kernels clip);
            # a smaller one would change the forward, which the hip kernels do not do.
            raise NotImplementedError(
                "sLSTMCell backend 'hip' implements gradient_recurrent_clipval >= 1 only: the reference clips the "
                "forward's y to the same bound, which the hip forward kernels do not do")
        # optional: keep the carried state in float32 instead of the input dtype
        self.keep_state_fp32 = False
        # workspaces of the sequence kernel, one per (device, stream), the status words of calls in flight, caches
        self._rt = _Runtime()
        self.reset_parameters()
        if not skip_backend_init:
            from . import _lib

            _lib.load()  # fail loudly here, not at the first forward, if the engine is missing

    def __repr__(self):
        return (
            f"{self.__class__.__name__}(function={self.config.function}, "
            f"hidden_size={self.config.hidden_size}, num_heads={self.config.num_heads})"
        )

    # ------------------------------------------------------------------ layouts
    @property
    def _recurrent_kernel(self):
        return self._recurrent_kernel_

    @property
    def _bias(self):
        return self._bias_

    @property
    def head_dim(self):
        return self.config.hidden_size // self.config.num_heads

    def _recurrent_kernel_ext2int(self, recurrent_kernel_ext: torch.Tensor) -> torch.Tensor:
        NH, dh, G = self.config.num_heads, self.head_dim, self.config.num_gates
        return recurrent_kernel_ext.reshape(NH, dh, G, dh).permute(0, 2, 3, 1).reshape(NH, G * dh, dh)

    def _recurrent_kernel_int2ext(self, recurrent_kernel_int: torch.Tensor) -> torch.Tensor:
        NH, dh, G = self.config.num_heads, self.head_dim, self.config.num_gates
        return recurrent_kernel_int.reshape(NH, G, dh, dh).permute(0, 3, 1, 2)

    def _bias_ext2int(self, bias_ext: torch.Tensor) -> torch.Tensor:
        return bias_ext.reshape(self.config.num_heads, self.config.num_gates, self.head_dim).reshape(-1)

    def _bias_int2ext(self, bias_int: torch.Tensor) -> torch.Tensor:
        return bias_int.reshape(self.config.num_heads, self.config.num_gates, self.head_dim)

    # ------------------------------------------------------------------ inits
    def reset_parameters(self):
        """Same distributions and loop order as cell.py:376-434."""
        cfg = self.config
        dh = self.head_dim
        for h in range(cfg.num_heads):
            for i, _gate in enumerate(["i", "f", "z", "o"]):
                if cfg.recurrent_weight_init == "zeros":
                    self.recurrent_kernel[h, :, i, :] = torch.zeros(dh, dh)
                elif cfg.recurrent_weight_init == "standard":
                    self.recurrent_kernel[h, :, i, :] = nn.init.uniform_(
                        torch.empty(dh, dh), -1.0 / sqrt(cfg.hidden_size), 1.0 / sqrt(cfg.hidden_size)
                    )
                else:
                    raise ValueError(f"unknown recurrent_weight_init {cfg.recurrent_weight_init}")
        for h in range(cfg.num_heads):
            for i, gate in enumerate(["i", "f", "z", "o"]):
                if cfg.bias_init == "powerlaw_blockdependent":
                    if gate == "f":
                        ratio_0_to_1 = cfg._block_idx / (cfg._num_blocks - 1) if cfg._num_blocks > 1 else 0.0
                        init_values = -(-5.0 + 12.0 * (torch.arange(dh) / (dh - 1)) ** (0.3 + 1.3 * ratio_0_to_1))
                        self.bias[h, i, :] = init_values
                    else:
                        self.bias[h, i] = torch.zeros(dh)
                elif cfg.bias_init == "small_init":
                    if gate == "f":
                        self.bias[h, i] = torch.linspace(3.0, 6.0, dh)
                    else:
                        self.bias[h, i] = torch.zeros(dh)
                elif cfg.bias_init == "zeros":
                    self.bias[h, i] = torch.zeros(dh)
                elif cfg.bias_init == "standard":
                    self.bias[h, i] = nn.init.uniform_(
                        torch.empty(dh), -1 / sqrt(cfg.hidden_size), 1 / sqrt(cfg.hidden_size)
                    )
                else:
                    raise ValueError(f"unknown bias_init {cfg.bias_init}")

    # ------------------------------------------------------------------ shapes
    def _check_input(self, input: torch.Tensor) -> None:
        assert self.config.hidden_size * self.config.num_gates == input.size(-1), (
            f"Input size mismatch: Expected input size {self.config.hidden_size * self.config.num_gates}, "
            f"but got {input.size(-1)}."
        )

    def _input_bs(self, x: torch.Tensor) -> torch.Tensor:
        """External input -> [B, S, 4H] (a view; the kernel takes strides)."""
        if x.dim() != 3:
            raise ValueError(f"input must be 3-dimensional, got {tuple(x.shape)}")
        if self.config.input_shape == "BSGNH":
            return x
        if self.config.input_shape == "SBGNH":
            return x.permute(1, 0, 2)
        raise ValueError("Bad input_shape value")

    def _permute_output(self, x: torch.Tensor) -> torch.Tensor:
        """[S, B, H] -> config.output_shape (cell.py:354-374)."""
        if self.config.output_shape == "SBH":
            return x
        if self.config.output_shape == "BSH":
            return x.permute(1, 0, 2)
        if self.config.output_shape == "BNSH":
            return x.view(x.shape[0], x.shape[1], self.config.num_heads, self.head_dim).permute(1, 2, 0, 3)
        if self.config.output_shape == "SBNH":
            return x.view(x.shape[0], x.shape[1], self.config.num_heads, self.head_dim)
        raise ValueError("Bad output_shape value")

    def _check_state(self, B: int, state: Optional[torch.Tensor]) -> None:
        if state is not None:
            assert tuple(state.shape) == (self.config.num_states, B, self.config.hidden_size), (
                f"state must be {(self.config.num_states, B, self.config.hidden_size)}, got {tuple(state.shape)}"
            )

    # ------------------------------------------------------------------ forward
    def _bf16_recurrent_kernel(self) -> torch.Tensor:
        """bf16 copy of R for decoding, refreshed when the parameter changes."""
        p = self._recurrent_kernel_
        key = (p.data_ptr(), p._version, p.device)
        cache = self._rt.r_bf16
        if cache is None or cache[0] != key:
            cache = (key, p.detach().to(torch.bfloat16).contiguous())
            self._rt.r_bf16 = cache
        return cache[1]

    # ------------------------------------------------------------------ status of calls in flight
    _STATUS_SLOTS = 16

    def _workspace(self, B: int, device) -> torch.Tensor:
        """The cell's workspace for calls on the current stream of ``device`` (calls on one stream run one after the
        other, so they can share it; calls on different streams may overlap and get one each)."""
        stream = torch.cuda.current_stream(device).cuda_stream
        NH, dh = self.config.num_heads, self.head_dim
        need = F_hip._lib.load().xs_slstm_workspace_bytes(B, 1, NH, dh)
        key = (device, stream)
        ws = self._rt.workspaces.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.empty(need, dtype=torch.uint8, device=device)
            self._rt.workspaces[key] = ws
        return ws

    def _watch(self, workspace: torch.Tensor) -> None:
        """Queues a copy of the call's ``aborted`` word to pinned host memory behind the kernel and looks at the
        words of earlier calls that have arrived: a sequence call whose wait between compute units ran out
        (its outputs are NaN by then) raises here, at the next call, or in :meth:`check_status`."""
        self._watch_word(workspace[:4].view(torch.int32))

    def _watch_word(self, word: torch.Tensor) -> None:
        """The same for any call's abort word (one int32 on the device): the backward pass hands its own here, so a
        backward call does not synchronise the host either."""
        if torch.cuda.is_current_stream_capturing():
            return
        ring = self._rt.status_ring
        if ring is None:
            ring = {"host": torch.zeros(self._STATUS_SLOTS, dtype=torch.int32).pin_memory(),
                    "events": [None] * self._STATUS_SLOTS, "next": 0}
            self._rt.status_ring = ring
        self._poll_status(block=False)
        i = ring["next"]
        if ring["events"][i] is not None:  # the ring is full of calls still running: wait for the oldest
            ring["events"][i].synchronize()
            self._poll_status(block=False)
        ring["host"][i:i + 1].copy_(word, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        ring["events"][i] = ev
        ring["next"] = (i + 1) % self._STATUS_SLOTS

    def _poll_status(self, block: bool) -> None:
        ring = self._rt.status_ring
        if ring is None:
            return
        bad = False
        for i, ev in enumerate(ring["events"]):
            if ev is None:
                continue
            if block:
                ev.synchronize()
            elif not ev.query():
                continue
            ring["events"][i] = None
            bad |= int(ring["host"][i]) != 0
        if bad:
            raise F_hip.EngineError(
                "an earlier sLSTM sequence call (forward or backward) on the hip backend gave up waiting for some of its "
                "compute units (they were held by other work on the GPU); its outputs were set to NaN"
            )

    def check_status(self) -> None:
        """Waits for this cell's calls in flight and raises ``EngineError`` if one of them was aborted."""
        self._poll_status(block=True)

    def last_status(self) -> dict:
        """The status block of this cell's most recent call (synchronises): ``aborted``, ``launches``,
        ``step_kernel`` (1 when the call ran the single-token kernel), ``max_spins``, ..."""
        ws = self._rt.last_workspace
        if ws is None:
            raise RuntimeError("the cell has not been called yet")
        return F_hip.read_status(ws)

    def _run(self, input, state, reset_mask, step: bool, state_out=None):
        self._check_input(input)
        x = self._input_bs(input)
        B = x.shape[0]
        step = step or x.shape[1] == 1  # one token: the step kernel (the reference layer decodes through forward)
        self._check_state(B, state)
        in_dtype = input.dtype
        if in_dtype == torch.float16:  # no fp16 kernels: compute in float32, round the results back
            x = x.float()
        elif in_dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"input dtype {in_dtype} not supported by the hip backend")
        r = self._recurrent_kernel_.detach()
        if step and x.dtype == torch.bfloat16:
            r = self._bf16_recurrent_kernel()  # the step kernel reads R every token: keep it in the operand type
        ws = self._workspace(B, x.device) if x.is_cuda else None
        wants_grad = torch.is_grad_enabled() and (
            input.requires_grad or self._recurrent_kernel_.requires_grad or self._bias_.requires_grad
            or (state is not None and state.requires_grad)
        )
        args = (x, r, self._bias_.detach().view(self.config.num_heads, 4, self.head_dim), state, reset_mask)
        coef = None
        if wants_grad and self.keep_backward_coefficients and x.is_cuda and not step:
            coef = F_hip.backward_coefficients_buffer(x, self.config.num_heads)
        h = s = None
        if coef is not None:
            try:
                h, s = F_hip.slstm_forward(*args, s_out=state_out, workspace=ws, coef_out=coef)
            except F_hip.CoefficientsUnsupported:  # (nothing has run: the plain forward, and the backward recomputes)
                coef = None
        if h is None:
            h, s = F_hip.slstm_forward(*args, step=step, s_out=state_out, workspace=ws)
        self._rt.last_workspace = ws
        if not step and x.shape[1] > 1:
            self._watch(ws)
        if wants_grad:
            if x.is_cuda and self.head_dim <= BACKWARD_MAX_HEAD_DIM.get(x.dtype, 0):
                h, s = _CellFunction.apply(x, self._recurrent_kernel_, self._bias_, state, h, s, reset_mask,
                                           self.config.num_heads, bool(self.config.gradient_recurrent_cut),
                                           self.config.gradient_recurrent_clipval, coef, self._watch_word)
            else:
                h, s = _ForwardOnly.apply(h, s, input, self._recurrent_kernel_, self._bias_)
        output = self._permute_output(h)
        if torch.is_autocast_enabled():
            return output, s
        return output.to(in_dtype), (s if self.keep_state_fp32 else s.to(in_dtype))

    def forward(self, input, state=None, lengths=None, reset_mask=None):
        """``input`` [B,S,4H] (or [S,B,4H] for input_shape 'SBGNH'), optional ``state`` [4,B,H],
        optional ``reset_mask`` [B,S].  Returns ``(output, state)`` like cell.py:496-506."""
        del lengths  # unused, as in the reference
        if input.dim() == 3 and input.shape[1 if self.config.input_shape == "BSGNH" else 0] == 1:
            fast = self._step_fast(input, state, reset_mask, None)
            if fast is not None:
                return fast
        return self._run(input, state, reset_mask, step=False)

    def step(self, input: torch.Tensor, state: Optional[torch.Tensor] = None, reset_mask=None,
             state_out: Optional[torch.Tensor] = None, h_out: Optional[torch.Tensor] = None,
             h_prev: Optional[torch.Tensor] = None):
        """One decode step (S == 1) through the step kernel.  Unlike the reference's
        ``step`` (cell.py:486-494, which hands back the state it was given) this
        returns the NEW state.  ``state_out`` (float32 [4,B,H], not overlapping ``state``)
        receives it without an allocation, for decode loops that alternate two buffers.
        ``h_out`` ([1,B,H] in the input dtype) likewise receives the hidden state; ``h_prev`` is the
        ``h_out`` of the previous step (bfloat16 inputs: the kernel then reads half the operand bytes,
        see ``functional.StepPlan``).  Both only take effect on the steady-state path (float32 state carried
        over, no mask); otherwise they are ignored and fresh tensors are returned."""
        if state_out is not None:
            B = self._input_bs(input).shape[0]
            if state_out.dtype != torch.float32 or not state_out.is_contiguous() or tuple(state_out.shape) != (
                    self.config.num_states, B, self.config.hidden_size):
                raise ValueError("state_out must be a contiguous float32 [4, B, H] tensor")
        fast = self._step_fast(input, state, reset_mask, state_out, h_out, h_prev)
        if fast is not None:
            return fast
        return self._run(input, state, reset_mask, step=True, state_out=state_out)

    def _step_fast(self, input, state, reset_mask, state_out, h_out=None, h_prev=None):
        """The decode steady state (float32 state carried over, no mask, no autograd) through a cached
        ``StepPlan``: the generic path spends more host time per token than the kernel runs."""
        if (reset_mask is not None or state is None or state.dtype != torch.float32 or not state.is_contiguous()
                or input.dtype not in (torch.float32, torch.bfloat16) or self.config.input_shape != "BSGNH"
                or input.dim() != 3 or input.shape[1] != 1 or not input.is_contiguous() or not input.is_cuda
                or torch.is_autocast_enabled()):
            return None
        if torch.is_grad_enabled() and (
                input.requires_grad or self._recurrent_kernel_.requires_grad or self._bias_.requires_grad
                or state.requires_grad):
            return None
        self._check_input(input)
        B = input.shape[0]
        self._check_state(B, state)
        r, b = self._recurrent_kernel_, self._bias_
        key = (B, input.dtype, input.device, r.data_ptr(), r._version, b.data_ptr(), b._version)
        cached = self._rt.step_plan
        if cached is None or cached[0] != key:
            plan = F_hip.StepPlan(B, r.detach(), b.detach().view(self.config.num_heads, 4, self.head_dim), wx_dtype=input.dtype)
            cached = (key, plan)
            self._rt.step_plan = cached
        H = self.config.hidden_size
        h = h_out if h_out is not None else torch.empty((1, B, H), dtype=input.dtype, device=input.device)
        if h.dtype != input.dtype or h.numel() != B * H or not h.is_contiguous():
            raise ValueError("h_out must be a contiguous [1, B, H] tensor in the input dtype")
        s_out = state_out if state_out is not None else torch.empty((4, B, H), dtype=torch.float32, device=input.device)
        if h_prev is None and input.dtype == torch.bfloat16:
            # The state this cell handed out last time comes back untouched: the h it returned with it is that state's
            # y plane in bfloat16, the operand the step kernel wants (half the bytes, and the pipelined kernel).
            last = self._rt.last_step
            if (last is not None and last[0] is state and state._version == last[1] and last[2]._version == last[3]
                    and last[2] is not h):
                h_prev = last[2]
        with torch.cuda.device(input.device):
            cached[1](input, state, s_out, h, h_prev=h_prev)
        self._rt.last_workspace = cached[1].workspace
        self._rt.last_step = (s_out, s_out._version, h, h._version) if self.keep_state_fp32 else None
        return self._permute_output(h), (s_out if self.keep_state_fp32 else s_out.to(input.dtype))


def reference_cell_params_to_hip(recurrent_kernel_int: torch.Tensor, bias_int: torch.Tensor, source_backend: str,
                                 num_heads: int):
    """``_recurrent_kernel_`` / ``_bias_`` as a reference checkpoint of backend ``source_backend``
    stores them -> the hip cell's layouts (R ``[NH, 4dh, dh]``, bias ``[4H]`` head-major).

    vanilla keeps R as ``[NH, 4dh, dh]`` (cell.py:601-617, the hip layout) and the bias gate-major
    (cell.py:635-642); cuda keeps R as ``[NH, dh, 4dh]`` (cell.py:694-706) and the bias head-major
    (cell.py:726-733, the hip layout)."""
    NH = num_heads
    if source_backend == "hip":
        return recurrent_kernel_int, bias_int
    if source_backend == "vanilla":
        if recurrent_kernel_int.dim() != 3 or recurrent_kernel_int.shape[1] != 4 * recurrent_kernel_int.shape[2]:
            raise ValueError(f"a vanilla checkpoint holds R as [NH, 4*dh, dh], got {tuple(recurrent_kernel_int.shape)}")
        dh = recurrent_kernel_int.shape[2]
        return recurrent_kernel_int, bias_int.reshape(4, NH, dh).permute(1, 0, 2).reshape(-1)
    if source_backend == "cuda":
        if recurrent_kernel_int.dim() != 3 or recurrent_kernel_int.shape[2] != 4 * recurrent_kernel_int.shape[1]:
            raise ValueError(f"a cuda checkpoint holds R as [NH, dh, 4*dh], got {tuple(recurrent_kernel_int.shape)}")
        return recurrent_kernel_int.permute(0, 2, 1).contiguous(), bias_int
    raise ValueError(f'unknown source backend {source_backend!r}, choose from ["vanilla", "cuda", "hip"]')


def reference_state_dict_to_hip(state_dict: dict, source_backend: str, num_heads: int) -> dict:
    """A state dict of any module that contains reference sLSTM cells (a cell, an ``sLSTMLayer``,
    a block stack) with every ``..._recurrent_kernel_`` / ``..._bias_`` pair rewritten for the hip
    cell; all other entries pass through untouched."""
    out = dict(state_dict)
    for key in state_dict:
        if key.endswith("_recurrent_kernel_"):
            bkey = key[: -len("_recurrent_kernel_")] + "_bias_"
            if bkey not in state_dict:
                raise KeyError(f"{key} has no matching {bkey}")
            out[key], out[bkey] = reference_cell_params_to_hip(state_dict[key], state_dict[bkey], source_backend, num_heads)
    return out


class sLSTMCell:
    """Backend switch (cell.py:777-788).  This package implements ``"hip"``."""

    config_class = sLSTMCellConfig

    def __new__(cls, config: sLSTMCellConfig, skip_backend_init: bool = False):
        if config.backend == "hip":
            return sLSTMCell_hip(config, skip_backend_init=skip_backend_init)
        raise RuntimeError(
            f'sLSTMCell unknown backend {config.backend}, choose from ["hip"] '
            '("cuda" and "vanilla" live in the reference package)'
        )
