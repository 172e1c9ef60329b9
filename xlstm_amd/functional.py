"""Tensor-level entry points of the HIP engine (torch is used for device memory,
streams and layout changes of the parameters only; all arithmetic happens in the HIP kernels).

Layouts are the external ones of the reference cell:
  wx    [B, S, 4*H]   gate pre-activations, last dim ordered (gate, head, unit)
                      (xlstm/blocks/slstm/cell.py:339-342, layer.py:151-153)
  r     [NH, 4*dh, dh] K-contiguous recurrent matrix (the vanilla internal
                      layout, cell.py:601-617)
  bias  [NH, 4, dh]   float32 (external view, cell.py:253-257)
  state [4, B, H]     y, c, n, m (cell.py:441-469)
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.XS_F32, torch.bfloat16: _lib.XS_BF16}


class EngineError(RuntimeError):
    """The C ABI returned an error code."""


def _require_cuda(name: str, t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); the hip backend has no CPU path")


def workspace_for(B: int, T: int, NH: int, dh: int, device) -> torch.Tensor:
    n = _lib.load().xs_slstm_workspace_bytes(B, T, NH, dh)
    return torch.empty(n, dtype=torch.uint8, device=device)


def read_status(workspace: torch.Tensor) -> dict:
    """Copies the status block back (synchronises the stream)."""
    raw = bytes(workspace[: ctypes.sizeof(_lib.SlstmStatus)].cpu().numpy().tobytes())
    st = _lib.SlstmStatus.from_buffer_copy(raw)
    return {k: getattr(st, k) for k, _ in _lib.SlstmStatus._fields_ if k != "reserved"}


_CU_COUNT = {}


def _compute_units(dev) -> int:
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    if idx not in _CU_COUNT:
        _CU_COUNT[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _CU_COUNT[idx]


def backward_kernel_head_dim(dh: int, dtype: torch.dtype) -> Optional[int]:
    """The head dim that the backward kernels run a head dim ``dh`` as: 64, 128, 256 (and 512 with bfloat16 inputs) for
    the kernels that take one launch for all steps; beyond those, up to the forward's range (1024 with bfloat16, 512 with
    float32), the next multiple of 64 for the kernels that take one launch per step.  Sizes in between are padded up by
    ``slstm_backward``.  None when there is none."""
    bf16 = dtype == torch.bfloat16
    for size in (64, 128, 256, 512):
        if dh <= size and (size < 512 or bf16):
            return size
    if dh <= (1024 if bf16 else 512):
        return (dh + 63) // 64 * 64
    return None


def stepwise_exchange_bytes(B: int, NH: int, dh: int, esz: int) -> int:
    """Bytes of the ``exchange`` buffer of a backward pass of one launch per step: the forward walk keeps a state
    ``[4,B,H]`` and R in its own order there, the reverse pass two sets of gate deltas in tiles of 64 rows."""
    H = NH * dh
    return max(16 * B * H + 4 * NH * dh * dh * esz, 8 * ((B + 63) // 64 * 64) * H * esz)


def backward_runs_stepwise(dh_kernel: int, dtype: torch.dtype) -> bool:
    """Whether the backward pass of that (kernel) head dim takes one launch per step (``split == 3`` of the C ABI)."""
    return dh_kernel > (512 if dtype == torch.bfloat16 else 256)


class CoefficientsUnsupported(EngineError):
    """A forward call was asked to leave the backward pass its coefficients and is not one of those that can."""


def backward_coefficients_buffer(wx: torch.Tensor, num_heads: int) -> Optional[torch.Tensor]:
    """The tensor a training forward (``slstm_forward(..., coef_out=)``) leaves the backward pass's coefficients in, or
    ``None`` where the forward cannot: it takes bfloat16 inputs, a head dim of 128 or 256 and a batch whose row tiles of
    4 rows fit the device in the forward (``ceil(B/4) * NH * dh/16`` workgroups) and, with their prefetching workgroups,
    in the backward.  36 bytes per step and element, held from the forward to the backward (the reference keeps the
    states and gate values of every step instead, ``slstm.cc:79-108``); without it the backward pass recomputes them."""
    B, T = int(wx.shape[0]), int(wx.shape[1])
    H = int(wx.shape[2]) // 4
    dh = H // num_heads
    if wx.dtype != torch.bfloat16 or dh not in (128, 256) or B < 1 or T < 2:
        return None
    cus = _compute_units(wx.device)
    groups4 = num_heads * ((B + 3) // 4)
    if (groups4 + 7) // 8 * 8 * (dh // 16) > cus or (groups4 + 7) // 8 * 8 * (dh // 64) + 8 > cus:
        return None
    return torch.empty((T, (B + 3) // 4 * 4, 9, H), dtype=torch.float32, device=wx.device)


def slstm_backward(
    wx: torch.Tensor,
    r: torch.Tensor,
    bias: torch.Tensor,
    s0: Optional[torch.Tensor],
    reset_mask: Optional[torch.Tensor],
    h_out: torch.Tensor,
    d_h: torch.Tensor,
    d_s_final: Optional[torch.Tensor] = None,
    timings: Optional[dict] = None,
    split_override: Optional[bool] = None,
    spin_limit: int = 0,
    row_tile_override: Optional[int] = None,
    coef: Optional[torch.Tensor] = None,
    recurrent_cut: bool = False,
    recurrent_clipval: Optional[float] = None,
    stepwise_override: Optional[bool] = None,
    d_wx_dtype: Optional[torch.dtype] = None,
    abort_sink=None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gradients of the cell, by the rule of the reference's native kernel (the stabiliser is a constant of the
    differentiation, ``slstm_pointwise.cu:118-196``).

    ``wx, r, bias, s0, reset_mask`` are the arguments of the forward call, ``h_out[S,B,H]`` what it returned, ``d_h`` the
    gradient with respect to ``h_out`` and ``d_s_final[4,B,H]`` (optional) with respect to the final state.  Returns
    ``(d_wx[B,S,4H] float32, d_r[NH,4*dh,dh], d_bias[NH,4,dh], d_s0[4,B,H])``.

    Three kernels of the engine: ``xs_slstm_backward_prepare`` (a forward walk over the stored outputs that leaves nine
    coefficients per step and element), ``xs_slstm_backward`` (the reverse pass) and ``xs_slstm_backward_params`` (the
    gradients of R and the bias, sums over all steps of products of the gate deltas with the outputs); what torch does
    here is allocating the buffers (R is brought into the reverse kernel's operand order by ``xs_slstm_backward_tile_r``).  ``timings`` (a dict) receives four
    events around the three kernels.  Where the head dim allows it (64, 128, 256; 512 in bfloat16) and the workgroups fit the device at once,
    a head is spread over ``dh/64`` compute units that wait for each other every step (``split_override`` forces either
    kernel), in row tiles of 4 rows where four times the workgroups fit (bfloat16, head dims up to 256;
    ``row_tile_override`` = 16 or 4 forces either); ``spin_limit`` bounds those waits, and a wait that runs out raises ``EngineError``.
    Head dims beyond those (up to 1024 with bfloat16, 512 with float32: the forward's range) take one launch per step,
    forward walk and reverse pass alike (``stepwise_override=True`` forces that for head dim 512 in bfloat16 and 256 in
    float32, which both ways cover).
    ``d_wx_dtype=torch.bfloat16`` (bfloat16 inputs only): ``d_wx`` comes back in bfloat16, as the reference returns its
    input gradient in the type of its kernels; the reverse kernel then writes and the parameter kernel reads half the bytes.
    ``abort_sink``: a callable that takes the call's abort word (an int32 tensor of one element on the device) instead
    of this function reading it, which synchronises the host; the cell queues an asynchronous copy and raises at a later call.
    ``coef``: what a training forward left (``slstm_forward(..., coef_out=)``); the forward walk is then skipped.
    ``recurrent_cut`` and ``recurrent_clipval`` are the reference's ``gradient_recurrent_cut`` (no gradient from a step
    to the y it started from, ``slstm_backward_cut.cu:265-312``) and ``gradient_recurrent_clipval`` (that gradient
    clipped to +-value before ``d_h`` is added, ``slstm_pointwise.cu:136-143``).
    """
    lib = _lib.load()
    _require_cuda("wx", wx)
    NH, dh = int(r.shape[0]), int(r.shape[2])
    H = NH * dh
    B, T = int(wx.shape[0]), int(wx.shape[1])
    if wx.dtype not in _DTYPE_CODE:
        raise TypeError(f"wx dtype {wx.dtype} not supported by the hip backend (float32 or bfloat16)")
    bf16 = wx.dtype == torch.bfloat16
    if tuple(h_out.shape) != (T, B, H) or tuple(d_h.shape) != (T, B, H):
        raise ValueError(f"h_out and d_h must be [S, B, H] = {(T, B, H)}")
    dh_k = backward_kernel_head_dim(dh, wx.dtype)
    if coef is not None and (dh_k != dh or not bf16 or tuple(coef.shape) != (T, (B + 3) // 4 * 4, 9, H)
                             or coef.dtype != torch.float32 or not coef.is_contiguous()):
        raise ValueError("coef must be the tensor that the forward call of the same inputs filled")
    if dh_k is None:
        raise EngineError(f"xlstm_amd: no backward kernel for head dim {dh} with {wx.dtype} inputs "
                          f"(up to 1024 with bfloat16, up to 512 with float32)")
    if dh_k != dh:
        # A head dim between the kernels' sizes runs as the next size up with units that are not there: their W.x, bias
        # and rows and columns of R are zero, so they neither see nor touch the real units, and their results are cut off.
        pad = dh_k - dh
        B_, T_ = int(wx.shape[0]), int(wx.shape[1])
        Fn = torch.nn.functional

        def widen(x, lead):  # [*lead, NH*dh] -> [*lead, NH, dh_k], zeros behind the real units
            return Fn.pad(x.reshape(*lead, NH, dh), (0, pad))

        wx_p = widen(wx, (B_, T_, 4)).reshape(B_, T_, 4 * NH * dh_k)
        r_p = Fn.pad(r.reshape(NH, 4, dh, dh), (0, pad, 0, pad)).reshape(NH, 4 * dh_k, dh_k)
        bias_p = Fn.pad(bias, (0, pad))
        s0_p = widen(s0, (4, B_)).reshape(4, B_, NH * dh_k) if s0 is not None else None
        h_p = widen(h_out, (T_, B_)).reshape(T_, B_, NH * dh_k)
        dh_p = widen(d_h, (T_, B_)).reshape(T_, B_, NH * dh_k)
        dsf_p = widen(d_s_final, (4, B_)).reshape(4, B_, NH * dh_k) if d_s_final is not None else None
        d_wx, d_r, d_bias, d_s0 = slstm_backward(wx_p, r_p, bias_p, s0_p, reset_mask, h_p, dh_p, dsf_p, timings=timings,
                                                 split_override=split_override, spin_limit=spin_limit, row_tile_override=row_tile_override,
                                                 recurrent_cut=recurrent_cut, recurrent_clipval=recurrent_clipval,
                                                 stepwise_override=stepwise_override, d_wx_dtype=d_wx_dtype, abort_sink=abort_sink)
        return (d_wx.view(B_, T_, 4, NH, dh_k)[..., :dh].reshape(B_, T_, 4 * H),
                d_r.view(NH, 4, dh_k, dh_k)[:, :, :dh, :dh].reshape(NH, 4 * dh, dh),
                d_bias[..., :dh].contiguous(),
                d_s0.view(4, B_, NH, dh_k)[..., :dh].reshape(4, B_, H))
    dev = wx.device
    # The kernel that spreads a head over dh/64 compute units needs all its workgroups on the device at once.  A batch
    # with more row tiles than that runs in slices of rows (rows do not meet in the backward pass but in the sums for
    # R and the bias), rather than with one workgroup per head, which takes 7 times as long per step.
    stepwise = backward_runs_stepwise(dh, wx.dtype)
    if stepwise_override and dh == (512 if bf16 else 256):
        stepwise = True
    if stepwise and coef is not None:
        raise EngineError("xlstm_amd: coefficients from the forward call do not go with the backward pass of one launch per step")
    if split_override is not False and coef is None and not stepwise:
        room = (_compute_units(dev) - 8) // (8 * (dh // 64)) * 8      # groups per launch, the prefetching workgroups kept
        tiles_per_launch = room // NH
        if tiles_per_launch >= 1 and (B + 15) // 16 > tiles_per_launch:
            rows = tiles_per_launch * 16
            parts = []
            for b0 in range(0, B, rows):
                b1 = min(B, b0 + rows)
                parts.append(slstm_backward(
                    wx[b0:b1], r, bias, None if s0 is None else s0[:, b0:b1], None if reset_mask is None else reset_mask[b0:b1],
                    h_out[:, b0:b1], d_h[:, b0:b1], None if d_s_final is None else d_s_final[:, b0:b1],
                    timings=None, split_override=split_override, spin_limit=spin_limit, row_tile_override=row_tile_override,
                    recurrent_cut=recurrent_cut, recurrent_clipval=recurrent_clipval, d_wx_dtype=d_wx_dtype, abort_sink=abort_sink))
            return (torch.cat([q[0] for q in parts], 0), sum(q[1] for q in parts), sum(q[2] for q in parts),
                    torch.cat([q[3] for q in parts], 1))
    esz = wx.element_size()
    if (wx.stride(2) != 1 or wx.data_ptr() % 16 or (wx.stride(0) * esz) % 16 or (wx.stride(1) * esz) % 16
            or wx.stride(1) < 4 * H or (B > 1 and wx.stride(0) < 4 * H)):
        wx = wx.contiguous()  # (the same condition as in the forward: the kernels fetch W.x in pieces of 16 bytes)
    bias = bias.to(torch.float32).contiguous()
    if s0 is not None:
        s0 = s0.to(torch.float32).contiguous()
    if reset_mask is not None:  # (bytes, any non-zero value marks a document start: as the forward takes it)
        if reset_mask.dtype == torch.bool:
            reset_mask = reset_mask.view(torch.uint8) if reset_mask.is_contiguous() else reset_mask.to(torch.uint8)
        elif reset_mask.dtype != torch.uint8:
            reset_mask = (reset_mask != 0).to(torch.uint8)
        reset_mask = reset_mask.contiguous()
    r_fwd = r.to(wx.dtype).contiguous()  # R as the forward multiplies by it (the forward rounds R to bf16)
    h_c = h_out if h_out.is_contiguous() and h_out.dtype == wx.dtype else h_out.to(wx.dtype).contiguous()
    if d_wx_dtype not in (None, torch.float32) and not (d_wx_dtype == torch.bfloat16 and bf16):
        raise TypeError("d_wx_dtype: float32, or bfloat16 with bfloat16 inputs")
    d_wx = torch.empty((B, T, 4 * H), dtype=d_wx_dtype or torch.float32, device=dev)
    d_s0 = torch.empty((4, B, H), dtype=torch.float32, device=dev)
    epc = 8 if bf16 else 4
    groups = NH * ((B + 15) // 16)
    S = dh // 64
    # a head over S compute units where the head dim allows it and all workgroups fit the device at once
    split = (dh in (64, 128, 256) or (dh == 512 and bf16)) and (groups + 7) // 8 * 8 * S <= _compute_units(dev)
    if split_override is not None:
        split = bool(split_override)
    if stepwise:
        split = False
    # row tiles of 4 rows (bf16, head dims up to 256) where four times the workgroups still fit (the prefetching ones
    # take what room is left: without any, at B 64 x 4 heads of 256, the reverse kernel still takes 2.6 ms against 4.2
    # with row tiles of 16 rows)
    groups4 = NH * ((B + 3) // 4)
    quad = (split and bf16 and dh <= 256 and (groups4 + 7) // 8 * 8 * S <= _compute_units(dev)
            and (reset_mask is None or 3 * reset_mask.stride(0) + T < 2 ** 31 - 256))
    if row_tile_override is not None:
        quad = split and row_tile_override == 4
    quad = quad and not stepwise
    if coef is not None:
        if not (split and quad):
            raise EngineError("xlstm_amd: coefficients from the forward call go with the reverse kernel for row tiles of 4 rows, "
                              "which this call does not run")
    # (the split kernels read the coefficients in pieces of a row tile: the buffer covers whole row tiles)
    coef_given = coef is not None
    if not coef_given:
        rows = ((B + 3) // 4 * 4 if quad else (B + 15) // 16 * 16) if split else ((B + 63) // 64 * 64 if stepwise else B)
        coef = torch.empty((T, rows, 9, H), dtype=torch.float32, device=dev)
    # R transposed in the operand order of the reverse kernel (xs_slstm_backward_tile_r), and what the kernels of a call
    # hand to each other
    r_t = torch.empty(NH * 4 * dh * dh, dtype=wx.dtype, device=dev)
    exchange = counters = None
    if quad:
        exchange = torch.empty(4 * groups4 * 4 * 4 * dh, dtype=wx.dtype, device=dev)
        counters = torch.empty(1 + 2 * groups4, dtype=torch.int32, device=dev)
    elif split:
        exchange = torch.empty(4 * groups * 16 * 4 * dh, dtype=wx.dtype, device=dev)
        counters = torch.empty(1 + 2 * groups, dtype=torch.int32, device=dev)
    elif stepwise:
        exchange = torch.empty(stepwise_exchange_bytes(B, NH, dh, esz), dtype=torch.uint8, device=dev)
    d_h = d_h.to(wx.dtype).contiguous()
    if d_s_final is not None:
        d_s_final = d_s_final.to(torch.float32).contiguous()

    a = _lib.SlstmBwdArgs()
    a.B, a.T, a.NH, a.dh = B, T, NH, dh
    a.dtype = _DTYPE_CODE[wx.dtype]
    a.wx = wx.data_ptr()
    a.wx_stride_b, a.wx_stride_t = wx.stride(0), wx.stride(1)
    a.ry = None
    a.r, a.h_out = r_fwd.data_ptr(), h_c.data_ptr()
    a.bias = bias.data_ptr()
    a.s0 = s0.data_ptr() if s0 is not None else None
    a.reset = reset_mask.data_ptr() if reset_mask is not None else None
    a.reset_stride_b = reset_mask.stride(0) if reset_mask is not None else 0
    a.coef = coef.data_ptr()
    a.d_h = d_h.data_ptr()
    a.d_s_final = d_s_final.data_ptr() if d_s_final is not None else None
    a.r_t = r_t.data_ptr()
    a.d_wx = d_wx.data_ptr()
    a.d_wx_stride_b, a.d_wx_stride_t = d_wx.stride(0), d_wx.stride(1)
    a.d_wx_dtype = _DTYPE_CODE[d_wx.dtype]
    a.d_s0 = d_s0.data_ptr()
    a.stream = torch.cuda.current_stream(dev).cuda_stream
    a.split = 3 if stepwise else ((2 if quad else 1) if split else 0)
    a.exchange = exchange.data_ptr() if exchange is not None else None
    a.counters = counters.data_ptr() if counters is not None else None
    a.spin_limit = int(spin_limit)
    a.recurrent_cut = 1 if recurrent_cut else 0
    a.recurrent_clipval = float(recurrent_clipval) if recurrent_clipval is not None else 0.0
    marks = []  # (measurement: events around the two kernels, read by the caller after a synchronisation)
    with torch.cuda.device(dev):
        rc = lib.xs_slstm_backward_tile_r(ctypes.byref(a))
        if rc != 0:
            raise EngineError(f"xlstm_amd error {rc}: {_lib.last_error()}")
        for fn in (lib.xs_slstm_backward_prepare, lib.xs_slstm_backward):
            if coef_given and fn is lib.xs_slstm_backward_prepare:
                if timings is not None:
                    marks.append(torch.cuda.Event(enable_timing=True))
                    marks[-1].record()
                continue
            if timings is not None:
                marks.append(torch.cuda.Event(enable_timing=True))
                marks[-1].record()
            rc = fn(ctypes.byref(a))
            if rc != 0:
                raise EngineError(f"xlstm_amd error {rc}: {_lib.last_error()}")
        if timings is not None:
            marks.append(torch.cuda.Event(enable_timing=True))
            marks[-1].record()
            timings["events"] = marks  # prepare = [0] -> [1], reverse kernel = [1] -> [2]
        # d R[h][g dh + a][d] = sum over steps and rows of delta[b,t,g,h,a] * y_{t-1}[b,h,d]; d bias = sum of delta: the
        # engine's third backward kernel, from d_wx as it lies and the forward's outputs
        d_r = torch.empty((NH, 4 * dh, dh), dtype=torch.float32, device=dev)
        d_bias = torch.empty((NH, 4, dh), dtype=torch.float32, device=dev)
        a.d_r, a.d_bias = d_r.data_ptr(), d_bias.data_ptr()
        rc = lib.xs_slstm_backward_params(ctypes.byref(a))
        if rc != 0:
            raise EngineError(f"xlstm_amd error {rc}: {_lib.last_error()}")
        if timings is not None:
            marks.append(torch.cuda.Event(enable_timing=True))
            marks[-1].record()  # parameter gradients = [2] -> [3]
    if split and abort_sink is not None:  # (the caller looks at the call's abort word later: no synchronisation here)
        abort_sink(counters[:1])
    elif split and timings is None and int(counters[0].item()):  # (a synchronisation)
        raise EngineError("xlstm_amd: a wait between the compute units of a head ran out in the backward pass "
                          "(other work held compute units, or the workgroups of a head were not placed on one XCD); "
                          "the gradients are invalid")
    return d_wx, d_r, d_bias, d_s0


def read_phase_stamps(workspace: torch.Tensor) -> torch.Tensor:
    """Per-phase cycle sums that a library built with ``-DXS_PROFILE`` leaves behind a sequence call: ``[6, 8]`` int64,
    one row per wave slot of workgroup 0 (which waves and phases: see ``bench.py --phase-profile``).  The product
    library writes nothing there."""
    off = 256 + 4 * (4096 - 128)
    return workspace[off: off + 6 * 8 * 8].cpu().view(torch.int64).view(6, 8)


def read_placement(workspace: torch.Tensor, max_wg: int = 4096) -> torch.Tensor:
    """Per-workgroup placement words written by the sequence kernel:
    bit 31 = workgroup was active, bits [30:8] head group, bits [3:0] XCD id."""
    off = 256
    return workspace[off: off + 4 * max_wg].cpu().view(torch.int32)


def slstm_forward(
    wx: torch.Tensor,
    r: torch.Tensor,
    bias: torch.Tensor,
    s0: Optional[torch.Tensor] = None,
    reset_mask: Optional[torch.Tensor] = None,
    *,
    step: bool = False,
    workspace: Optional[torch.Tensor] = None,
    h_out: Optional[torch.Tensor] = None,
    s_out: Optional[torch.Tensor] = None,
    spin_limit: int = 0,
    h_prev: Optional[torch.Tensor] = None,
    coef_out: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Runs the cell over ``wx`` and returns ``(h[S,B,H] in wx.dtype, state[4,B,H] float32)``.

    ``coef_out`` (a training forward; a float32 tensor from ``backward_coefficients_buffer``): the kernel also leaves
    the coefficients of the backward pass there, and ``slstm_backward(..., coef=coef_out)`` skips its own forward walk.
    Raises ``CoefficientsUnsupported`` (nothing has run) for calls that cannot: see ``backward_coefficients_buffer``.

    ``reset_mask[B,S]`` (bool/uint8) marks document starts: the row's state is
    zeroed before that step.  ``step=True`` uses the decode entry point (S == 1).
    ``h_prev`` (bfloat16 decode steps only): the ``h`` the previous step returned, i.e.
    ``s0[0]`` already rounded to bfloat16; the kernel then reads half the operand bytes.
    """
    lib = _lib.load()
    _require_cuda("wx", wx)
    if wx.dim() != 3:
        raise ValueError(f"wx must be [B, S, 4*H], got {tuple(wx.shape)}")
    if wx.dtype not in _DTYPE_CODE:
        raise TypeError(f"wx dtype {wx.dtype} not supported by the hip backend (float32 or bfloat16)")
    if r.dim() != 3 or r.shape[1] != 4 * r.shape[2]:
        raise ValueError(f"r must be [NH, 4*dh, dh], got {tuple(r.shape)}")
    NH, dh = int(r.shape[0]), int(r.shape[2])
    H = NH * dh
    B, T = int(wx.shape[0]), int(wx.shape[1])
    if wx.shape[2] != 4 * H:
        raise ValueError(f"Input size mismatch: Expected input size {4 * H}, but got {wx.shape[2]}.")
    if r.dtype not in _DTYPE_CODE:
        raise TypeError(f"r dtype {r.dtype} not supported")
    if wx.dtype == torch.float32 and r.dtype != torch.float32:
        r = r.float()
    if step and r.dtype != wx.dtype:
        r = r.to(wx.dtype)  # callers that decode many tokens pass a cached copy (see sLSTMCell_hip)
    if tuple(bias.shape) != (NH, 4, dh):
        raise ValueError(f"bias must be [NH, 4, dh] = {(NH, 4, dh)}, got {tuple(bias.shape)}")
    for name, t in (("r", r), ("bias", bias)):
        _require_cuda(name, t)
    r = r.contiguous()
    bias = bias.to(torch.float32).contiguous()
    if wx.numel():
        esz = wx.element_size()
        if (wx.stride(2) != 1 or wx.data_ptr() % 16 or (wx.stride(0) * esz) % 16 or (wx.stride(1) * esz) % 16
                or wx.stride(1) < 4 * H or (B > 1 and wx.stride(0) < 4 * H)):
            wx = wx.contiguous()
    if s0 is not None:
        _require_cuda("state", s0)
        if tuple(s0.shape) != (4, B, H):
            raise ValueError(f"state must be [4, B, H] = {(4, B, H)}, got {tuple(s0.shape)}")
        s0 = s0.to(torch.float32).contiguous()
    if reset_mask is not None:
        _require_cuda("reset_mask", reset_mask)
        if tuple(reset_mask.shape) != (B, T):
            raise ValueError(f"reset_mask must be [B, S] = {(B, T)}, got {tuple(reset_mask.shape)}")
        if reset_mask.dtype == torch.bool:
            reset_mask = reset_mask.view(torch.uint8) if reset_mask.is_contiguous() else reset_mask.to(torch.uint8)
        elif reset_mask.dtype != torch.uint8:
            reset_mask = (reset_mask != 0).to(torch.uint8)
        if T and reset_mask.stride(1) != 1:
            reset_mask = reset_mask.contiguous()
    dev = wx.device
    if h_out is None:
        h_out = torch.empty((T, B, H), dtype=wx.dtype, device=dev)
    if s_out is None:
        s_out = torch.empty((4, B, H), dtype=torch.float32, device=dev)
    if workspace is None:
        workspace = workspace_for(B, T, NH, dh, dev)

    a = _lib.SlstmArgs()
    a.B, a.T, a.NH, a.dh = B, T, NH, dh
    a.wx_dtype = _DTYPE_CODE[wx.dtype]
    a.r_dtype = _DTYPE_CODE[r.dtype]
    a.wx = wx.data_ptr()
    a.wx_stride_b = wx.stride(0) if B else 0
    a.wx_stride_t = wx.stride(1) if T else 0
    a.r = r.data_ptr()
    a.bias = bias.data_ptr()
    a.s0 = s0.data_ptr() if s0 is not None else None
    a.reset = reset_mask.data_ptr() if reset_mask is not None else None
    a.reset_stride_b = reset_mask.stride(0) if reset_mask is not None else 0
    a.h_out = h_out.data_ptr()
    a.s_out = s_out.data_ptr()
    a.workspace = workspace.data_ptr()
    a.workspace_bytes = workspace.numel()
    a.stream = torch.cuda.current_stream(dev).cuda_stream
    a.spin_limit = int(spin_limit)
    a.h_prev = None
    if h_prev is not None and step and wx.dtype == torch.bfloat16 and s0 is not None:
        if h_prev.dtype != torch.bfloat16 or h_prev.numel() != B * H or not h_prev.is_contiguous():
            raise ValueError(f"h_prev must be a contiguous bfloat16 tensor of {B * H} elements")
        a.h_prev = h_prev.data_ptr()
    a.coef_out = None
    if coef_out is not None:
        if step:
            raise CoefficientsUnsupported("xlstm_amd: a decode step keeps no coefficients")
        if coef_out.dtype != torch.float32 or not coef_out.is_contiguous() or coef_out.numel() != T * ((B + 3) // 4 * 4) * 9 * H:
            raise ValueError("coef_out must be the tensor backward_coefficients_buffer returns for this call")
        a.coef_out = coef_out.data_ptr()
    with torch.cuda.device(dev):
        rc = (lib.xs_slstm_step if step else lib.xs_slstm_forward)(ctypes.byref(a))
    if rc != 0:
        if coef_out is not None and rc == _lib.XS_ERR_UNSUPPORTED:
            raise CoefficientsUnsupported(f"xlstm_amd error {rc}: {_lib.last_error()}")
        raise EngineError(f"xlstm_amd error {rc}: {_lib.last_error()}")
    return h_out, s_out


class StepPlan:
    """Single-token steps with fixed shapes, validated once.

    ``slstm_forward(..., step=True)`` checks and normalises every argument on every call, which costs
    more host time than the step kernel runs.  A plan does that work once; calling it only swaps
    the five pointers that change between tokens and launches ``xs_slstm_step``::

        plan = StepPlan(B, r, bias, wx_dtype=torch.bfloat16)
        for x_t in tokens:                       # x_t: [B, 1, 4H], contiguous
            plan(x_t, s_in, s_out, h_out)        # s_in / s_out: float32 [4, B, H], distinct buffers
            s_in, s_out = s_out, s_in

    The caller keeps the plan's contract: tensors on the plan's device, which is the current one,
    the dtypes and shapes given at construction, contiguous, ``s_out`` not overlapping ``s_in``.
    A plan is NOT re-entrant: every call rewrites the one argument block the plan owns, so a plan
    belongs to one host thread at a time (calls from one thread onto different streams are fine,
    the block is read before the call returns).
    """

    def __init__(self, B: int, r: torch.Tensor, bias: torch.Tensor, wx_dtype: torch.dtype = torch.bfloat16,
                 workspace: Optional[torch.Tensor] = None):
        lib = _lib.load()
        _require_cuda("r", r)
        if wx_dtype not in _DTYPE_CODE:
            raise TypeError(f"wx dtype {wx_dtype} not supported by the hip backend (float32 or bfloat16)")
        if r.dim() != 3 or r.shape[1] != 4 * r.shape[2]:
            raise ValueError(f"r must be [NH, 4*dh, dh], got {tuple(r.shape)}")
        NH, dh = int(r.shape[0]), int(r.shape[2])
        if tuple(bias.shape) != (NH, 4, dh):
            raise ValueError(f"bias must be [NH, 4, dh] = {(NH, 4, dh)}, got {tuple(bias.shape)}")
        self.B, self.NH, self.dh, self.H = int(B), NH, dh, NH * dh
        self.wx_dtype = wx_dtype
        self.device = r.device
        # the plan owns what it points to: R in the operand type, float32 bias, the workspace
        self.r = r.detach().to(wx_dtype).contiguous()
        self.bias = bias.detach().to(torch.float32).contiguous()
        self.workspace = workspace if workspace is not None else workspace_for(self.B, 1, NH, dh, self.device)
        a = _lib.SlstmArgs()
        a.B, a.T, a.NH, a.dh = self.B, 1, NH, dh
        a.wx_dtype = a.r_dtype = _DTYPE_CODE[wx_dtype]
        a.wx_stride_b, a.wx_stride_t = 4 * self.H, 4 * self.H
        a.r, a.bias = self.r.data_ptr(), self.bias.data_ptr()
        a.reset, a.reset_stride_b = None, 0
        a.workspace, a.workspace_bytes = self.workspace.data_ptr(), self.workspace.numel()
        a.spin_limit = 0
        # Head dims whose K range the step kernel walks in slabs (beyond 256 in bfloat16, 128 in float32): R once more, slab
        # by slab, for the kernel whose feeder waves bring the slabs to LDS (bfloat16: when the caller passes ``h_prev``)
        self.r_tiled = None
        if dh % 64 == 0 and dh > (256 if wx_dtype == torch.bfloat16 else 128):
            self.r_tiled = torch.empty_like(self.r)
            with torch.cuda.device(self.device):
                rc = lib.xs_slstm_tile_r_for_steps(self.r.data_ptr(), self.r_tiled.data_ptr(), NH, dh, _DTYPE_CODE[wx_dtype],
                                                   torch.cuda.current_stream(self.device).cuda_stream)
            if rc != 0:
                raise EngineError(f"xlstm_amd error {rc}: {_lib.last_error()}")
            a.r_tiled = self.r_tiled.data_ptr()
        self._args, self._ref, self._fn = a, ctypes.byref(a), lib.xs_slstm_step
        self._wx_numel, self._s_numel = self.B * 4 * self.H, 4 * self.B * self.H

    def __call__(self, wx: torch.Tensor, s_in: torch.Tensor, s_out: torch.Tensor, h_out: torch.Tensor,
                 stream: Optional[int] = None, h_prev: Optional[torch.Tensor] = None) -> None:
        """``h_prev`` (bfloat16 plans): the ``h_out`` buffer the previous call filled, a different buffer
        than this call's ``h_out``; it must hold ``s_in[0]`` rounded to bfloat16."""
        if (wx.dtype != self.wx_dtype or wx.numel() != self._wx_numel or s_in.numel() != self._s_numel
                or s_out.numel() != self._s_numel or s_in.dtype != torch.float32 or s_out.dtype != torch.float32
                or h_out.dtype != self.wx_dtype or h_out.numel() * 4 != self._s_numel):
            raise ValueError("tensor does not fit the plan (dtype or size)")
        a = self._args
        a.wx, a.s0, a.s_out, a.h_out = wx.data_ptr(), s_in.data_ptr(), s_out.data_ptr(), h_out.data_ptr()
        if h_prev is not None and self.wx_dtype == torch.bfloat16:
            if h_prev.dtype != torch.bfloat16 or h_prev.numel() * 4 != self._s_numel:
                raise ValueError("h_prev does not fit the plan (dtype or size)")
            a.h_prev = h_prev.data_ptr()
        else:
            a.h_prev = None
        a.stream = stream if stream is not None else torch.cuda.current_stream().cuda_stream
        rc = self._fn(self._ref)
        if rc != 0:
            raise EngineError(f"xlstm_amd error {rc}: {_lib.last_error()}")


def _mask_u8(reset_mask: torch.Tensor, B: int, T: int) -> torch.Tensor:
    _require_cuda("reset_mask", reset_mask)
    if tuple(reset_mask.shape) != (B, T):
        raise ValueError(f"reset_mask must be [B, S] = {(B, T)}, got {tuple(reset_mask.shape)}")
    if reset_mask.dtype == torch.bool:
        reset_mask = reset_mask.view(torch.uint8) if reset_mask.is_contiguous() else reset_mask.to(torch.uint8)
    elif reset_mask.dtype != torch.uint8:
        reset_mask = (reset_mask != 0).to(torch.uint8)
    if T and reset_mask.stride(1) != 1:
        reset_mask = reset_mask.contiguous()
    return reset_mask


def fused_layer_ops_supported(x: torch.Tensor, num_heads: int, kernel_size: int) -> bool:
    """Whether :func:`causal_conv_silu` and :func:`headwise_gates` cover this input (bfloat16 on the GPU,
    head dim a multiple of 64, 2..4 taps)."""
    D = int(x.shape[-1])
    return (x.is_cuda and x.dtype == torch.bfloat16 and D % num_heads == 0 and (D // num_heads) % 64 == 0
            and (kernel_size == 0 or 2 <= kernel_size <= 4))


def causal_conv_silu(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     conv_state: Optional[torch.Tensor] = None, reset_mask: Optional[torch.Tensor] = None,
                     out: Optional[torch.Tensor] = None, ring_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(causal_conv1d(x))`` of an sLSTM layer (xlstm/components/conv.py:113-127,
    xlstm/blocks/slstm/layer.py:136-137) in one kernel.  ``x`` [B,S,D] bfloat16, ``weight`` [D,1,K] or [D,K],
    ``conv_state`` [B,K-1,D] = the inputs before ``x``; ``reset_mask`` [B,S] stops the taps at document starts.
    ``ring_out`` (S == 1): a contiguous bfloat16 [B,K,D] buffer, not overlapping ``conv_state``, that receives the
    state of the next step (``conv_state`` followed by ``x``, conv.py:142-149)."""
    lib = _lib.load()
    _require_cuda("x", x)
    if x.dim() != 3 or x.dtype != torch.bfloat16:
        raise TypeError(f"x must be a bfloat16 [B, S, D] tensor, got {x.dtype} {tuple(x.shape)}")
    B, T, D = (int(v) for v in x.shape)
    w = weight.reshape(D, -1)
    K = int(w.shape[1])
    if w.dtype != torch.bfloat16 or not w.is_contiguous():
        w = w.to(torch.bfloat16).contiguous()
    if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_contiguous()):
        bias = bias.to(torch.bfloat16).contiguous()
    if x.numel() and (x.stride(2) != 1 or x.data_ptr() % 16 or x.stride(0) % 8 or x.stride(1) % 8
                      or x.stride(1) < D or (B > 1 and x.stride(0) < D)):
        x = x.contiguous()
    if conv_state is not None:
        if tuple(conv_state.shape) != (B, K - 1, D):
            raise ValueError(f"conv_state must be [B, K-1, D] = {(B, K - 1, D)}, got {tuple(conv_state.shape)}")
        if (conv_state.dtype != torch.bfloat16 or conv_state.stride(2) != 1 or conv_state.stride(1) != D
                or conv_state.stride(0) % 8 or conv_state.data_ptr() % 16):  # a [:, :K-1] view of a ring is taken as it is
            conv_state = conv_state.to(torch.bfloat16).contiguous()
    if reset_mask is not None:
        reset_mask = _mask_u8(reset_mask, B, T)
    if out is None:
        out = torch.empty((B, T, D), dtype=torch.bfloat16, device=x.device)
    elif out.dtype != torch.bfloat16 or out.numel() != B * T * D or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous bfloat16 tensor of {B * T * D} elements")
    a = _lib.ConvArgs()
    a.B, a.T, a.D, a.K = B, T, D, K
    a.dtype = _lib.XS_BF16
    a.x = x.data_ptr()
    a.x_stride_b = x.stride(0) if B else 0
    a.x_stride_t = x.stride(1) if T else 0
    a.conv_state = conv_state.data_ptr() if conv_state is not None else None
    a.conv_state_stride_b = conv_state.stride(0) if conv_state is not None and B > 1 else 0
    a.weight = w.data_ptr()
    a.bias = bias.data_ptr() if bias is not None else None
    a.reset = reset_mask.data_ptr() if reset_mask is not None else None
    a.reset_stride_b = reset_mask.stride(0) if reset_mask is not None else 0
    a.out = out.data_ptr()
    a.ring_out = None
    if ring_out is not None:
        if ring_out.dtype != torch.bfloat16 or tuple(ring_out.shape) != (B, K, D) or not ring_out.is_contiguous():
            raise ValueError(f"ring_out must be a contiguous bfloat16 [B, K, D] = {(B, K, D)} tensor")
        a.ring_out = ring_out.data_ptr()
    a.stream = torch.cuda.current_stream(x.device).cuda_stream
    with torch.cuda.device(x.device):
        rc = lib.xs_causal_conv_silu(ctypes.byref(a))
    if rc != 0:
        raise EngineError(f"xs_causal_conv_silu failed ({rc}): {_lib.last_error()}")
    return out


def headwise_gates(x: torch.Tensor, x_conv: torch.Tensor, weights, num_heads: int,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The cell input of an sLSTM layer in one kernel: ``cat([W_i x_conv, W_f x_conv, W_z x, W_o x], -1)`` with
    block-diagonal ("headwise") matrices (xlstm/blocks/slstm/layer.py:144-153,
    xlstm/components/linear_headwise.py:75-82).  ``weights``: four [NH, dh, dh] tensors in slot order i, f, z, o."""
    lib = _lib.load()
    _require_cuda("x", x)
    if x.dtype != torch.bfloat16 or x_conv.dtype != torch.bfloat16 or x.shape != x_conv.shape:
        raise TypeError("x and x_conv must be bfloat16 tensors of one shape")
    H = int(x.shape[-1])
    dh = H // num_heads
    x2 = x.reshape(-1, H)
    xc2 = x_conv.reshape(-1, H)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    if xc2.stride(1) != 1 or xc2.stride(0) % 8 or xc2.data_ptr() % 16:
        xc2 = xc2.contiguous()
    M = int(x2.shape[0])
    ws = []
    for w in weights:
        if tuple(w.shape) != (num_heads, dh, dh):
            raise ValueError(f"gate weight must be [NH, dh, dh] = {(num_heads, dh, dh)}, got {tuple(w.shape)}")
        ws.append(w if (w.dtype == torch.bfloat16 and w.is_contiguous()) else w.to(torch.bfloat16).contiguous())
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (4 * H,), dtype=torch.bfloat16, device=x.device)
    elif out.dtype != torch.bfloat16 or out.numel() != M * 4 * H or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous bfloat16 tensor of {M * 4 * H} elements")
    a = _lib.GatesArgs()
    a.M, a.NH, a.dh = M, num_heads, dh
    a.dtype = _lib.XS_BF16
    a.x = x2.data_ptr()
    a.x_stride_row = x2.stride(0) if M else H
    a.x_conv = xc2.data_ptr()
    a.x_conv_stride_row = xc2.stride(0) if M else H
    for g in range(4):
        a.w[g] = ws[g].data_ptr()
    a.out = out.data_ptr()
    a.out_stride_row = 4 * H
    a.stream = torch.cuda.current_stream(x.device).cuda_stream
    with torch.cuda.device(x.device):
        rc = lib.xs_headwise_gates(ctypes.byref(a))
    if rc != 0:
        raise EngineError(f"xs_headwise_gates failed ({rc}): {_lib.last_error()}")
    return out


def headwise_group_norm(y: torch.Tensor, weight: Optional[torch.Tensor] = None, eps: float = 1e-5,
                        out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The layer's group norm behind the cell in one kernel (xlstm/components/ln.py:51-68 with the residual
    weight, then the transpose + view of xlstm/blocks/slstm/layer.py:159): ``y`` [B,NH,S,DH] bfloat16 - the cell's
    output, any strides with a contiguous last dim - to ``[B,S,NH*DH]``."""
    lib = _lib.load()
    _require_cuda("y", y)
    if y.dim() != 4 or y.dtype != torch.bfloat16:
        raise TypeError(f"y must be a bfloat16 [B, NH, S, DH] tensor, got {y.dtype} {tuple(y.shape)}")
    B, NH, T, dh = (int(v) for v in y.shape)
    if y.numel() and (y.stride(3) != 1 or y.data_ptr() % 8 or any(y.stride(i) % 4 for i in range(3))):
        y = y.contiguous()
    if weight is not None and (weight.dtype != torch.bfloat16 or not weight.is_contiguous()):
        weight = weight.to(torch.bfloat16).contiguous()
    if out is None:
        out = torch.empty((B, T, NH * dh), dtype=torch.bfloat16, device=y.device)
    elif out.dtype != torch.bfloat16 or out.numel() != B * T * NH * dh or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous bfloat16 tensor of {B * T * NH * dh} elements")
    a = _lib.NormArgs()
    a.B, a.T, a.NH, a.dh = B, T, NH, dh
    a.dtype = _lib.XS_BF16
    a.eps = float(eps)
    a.x = y.data_ptr()
    a.x_stride_b, a.x_stride_h, a.x_stride_t = y.stride(0), y.stride(1), y.stride(2)
    a.weight = weight.data_ptr() if weight is not None else None
    a.out = out.data_ptr()
    a.stream = torch.cuda.current_stream(y.device).cuda_stream
    with torch.cuda.device(y.device):
        rc = lib.xs_headwise_group_norm(ctypes.byref(a))
    if rc != 0:
        raise EngineError(f"xs_headwise_group_norm failed ({rc}): {_lib.last_error()}")
    return out
