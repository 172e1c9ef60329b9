"""Benchmark of the sLSTM forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one forward pass of the cell over one packed batch (BASELINE config 2:
B=16, T=2048, D=1024, 4 heads, bf16 W.x, documents of geometric length (mean 512)
packed into every row with a reset mask).  Inputs are resident in HBM before the
timed region.  Prints ONE JSON line:

  value        tokens/s over the K timed steps (wall clock, synchronised on both sides)
  roofline     the persistent sequence kernel against the HBM roofline: algorithmic
               bytes per launch / average launch duration (HIP events on the launch stream)
  cpu_baseline the vanilla-structured PyTorch CPU port (oracle/vanilla_port.py) timed on
               a bounded slice of the same workload on this box's host cores
  decode       BASELINE config 3: us per single-token step at B=256, D=2048 (8 heads),
               1024 consecutive steps after a 128-token prefill, state carried on device
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "sLSTM fwd tokens/s @ D=1024 packed B16×T2048; decode step µs @ B=256"
HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA rate
CONFIG5_NAME = "config 5: B=64 T=4096 D=4096 NH=4 bf16, no resets"


def algorithmic_bytes(B, T, NH, dh, wx_bytes, h_bytes, r_bytes, with_mask=True):
    """One read of W.x, one write of h, the reset mask, one read of R and bias, the final state."""
    H = NH * dh
    return (B * T * 4 * H * wx_bytes + B * T * H * h_bytes + (B * T if with_mask else 0)
            + NH * 4 * dh * dh * r_bytes + 4 * H * 4 + 4 * B * H * 4)


def make_inputs(B, T, NH, dh, mean_doc, device, seed=0):
    import numpy as np
    import torch

    from tests._util import geometric_reset_mask

    g = torch.Generator().manual_seed(seed)
    H = NH * dh
    wx = torch.randn(B, T, 4 * H, generator=g).bfloat16()
    r_ext = (torch.rand(NH, dh, 4, dh, generator=g) * 2 - 1) / float(np.sqrt(H))  # "standard" init
    bias = torch.zeros(NH, 4, dh)
    bias[:, 1] = torch.linspace(3.0, 6.0, dh)  # "small_init"
    mask = torch.from_numpy(geometric_reset_mask(seed, B, T, mean_doc)) if mean_doc else None
    return wx, r_ext, bias, mask


def cpu_baseline(wx, r_ext, bias, mask, budget_s=15.0):
    """Times the vanilla-structured CPU port on the first T_s steps of the same batch."""
    import torch

    from oracle import vanilla_port as vp

    B, T = wx.shape[0], wx.shape[1]
    cores = os.cpu_count() or 1
    cores = min(cores, 16)  # the GPU box gives one job 16 cores' worth of CPU
    torch.set_num_threads(cores)
    wx32 = wx.float()
    probe = 32
    t0 = time.perf_counter()
    vp.slstm_forward(wx32[:, :probe], r_ext, bias, None, mask[:, :probe] if mask is not None else None)
    per_step = (time.perf_counter() - t0) / probe
    Ts = int(max(64, min(T, budget_s / max(per_step, 1e-6))))
    runs = []
    while (sum(runs) < 10.0 and len(runs) < 40) or len(runs) < 2:  # 10-30 s of CPU work in total, whatever the host's speed
        t0 = time.perf_counter()
        vp.slstm_forward(wx32[:, :Ts], r_ext, bias, None, mask[:, :Ts] if mask is not None else None)
        runs.append(time.perf_counter() - t0)
    dt = sorted(runs)[len(runs) // 2]
    return {
        "value": B * Ts / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"first {Ts} of {T} steps of the same packed batch (B={B}), fp32, torch {torch.__version__} CPU, "
                  f"median of {len(runs)} runs of {dt:.1f} s after a {probe}-step warm-up",
    }


def bench_decode(device, steps=1024, prefill=128):
    """BASELINE config 3: B=256, D=2048 (8 heads x 256), bf16 W.x, state carried on device."""
    import torch

    from xlstm_amd import functional as F

    B, NH, dh = 256, 8, 256
    H = NH * dh
    wx_pre, r_ext, bias, _ = make_inputs(B, prefill, NH, dh, 0, device, seed=1)
    r = r_ext.permute(0, 2, 3, 1).reshape(NH, 4 * dh, dh).contiguous().to(device).bfloat16()  # bf16 R for decode
    bias = bias.to(device)
    g = torch.Generator().manual_seed(2)
    wx_dec = torch.randn(steps, B, 1, 4 * H, generator=g).bfloat16().to(device)  # pre-generated, RNG not timed
    ws = F.workspace_for(B, prefill, NH, dh, device)
    _, state = F.slstm_forward(wx_pre.to(device), r, bias, None, None, workspace=ws)
    h1 = torch.empty(1, B, H, dtype=torch.bfloat16, device=device)
    h2 = [torch.empty(1, B, H, dtype=torch.bfloat16, device=device) for _ in range(2)]  # h ping-pong: h of step t is the
    s_a, s_b = state.clone(), torch.empty_like(state)  # bf16 operand of step t+1.  State ping-pong: s_out must not alias s0
    for t in range(16):  # warm-up
        F.slstm_forward(wx_dec[t], r, bias, s_a, None, step=True, workspace=ws, h_out=h1, s_out=s_b)
        s_a, s_b = s_b, s_a
    s_a.copy_(state)
    torch.cuda.synchronize()
    # eager loop: one xs_slstm_step call per token from Python through a StepPlan (arguments validated once)
    plan = F.StepPlan(B, r, bias, wx_dtype=torch.bfloat16, workspace=ws)
    stream = torch.cuda.current_stream().cuda_stream
    # (three passes over the same 1024 steps from the same state, the median pass is reported: one pass is at the mercy
    # of whatever else the box does in those 7 ms)
    walls, gpus = [], []
    for rep in range(3):
        s_a.copy_(state)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for t in range(steps):
            plan(wx_dec[t], s_a, s_b, h2[t & 1], stream, h2[(t + 1) & 1] if t else None)
            s_a, s_b = s_b, s_a
        e1.record()
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
        gpus.append(e0.elapsed_time(e1) * 1e3 / steps)
    wall = sorted(walls)[1]
    gpu_us = sorted(gpus)[1]
    nbytes = algorithmic_bytes(B, 1, NH, dh, 2, 2, 2, with_mask=False) + 4 * B * H * 4  # state is read AND written
    eager_state = s_a.clone()

    # The same steps replayed from a HIP graph (64 step launches per graph, no host work between them):
    # what a serving loop that captures its decode step sees.  Every replay is checked against the eager run.
    per_graph = 64
    graph_us, graph_ok = None, None
    if steps % per_graph == 0:
        g_a, g_b = state.clone(), torch.empty_like(state)
        wx_g = torch.empty(per_graph, B, 1, 4 * H, dtype=wx_dec.dtype, device=device)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            def chain():
                a, b = g_a, g_b
                for t in range(per_graph):  # an even count: the state ends in g_a again
                    F.slstm_forward(wx_g[t], r, bias, a, None, step=True, workspace=ws, h_out=h2[t & 1], s_out=b,
                                    h_prev=h2[(t + 1) & 1] if t else None)
                    a, b = b, a
            chain()  # warm-up outside the capture
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                chain()
        torch.cuda.synchronize()
        g_a.copy_(state)
        g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        total = 0.0
        for rep in range(steps // per_graph):
            wx_g.copy_(wx_dec[rep * per_graph:(rep + 1) * per_graph])
            g0.record()
            graph.replay()
            g1.record()
            torch.cuda.synchronize()
            total += g0.elapsed_time(g1)
        graph_us = total * 1e3 / steps
        graph_ok = bool(torch.equal(g_a, eager_state))
    best_us = min(gpu_us, graph_us) if graph_us else gpu_us
    traffic = None
    traffic_file = os.path.join(ROOT, "profiles", "traffic_step_cfg3.json")
    if os.path.exists(traffic_file):
        traffic = json.load(open(traffic_file)).get("hbm_bytes_per_launch")
    return {
        "workload": f"decode B={B} D={H} NH={NH}, {steps} consecutive T=1 steps after a {prefill}-token prefill",
        "us_per_step": wall * 1e6 / steps, "gpu_us_per_step": gpu_us, "gpu_us_per_step_passes": gpus,
        "graph_us_per_step": graph_us,
        "graph_equals_eager": graph_ok, "steps": steps,
        "finite": bool(torch.isfinite(s_a).all()),
        "roofline": {"bound": "hbm", "achieved": nbytes / (best_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": nbytes / (best_us * 1e-6) / 1e9 / HBM_PEAK_GBS, "traffic": traffic,
                     "kernel": "slstm_step_pipe_kernel<NK=8>", "algorithmic_bytes_per_launch": nbytes,
                     "traffic_source": "profiles/traffic_step_cfg3.json (rocprofv3 counters of a separate run, not of this one)"},
    }


def measure_stage(device, stage, steps, members=16, two_xcds=0, rows=4, reps=5):
    """Median time (us) of one call of ``xs_measure_stage`` with ``steps`` iterations, by HIP events on the stream the
    kernel is launched on; ``None`` if one of its bounded waits ran out."""
    import ctypes

    import numpy as np
    import torch

    from xlstm_amd import _lib

    lib = _lib.load()
    ws = torch.zeros(256 + 32 * 8 * 16 * 512, dtype=torch.uint8, device=device)
    a = _lib.MeasureArgs()
    a.stage, a.members, a.two_xcds, a.rows, a.steps = stage, members, two_xcds, rows, steps
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.stream = torch.cuda.current_stream(device).cuda_stream
    times = []
    for i in range(reps + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        rc = lib.xs_measure_stage(ctypes.byref(a))
        e1.record()
        torch.cuda.synchronize()
        if rc != 0:
            raise RuntimeError(f"xs_measure_stage failed ({rc}): {_lib.last_error()}")
        if stage in (_lib.STAGE_EXCHANGE, _lib.STAGE_CHAIN) and int(ws[:4].view(torch.int32)[0]):
            return None
        if i:
            times.append(e0.elapsed_time(e1) * 1e3)
    return float(np.median(times))


def serial_bound(device):
    """The dependency chain of one timestep, measured by ``xs_measure_stage`` (the product kernel's instructions, layouts
    and exchange protocol; every iteration needs the result of the one before).  ``config2_chain``: the whole chain as
    one loop - barrier, poll, MFMAs, fold and row shifts, gating, publication - on 16 head groups of 16 compute
    units, with none of the product kernel's other work: the serial bound of a step of this structure.  The stages alone
    (each its own loop, so their sum is more than the chain: every loop pays its own entry and waits) say where it
    goes.  Per-iteration times are differences between two step counts, so launches and set-up cancel.  Also the floor
    of a dependent launch (the decode step's)."""
    from xlstm_amd import _lib

    def per_step(stage, n=20000, **kw):
        lo, hi = measure_stage(device, stage, n, **kw), measure_stage(device, stage, 3 * n, **kw)
        return None if lo is None or hi is None else (hi - lo) / (2 * n)

    chain = per_step(_lib.STAGE_CHAIN, rows=4)
    ex16 = per_step(_lib.STAGE_EXCHANGE, members=16, rows=4)
    mm = per_step(_lib.STAGE_CONTRACTION)
    ga = per_step(_lib.STAGE_GATING)
    ex64 = per_step(_lib.STAGE_EXCHANGE, n=5000, members=64, two_xcds=1, rows=16)
    ex32 = per_step(_lib.STAGE_EXCHANGE, n=5000, members=32, rows=16)
    launch = per_step(_lib.STAGE_LAUNCH, n=2000)
    return {"config2_chain_us_per_step": chain,
            "stages_alone_us": {"exchange_16_units_one_xcd_4_rows": ex16, "mfma_fold_and_row_shifts": mm, "gating": ga},
            "exchange_32_units_one_xcd_16_rows_us": ex32, "exchange_64_units_two_xcds_16_rows_us": ex64,
            "dependent_launch_us": launch}


def bench_backward(device, iters=3):
    """The backward pass at BASELINE config 2 (B=16, T=2048, D=1024, NH=4, bf16, packed documents): the whole call
    and the engine's three kernels by HIP events."""
    import numpy as np
    import torch

    from tests._util import geometric_reset_mask
    from xlstm_amd import functional as F

    B, T, NH, dh = 16, 2048, 4, 256
    H = NH * dh
    torch.manual_seed(0)
    wx = torch.randn(B, T, 4 * H, device=device).bfloat16()
    r = (torch.rand(NH, 4 * dh, dh, device=device) * 2 - 1) / np.sqrt(H)
    bias = torch.zeros(NH, 4, dh, device=device)
    bias[:, 1] = torch.linspace(3, 6, dh, device=device)
    mask = torch.from_numpy(geometric_reset_mask(0, B, T, 512)).to(device)
    h, _ = F.slstm_forward(wx, r, bias, None, mask)
    d_h = torch.randn(T, B, H, device=device).bfloat16()
    total, prep, rev, par = [], [], [], []
    for i in range(iters + 1):
        tm = {}
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = F.slstm_backward(wx, r, bias, None, mask, h, d_h, timings=tm)
        torch.cuda.synchronize()
        if i:
            total.append((time.perf_counter() - t0) * 1e3)
            ev = tm["events"]
            prep.append(ev[0].elapsed_time(ev[1]))
            rev.append(ev[1].elapsed_time(ev[2]))
            par.append(ev[2].elapsed_time(ev[3]))
    rev_ms = float(np.median(rev))
    # the same with a training forward that leaves the coefficients (no forward walk in the backward call)
    keep = {}
    coef = F.backward_coefficients_buffer(wx, NH)
    if coef is not None:
        fwd_plain, fwd_keep, tot_keep, tot_cell = [], [], [], []
        for i in range(iters + 1):
            e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
            e[0].record()
            F.slstm_forward(wx, r, bias, None, mask)
            e[1].record()
            F.slstm_forward(wx, r, bias, None, mask, coef_out=coef)
            e[2].record()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out2 = F.slstm_backward(wx, r, bias, None, mask, h, d_h, coef=coef)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            # ... and with the gate deltas returned in the input's type, as sLSTMCell_hip asks for them
            out3 = F.slstm_backward(wx, r, bias, None, mask, h, d_h, coef=coef, d_wx_dtype=torch.bfloat16)
            torch.cuda.synchronize()
            if i:
                tot_cell.append((time.perf_counter() - t1) * 1e3)
                tot_keep.append((t1 - t0) * 1e3)
                fwd_plain.append(e[0].elapsed_time(e[1]))
                fwd_keep.append(e[1].elapsed_time(e[2]))
        keep = {"with_forward_coefficients": {
            "backward_ms": float(np.median(tot_keep)), "forward_ms": float(np.median(fwd_keep)),
            "plain_forward_ms": float(np.median(fwd_plain)),
            "backward_ms_with_bf16_gate_deltas": float(np.median(tot_cell)),
            "bf16_gate_deltas_are_the_float32_ones_rounded": bool(torch.equal(out3[0], out2[0].bfloat16())),
            "same_gradients": bool(torch.allclose(out2[0], out[0], rtol=0, atol=2e-3 * float(out[0].abs().max())))}}
    # what the reverse kernel has to move per step and element: nine coefficients and the four gate deltas in float32,
    # the output gradient in bf16; R transposed once (the gate deltas that the compute units of a head exchange stay in the L2)
    nbytes = (9 * 4 + 4 * 4 + 2) * B * T * H + NH * 4 * dh * dh * 2
    traffic = None
    traffic_file = os.path.join(ROOT, "profiles", "traffic_bwd_cfg2.json")
    if os.path.exists(traffic_file):
        traffic = json.load(open(traffic_file)).get("hbm_bytes_per_launch")
    return {"workload": "backward pass at config 2: B=16 T=2048 D=1024 NH=4 bf16, documents mean 512",
            "ms": float(np.median(total)), "prepare_kernel_ms": float(np.median(prep)), "reverse_kernel_ms": rev_ms,
            "parameter_gradient_kernel_ms": float(np.median(par)),
            "tokens_per_s": B * T / (float(np.median(total)) * 1e-3), "finite": bool(torch.isfinite(out[0]).all()), **keep,
            "roofline": {"bound": "hbm", "achieved": nbytes / (rev_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": nbytes / (rev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": traffic,
                         "kernel": "slstm_bwd_quad_kernel<S=4>", "algorithmic_bytes_per_launch": nbytes,
                         "traffic_source": "profiles/traffic_bwd_cfg2.json (rocprofv3 counters of a separate run, not of this one)"}}


def bench_backward_large(device, T=4096, iters=2):
    """The backward pass at BASELINE config 5's shape (B=64, 4 heads of 1024, bf16): the kernels of one launch per step
    (``split == 3`` of the C ABI), the whole call and its three parts by HIP events.  Per step the walk and the reverse
    pass each read R once (32 MiB: it does not stay in any cache level below the Infinity Cache) and the operand rows
    once per tile of 32 units; the roofline line prices those bytes of the reverse kernel against the HBM peak."""
    import numpy as np
    import torch

    from xlstm_amd import functional as F

    B, NH, dh = 64, 4, 1024
    H = NH * dh
    g = torch.Generator(device=device).manual_seed(11)
    wx = torch.empty(B, T, 4 * H, dtype=torch.bfloat16, device=device)
    for row in range(B):
        wx[row] = torch.randn(T, 4 * H, generator=g, device=device).bfloat16()
    r = (torch.rand(NH, 4 * dh, dh, generator=g, device=device) * 2 - 1) / float(np.sqrt(H))
    bias = torch.zeros(NH, 4, dh, device=device)
    bias[:, 1] = torch.linspace(3.0, 6.0, dh, device=device)
    h, _ = F.slstm_forward(wx, r, bias)
    d_h = torch.empty(T, B, H, dtype=torch.bfloat16, device=device)
    for t0 in range(0, T, 256):
        d_h[t0:t0 + 256] = torch.randn(min(256, T - t0), B, H, generator=g, device=device).bfloat16()
    total, prep, rev, par = [], [], [], []
    for i in range(iters + 1):
        tm = {}
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = F.slstm_backward(wx, r, bias, None, None, h, d_h, timings=tm)
        torch.cuda.synchronize()
        if i:
            total.append((time.perf_counter() - t0) * 1e3)
            ev = tm["events"]
            prep.append(ev[0].elapsed_time(ev[1]))
            rev.append(ev[1].elapsed_time(ev[2]))
            par.append(ev[2].elapsed_time(ev[3]))
        finite = bool(torch.isfinite(out[0][:, -1]).all() and torch.isfinite(out[3]).all())
        del out
    rev_ms = float(np.median(rev))
    # a launch of the reverse kernel: R transposed once, nine coefficients in and four gate deltas out per element in
    # float32, the deltas in bf16 out and (the step behind's) in, d_h in bf16, the gradients of c and n in and out
    nbytes = NH * 4 * dh * dh * 2 + (9 * 4 + 4 * 4 + 2 + 2 + 2 + 4 * 4) * B * H
    return {"workload": "backward pass at config 5's shape: B=64 T=%d D=4096 NH=4 bf16, one launch per step" % T,
            "ms": float(np.median(total)), "forward_walk_ms": float(np.median(prep)), "reverse_ms": rev_ms,
            "parameter_gradient_kernel_ms": float(np.median(par)),
            "us_per_step": {"forward_walk": float(np.median(prep)) * 1e3 / T, "reverse": rev_ms * 1e3 / (T + 1)},
            "finite": finite,
            "roofline": {"bound": "hbm", "achieved": nbytes / (rev_ms / (T + 1) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": nbytes / (rev_ms / (T + 1) * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                         "kernel": "slstm_bwd_step_kernel<bf16>", "algorithmic_bytes_per_launch": nbytes}}


def bench_decode_other_head_dims(device, steps=300):
    """Decode steps at the head dims that `slstm_step_feed_kernel` takes (beyond 256 in bf16): eager launches back to
    back through a `StepPlan` with the previous step's h handed on, us per step; `r_tiled_off` the same plan without R
    in slabs (the tile kernel that reads R as it lies)."""
    import numpy as np
    import torch

    from xlstm_amd import functional as F

    rows = []
    for B, NH, dh in ((256, 4, 512), (64, 4, 1024)):
        H = NH * dh
        g = torch.Generator(device=device).manual_seed(5)
        r = ((torch.rand(NH, 4 * dh, dh, generator=g, device=device) * 2 - 1) / float(np.sqrt(H))).bfloat16()
        bias = torch.zeros(NH, 4, dh, device=device)
        bias[:, 1] = torch.linspace(3.0, 6.0, dh, device=device)
        wx = torch.randn(B, 1, 4 * H, generator=g, device=device).bfloat16()
        row = {"workload": "decode step B=%d NH=%d dh=%d bf16" % (B, NH, dh)}
        for key in ("us_per_step", "r_tiled_off_us_per_step"):
            plan = F.StepPlan(B, r, bias, wx_dtype=torch.bfloat16)
            if key != "us_per_step":
                plan._args.r_tiled = None
            s = [torch.zeros(4, B, H, device=device), torch.zeros(4, B, H, device=device)]
            s[0][1:3] = 0.1
            h = [torch.zeros(B, H, device=device, dtype=torch.bfloat16) for _ in range(2)]
            for i in range(20):
                plan(wx, s[i & 1], s[(i + 1) & 1], h[(i + 1) & 1], h_prev=h[i & 1])
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(steps):
                plan(wx, s[i & 1], s[(i + 1) & 1], h[(i + 1) & 1], h_prev=h[i & 1])
            e1.record()
            torch.cuda.synchronize()
            row[key] = e0.elapsed_time(e1) * 1e3 / steps
            row["finite"] = bool(torch.isfinite(s[steps & 1]).all())
        nbytes = NH * 4 * dh * dh * 2 + B * H * (4 * 2 + 7 * 4 + 2 + 2)  # R, W.x, state in (c, n, m) and out, h in and out
        row["roofline"] = {"bound": "hbm", "achieved": nbytes / row["us_per_step"] / 1e3, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": nbytes / row["us_per_step"] / 1e3 / HBM_PEAK_GBS, "kernel": "slstm_step_feed_kernel<bf16>",
                           "algorithmic_bytes_per_launch": nbytes}
        rows.append(row)
    return rows


def bench_config(device, name, B, T, NH, dh, bf16, mean_doc, iters=5):
    """Times one forward call of the cell at another BASELINE shape (median of `iters`)."""
    import numpy as np
    import torch

    from tests._util import geometric_reset_mask
    from xlstm_amd import functional as F

    H = NH * dh
    g = torch.Generator(device=device).manual_seed(7)
    wx = torch.empty(B, T, 4 * H, dtype=torch.bfloat16 if bf16 else torch.float32, device=device)
    for row in range(B):
        wx[row] = torch.randn(T, 4 * H, generator=g, device=device).to(wx.dtype)
    r = ((torch.rand(NH, 4 * dh, dh, generator=g, device=device) * 2 - 1) / float(np.sqrt(H)))
    bias = torch.zeros(NH, 4, dh, device=device)
    bias[:, 1] = torch.linspace(3.0, 6.0, dh, device=device)
    mask = torch.from_numpy(geometric_reset_mask(7, B, T, mean_doc)).to(device) if mean_doc else None
    ws = F.workspace_for(B, T, NH, dh, device)
    h = torch.empty(T, B, H, dtype=wx.dtype, device=device)
    s = torch.empty(4, B, H, dtype=torch.float32, device=device)
    times = []
    for i in range(iters + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        F.slstm_forward(wx, r, bias, None, mask, workspace=ws, h_out=h, s_out=s)
        e1.record()
        torch.cuda.synchronize()
        if i:
            times.append(e0.elapsed_time(e1))
    ms = float(np.median(times))
    esz = 2 if bf16 else 4
    nbytes = algorithmic_bytes(B, T, NH, dh, esz, esz, 4, with_mask=bool(mean_doc))
    flops = 8.0 * B * T * H * dh
    return {"workload": name, "ms": ms, "us_per_timestep": ms * 1e3 / T, "tokens_per_s": B * T / ms * 1e3,
            "hbm_GBs": nbytes / ms / 1e6, "tflops": flops / ms / 1e9,
            "aborted": F.read_status(ws)["aborted"]}


def bench_small_batch(device, T=1024):
    """The sequence kernel at the batch sizes where an MFMA row tile is mostly padding: B = 1, 2, 4 at head dims 128
    and 256 (4 heads), bf16 and fp32, plus the reference test's shape (B 1, 4 heads of 16, one step:
    tests/test_slstm_cell_vanilla_vs_cuda.py:12-40).  Run once with the shipped library (MFMA contraction) and once
    with a library built with -DXS_SMALL_BATCH_FMA (XLSTM_AMD_LIB=...) to compare the two contractions."""
    rows = []
    for bf16 in (True, False):
        for dh in (128, 256):
            if not bf16 and dh == 256:
                continue  # (a float32 head of 256 is not a whole K range of the small variants)
            for B in (1, 2, 4):
                r = bench_config(device, f"B={B} T={T} NH=4 dh={dh} {'bf16' if bf16 else 'fp32'}", B, T, 4, dh, bf16, 0, iters=5)
                rows.append({k: r[k] for k in ("workload", "ms", "us_per_timestep", "aborted")})
    r = bench_config(device, "reference test shape: B=1 T=1 NH=4 dh=16 fp32 (one step)", 1, 1, 4, 16, False, 0, iters=20)
    rows.append({"workload": r["workload"], "us_per_call": r["ms"] * 1e3})
    return {"library": os.environ.get("XLSTM_AMD_LIB", "xlstm_amd/lib/libxlstm_amd.so"), "rows": rows}


PROFILE_LIB = os.path.join(ROOT, "xlstm_amd", "lib", "libxlstm_amd_profile.so")


def phase_profile(device):
    """Per-phase cycle table of the sequence kernels, from the cycle stamps of the measurement build of the library
    (``-DXS_PROFILE``: every wave of workgroup 0 sums the cycles between fixed points of its loop).  The stamps cost
    time themselves (a step of config 2 takes about a quarter longer than in the product build), so the table says where
    a step's time goes, not how long a step takes."""
    import torch

    from xlstm_amd import functional as F

    def run(B, T, NH, dh, mean_doc):
        H = NH * dh
        wx_c, r_ext_c, bias_c, mask_c = make_inputs(B, T, NH, dh, mean_doc, torch.device("cpu"))
        wx = wx_c.to(device)
        r = r_ext_c.permute(0, 2, 3, 1).reshape(NH, 4 * dh, dh).contiguous().to(device)
        bias = bias_c.to(device)
        mask = mask_c.to(device) if mean_doc else None
        ws = F.workspace_for(B, T, NH, dh, device)
        h = torch.empty(T, B, H, dtype=torch.bfloat16, device=device)
        s = torch.empty(4, B, H, dtype=torch.float32, device=device)
        ms = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            F.slstm_forward(wx, r, bias, None, mask, workspace=ws, h_out=h, s_out=s)
            e1.record()
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1))
        if F.read_status(ws)["aborted"]:
            sys.exit("bench.py: the engine flagged the run as aborted")
        return F.read_phase_stamps(ws).double(), sorted(ms)[1]

    out = {}
    # config 2: slstm_seq_kernel, one row tile of 4 rows; per timestep
    T = 2048
    st, ms = run(16, T, 4, 256, 512)
    names = {5: "loop top", 2: "barrier", 1: "W.x and flags out of LDS + s_sleep", 0: "poll (request to complete operand)",
             7: "8 MFMAs + fold + row shifts", 3: "exponential gating", 4: "publish + re-arm + stage h"}
    out["config 2 (slstm_seq_kernel<bf16,NCH=2,MT=1,FULL,QUAD>), cycles per timestep, workgroup 0"] = {
        "ms_per_call_with_stamps": ms,
        "compute waves 0-3": {n: [round(float(st[w][i] / T)) for w in range(4)] for i, n in names.items()},
        "compute waves: sum": [round(float((st[w][:6].sum() + st[w][7]) / T)) for w in range(4)],
        "compute waves: polls repeated per step": [round(float(st[w][6] / T), 2) for w in range(4)],
        "feeder wave": {"W.x into LDS": round(float(st[4][0] / T)), "issue": round(float(st[4][1] / T)),
                        "barrier": round(float(st[4][2] / T))},
        "drainer wave": {"h to HBM": round(float(st[5][0] / T)), "barrier": round(float(st[5][1] / T))},
    }
    # config 5 at a quarter of its length and config 3's prefill: slstm_seq_roles_kernel; per tile iteration (4 per step)
    for label, (B, T, NH, dh) in (("config 5, T = 1024 (slstm_seq_roles_kernel<bf16,NCH=8,FULL>)", (64, 1024, 4, 1024)),
                                  ("config 3 prefill, T = 128 (slstm_seq_roles_kernel<bf16,NCH=2,FULL>)", (256, 128, 8, 256))):
        st, ms = run(B, T, NH, dh, 0)
        n = 4.0 * T
        mnames = ["loop top", "wait for the operand tile", "request next tile + arrival test", "mfma", "partial sums to LDS", "barrier"]
        out[label + ", cycles per tile iteration, workgroup 0"] = {
            "ms_per_call_with_stamps": ms,
            "MFMA waves 0-3": {nm: [round(float(st[w][i] / n)) for w in range(4)] for i, nm in enumerate(mnames)},
            "MFMA waves: sum": [round(float(st[w][:6].sum() / n)) for w in range(4)],
            "gating wave 4": {"barrier": round(float(st[5][0] / n)), "partial sums out of LDS + sums": round(float(st[5][4] / n)),
                              "gating": round(float(st[5][5] / n)), "3 stores": round(float(st[5][2] / n)),
                              "fetch of W.x D iterations ahead + loop top + wait for this iteration's W.x":
                                  round(float(st[5][1] / n)),
                              "W.x through the LDS corner": round(float(st[5][3] / n)),
                              "sum": round(float(st[5][:6].sum() / n))},
        }
    out["backward, config 2 (slstm_bwd_quad_kernel<S=4>), cycles since the step's barrier, first workgroup"] = backward_phase_profile(device)
    return out


def backward_phase_profile(device):
    """When three waves of the reverse kernel's first workgroup pass fixed points of a timestep, in cycles since they left
    the step's barrier (the measurement build leaves the sums in the m plane of ``d_s0``, which is zero otherwise)."""
    import torch

    from xlstm_amd import functional as F

    B, T, NH, dh = 16, 2048, 4, 256
    H = NH * dh
    wx_c, r_ext_c, bias_c, mask_c = make_inputs(B, T, NH, dh, 512, torch.device("cpu"))
    wx = wx_c.to(device)
    r = r_ext_c.permute(0, 2, 3, 1).reshape(NH, 4 * dh, dh).contiguous().to(device)
    bias, mask = bias_c.to(device), mask_c.to(device)
    h, _ = F.slstm_forward(wx, r, bias, None, mask)
    d_h = torch.randn(T, B, H, device=device).bfloat16()
    ms = []
    for _ in range(3):
        tm = {}
        out = F.slstm_backward(wx, r, bias, None, mask, h, d_h, timings=tm)
        torch.cuda.synchronize()
        ms.append(tm["events"][1].elapsed_time(tm["events"][2]))
    words = out[3][3].reshape(-1)[:60].view(torch.int64).cpu().double()
    st, fd = words[:24].view(3, 8) / T, words[24:30]
    points = ["partial results added up", "deltas published", "first look issued at the earliest", "deltas complete",
              "partial tile written", "barrier left (= the step)"]
    res = {"reverse_kernel_ms_with_stamps": sorted(ms)[1]}
    for w, row in zip(("wave 0 (forms the gradient; polls its own workgroup)", "wave 4 (polls its own workgroup)",
                       "wave 6 (polls another workgroup)"), st):
        res[w] = {n: round(float(v)) for n, v in zip(points, row[:6])}
        res[w]["looks repeated per step"] = round(float(row[6]), 2)
        res[w]["the look that found them issued"] = round(float(row[7]))
    res["feeder wave 0"] = {"a request, issue to landed (sampled)": round(float(fd[0] / max(1.0, float(fd[1])))),
                            "its request goes out (every fourth step)": round(float(fd[2] / (T / 4))),
                            "its wait is over, per step": round(float(fd[4] / T)), "step": round(float(fd[5] / T))}
    return res


def bench_config4(device, iters=3):
    """BASELINE config 4: 24 blocks (sLSTM at 3, 11, 19), D=1024, 4 heads, vocab 50304, bf16, B=8, T=2048,
    packed documents of mean length 768.  Only the sLSTM cells run on the HIP engine."""
    import numpy as np
    import torch

    from tests._util import geometric_reset_mask
    from xlstm_amd.lm_harness import HarnessConfig, xLSTMLMHarness

    torch.manual_seed(4)
    B, T = 8, 2048
    model = xLSTMLMHarness(HarnessConfig()).to(device).bfloat16().eval()
    idx = torch.randint(0, 50304, (B, T), device=device)
    mask = torch.from_numpy(geometric_reset_mask(4, B, T, 768)).to(device)
    total, cells, layers = [], [], []
    with torch.no_grad():
        for i in range(iters + 1):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            logits = model(idx, reset_mask=mask, time_cells=True)
            e1.record()
            torch.cuda.synchronize()
            if i:
                total.append(e0.elapsed_time(e1))
                cells.append(list(model.cell_ms))
                layers.append(list(model.layer_ms))
    cell_ms = np.median(np.array(cells), axis=0)
    layer_ms = np.median(np.array(layers), axis=0)
    return {"workload": "config 4: 24-block xLSTM LM harness, sLSTM layers at blocks 3/11/19 on HIP (conv, gate projections, "
                        "cell, group norm), rest PyTorch-ROCm, "
                        "B=8 T=2048 D=1024 NH=4 bf16, documents mean 768",
            "forward_ms": float(np.median(total)), "slstm_cell_ms": [float(c) for c in cell_ms],
            "slstm_layer_ms": [float(c) for c in layer_ms], "cell_share_of_slstm_layer": float(cell_ms.sum() / layer_ms.sum()),
            "slstm_cells_share": float(cell_ms.sum() / np.median(total)),
            "slstm_tokens_per_s_per_cell": float(B * T / cell_ms.mean() * 1e3),
            "finite": bool(torch.isfinite(logits.float()).all())}


def bench_layer(device, iters=10, decode_steps=512):
    """The caller of the path: one sLSTM layer (conv + SiLU, gate projections, cell, group norm) at the layer shape of
    BASELINE config 4 (B=8, T=2048, D=1024, NH=4, bf16, documents of mean length 768), once with the engine's kernels
    around the cell and once with the PyTorch ops they replace; and one decode step of the layer at the shape of
    config 3 (B=256, D=2048, NH=8) replayed from HIP graphs."""
    import numpy as np
    import torch

    from tests._util import geometric_reset_mask
    from xlstm_amd.decode import GraphedLayerDecoder
    from xlstm_amd.layer import sLSTMLayer, sLSTMLayerConfig

    def timed(fn, n):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    torch.manual_seed(0)
    out = {}
    B, T, D, NH = 8, 2048, 1024, 4
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=D, num_heads=NH, backend="hip", recurrent_weight_init="standard"))
    layer = layer.to(device).bfloat16().eval()
    x = torch.randn(B, T, D, device=device).bfloat16()
    mask = torch.from_numpy(geometric_reset_mask(4, B, T, 768)).to(device)
    with torch.no_grad():
        res = {}
        for name, fused in (("engine_ops", True), ("torch_ops", False)):
            layer.fused_pre_ops = fused
            res[name] = layer(x, reset_mask=mask).float()
            out["forward_ms_" + name] = timed(lambda: layer(x, reset_mask=mask), iters)
        layer.fused_pre_ops = True
        wx = layer._gates(x, x)
        out["cell_ms"] = timed(lambda: layer.slstm_cell(wx, reset_mask=mask), iters)
        out["max_abs_difference_between_the_two"] = float((res["engine_ops"] - res["torch_ops"]).abs().max())
    out["forward_workload"] = "one sLSTM layer, B=8 T=2048 D=1024 NH=4 bf16, documents mean 768"
    if decode_steps <= 0:
        return out

    B, D, NH = 256, 2048, 8
    layer = sLSTMLayer(sLSTMLayerConfig(embedding_dim=D, num_heads=NH, backend="hip", recurrent_weight_init="standard"))
    layer = layer.to(device).bfloat16().eval()
    layer.slstm_cell.keep_state_fp32 = True
    xs = torch.randn(B, 64, D, device=device).bfloat16()
    with torch.no_grad():
        for name, fused in (("engine_ops", True), ("torch_ops", False)):
            layer.fused_pre_ops = fused
            dec = GraphedLayerDecoder(layer, B)
            for t in range(8):
                dec.step(xs[:, t:t + 1])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for t in range(decode_steps):
                dec.step(xs[:, t % 64:t % 64 + 1])
            torch.cuda.synchronize()
            out["decode_step_us_graphed_" + name] = (time.perf_counter() - t0) / decode_steps * 1e6
            out["decode_finite"] = bool(torch.isfinite(dec.out.float()).all())
            if fused:  # the token already in the decoder's input buffer (written there by its producer): no copy kernel
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for t in range(decode_steps):
                    dec.step()
                torch.cuda.synchronize()
                out["decode_step_us_graphed_engine_ops_input_in_place"] = (time.perf_counter() - t0) / decode_steps * 1e6
    out["decode_workload"] = "one sLSTM layer decode step, B=256 D=2048 NH=8 bf16, two alternating HIP graphs"
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode leg (profiling runs)")
    ap.add_argument("--decode-only", action="store_true", help="only run the decode leg (profiling runs)")
    ap.add_argument("--all-configs", action="store_true",
                    help="also time the cell at BASELINE configs 1, 4 and 5 (adds an 'all_configs' object)")
    ap.add_argument("--config4", action="store_true",
                    help="also run BASELINE config 4: the 24-block LM harness, timing its three sLSTM cells")
    ap.add_argument("--layer", action="store_true",
                    help="also time one sLSTM layer around the cell (adds a 'layer' object); --layer-only: nothing else")
    ap.add_argument("--layer-only", action="store_true")
    ap.add_argument("--layer-iters", type=int, default=10, help="timed forward calls of the layer leg")
    ap.add_argument("--layer-decode-steps", type=int, default=512,
                    help="graphed decode steps of the layer leg; 0 skips them (short counter runs)")
    ap.add_argument("--config5-only", action="store_true",
                    help="only time the cell at BASELINE config 5 (B=64 T=4096 D=4096 NH=4 bf16), the shape bound by "
                         "the bf16 MFMA roofline (profiling runs)")
    ap.add_argument("--small-batch-only", action="store_true",
                    help="only time the sequence kernel at B = 1, 2, 4 (head dims 128 and 256) and the reference test's shape")
    ap.add_argument("--backward-only", action="store_true",
                    help="only time the backward pass at config 2 (its own JSON line)")
    ap.add_argument("--backward-large-only", action="store_true",
                    help="only the backward pass at config 5's shape (4 heads of 1024: one launch per step)")
    ap.add_argument("--backward-large-steps", type=int, default=4096, help="sequence length of --backward-large-only")
    ap.add_argument("--phase-profile", action="store_true",
                    help="per-phase cycle tables of the sequence kernels from the measurement build of the library "
                         "(python -m xlstm_amd.build -DXS_PROFILE -o xlstm_amd/lib/libxlstm_amd_profile.so)")
    ap.add_argument("--serial-bound", action="store_true",
                    help="only measure the stages of a timestep's dependency chain and the launch floor (their own JSON line)")
    ap.add_argument("--headline-only", action="store_true",
                    help="leave out the other BASELINE configs, the backward pass and the serial bound (profiling runs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 1 GiB device copy 5 times (scales the rocprofv3 FETCH_SIZE/WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU; the path shards over batch rows / heads without "
                 "communication, and no multi-GPU figure is produced (run with --gpus 1)")

    if args.phase_profile:  # (before the package loads its library)
        if not os.path.exists(PROFILE_LIB):
            sys.exit(f"bench.py --phase-profile needs {PROFILE_LIB}: "
                     "python -m xlstm_amd.build -DXS_PROFILE -o xlstm_amd/lib/libxlstm_amd_profile.so")
        os.environ["XLSTM_AMD_LIB"] = PROFILE_LIB

    import torch

    from xlstm_amd import functional as F

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the hip backend has no CPU path)")
    device = torch.device("cuda:0")
    if args.phase_profile:
        print(json.dumps({"phase_profile": phase_profile(device)}, indent=1))
        return
    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device=device)  # 1 GiB read + 1 GiB written per copy
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_each_way": src.numel() * 4, "copies": 5}))
        return
    if args.serial_bound:
        print(json.dumps({"serial_bound": serial_bound(device)}))
        return
    if args.decode_only:
        dec = bench_decode(device)
        dec["other_head_dims"] = bench_decode_other_head_dims(device)
        print(json.dumps({"decode": dec}))
        return
    if args.small_batch_only:
        print(json.dumps({"small_batch": bench_small_batch(device)}))
        return
    if args.backward_only:
        print(json.dumps({"backward": bench_backward(device, iters=max(1, min(args.steps, 5)))}))
        return
    if args.backward_large_only:
        print(json.dumps({"backward_config5_shape": bench_backward_large(device, T=args.backward_large_steps,
                                                                           iters=max(1, min(args.steps, 3)))}))
        return
    if args.config5_only:
        c5 = bench_config(device, CONFIG5_NAME, 64, 4096, 4, 1024, True, 0, iters=max(1, min(args.steps, 5)))
        c5["roofline"] = {"bound": "mfma", "achieved": c5["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                          "frac": c5["tflops"] / MFMA_BF16_PEAK_TFLOPS, "traffic": None,
                          "kernel": "slstm_seq_roles_kernel<bf16,NCH=8,FULL>",
                          "algorithmic_flops_per_launch": 8.0 * 64 * 4096 * 4096 * 1024}
        print(json.dumps({"config5": c5}))
        return
    if args.layer_only:
        print(json.dumps({"layer": bench_layer(device, args.layer_iters, args.layer_decode_steps)}))
        return
    B, T, NH, dh = 16, 2048, 4, 256
    H = NH * dh
    wx_c, r_ext_c, bias_c, mask_c = make_inputs(B, T, NH, dh, 512, device)
    wx = wx_c.to(device)
    r = r_ext_c.permute(0, 2, 3, 1).reshape(NH, 4 * dh, dh).contiguous().to(device)  # fp32, K-contiguous
    bias = bias_c.to(device)
    mask = mask_c.to(device)
    ws = F.workspace_for(B, T, NH, dh, device)
    h = torch.empty(T, B, H, dtype=torch.bfloat16, device=device)
    s = torch.empty(4, B, H, dtype=torch.float32, device=device)

    def step():
        F.slstm_forward(wx, r, bias, None, mask, workspace=ws, h_out=h, s_out=s)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for e0, e1 in evs:
        e0.record()  # torch's current stream is the stream the kernel is launched on
        step()
        e1.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    status = F.read_status(ws)
    if status["aborted"]:
        sys.exit(f"bench.py: the engine flagged the run as aborted: {status}")
    kern_ms = sum(e0.elapsed_time(e1) for e0, e1 in evs) / args.steps
    nbytes = algorithmic_bytes(B, T, NH, dh, 2, 2, 4)
    achieved = nbytes / (kern_ms * 1e-3) / 1e9
    out = {
        "metric": METRIC,
        "value": B * T * args.steps / elapsed,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed * 1e3 / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "sLSTM cell forward, packed documents (geometric, mean 512) with reset mask, "
                               "B=16 T=2048 D=1024 NH=4, bf16 W.x/h, fp32 R and state (BASELINE configs[1])",
                   "tokens_per_step": B * T},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "slstm_seq_kernel<bf16,NCH=2,MT=1,FULL,BURST=0,FMAC=0,QUAD=1>", "kernel_ms": kern_ms,
                     "algorithmic_bytes_per_launch": nbytes, "us_per_timestep": kern_ms * 1e3 / T,
                     "max_poll_rounds": status["max_spins"],
                     "tflops": 8.0 * B * T * NH * dh * dh / (kern_ms * 1e-3) / 1e12},
    }
    traffic_file = os.path.join(ROOT, "profiles", "traffic_seq_cfg2.json")
    if os.path.exists(traffic_file):
        out["roofline"]["traffic"] = json.load(open(traffic_file)).get("hbm_bytes_per_launch")
        out["roofline"]["traffic_source"] = "profiles/traffic_seq_cfg2.json (rocprofv3 counters of a separate run, not of this one)"
    lean = args.headline_only or args.no_decode  # (profiling runs want the one kernel)
    if not lean:
        # the stages of the chain measured in this run, and what the measured step is against their sum
        sb = serial_bound(device)
        out["roofline"]["serial_bound_stages_us"] = sb
        if sb.get("config2_chain_us_per_step"):
            out["roofline"]["serial_bound_us_per_step"] = sb["config2_chain_us_per_step"]
            out["roofline"]["frac_of_serial_bound"] = sb["config2_chain_us_per_step"] / (kern_ms * 1e3 / T)
            out["roofline"]["serial_bound_source"] = ("measured in this run: xs_measure_stage(XS_STAGE_CHAIN), the step's "
                                                      "dependency chain alone on 16 head groups of 16 compute units")
        # the other BASELINE configurations and the backward pass, compact (full rows: --all-configs)
        c1 = bench_config(device, "config 1: B=4 T=256 D=512 NH=4 fp32, no resets", 4, 256, 4, 128, False, 0)
        c4 = bench_config(device, "config 4 (one sLSTM cell): B=8 T=2048 D=1024 NH=4 bf16, documents mean 768", 8, 2048, 4, 256, True, 768)
        c5 = bench_config(device, CONFIG5_NAME, 64, 4096, 4, 1024, True, 0, iters=3)
        bw = bench_backward(device)
        out["other_configs"] = [
            {"workload": c["workload"], "ms": c["ms"], "us_per_timestep": c["us_per_timestep"], "aborted": c["aborted"],
             "roofline": ({"bound": "mfma", "frac": c["tflops"] / MFMA_BF16_PEAK_TFLOPS, "achieved": c["tflops"], "unit": "TFLOP/s",
                           "peak": MFMA_BF16_PEAK_TFLOPS, "kernel": "slstm_seq_roles_kernel<bf16,NCH=8,FULL>"} if c is c5 else
                          {"bound": "hbm", "frac": c["hbm_GBs"] / HBM_PEAK_GBS, "achieved": c["hbm_GBs"], "unit": "GB/s",
                           "peak": HBM_PEAK_GBS})}
            for c in (c1, c4, c5)]
        out["backward"] = {k: bw[k] for k in ("workload", "ms", "finite") if k in bw}
        out["backward"]["kernels_ms"] = {k: v for k, v in bw.items() if k.endswith("_ms")}
        out["backward"]["roofline"] = bw["roofline"]
        if "with_forward_coefficients" in bw:
            out["backward"]["with_forward_coefficients"] = bw["with_forward_coefficients"]
        out["backward_config5_shape"] = bench_backward_large(device, iters=1)
    if args.all_configs:
        out["all_configs"] = [
            bench_config(device, "config 1: B=4 T=256 D=512 NH=4 fp32, no resets", 4, 256, 4, 128, False, 0),
            bench_config(device, "config 4 (one sLSTM cell): B=8 T=2048 D=1024 NH=4 bf16, documents mean 768", 8, 2048, 4, 256, True, 768),
            bench_config(device, CONFIG5_NAME, 64, 4096, 4, 1024, True, 0, iters=2),
            bench_config(device, "reference test shape: B=1 T=1 NH=4 dh=16 fp32 (one step, the step kernel)", 1, 1, 4, 16, False, 0, iters=20),
        ]
        out["backward"] = bench_backward(device)
        out["backward_config5_shape"] = bench_backward_large(device)
    if args.config4:
        out["config4"] = bench_config4(device)
    if args.layer:
        out["layer"] = bench_layer(device, args.layer_iters, args.layer_decode_steps)
    if not args.no_decode:
        out["decode"] = bench_decode(device)
        if not lean:
            out["decode"]["other_head_dims"] = bench_decode_other_head_dims(device)
        if not lean:
            # a decode step is one dependent launch: its floor is the launch itself plus the step's bytes at the HBM peak
            launch = out["roofline"]["serial_bound_stages_us"].get("dependent_launch_us")
            if launch:
                dr = out["decode"]["roofline"]
                dr["dependent_launch_floor_us"] = launch
                dr["serial_bound_us_per_step"] = launch + dr["algorithmic_bytes_per_launch"] / (HBM_PEAK_GBS * 1e3)
                dr["frac_of_serial_bound"] = dr["serial_bound_us_per_step"] / min(
                    out["decode"]["gpu_us_per_step"], out["decode"]["graph_us_per_step"] or 1e9)
                dr["serial_bound_source"] = "measured in this run: back-to-back launches of an empty kernel + bytes / HBM peak"
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wx_c, r_ext_c, bias_c, mask_c)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
