"""Shared helpers of the test-suite: seeded problems in the external layouts."""
import numpy as np
import torch


def make_problem(seed, B, T, NH, dh, rscale=1.0, bf16=False, with_state=False, bias="small_init"):
    """Seeded inputs shaped like the reference cell's: wx ~ N(0,1) [B,T,4H],
    R ~ U(+-rscale/sqrt(H)) in the external layout [NH,dh,4,dh], forget-gate
    bias linspace(3,6) per head (cell.py:420-426) or random."""
    rng = np.random.default_rng(seed)
    H = NH * dh
    wx = rng.standard_normal((B, T, 4 * H)).astype(np.float32)
    r_ext = (rng.uniform(-1, 1, (NH, dh, 4, dh)) * rscale / np.sqrt(H)).astype(np.float32)
    if bias == "small_init":
        b_ext = np.zeros((NH, 4, dh), np.float32)
        b_ext[:, 1, :] = np.linspace(3.0, 6.0, dh, dtype=np.float32)
    else:
        b_ext = rng.standard_normal((NH, 4, dh)).astype(np.float32)
    s0 = None
    if with_state:
        s0 = rng.standard_normal((4, B, H)).astype(np.float32)
        s0[0] = np.tanh(s0[0])
        s0[2] = np.abs(s0[2]) + 1.0
    if bf16:
        wx = torch.from_numpy(wx).bfloat16().float().numpy()
    return wx, r_ext, b_ext, s0


def r_ext_to_kernel(r_ext: torch.Tensor) -> torch.Tensor:
    """[NH, dh_in, 4, dh_out] -> [NH, 4*dh_out, dh_in]."""
    NH, dh = r_ext.shape[0], r_ext.shape[1]
    return r_ext.permute(0, 2, 3, 1).reshape(NH, 4 * dh, dh).contiguous()


def geometric_reset_mask(seed, B, T, mean_len):
    """Document starts for rows packed with documents of Geometric(1/mean_len)
    length (support >= 1); 1 at every document start including t = 0."""
    rng = np.random.default_rng(seed)
    mask = np.zeros((B, T), np.uint8)
    for b in range(B):
        t = 0
        while t < T:
            mask[b, t] = 1
            t += int(rng.geometric(1.0 / mean_len))
    return mask


def max_err(actual, desired):
    """max |a - d| / max(1, |d|): the parity measure used throughout."""
    a = np.asarray(actual, np.float64)
    d = np.asarray(desired, np.float64)
    return float(np.max(np.abs(a - d) / np.maximum(1.0, np.abs(d)))) if a.size else 0.0
