"""CPU tests of the host-side mirror of the reference cell interface (no kernels run)."""
import dataclasses

import pytest
import torch

from xlstm_amd.cell import ParameterProxy, sLSTMCell, sLSTMCell_hip, sLSTMCellConfig


def _cell(**kw):
    cfg = sLSTMCellConfig(hidden_size=kw.pop("hidden_size", 64), num_heads=kw.pop("num_heads", 4), **kw)
    return sLSTMCell(cfg, skip_backend_init=True)


def test_backend_switch():
    assert isinstance(_cell(), sLSTMCell_hip)
    with pytest.raises(RuntimeError, match="unknown backend"):
        sLSTMCell(sLSTMCellConfig(hidden_size=64, backend="nope"))


def test_config_defaults_match_reference_fields():
    # field names and defaults of xlstm/blocks/slstm/cell.py:61-119 (backend default aside)
    cfg = sLSTMCellConfig(hidden_size=128)
    d = dataclasses.asdict(cfg)
    for k, v in dict(num_heads=4, num_states=4, function="slstm", bias_init="powerlaw_blockdependent",
                     recurrent_weight_init="zeros", num_gates=4, input_shape="BSGNH", output_shape="BNSH",
                     dtype="bfloat16", dtype_b="float32", enable_automatic_mixed_precision=True).items():
        assert d[k] == v, k
    assert cfg.dtype_r == "bfloat16" and cfg.dtype_s == "bfloat16" and cfg.dtype_a == "float32"
    assert cfg.head_dim == 32 and cfg.input_dim == 512


def test_hidden_size_must_divide():
    with pytest.raises(ValueError, match="must be divisible"):
        _cell(hidden_size=66, num_heads=4)


def test_layout_round_trips():
    # the doctests of cell.py:623-626,646-649 for the hip layouts
    cell = _cell(hidden_size=64, num_heads=2, recurrent_weight_init="standard", bias_init="standard")
    rk, b = cell._recurrent_kernel, cell._bias
    assert torch.equal(cell._recurrent_kernel_ext2int(cell._recurrent_kernel_int2ext(rk)), rk)
    assert torch.equal(cell._bias_ext2int(cell._bias_int2ext(b)), b)
    assert tuple(cell.recurrent_kernel.shape) == (2, 32, 4, 32)
    assert tuple(cell.bias.shape) == (2, 4, 32)


def test_internal_layout_is_k_contiguous_vanilla_layout():
    cell = _cell(hidden_size=32, num_heads=2, recurrent_weight_init="standard")
    ext = cell.recurrent_kernel[:]
    NH, dh = 2, 16
    for h, d, g, a in [(0, 3, 1, 5), (1, 15, 3, 0), (1, 0, 0, 15)]:
        assert cell._recurrent_kernel_[h, g * dh + a, d] == ext[h, d, g, a]
    bext = cell.bias[:]
    for h, g, a in [(0, 1, 3), (1, 3, 15)]:
        assert cell._bias_[h * 4 * dh + g * dh + a] == bext[h, g, a]


def test_inits_closed_forms():
    cell = _cell(hidden_size=64, num_heads=4)  # defaults: zeros R, power-law forget bias
    assert torch.count_nonzero(cell.recurrent_kernel[:]) == 0
    b = cell.bias[:]
    dh = 16
    want = -(-5.0 + 12.0 * (torch.arange(dh) / (dh - 1)) ** 0.3)
    for h in range(4):
        assert torch.allclose(b[h, 1], want)
        assert torch.count_nonzero(b[h, [0, 2, 3]]) == 0
    cell = _cell(hidden_size=64, num_heads=4, bias_init="small_init", recurrent_weight_init="standard")
    b = cell.bias[:]
    assert torch.allclose(b[2, 1], torch.linspace(3.0, 6.0, dh))
    r = cell.recurrent_kernel[:]
    assert r.abs().max() <= 1 / 8 and r.std() > 0.05  # U(+-1/sqrt(64))
    blockdep = sLSTMCell(sLSTMCellConfig(hidden_size=64, _block_idx=3, _num_blocks=7), skip_backend_init=True)
    want = -(-5.0 + 12.0 * (torch.arange(dh) / (dh - 1)) ** (0.3 + 1.3 * 0.5))
    assert torch.allclose(blockdep.bias[0, 1], want)


def test_proxy_setitem_writes_internal_layout():
    cell = _cell(hidden_size=32, num_heads=2)
    cell.recurrent_kernel[1, 2, 3, 4] = 7.0
    assert cell._recurrent_kernel_[1, 3 * 16 + 4, 2] == 7.0
    assert isinstance(cell.recurrent_kernel, ParameterProxy)


def test_permute_output_shapes():
    # shapes documented at cell.py:355-362
    for shape, want in (("SBH", (5, 3, 16)), ("BSH", (3, 5, 16)), ("BNSH", (3, 2, 5, 8)), ("SBNH", (5, 3, 2, 8))):
        cell = _cell(hidden_size=16, num_heads=2, output_shape=shape)
        assert tuple(cell._permute_output(torch.zeros(5, 3, 16)).shape) == want


def test_bad_input_size_and_cpu_tensor_fail_loudly():
    cell = _cell(hidden_size=64, num_heads=4)
    with pytest.raises(AssertionError, match="Input size mismatch"):
        cell(torch.zeros(1, 1, 255))
    with pytest.raises(ValueError, match="no CPU path"):
        with torch.no_grad():
            cell(torch.zeros(1, 1, 256))
    with pytest.raises(AssertionError, match="state must be"):
        with torch.no_grad():
            cell(torch.zeros(1, 1, 256), torch.zeros(4, 2, 64))


def test_state_dict_names_match_reference():
    assert set(_cell().state_dict().keys()) == {"_recurrent_kernel_", "_bias_"}


def test_reference_checkpoint_layouts_convert_to_hip():
    """Internal tensors as the reference's vanilla and cuda cells store them (fixture written from
    those classes) land in the hip cell with the same EXTERNAL view."""
    import os

    import numpy as np
    import torch

    from xlstm_amd.cell import reference_cell_params_to_hip, reference_state_dict_to_hip, sLSTMCell, sLSTMCellConfig

    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "ckpt_layouts.npz"))
    NH = int(z["num_heads"])
    r_ext, b_ext = torch.from_numpy(z["r_ext"]), torch.from_numpy(z["b_ext"])
    for backend in ("vanilla", "cuda"):
        cell = sLSTMCell(sLSTMCellConfig(hidden_size=r_ext.shape[0] * r_ext.shape[1], num_heads=NH, backend="hip",
                                         dtype="float32"), skip_backend_init=True)
        sd = {"slstm_cell._recurrent_kernel_": torch.from_numpy(z[f"r_{backend}"]),
              "slstm_cell._bias_": torch.from_numpy(z[f"b_{backend}"]), "other.weight": torch.ones(2)}
        conv = reference_state_dict_to_hip(sd, backend, NH)
        assert conv["other.weight"] is sd["other.weight"]
        cell.load_state_dict({"_recurrent_kernel_": conv["slstm_cell._recurrent_kernel_"],
                              "_bias_": conv["slstm_cell._bias_"]})
        assert torch.equal(cell.recurrent_kernel[:], r_ext), backend
        assert torch.equal(cell.bias[:], b_ext), backend
    # the two source layouts really differ from each other (the fixture is not vacuous)
    assert z["r_vanilla"].shape != z["r_cuda"].shape and not np.array_equal(z["b_vanilla"], z["b_cuda"])
    import pytest
    with pytest.raises(ValueError):
        reference_cell_params_to_hip(torch.from_numpy(z["r_cuda"]), torch.from_numpy(z["b_cuda"]), "vanilla", NH)
    with pytest.raises(ValueError):
        reference_cell_params_to_hip(torch.from_numpy(z["r_cuda"]), torch.from_numpy(z["b_cuda"]), "triton", NH)


def test_cell_can_be_copied_and_pickled():
    """copy.deepcopy / pickle of a cell (torch does it for EMA copies, DDP, checkpoints of whole modules): the
    parameter proxies follow the copy, the per-cell runtime objects (workspaces, events, decode plan) do not."""
    import copy
    import pickle

    import torch

    from xlstm_amd.cell import sLSTMCell, sLSTMCellConfig

    c = sLSTMCell(sLSTMCellConfig(hidden_size=64, num_heads=4, backend="hip", recurrent_weight_init="standard"),
                  skip_backend_init=True)
    for other in (copy.deepcopy(c), pickle.loads(pickle.dumps(c))):
        assert other._rt is not c._rt and other.recurrent_kernel.module is other
        assert torch.equal(other.recurrent_kernel[:], c.recurrent_kernel[:]) and torch.equal(other.bias[:], c.bias[:])
        other.bias[0, 1] = torch.zeros(16)
        assert not torch.equal(other.bias[:], c.bias[:])
