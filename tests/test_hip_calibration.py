"""GPU parity of the calibration statistics (row filter, std over kept rows, exact quantile by
radix selection, moving-average update) and of `calibrate_input_ranges` for every strategy,
against the CPU oracle and the ranges written by the real reference.

Tolerances: the row filter, the selection itself and the update arithmetic are exact; the
interpolated quantile and the std are fp32 expressions (1e-6 relative); calibrated ranges 1e-5
(fp32) / 1e-2 (bf16) relative, the path's stated tolerance.
"""
import os

import numpy as np
import pytest
import torch

from calib_cases import CALIB_CASES, RANDPERM_SEED, make_batches
from golden_cases import DTYPES
from oracle import torch_mode as om
from test_oracle_calibration import oracle_ranges

pytestmark = pytest.mark.gpu

CALIB_GOLDEN = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                         "calib_cases.npz")))


def ops():
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS
    return OPS


def sample(rows, cols, dtype, seed, zero_rows=(), ties=True):
    x = torch.randn(rows, cols, generator=torch.Generator().manual_seed(seed)) * 3.0
    if ties and rows > 2:
        x[0, : cols // 2] = x[2, : cols // 2]
        x[:, 0] = 0.5
    for r in zero_rows:
        x[r] = 0.0
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("rows,cols,max_size,zero_rows", [
    (1, 7, 3, ()), (12, 40, 16, (1, 4)), (130, 257, 128, (0, 129)), (64, 1024, 512, (5,)),
    (5, 33, -1, (0, 1, 2, 3, 4)),
])
def test_row_filter_and_std_over_kept_rows(rows, cols, max_size, zero_rows, dtype):
    x = sample(rows, cols, dtype, 11, zero_rows)
    sizes = om.split_sizes(cols, max_size)
    kept = ops().row_nonzero(x.cuda()).cpu().bool()
    assert torch.equal(kept, ~(x == 0).all(-1))
    got = ops().sliced_std_kept(x.cuda(), sizes).cpu()
    rows_kept = om.kept_rows(x)
    for t, (lo, hi) in enumerate(om.tile_bounds(sizes)):
        want = rows_kept[:, lo:hi].double().std()
        if torch.isnan(want):
            assert torch.isnan(got[t])
        else:
            assert abs(float(got[t]) - float(want)) <= 1e-6 * float(want) + 1e-12


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("q", [0.0, 0.25, 0.5, 0.99, 0.99995, 1.0])
@pytest.mark.parametrize("rows,cols,max_size,zero_rows", [
    (1, 7, 3, ()), (12, 40, 16, (1, 4)), (130, 257, 128, (0, 129)), (300, 96, 32, (7,)),
])
def test_quantile_by_selection(rows, cols, max_size, zero_rows, q, dtype):
    x = sample(rows, cols, dtype, 12, zero_rows)
    sizes = om.split_sizes(cols, max_size)
    got = ops().sliced_quantile(x.cuda(), sizes, q).cpu()
    rows_kept = om.kept_rows(x)
    for t, (lo, hi) in enumerate(om.tile_bounds(sizes)):
        want = float(om.quantile_linear(rows_kept[:, lo:hi], q))
        assert abs(float(got[t]) - want) <= 1e-6 * max(1.0, abs(want)), (t, float(got[t]), want)


def test_quantile_edge_cases():
    sizes = [4, 4]
    x = torch.zeros(3, 8)
    assert torch.isnan(ops().sliced_quantile(x.cuda(), sizes, 0.5).cpu()).all(), "no kept row"
    x = torch.randn(6, 8, generator=torch.Generator().manual_seed(1))
    x[2, 5] = float("nan")
    got = ops().sliced_quantile(x.cuda(), sizes, 0.5).cpu()
    assert not torch.isnan(got[0]) and torch.isnan(got[1]), "NaN poisons its own tile only"
    x = torch.full((4, 8), -2.5)
    assert torch.equal(ops().sliced_quantile(x.cuda(), sizes, 0.7).cpu(), torch.full((2,), -2.5))
    x = torch.tensor([[-0.0, 0.0, 1.0, -1.0, float("inf"), -float("inf"), 2.0, -2.0]])
    # torch.quantile's lerp turns an infinite order statistic into NaN (inf - inf); same here
    assert torch.isnan(ops().sliced_quantile(x.cuda(), [8], 0.0).cpu()[0])
    assert torch.isnan(torch.quantile(x, 0.0))
    assert float(ops().sliced_quantile(x.cuda(), [8], 0.5).cpu()[0]) == float(torch.quantile(x, 0.5))


def test_quantile_full_size_order_property():
    """Calibration size (2048 x 3072 activations, tiles of 512): the selected value has the
    wanted rank, checked by counting (ranks with weight 0, so no interpolation is involved)."""
    rows, cols = 2048, 3072
    x = (torch.randn(rows, cols, generator=torch.Generator().manual_seed(13)) * 2.0).cuda()
    sizes = om.split_sizes(cols, 512)
    n = rows * 512
    for lo in (0, 12345, n // 2, n - 2, n - 1):
        q = lo / (n - 1)
        if float(torch.tensor(q, dtype=torch.float32) * torch.tensor(float(n - 1))) != float(lo):
            continue  # the fp32 rank is not this integer: interpolation would be involved
        got = ops().sliced_quantile(x, sizes, q)
        for t, (c0, c1) in enumerate(om.tile_bounds(sizes)):
            part = x[:, c0:c1]
            below, at_most = int((part < got[t]).sum()), int((part <= got[t]).sum())
            assert below <= lo < at_most, (t, lo, below, at_most)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_moving_update_bit_exact(dtype):
    vals = [torch.tensor([0.1234567, 7.25, 1e-3]), torch.tensor([2.5, 0.3333333, 9.75]),
            torch.tensor([1.0, 1.0, 1.0])]
    ir = torch.full((3,), 3.0, dtype=dtype)
    idx = torch.zeros(3, dtype=torch.int32)
    ir_d, idx_d = ir.cuda(), idx.cuda()
    for alpha, in_dtype, v in ((3.0, True, vals[0]), (2.5, True, vals[1]), (1.0, False, vals[2])):
        ops().ir_moving_update(ir_d, idx_d, v.cuda(), alpha, in_dtype)
        for t in range(3):
            stat = float(v[t].to(dtype)) if in_dtype else float(v[t])
            om.moving_update(ir, idx, t, alpha * stat)
        assert torch.equal(ir_d.cpu(), ir) and torch.equal(idx_d.cpu(), idx)


@pytest.mark.parametrize("kind", ["MOVING_STD", "MOVING_QUANTILE", "MAX", "CACHE_QUANTILE"])
def test_a_batch_of_all_zero_rows_is_passed_over(kind):
    """The hidden projection of a recurrent layer sees an all-zero batch at the first step. The
    reference's statistics of the empty row selection are NaN or an error; here such a batch
    leaves the calibration state alone (the same as the oracle's statement of it)."""
    from aihwkit_lightning.inference.calibration import (InputRangeCalibrationType,
                                                         calibrate_input_ranges)
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig

    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 16
    layer = AnalogLinear(40, 8, rpu_config=cfg).cuda().eval()
    gen = torch.Generator().manual_seed(11)
    data = [torch.randn(32, 40, generator=gen) for _ in range(3)]
    batches = [torch.zeros(32, 40), data[0], torch.zeros(32, 40), data[1], data[2]]
    calibrate_input_ranges(layer, InputRangeCalibrationType[kind],
                           (((b.cuda(),), {}) for b in batches), quantile=0.99, max_samples=64,
                           std_alpha=3.0, verbose=False)
    got = layer.input_range.detach().cpu()
    assert torch.isfinite(got).all() and (got > 0).all()
    sizes = [14, 13, 13]
    if kind in ("MOVING_STD", "MOVING_QUANTILE"):
        want, _ = om.calibrate_moving(batches, sizes, InputRangeCalibrationType[kind].value,
                                      torch.float32, alpha=3.0, q=0.99)
        assert torch.allclose(got, want, rtol=1e-6)
        assert int(layer.input_range_update_idx.isinf().sum()) == 3  # marked as finished
    elif kind == "MAX":
        assert torch.equal(got, om.calibrate_max(data, sizes))


def build_layer(case):
    from aihwkit_lightning.nn import AnalogConv2d, AnalogLinear
    from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig

    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = case["max_input_size"]
    cfg.pre_post.input_range.enable = False
    cfg.forward.inp_res = -1
    dtype = DTYPES[case["dtype"]]
    if case["conv"]:
        layer = AnalogConv2d(3, case["N"], 3, padding=1, dtype=dtype, rpu_config=cfg)
    else:
        layer = AnalogLinear(case["K"], case["N"], dtype=dtype, rpu_config=cfg)
    return layer.cuda().eval()


@pytest.mark.parametrize("case", CALIB_CASES, ids=[c["name"] for c in CALIB_CASES])
def test_calibrate_input_ranges_matches_oracle_and_reference(case):
    from aihwkit_lightning.inference import InputRangeCalibrationType, calibrate_input_ranges

    layer = build_layer(case)
    batches = make_batches(case)
    trace = []

    def loader():
        for x in batches:
            if layer.input_range is not None:
                trace.append(layer.input_range.detach().float().cpu().clone())
            yield (x.cuda(),), {}

    torch.manual_seed(RANDPERM_SEED)
    kwargs = {} if case["std_alpha"] is None else {"std_alpha": case["std_alpha"]}
    calibrate_input_ranges(layer, InputRangeCalibrationType(case["kind"]), loader(),
                           quantile=case["quantile"], max_samples=case["max_samples"],
                           verbose=False, **kwargs)
    got = layer.input_range.detach().float().cpu()
    rtol = 1e-5 if case["dtype"] == "f32" else 1e-2
    want, want_trace = oracle_ranges(case)
    gold = torch.from_numpy(CALIB_GOLDEN[f"{case['name']}/ir"])
    assert torch.allclose(got, want.float(), rtol=rtol, atol=0), f"oracle: {got} vs {want}"
    assert torch.allclose(got, gold, rtol=rtol, atol=0), f"reference: {got} vs {gold}"
    if want_trace is not None:
        assert torch.allclose(torch.stack(trace), want_trace, rtol=rtol, atol=0)
    # state after calibration as in the reference: range enabled, parameter in the layer dtype
    assert layer.rpu_config.pre_post.input_range.enable
    assert layer.input_range.dtype == DTYPES[case["dtype"]]
    out = layer(batches[0].cuda())
    assert torch.isfinite(out.float()).all()
