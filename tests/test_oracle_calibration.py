"""Pins the calibration part of the oracle: the quantile restatement against torch.quantile (an
independent library routine) and every strategy against ranges written by the real reference."""
import os

import numpy as np
import pytest
import torch

from calib_cases import CALIB_CASES, RANDPERM_SEED, make_batches
from golden_cases import DTYPES
from oracle import conv_mode as oc
from oracle import torch_mode as om

CALIB_GOLDEN = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                         "calib_cases.npz")))


@pytest.mark.parametrize("n", [1, 2, 3, 10, 257, 5000])
@pytest.mark.parametrize("q", [0.0, 0.3, 0.5, 0.9, 0.99995, 1.0])
def test_quantile_restatement_matches_torch(n, q):
    gen = torch.Generator().manual_seed(n)
    values = torch.randn(n, generator=gen)
    values[: n // 3] = values[0]  # ties
    got, want = om.quantile_linear(values, q), torch.quantile(values, q)
    assert abs(float(got) - float(want)) <= 1e-6 * max(1.0, abs(float(want)))
    assert float(om.quantile_linear(values.sort().values.flip(0), q)) == float(got), "order free"


def test_quantile_special_cases():
    assert torch.isnan(om.quantile_linear(torch.zeros(0), 0.5))
    assert torch.isnan(om.quantile_linear(torch.tensor([1.0, float("nan")]), 0.5))
    assert float(om.quantile_linear(torch.tensor([1.0, 3.0]), 0.5)) == 2.0
    assert float(om.quantile_linear(torch.tensor([-2.0, 5.0, 1.0]), 1.0)) == 5.0


def tile_rows(case, batches):
    """What the tiles see: the batch itself, or the patches of a convolution input."""
    if not case["conv"]:
        return batches
    return [oc.conv_patches(x.unsqueeze(2), [1, 3, 3], [1, 1, 1], [0, 1, 1], [1, 1, 1])[0]
            .reshape(-1, 27) for x in batches]


def oracle_ranges(case):
    dtype = DTYPES[case["dtype"]]
    rows = tile_rows(case, make_batches(case))
    sizes = om.split_sizes(case["K"], case["max_input_size"])
    if case["kind"] == "Max":
        return om.calibrate_max(rows, sizes), None
    if case["kind"] == "CacheQuantile":
        torch.manual_seed(RANDPERM_SEED)
        return om.calibrate_cache_quantile(rows, sizes, case["quantile"], case["max_samples"], dtype), None
    alpha = 3.0 if case["std_alpha"] is None else case["std_alpha"]
    return om.calibrate_moving(rows, sizes, case["kind"], dtype, alpha=alpha, q=case["quantile"])


@pytest.mark.parametrize("case", CALIB_CASES, ids=[c["name"] for c in CALIB_CASES])
def test_calibrated_ranges_match_reference(case):
    ir, trace = oracle_ranges(case)
    gold = torch.from_numpy(CALIB_GOLDEN[f"{case['name']}/ir"])
    if case["dtype"] == "bf16":
        assert torch.equal(ir.float(), gold), f"{ir.float()} vs {gold}"
    else:
        assert torch.allclose(ir.float(), gold, rtol=1e-6, atol=0), f"{ir} vs {gold}"
    if trace is not None:
        gtrace = torch.from_numpy(CALIB_GOLDEN[f"{case['name']}/trace"])
        assert torch.allclose(trace, gtrace, rtol=1e-6, atol=0)


def test_zeroed_rows_matter():
    """The cases must be sensitive to the row filter, or they would not pin it."""
    case = [c for c in CALIB_CASES if c["name"] == "moving_std_f32"][0]
    batches = make_batches(case)
    assert any(bool((b == 0).all(-1).any()) for b in batches)
    sizes = om.split_sizes(case["K"], case["max_input_size"])
    filtered = batches[1][~(batches[1] == 0).all(-1)][:, :sizes[0]].std()
    assert abs(float(filtered) - float(batches[1][:, :sizes[0]].std())) > 1e-3
