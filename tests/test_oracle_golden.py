"""Pins the CPU oracle against vectors produced by the real reference (tests/golden)."""
import pytest
import torch

from golden_cases import CASES, DTYPES, make_inputs, make_learnable_clip
from helpers import golden, golden_tensor, oracle_cfg, oracle_fwd_bwd, case_input_range
from oracle import torch_mode as om

FWD_BWD = [c for c in CASES if c["kind"] == "fwd_bwd"]


def _exact_or_close(got, ref, dtype, what):
    """bf16 / f16 results must be identical; fp32 results may differ by accumulation order only."""
    got = got.float()
    if dtype in (torch.bfloat16, torch.float16):
        mism = int((got != ref).sum())
        assert mism == 0, f"{what}: {mism} of {ref.numel()} 16-bit elements differ"
    else:
        scale = ref.abs().mean().clamp_min(1e-30)
        err = ((got - ref).abs() / (ref.abs() + scale)).max()
        assert err < 2e-6, f"{what}: relative error {err:.2e}"


@pytest.mark.parametrize("case", FWD_BWD, ids=[c["name"] for c in FWD_BWD])
def test_forward_backward_matches_reference(case):
    res = oracle_fwd_bwd(case)
    dtype = DTYPES[case["dtype"]]
    name = case["name"]
    for key in ("out", "dx", "dw", "db", "dir", "dlwc"):
        gkey = f"{name}/{key}"
        if gkey not in golden():
            continue
        assert res[key] is not None, f"oracle produced no {key}"
        _exact_or_close(res[key], golden_tensor(gkey), dtype, gkey)
    if case["ir_mode"] in ("static", "fast"):
        assert f"{name}/dir" in golden(), "reference wrote an input-range gradient"
    if case["clip"] == "learnable":
        assert f"{name}/dlwc" in golden(), "reference wrote a gradient of the learnable clip"


@pytest.mark.parametrize("name", ["f32_ir_init", "bf16_ir_init"])
def test_input_range_initialisation_sequence(name):
    case = [c for c in CASES if c["name"] == name][0]
    dtype = DTYPES[case["dtype"]]
    _, w, b, _ = make_inputs(case)
    cfg = oracle_cfg(case)
    in_sizes = om.split_sizes(case["K"], case["max_input_size"])
    ir = case_input_range(case, len(in_sizes))
    idx = torch.zeros(len(in_sizes), dtype=dtype)
    for step in range(case["steps"]):
        xs = golden_tensor(f"{name}/x{step}", dtype)
        for t, (lo, hi) in enumerate(om.tile_bounds(in_sizes)):
            om.ir_init_update(xs[:, lo:hi], ir, idx, t, case["init_from_data"], case["init_std_alpha"])
        out, _ = om.linear_forward(xs, w, b, cfg, ir, True)
        _exact_or_close(ir, golden_tensor(f"{name}/ir{step}"), dtype, f"ir after step {step}")
        _exact_or_close(idx, golden_tensor(f"{name}/idx{step}"), dtype, f"idx after step {step}")
        _exact_or_close(out, golden_tensor(f"{name}/out{step}"), dtype, f"out step {step}")
    assert float(idx.max()) == case["init_from_data"], "initialisation must stop at init_from_data"


@pytest.mark.parametrize("name", ["f32_fast_init", "bf16_fast_init", "f32_fast_init_minmax"])
def test_fast_mode_range_sequence(name):
    case = [c for c in CASES if c["name"] == name][0]
    dtype = DTYPES[case["dtype"]]
    _, w, b, _ = make_inputs(case)
    cfg = oracle_cfg(case)
    in_sizes = om.split_sizes(case["K"], case["max_input_size"])
    n_tiles = len(in_sizes)
    ir = case_input_range(case, n_tiles)
    idx = torch.zeros(n_tiles, dtype=dtype)
    x_min = torch.full((n_tiles,), -1e-5, dtype=dtype)  # nn/modules/base.py:149-154
    x_max = torch.full((n_tiles,), 1e-5, dtype=dtype)
    for step in range(case["steps"]):
        xs = golden_tensor(f"{name}/x{step}", dtype)
        for t, (lo, hi) in enumerate(om.tile_bounds(in_sizes)):
            om.ir_fast_update(xs[:, lo:hi], ir, idx, x_min, x_max, t, case["init_from_data"],
                              case["act_range_momentum"])
        out, _ = om.linear_forward(xs, w, b, cfg, ir, True)
        for key, val in (("ir", ir), ("idx", idx), ("xmin", x_min), ("xmax", x_max), ("out", out)):
            _exact_or_close(val, golden_tensor(f"{name}/{key}{step}"), dtype, f"{key} after step {step}")
    assert float(idx.max()) == case["init_from_data"], "the updates must stop at init_from_data"


@pytest.mark.parametrize("name", ["f32_clip_layer", "f32_clip_channel", "bf16_clip_channel"])
def test_clip_weights(name):
    case = [c for c in CASES if c["name"] == name][0]
    _, w, _, _ = make_inputs(case)
    got = om.clip_weights(w, case["clip_sigma"], case["clip"] == "channel")
    assert torch.equal(got.float(), golden_tensor(f"{name}/w_clipped"))
    assert not torch.equal(got, w), "the case must actually clip something"


QUANTIZE_CASES = ["f32_quantize_channel", "f32_quantize_odd", "bf16_quantize_tensor",
                  "f32_quantize_lsq_clip", "bf16_quantize_lsq_clip", "f32_quantize_lsq_quant",
                  "bf16_quantize_lsq_quant", "f32_quantize_lsq_clip_big"]


@pytest.mark.parametrize("name", QUANTIZE_CASES)
def test_quantize_weights(name):
    case = [c for c in CASES if c["name"] == name][0]
    dtype = DTYPES[case["dtype"]]
    x, w, b, _ = make_inputs(case)
    in_sizes = om.split_sizes(case["K"], case["max_input_size"])
    lwc = make_learnable_clip(case, w) if case["clip"] == "learnable" else None
    got = om.quantize_weights(w, in_sizes, case["weight_quant"], case["modifier_res"], lwc)
    if lwc is not None:
        assert not torch.equal(got, w), "the case must actually change weights"
    _exact_or_close(got, golden_tensor(f"{name}/w_quantized"), dtype, "quantised weights")
    # the reference switches quantisation off afterwards and evaluates the layer plainly
    cfg = oracle_cfg(case)
    cfg.weight_quant = om.NONE
    cfg.clip_learnable = cfg.bound_per_channel = False   # ... and the clipping (base.py:208-212)
    out, _ = om.linear_forward(x, got, b, cfg, None, False)
    _exact_or_close(out, golden_tensor(f"{name}/out"), dtype, "output after quantisation")
