"""Pins the convolution oracle: torch's own unfold / convolutions (independent library routines),
the adjoint identity of the fold, and vectors written by the real reference."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conv_cases import CONV_CASES, make_conv_inputs
from golden_cases import DTYPES
from helpers import case_input_range, oracle_cfg
from oracle import conv_mode as oc
from oracle import torch_mode as om

CONV_GOLDEN = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                        "conv_cases.npz")))
GEOMS_2D = [
    # C, size, kernel, stride, padding, dilation
    (3, (7, 6), (3, 3), (1, 1), (1, 1), (1, 1)),
    (2, (9, 8), (3, 2), (2, 1), (1, 0), (1, 2)),
    (4, (5, 11), (1, 4), (1, 3), (0, 2), (1, 1)),
    (1, (8, 8), (3, 3), (3, 2), (2, 2), (2, 1)),
]


@pytest.mark.parametrize("geom", GEOMS_2D)
def test_patches_match_torch_unfold(geom):
    chan, size, kernel, stride, padding, dilation = geom
    x = torch.randn(3, chan, *size, generator=torch.Generator().manual_seed(1))
    cols, out = oc.conv_patches(x.unsqueeze(2), [1, *kernel], [1, *stride], [0, *padding],
                                [1, *dilation])
    want = F.unfold(x, kernel, dilation=dilation, padding=padding, stride=stride).transpose(1, 2)
    assert torch.equal(cols, want)
    assert out[0] == 1 and out[1] * out[2] == want.size(1)


@pytest.mark.parametrize("geom", GEOMS_2D)
def test_fold_is_the_adjoint_of_patches(geom):
    chan, size, kernel, stride, padding, dilation = geom
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(2, chan, 1, *size, generator=gen, dtype=torch.float64).float()
    args = ([1, *kernel], [1, *stride], [0, *padding], [1, *dilation])
    cols, _ = oc.conv_patches(x, *args)
    g = torch.randn(cols.shape, generator=gen)
    dx = oc.conv_fold(g, x.shape, *args)
    lhs = (cols.double() * g.double()).sum()
    rhs = (x.double() * dx.double()).sum()
    assert abs(lhs - rhs) <= 1e-5 * max(1.0, abs(lhs))
    # and it is torch's fold
    want = F.fold(g.transpose(1, 2), size, kernel, dilation=dilation, padding=padding, stride=stride)
    assert torch.allclose(dx.squeeze(2), want, rtol=1e-5, atol=1e-6)


PLAIN = [c for c in CONV_CASES if c["name"].endswith("_plain")]


@pytest.mark.parametrize("case", PLAIN, ids=[c["name"] for c in PLAIN])
def test_plain_convolution_is_torch_convolution(case):
    """Without non-idealities the layer is torch's convolution, forward and all gradients."""
    x, w, b, g = make_conv_inputs(case)
    out, saved = oc.conv_forward(x, w, b, case["stride"], case["padding"], case["dilation"],
                                 oracle_cfg(case), None, True)
    dx, dw, db, _ = oc.conv_backward(g, saved)
    conv = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[case["ndim"]]
    xr, wr, br = (t.clone().requires_grad_(True) for t in (x, w, b))
    ref = conv(xr, wr, br, stride=case["stride"], padding=case["padding"], dilation=case["dilation"])
    ref.backward(g)
    for got, want, what in ((out, ref, "out"), (dx, xr.grad, "dx"), (dw, wr.grad, "dw"),
                            (db, br.grad, "db")):
        assert got.shape == want.shape, what
        assert torch.allclose(got, want.detach(), rtol=1e-5, atol=1e-5), what


def _compare(got, ref, dtype, what, exact_bf16=True):
    got = got.float()
    assert got.shape == ref.shape, f"{what}: {tuple(got.shape)} vs {tuple(ref.shape)}"
    if dtype == torch.bfloat16 and exact_bf16:
        mism = int((got != ref).sum())
        assert mism == 0, f"{what}: {mism} of {ref.numel()} bf16 elements differ"
        return
    # fp32: summation order only; bf16 input gradient: the reference folds in bf16 (one rounding
    # per added patch entry), the oracle in fp32 with one rounding
    rtol = 2e-6 if dtype == torch.float32 else 2e-2
    scale = ref.abs().mean().clamp_min(1e-30)
    err = ((got - ref).abs() / (ref.abs() + scale)).max()
    assert err < rtol, f"{what}: relative error {err:.2e}"


@pytest.mark.parametrize("case", CONV_CASES, ids=[c["name"] for c in CONV_CASES])
def test_convolution_matches_reference(case):
    dtype = DTYPES[case["dtype"]]
    name = case["name"]
    x, w, b, g = make_conv_inputs(case)
    batched = case["batch"] > 0
    xb, gb = (x, g) if batched else (x.unsqueeze(0), g.unsqueeze(0))
    k_in = w[0].numel()
    ir = case_input_range(case, len(om.split_sizes(k_in, case["max_input_size"])))
    torch.manual_seed(case["noise_seed"])
    out, saved = oc.conv_forward(xb, w, b, case["stride"], case["padding"], case["dilation"],
                                 oracle_cfg(case), ir, case["training"])
    dx, dw, db, dir_ = oc.conv_backward(gb, saved)
    if not batched:
        out, dx = out.squeeze(0), dx.squeeze(0)
    gold = {k: torch.from_numpy(CONV_GOLDEN[f"{name}/{k}"]) for k in ("out", "dx", "dw", "db")}
    _compare(out, gold["out"], dtype, "out")
    _compare(dw, gold["dw"], dtype, "dw")
    _compare(db, gold["db"], dtype, "db")
    _compare(dx, gold["dx"], dtype, "dx", exact_bf16=False)
    if case["ir_mode"] == "static":
        _compare(dir_, torch.from_numpy(CONV_GOLDEN[f"{name}/dir"]), dtype, "dir")


def test_cases_exercise_the_nonidealities():
    """The ADC cases must clip inputs and clamp outputs, or they would pin nothing."""
    case = [c for c in CONV_CASES if c["name"] == "conv2d_f32_adc"][0]
    x, w, b, _ = make_conv_inputs(case)
    ir = case_input_range(case, 3)
    _, saved = oc.conv_forward(x, w, b, case["stride"], case["padding"], case["dilation"],
                               oracle_cfg(case), ir, True)
    assert any(bool(rec["up"].any()) for rec in saved["tiles"])
    assert any(not bool(rec["keep"].all()) for rec in saved["tiles"])
