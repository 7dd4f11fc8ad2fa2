"""Shared test helpers: golden fixtures, oracle drivers, comparison with the stated tolerances."""
import os

import numpy as np
import torch

from golden_cases import CASES_BY_NAME, DTYPES, make_inputs, make_learnable_clip
from oracle import torch_mode as om

GOLDEN_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "linear_cases.npz")
_GOLDEN = None


def golden():
    """The fixture arrays written by the reference (tests/golden/make_golden.py)."""
    global _GOLDEN  # pylint: disable=global-statement
    if _GOLDEN is None:
        _GOLDEN = dict(np.load(GOLDEN_PATH))
    return _GOLDEN


def golden_tensor(key, dtype=torch.float32):
    return torch.from_numpy(golden()[key]).to(dtype)


def oracle_cfg(c) -> om.OracleCfg:
    """OracleCfg of a golden case dict."""
    return om.OracleCfg(
        max_input_size=c["max_input_size"], inp_res=c["inp_res"], out_res=c["out_res"],
        out_bound=c["out_bound"], out_noise=c["out_noise"],
        out_noise_per_channel=c["out_noise_per_channel"],
        bound_per_channel=c["clip"] in ("channel", "learnable"), clip_learnable=c["clip"] == "learnable",
        ir_mode=c["ir_mode"], ir_decay=c["ir_decay"], ir_input_min_percentage=c["ir_min_pct"],
        weight_quant=c["weight_quant"], weight_noise=c["weight_noise"],
        modifier_res=c["modifier_res"], modifier_std=c["modifier_std"],
    )


def case_input_range(c, n_tiles):
    """Initial per-tile input range of a case (None unless the range is a stored parameter)."""
    if c["ir_mode"] not in ("static", "fast"):
        return None
    dtype = DTYPES[c["dtype"]]
    if c["ir_values"] is not None:
        return torch.tensor(c["ir_values"], dtype=dtype)
    return torch.full((n_tiles,), c["ir_init"], dtype=dtype)


def oracle_fwd_bwd(c):
    """Run the oracle on a 'fwd_bwd' case; returns dict(out, dx, dw, db, dir)."""
    x, w, b, g = make_inputs(c)
    cfg = oracle_cfg(c)
    in_sizes = om.split_sizes(c["K"], c["max_input_size"])
    ir = case_input_range(c, len(in_sizes))
    torch.manual_seed(c["noise_seed"])
    lwc = make_learnable_clip(c, w) if c["clip"] == "learnable" else None
    out, saved = om.linear_forward(x, w, b, cfg, ir, c["training"], learnable_weight_clip=lwc)
    dx, dw, db, dir_ = om.linear_backward(g, saved)
    return dict(out=out, dx=dx, dw=dw, db=db if b is not None else None, dir=dir_,
                dlwc=saved.get("dlwc"))


def rel_scale_mismatch(got, ref, rtol):
    """Boolean mask of elements outside |got - ref| <= rtol * (|ref| + mean|ref|)."""
    got, ref = got.double(), ref.double()
    scale = ref.abs().mean()
    return (got - ref).abs() > rtol * (ref.abs() + scale)


def assert_close_lsb(got, ref, rtol, lsb=None, max_frac=1e-3, what=""):
    """The acceptance rule of the path: every element within ``rtol`` relative to the tensor's
    scale; elements outside it must be at most one ADC LSB away (``lsb``: scalar or tensor
    broadcastable to ref) and at most ``max_frac`` (0.1 %) of all elements."""
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    bad = rel_scale_mismatch(got, ref, rtol)
    n_bad = int(bad.sum())
    if n_bad == 0:
        return
    diff = (got.double() - ref.double()).abs()
    assert lsb is not None, f"{what}: {n_bad} elements differ, max |diff| {diff.max():.3e}"
    lsb_t = torch.as_tensor(lsb, dtype=torch.float64).expand_as(diff)
    over = bad & (diff > lsb_t * 1.01 + rtol * ref.double().abs())
    assert int(over.sum()) == 0, (
        f"{what}: {int(over.sum())} elements differ by more than one LSB "
        f"(max |diff| {diff[bad].max():.3e})"
    )
    frac = n_bad / ref.numel()
    assert frac <= max_frac, f"{what}: {n_bad} of {ref.numel()} elements ({frac:.3%}) differ by an LSB"
