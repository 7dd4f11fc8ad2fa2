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


# Bound of the error of an fp32-accumulated product of K terms relative to the sum of the terms'
# magnitudes: 8 units in the last place of fp32. The worst case of a plain running sum is (K - 1)
# units, that of a pairwise sum log2(K); the MFMA kernels add 16 products exactly-ish per
# instruction and chain K / 16 of those, the CPU library sums in vector lanes.
ACC_ERR = 8.0 * 2.0 ** -24


class TieLog:
    """``om.PRODUCT_HOOK`` that finds the tile products whose result depends on the order of the
    fp32 accumulation: the exact product (float64) is moved down and up by the accumulation error
    bound, both values are rounded to the tensor dtype and taken through the rest of the tile's
    pipeline (noise, ADC, clamp: ``om.tile_output``, monotone in the product). Where the two
    tile outputs differ the element is a *tie* of the ADC level (``near_out``), where the two
    clamp decisions differ a tie of the clamp mask (``near_keep``). Two correct implementations
    may disagree exactly there and nowhere else.

    ``flip``: ties, as ``(call, row, column)``, to resolve the other way than the oracle's own
    product did (``call`` counts the tile products of the run, in order)."""

    def __init__(self, flip=(), input_err=0.0):
        self.flip = set(flip)
        self.calls = []       # per tile product: dict(near_out, near_keep) of bool [M, N]
        self.ties = []        # (call, row, column) of every tie found
        self.outside = 0      # products of the oracle outside the interval of the two candidates
        # DAC ties (networks only): a layer input that comes out of another layer's activation
        # functions carries their last-place differences between CPU and GPU; ``input_err`` is
        # the relative size of that difference, 0 for a layer whose input is given
        self.input_err = input_err
        self.dac_calls = 0
        self.dac_ties = []    # ("dac", call, row, column)

    def dac(self, xc, step, xq, skip_rounding):
        """``om.DAC_HOOK``: DAC levels that change when the input moves by ``input_err``."""
        call = self.dac_calls
        self.dac_calls += 1
        if self.input_err <= 0.0 or skip_rounding:
            return xq
        v = (xc / step.clamp_min(om._tiny(xc.dtype))).double()
        # with a per-row range the step moves with the row's largest input as well
        err = 2.0 * self.input_err * v.abs()
        lo, hi = (v - err).to(xc.dtype).round(), (v + err).to(xc.dtype).round()
        here = [("dac", call, m, k) for m, k in (lo != hi).nonzero().tolist()]
        self.dac_ties.extend(here)
        flips = [tie for tie in here if tie in self.flip]
        if flips:
            xq = xq.clone()
            mine = (xc / step.clamp_min(om._tiny(xc.dtype))).round()
            for _, _, m, k in flips:
                other = hi[m, k] if mine[m, k] == lo[m, k] else lo[m, k]
                xq[m, k] = (other * step.expand_as(xq)[m, k]).to(xq.dtype)
        return xq

    def __call__(self, xq, w_eff, y, post):
        exact = xq.double() @ w_eff.double().T
        err = ACC_ERR * (xq.double().abs() @ w_eff.double().abs().T)
        lo, hi = (exact - err).to(y.dtype), (exact + err).to(y.dtype)
        self.outside += int(((y < torch.minimum(lo, hi)) | (y > torch.maximum(lo, hi))).sum())
        out_lo, keep_lo = om.tile_output(lo, post)
        out_hi, keep_hi = om.tile_output(hi, post)
        near_out = out_lo != out_hi
        near_keep = torch.zeros_like(near_out) if keep_lo is None else keep_lo != keep_hi
        call = len(self.calls)
        self.calls.append(dict(near_out=near_out, near_keep=near_keep))
        here = [(call, m, n) for m, n in (near_out | near_keep).nonzero().tolist()]
        self.ties.extend(here)
        flips = [tie for tie in here if tie in self.flip]
        if flips:
            y = y.clone()
            for _, m, n in flips:
                y[m, n] = hi[m, n] if y[m, n] == lo[m, n] else lo[m, n]
        return y


class product_hook:
    """``with product_hook(log): ...`` installs a TieLog as the oracle's product hook."""

    def __init__(self, log):
        self.log = log

    def __enter__(self):
        assert om.PRODUCT_HOOK is None and om.DAC_HOOK is None
        om.PRODUCT_HOOK = self.log
        om.DAC_HOOK = self.log.dac
        return self.log

    def __exit__(self, *exc):
        om.PRODUCT_HOOK = None
        om.DAC_HOOK = None
        return False


def tie_allowances(c, saved, g, log):
    """What a flipped clamp decision may change in each gradient, from the oracle's own record:
    one flipped (row m, channel n, tile t) adds or removes g[m, n] * w_eff[n, k] in dx[m, k] and
    g[m, n] * xq[m, k] in dw[n, k] for the columns k of tile t. Returns float64 tensors (upper
    bounds of the change if every tie of the clamp mask went the other way) for dx, dw, the
    input-range gradient and the gradient of a learnable clip, plus the ties themselves."""
    cfg = saved["cfg"]
    bounds = om.tile_bounds(saved["in_sizes"])
    x = saved["x"]
    gd = g.double().abs()
    tol_dx = torch.zeros(x.shape, dtype=torch.float64)
    tol_dw = torch.zeros(g.shape[1], x.shape[1], dtype=torch.float64)
    tol_dir = torch.zeros(len(bounds), dtype=torch.float64)
    tol_dlwc = torch.zeros(len(bounds), g.shape[1], dtype=torch.float64)
    near_out = torch.zeros(g.shape, dtype=torch.bool)
    n_keep = 0
    for t, (lo, hi) in enumerate(bounds):
        rec, call = saved["tiles"][t], log.calls[t]
        near_out |= call["near_out"] | call["near_keep"]
        n_keep += int(call["near_keep"].sum())
        if not bool(call["near_keep"].any()):
            continue
        gk = gd * call["near_keep"]
        tol_dx[:, lo:hi] = gk @ rec["w_eff"].double().abs()
        tol_dw[:, lo:hi] = gk.T @ rec["xq"].double().abs()
        x_t = x[:, lo:hi]
        if cfg.ir_mode == om.IR_STATIC:
            outside = rec["up"] | rec["lo"]
        elif cfg.ir_mode == om.IR_FAST:
            outside = (x_t > rec["ir"]) | (x_t < -rec["ir"])
        else:
            outside = None
        if outside is not None:
            tol_dir[t] = float(rec["ir"].double().abs()) * float((tol_dx[:, lo:hi] * outside).sum())
        if "lsq" in rec:
            lsq = rec["lsq"]
            tol_dlwc[t] = tol_dw[:, lo:hi].sum(dim=1) * lsq["max_q"] * lsq["grad_scale"] / lsq["chain"]
    return dict(dx=tol_dx, dw=tol_dw, dir=tol_dir, dlwc=tol_dlwc, db=None, near_out=near_out,
                n_keep=n_keep, spans=bounds, decisions=g.numel() * len(bounds))


def oracle_fwd_bwd(c, ties=True):
    """Run the oracle on a 'fwd_bwd' case; returns dict(out, dx, dw, db, dir). With ``ties`` the
    run is watched by a :class:`TieLog` and ``"_ties"`` holds :func:`tie_allowances`."""
    x, w, b, g = make_inputs(c)
    cfg = oracle_cfg(c)
    in_sizes = om.split_sizes(c["K"], c["max_input_size"])
    ir = case_input_range(c, len(in_sizes))
    torch.manual_seed(c["noise_seed"])
    lwc = make_learnable_clip(c, w) if c["clip"] == "learnable" else None
    log = TieLog() if ties else None
    if ties:
        with product_hook(log):
            out, saved = om.linear_forward(x, w, b, cfg, ir, c["training"], learnable_weight_clip=lwc)
    else:
        out, saved = om.linear_forward(x, w, b, cfg, ir, c["training"], learnable_weight_clip=lwc)
    dx, dw, db, dir_ = om.linear_backward(g, saved)
    res = dict(out=out, dx=dx, dw=dw, db=db if b is not None else None, dir=dir_,
               dlwc=saved.get("dlwc"))
    if ties:
        res["_ties"] = tie_allowances(c, saved, g, log)
    return res


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


def assert_close_ties(got, ref, rtol, ties, key, what=""):
    """Acceptance rule of a gradient: within ``rtol`` relative to the tensor's scale, except
    where a clamp decision that the oracle itself places within the accumulation error of the
    clamp (``ties`` from :func:`tie_allowances`) may have gone the other way: there by at most
    what those decisions carry, and on at most 0.1 % of the (row, channel, tile) decisions
    (counted by the tile spans of rows that show a difference; always at least one)."""
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    bad = rel_scale_mismatch(got, ref, rtol)
    n_bad = int(bad.sum())
    if n_bad == 0:
        return
    diff = (got.double() - ref.double()).abs()
    tol = None if ties is None else ties.get(key)
    assert tol is not None and ties["n_keep"] > 0, (
        f"{what}: {n_bad} elements differ, max |diff| {diff.max():.3e}, and the oracle has no clamp "
        f"decision within the accumulation error of its bound")
    tol = tol.reshape(ref.shape)
    slack = rtol * (ref.double().abs() + ref.double().abs().mean())
    over = bad & (diff > 1.01 * tol + slack)
    assert int(over.sum()) == 0, (
        f"{what}: {int(over.sum())} elements differ by more than the clamp ties of the oracle allow "
        f"(max |diff| {diff[over].max():.3e}, {ties['n_keep']} ties)")
    if bad.dim() == 2:
        spans = sum(int(bad[:, lo:hi].any(dim=1).sum()) for lo, hi in ties["spans"])
        cap = max(1, int(1e-3 * ties["decisions"]))
        assert spans <= cap, f"{what}: {spans} tile spans differ, more than 0.1 % of the clamp decisions ({cap})"
