"""CPU oracle for the AnalogLinear hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A from-scratch restatement, in plain CPU torch tensor ops, of what the reference's torch-mode
computes for one AnalogLinear layer: forward, the explicit (hand-derived) backward that its
autograd graph implies, and the memory-bound helpers around it. Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module,
and only as a checker or a timed baseline; nothing in ``aihwkit-lightning_amd/`` does.

Every function cites the reference lines it follows (paths relative to the reference's
``src/aihwkit_lightning/``). Tensors stay in the layer dtype throughout, so each elementwise
op rounds to that dtype exactly as torch does for the reference.

How the oracle itself is pinned (see ``tests/test_oracle_*.py``): golden vectors written by the
real reference (``tests/golden/make_golden.py``), the closed forms in the reference's own tests
(clipping, weight modifier, calibration max, quantisation idempotence), reductions to
``F.linear`` / brute force, ``torch.quantile`` for the quantile restatement, and Philox
known-answer vectors.
"""
from dataclasses import dataclass
from math import sqrt
from typing import Dict, List, Optional, Sequence, Tuple

import torch
from torch import Tensor

# quantisation / noise / clip selectors (plain strings: the oracle does not depend on the package)
NONE = "none"
DISCRETIZE = "discretize"
DISCRETIZE_PER_CHANNEL = "discretize_per_channel"
ADD_NORMAL = "add_normal"
ADD_NORMAL_PER_CHANNEL = "add_normal_per_channel"
IR_NONE, IR_STATIC, IR_DYNAMIC, IR_FAST = "none", "static", "dynamic", "fast"


@dataclass
class OracleCfg:
    """Flat view of the settings that influence one layer call."""

    max_input_size: int = -1
    inp_res: float = -1.0
    out_res: float = -1.0
    out_bound: float = 0.0
    out_noise: float = 0.0
    out_noise_per_channel: bool = False
    bound_per_channel: bool = False  # clip type is one of the per-channel kinds
    clip_learnable: bool = False     # clip type LEARNABLE_PER_CHANNEL
    ir_mode: str = IR_NONE
    ir_decay: float = 0.001
    ir_input_min_percentage: float = 0.95
    weight_quant: str = NONE
    weight_noise: str = NONE
    modifier_res: float = 0.0
    modifier_std: float = 0.0
    skip_rounding: bool = False


# --------------------------------------------------------------------------------------------
def split_sizes(size: int, max_size: int) -> List[int]:
    """K-tile sizes (nn/modules/linear.py:155-170)."""
    if max_size <= 0:
        return [size]
    n_tiles = -(-size // max_size)
    base, extra = divmod(size, n_tiles)
    return [base + 1 if i < extra else base for i in range(n_tiles)]


def tile_bounds(in_sizes: Sequence[int]) -> List[Tuple[int, int]]:
    """[(lo, hi)] column ranges of the tiles."""
    out, lo = [], 0
    for size in in_sizes:
        out.append((lo, lo + size))
        lo += size
    return out


def _acc(dtype: torch.dtype) -> torch.dtype:
    """Accumulation dtype of a matrix product: fp32 for bf16/fp32 tensors, fp64 for fp64."""
    return torch.float64 if dtype == torch.float64 else torch.float32


def matmul_rounded(a: Tensor, b: Tensor) -> Tensor:
    """a @ b accumulated in fp32 (fp64 for fp64 inputs) and rounded once to a's dtype."""
    acc = _acc(a.dtype)
    return (a.to(acc) @ b.to(acc)).to(a.dtype)


def _tiny(dtype: torch.dtype) -> float:
    return torch.finfo(dtype).tiny


def quant_step(bound: Tensor, res: float) -> Tensor:
    """Step of a quantiser given as #states (res > 1) or 1/#states, for a tensor bound
    (torch_utils/quant_utils.py:63-66)."""
    alpha = 2 * bound
    return alpha / res if res > 1.0 else alpha * res


def quantize(values: Tensor, step: Tensor, skip_rounding: bool = False,
             max_state: Optional[float] = None) -> Tensor:
    """round(clamp(values / max(step, tiny))) * step (torch_utils/quant_utils.py:78-99)."""
    out = values / step.clamp_min(_tiny(values.dtype))
    if max_state is not None:
        out = torch.clamp(out, min=-max_state, max=max_state)
    if not skip_rounding:
        out = out.round()
    return out * step


def sliced_abs_max(weights: Tensor, in_sizes: Sequence[int]) -> Tensor:
    """[T, N] per-tile per-row abs-max (torch_utils/torch_abs_max.py:17-39)."""
    return torch.stack([weights[:, lo:hi].abs().amax(dim=1) for lo, hi in tile_bounds(in_sizes)])


def sliced_std(x: Tensor, in_sizes: Sequence[int]) -> Tensor:
    """[T] unbiased std of each tile over all rows (torch_utils/torch_linear.py:342)."""
    return torch.stack([x[:, lo:hi].std() for lo, hi in tile_bounds(in_sizes)])


def quantize_weight_tile(w_t: Tensor, wmax_t: Tensor, kind: str, res: float) -> Tensor:
    """On-the-fly weight quantiser of one tile without learnable clipping
    (torch_utils/quant_utils.py:204-233): scale = wmax / n_states (per tile or per channel),
    UniformQuantize(w, scale, bound=1.0, max_quant_state=n_states/2)."""
    if kind == NONE:
        return w_t
    n_states = max(res, 1 / res)
    scale = wmax_t.max() / n_states if kind == DISCRETIZE else wmax_t / n_states
    step = 2.0 / scale if bool((scale > 1.0).all()) else 2.0 * scale
    step = step.clone()
    step[step == 0.0] = 1.0
    return quantize(w_t, step, False, n_states / 2)


def learned_clip_tile(w_t: Tensor, lwc_t: Tensor, kind: str, res: float) -> Tuple[Tensor, Dict]:
    """Weights of one tile under LEARNABLE_PER_CHANNEL clipping (clip_and_quantize,
    torch_utils/quant_utils.py:184-233, through UniformQuantize.forward :63-107). ``lwc_t`` is the
    learnable clip of the tile, [N, 1].
    No quantiser: clamp(w / c, -1, 1) * c (res = c, bound 0.5, max state 1, no rounding);
    DISCRETIZE_PER_CHANNEL: round(clamp(w / (2 c / n), +-n/2)) * (2 c / n).
    Returns the weights and what :func:`learned_clip_backward` needs."""
    assert kind in (NONE, DISCRETIZE_PER_CHANNEL), "per-channel clip cannot feed a per-tensor quantiser"
    tiny = _tiny(w_t.dtype)
    if kind == NONE:
        alpha, max_q, skip, passed = 1.0, 1.0, True, lwc_t
        chain = 1.0
    else:
        n_states = max(res, 1 / res)
        alpha, max_q, skip, passed = 2.0, n_states / 2, False, lwc_t / n_states
        chain = n_states
    step = alpha / passed if bool((passed > 1.0).all()) else alpha * passed
    step = step.clone()
    step[step == 0.0] = 1.0
    cstep = step.clamp_min(tiny)
    out = torch.clamp(w_t / cstep, min=-max_q, max=max_q)
    if not skip:
        out = out.round()
    out = out * step
    numel = w_t.numel()
    grad_scale = 1 / sqrt(numel) if skip else 2 * sqrt(max_q / numel)
    return out, dict(w=w_t, cstep=cstep, max_q=max_q, skip=skip, grad_scale=grad_scale, chain=chain)


def learned_clip_backward(grad_w_eff: Tensor, ctx: Dict) -> Tuple[Tensor, Tensor]:
    """LSQ backward of :func:`learned_clip_tile` (UniformQuantize.backward,
    torch_utils/quant_utils.py:123-153, written with the same tensor expressions so that the
    dtype promotions are torch's own): gradient to the weights where they were not clipped, and
    to the clip value [N] (through ``lwc / n_states`` when a quantiser follows)."""
    w, cstep, max_q = ctx["w"], ctx["cstep"], ctx["max_q"]
    q_w = w / cstep
    small = (q_w < -max_q).float()
    big = (q_w > max_q).float()
    middle = 1.0 - small - big
    if ctx["skip"]:
        grad_res = (small * (-max_q) + big * max_q) * grad_w_eff * ctx["grad_scale"]
    else:
        grad_res = ((small * (-max_q) + big * max_q + middle * (-q_w + q_w.round()))
                    * grad_w_eff * ctx["grad_scale"])
    grad_res = torch.sum(grad_res, dim=-1, keepdim=True).to(w.dtype)  # autograd casts to the input dtype
    grad_w = (middle * grad_w_eff).to(w.dtype)
    if ctx["chain"] != 1.0:
        grad_res = grad_res / ctx["chain"]
    return grad_w, grad_res.view(-1)


def noisy_weight_tile(w_t: Tensor, wmax_t: Tensor, kind: str, std_dev: float,
                      xi: Optional[Tensor] = None) -> Tensor:
    """w + std_dev * wmax * N(0,1) per tile (ADD_NORMAL) or per tile and channel
    (torch_utils/torch_linear.py:444-462). ``xi`` overrides the normal draw."""
    if kind == NONE:
        return w_t
    if xi is None:
        xi = torch.randn_like(w_t)
    ref = wmax_t.max() if kind == ADD_NORMAL else wmax_t
    return w_t + std_dev * ref * xi


# --------------------------------------------------------------------------------------------
def ir_init_update(x_t: Tensor, ir: Tensor, idx: Tensor, t: int, init_from_data: float,
                   alpha: float) -> None:
    """One data-initialisation step of tile t's input range, in place
    (torch_utils/torch_linear.py:338-352)."""
    i = idx[t]
    if i < init_from_data:
        std = x_t.std()
        if std > 0.0:
            ir[t] = ((ir[t].float() * i + alpha * std.float()) / (i + 1)).to(ir.dtype)
            idx[t] += 1
        ir[t] = ir[t].abs()


def ir_fast_update(x_t: Tensor, ir: Tensor, idx: Tensor, x_min: Tensor, x_max: Tensor, t: int,
                   init_from_data: float, momentum: float) -> None:
    """One fast_mode range update of tile t from the data x_t, in place
    (torch_utils/torch_linear.py:387-419): the running min / max start from the first batch, then
    follow with momentum (or as plain running extrema for momentum -1); the range is the larger
    magnitude of the two. All arithmetic is in the dtype of the buffers."""
    if not idx[t] < init_from_data:
        return
    act_min, act_max = x_t.min(), x_t.max()
    if x_min[t] > -1.1e-5 and x_max[t] < 1.1e-5:
        x_min[t] = x_min[t] + act_min
        x_max[t] = x_max[t] + act_max
    elif momentum == -1:
        x_min[t] = min(x_min[t], act_min)
        x_max[t] = max(x_max[t], act_max)
    else:
        x_min[t] = x_min[t] * momentum + act_min * (1 - momentum)
        x_max[t] = x_max[t] * momentum + act_max * (1 - momentum)
    idx[t] += 1
    ir[t] = max(x_min[t].abs(), x_max[t].abs())


# Test instrumentation: when set, ``PRODUCT_HOOK(xq, w_eff, y, post)`` sees every tile product of
# :func:`linear_forward` before noise / ADC / clamp and returns the product to go on with. The tie
# analysis of the GPU parity tests uses it to find (and to resolve the other way) products whose
# exact value lies within the fp32 accumulation error of a rounding decision; nothing else sets it.
PRODUCT_HOOK = None
# The same for the DAC: ``DAC_HOOK(xc, step, xq, skip_rounding)`` sees the clamped input of a tile,
# its quantisation step and the quantised input, and returns the quantised input to go on with.
# Networks of several layers use it: the input of a later layer comes out of exp / tanh, whose
# last place differs between a CPU and a GPU, so a DAC level can hang on that last place.
DAC_HOOK = None


def tile_output(y: Tensor, post: Dict) -> Tuple[Tensor, Optional[Tensor]]:
    """What follows the product of one tile (torch_utils/torch_linear.py:255-309): output noise
    (``post["noise"]``: the scaled normal draw), ADC with step ``post["step"]``, clamp to
    ``post["bound"]``. Returns the tile output and the mask of unclamped elements (or None)."""
    if post["noise"] is not None:
        y = y + post["noise"]
    keep = None
    if post["bound"] is not None:
        bound = post["bound"]
        if post["step"] is not None:
            y = quantize(y, post["step"], post["skip_rounding"])
        if post["clamp"]:
            keep = (y >= -bound) & (y <= bound)
            y = torch.clamp(y, min=-bound, max=bound)
    return y, keep


def linear_forward(
    x: Tensor,
    weights: Tensor,
    bias: Optional[Tensor],
    cfg: OracleCfg,
    input_range: Optional[Tensor],
    training: bool,
    out_xi: Optional[Sequence[Tensor]] = None,
    w_xi: Optional[Sequence[Tensor]] = None,
    learnable_weight_clip: Optional[Tensor] = None,
) -> Tuple[Tensor, Dict]:
    """Forward of one layer call on x[M, K] (torch_utils/torch_linear.py:116-314), tile by tile:
    input range -> DAC -> weight quantiser/noise -> product -> output noise -> ADC -> clamp ->
    sum in dtype -> bias. Returns the output and what the explicit backward needs.

    Normal draws come from torch's global generator in the reference's order (per tile: weight
    noise, then output noise) unless ``w_xi`` / ``out_xi`` (lists per tile) are given.
    """
    assert x.dim() == 2
    in_sizes = split_sizes(x.size(1), cfg.max_input_size)
    n_tiles = len(in_sizes)
    adc_on = cfg.out_res > 0
    bound_on = adc_on or cfg.out_bound > 0
    noise_on = training and cfg.out_noise > 0
    w_noise_on = training and cfg.weight_noise != NONE
    need_wmax = bound_on or noise_on or w_noise_on or cfg.weight_quant != NONE or cfg.clip_learnable
    out = 0.0
    saved: Dict = {"cfg": cfg, "in_sizes": in_sizes, "x": x, "tiles": []}
    for t, (lo, hi) in enumerate(tile_bounds(in_sizes)):
        x_t = x[:, lo:hi]
        rec: Dict = {}
        ir_t = None
        if cfg.ir_mode == IR_STATIC:
            ir_t = input_range[t]
            rec["up"] = x_t >= ir_t
            rec["lo"] = x_t <= -ir_t
            xc = torch.clamp(x_t, min=-ir_t, max=ir_t)
        elif cfg.ir_mode == IR_FAST:
            # plain torch.clamp with tensor bounds (torch_linear.py:421); its autograd rule is
            # restated in linear_backward
            ir_t = input_range[t]
            xc = torch.clamp(x_t, min=-ir_t, max=ir_t)
        elif cfg.ir_mode == IR_DYNAMIC:
            ir_t = x_t.abs().max(dim=-1, keepdim=True)[0]
            xc = x_t
        else:
            xc = x_t
        rec["ir"] = ir_t
        if cfg.inp_res > 0:
            dac_step = quant_step(ir_t, cfg.inp_res)
            xq = quantize(xc, dac_step, cfg.skip_rounding)
            if DAC_HOOK is not None:
                xq = DAC_HOOK(xc, dac_step, xq, cfg.skip_rounding)
        else:
            xq = xc
        w_t = weights[:, lo:hi]
        wmax_t = w_t.abs().amax(dim=-1, keepdim=True) if need_wmax else None
        if cfg.clip_learnable:
            # the clipped weights, and from here on the learned clip is the tile's "wmax"
            # (torch_linear.py:222-244)
            lwc_t = learnable_weight_clip[t].unsqueeze(-1)
            w_eff, rec["lsq"] = learned_clip_tile(w_t, lwc_t, cfg.weight_quant, cfg.modifier_res)
            wmax_t = lwc_t.view_as(wmax_t)
        else:
            w_eff = quantize_weight_tile(w_t, wmax_t, cfg.weight_quant, cfg.modifier_res)
        if w_noise_on:
            w_eff = noisy_weight_tile(w_eff, wmax_t, cfg.weight_noise, cfg.modifier_std,
                                      None if w_xi is None else w_xi[t])
        # one fp32-accumulated product, rounded once to the tensor dtype
        y = matmul_rounded(xq, w_eff.T)
        post: Dict = {"noise": None, "bound": None, "step": None, "clamp": cfg.out_bound > 0,
                      "skip_rounding": cfg.skip_rounding}
        if noise_on:
            wr = wmax_t.view(1, -1) if cfg.out_noise_per_channel else wmax_t.max()
            xi = torch.randn_like(y) if out_xi is None else out_xi[t]
            post["noise"] = wr * (cfg.out_noise / sqrt(n_tiles) * ir_t) * xi
        if bound_on:
            wb = wmax_t.view(1, -1) if cfg.bound_per_channel else wmax_t.max()
            post["bound"] = (ir_t * cfg.out_bound) * wb
            if adc_on:
                post["step"] = quant_step(post["bound"], cfg.out_res)
        if PRODUCT_HOOK is not None:
            y = PRODUCT_HOOK(xq, w_eff, y, post)
        y, keep = tile_output(y, post)
        out = out + y
        rec.update(xq=xq, w_eff=w_eff, keep=keep)
        saved["tiles"].append(rec)
    if bias is not None:
        out = out + bias
    return out, saved


def linear_backward(grad_out: Tensor, saved: Dict) -> Tuple[Tensor, Tensor, Tensor, Optional[Tensor]]:
    """Explicit backward of :func:`linear_forward` = what autograd computes for the reference
    graph: clamp mask (torch.clamp), straight-through ADC/DAC (quant_utils.py:152-156), product,
    input-range gradient (torch_linear.py:92-106) and straight-through input clamp
    (torch_linear.py:44-54). Returns (dx, dw, dbias, ir_grad or None); with a learnable weight
    clip its gradient [T, N] is stored as ``saved["dlwc"]``."""
    cfg: OracleCfg = saved["cfg"]
    x = saved["x"]
    dtype = x.dtype
    n_tiles = len(saved["in_sizes"])
    dx = torch.zeros_like(x)
    dw_parts = []
    ir_grad = torch.zeros(n_tiles, dtype=dtype) if cfg.ir_mode in (IR_STATIC, IR_FAST) else None
    for t, (lo, hi) in enumerate(tile_bounds(saved["in_sizes"])):
        rec = saved["tiles"][t]
        gy = grad_out if rec["keep"] is None else grad_out * rec["keep"]
        dw_t = matmul_rounded(gy.T, rec["xq"])
        if "lsq" in rec:
            dw_t, dlwc_t = learned_clip_backward(dw_t, rec["lsq"])
            saved.setdefault("dlwc", []).append(dlwc_t)
        dw_parts.append(dw_t)
        d = matmul_rounded(gy, rec["w_eff"])
        if cfg.ir_mode == IR_STATIC:
            ir_t, up, low = rec["ir"], rec["up"], rec["lo"]
            grad = torch.zeros_like(ir_t)
            grad += torch.clamp(d[up], min=None, max=0.0).sum()
            grad -= torch.clamp(d[low], min=0.0, max=None).sum()
            grad *= ir_t
            if cfg.ir_decay > 0:
                pct = 1.0 - (up | low).sum().div(up.numel())
                grad += cfg.ir_decay * ir_t * (pct > cfg.ir_input_min_percentage)
            ir_grad[t] = grad
            x_t = x[:, lo:hi]
            d = d.clone()
            d[(up | low) & (x_t.abs() != ir_t)] = 0.0
        elif cfg.ir_mode == IR_FAST:
            # autograd of clamp(x, min=-ir, max=ir) with tensor bounds: the gradient goes to x
            # inside [-ir, ir] (bounds included), to `max` where x > ir and to `min` where
            # x < -ir; each is reduced to a scalar in the tensor dtype, and min = -ir
            ir_t, x_t = rec["ir"], x[:, lo:hi]
            zero = torch.zeros_like(d)
            g_max = torch.where(x_t > ir_t, d, zero).sum()
            g_min = torch.where(x_t < -ir_t, d, zero).sum()
            ir_grad[t] = g_max + (-g_min)
            d = torch.where((x_t >= -ir_t) & (x_t <= ir_t), d, zero)
        dx[:, lo:hi] = d
    dw = torch.cat(dw_parts, dim=1)
    dbias = grad_out.sum(dim=0)
    if "dlwc" in saved:  # gradient of learnable_weight_clip [T, N], left in ``saved``
        saved["dlwc"] = torch.stack(saved["dlwc"])
    return dx, dw, dbias, ir_grad


# --------------------------------------------------------------------------------------------
def clip_weights(weights: Tensor, sigma: float, per_channel: bool) -> Tensor:
    """clamp(W, +-sigma * std) with the std of each row or of the whole matrix
    (nn/modules/linear.py:269-283). Returns a new tensor."""
    bound = sigma * (weights.std(1, keepdim=True) if per_channel else weights.std())
    return torch.clamp(weights, -bound, bound)


def quantize_weights(weights: Tensor, in_sizes: Sequence[int], kind: str, res: float,
                     learnable_clip: Optional[Tensor] = None) -> Tensor:
    """Post-training per-tile quantisation (nn/modules/linear.py:285-303 -> clip_and_quantize,
    torch_utils/quant_utils.py:159-236): with the slice's own abs-max, or -- under a learned
    per-channel clip ``learnable_clip [T, N]`` -- the clamp at the learned clip (no quantiser) /
    the quantiser whose range is the learned clip. Returns a new tensor."""
    out = weights.clone()
    for t, (lo, hi) in enumerate(tile_bounds(in_sizes)):
        w_t = weights[:, lo:hi]
        if learnable_clip is not None:
            out[:, lo:hi] = learned_clip_tile(w_t, learnable_clip[t].unsqueeze(-1), kind, res)[0]
        else:
            out[:, lo:hi] = quantize_weight_tile(w_t, w_t.abs().amax(dim=1, keepdim=True), kind, res)
    return out


def calibrate_max(batches: Sequence[Tensor], in_sizes: Sequence[int]) -> Tensor:
    """Running per-tile abs-max over batches (inference/calibration/calibration.py:110-124)."""
    cache = torch.full((len(in_sizes),), float("-inf"), dtype=batches[0].dtype)
    for x in batches:
        x = x.reshape(-1, x.size(-1))
        for t, (lo, hi) in enumerate(tile_bounds(in_sizes)):
            cache[t] = max(cache[t], x[:, lo:hi].abs().max())
    return cache


def kept_rows(x: Tensor) -> Tensor:
    """Rows of x[n, K] that are not all zero (calibration.py:94-95)."""
    x = x.reshape(-1, x.size(-1))
    return x[~(x == 0.0).all(-1)]


def quantile_linear(values: Tensor, q: float) -> Tensor:
    """q-quantile with linear interpolation of a 1-d fp32 tensor, restated from the definition
    torch.quantile implements (aten/src/ATen/native/Sorting.cpp, quantile_compute): the rank
    q * (n - 1) is evaluated in fp32, the two neighbouring order statistics are blended with the
    two-sided lerp formula. NaN for an empty input or one that holds a NaN."""
    values = values.float().flatten()
    n = values.numel()
    if n == 0 or bool(torch.isnan(values).any()):
        return torch.tensor(float("nan"))
    ordered = torch.sort(values).values
    rank = torch.tensor(q, dtype=torch.float32) * torch.tensor(float(n - 1), dtype=torch.float32)
    below = torch.floor(rank)
    weight = rank - below
    lo = ordered[int(below)]
    hi = ordered[int(torch.ceil(rank))]
    diff = hi - lo
    return lo + weight * diff if float(weight) < 0.5 else hi - diff * (1.0 - weight)


def moving_update(ir: Tensor, idx: Tensor, t: int, val: float) -> None:
    """input_range[t] <- (input_range[t] * idx[t] + val) / (idx[t] + 1); idx[t] += 1, evaluated as
    the reference does: Python float times an int32 tensor element gives an fp32 0-dim tensor,
    the result is cast to the range's dtype (calibration.py:144-147)."""
    old_val = ir[t].item()
    new_val = (old_val * idx[t] + val) / (idx[t] + 1)
    ir[t] = new_val.type_as(ir)
    idx[t] += 1


def calibrate_moving(batches: Sequence[Tensor], in_sizes: Sequence[int], kind: str, dtype,
                     alpha: float = 3.0, q: float = 0.99995) -> Tuple[Tensor, Tensor]:
    """MOVING_STD / MOVING_QUANTILE (calibration.py:126-147): per batch and tile the statistic
    of the kept rows (alpha * std in the data dtype, or the quantile of the fp32 values, or the
    abs-max when q == 1), folded into a running mean that starts from 3.0. Returns the final
    ranges and the trace of ranges seen before each batch."""
    n_tiles = len(in_sizes)
    ir = torch.full((n_tiles,), 3.0, dtype=dtype)
    idx = torch.zeros(n_tiles, dtype=torch.int32)
    trace = []
    for x in batches:
        trace.append(ir.float().clone())
        rows = kept_rows(x)
        if rows.size(0) == 0:
            # A batch of all-zero rows (the hidden state of a recurrent layer's first step): the
            # reference's statistic of the empty selection is NaN (std) or an error (quantile,
            # max), which ruins the range for good. Stated here as what the product does
            # instead: such a batch is passed over.
            continue
        for t, (lo, hi) in enumerate(tile_bounds(in_sizes)):
            part = rows[:, lo:hi]
            if kind == "MovingStd":
                val = alpha * part.std().item()
            elif q == 1.0:
                val = part.abs().max().item()
            else:
                val = quantile_linear(part, q).item()
            moving_update(ir, idx, t, val)
    return ir, torch.stack(trace)


def calibrate_cache_quantile(batches: Sequence[Tensor], in_sizes: Sequence[int], q: float,
                             max_samples: int, dtype) -> Tensor:
    """CACHE_QUANTILE (calibration.py:100-110, :305-313): the kept rows of every batch join a
    cache that is re-drawn to at most max_samples rows with torch.randperm (global CPU
    generator); the range of a tile is the quantile of the cached fp32 values."""
    cache = torch.zeros(0, sum(in_sizes))
    for x in batches:
        cache = torch.cat([cache, kept_rows(x).float()])
        cache = cache[torch.randperm(cache.size(0))[:max_samples]]
    out = torch.empty(len(in_sizes), dtype=dtype)
    for t, (lo, hi) in enumerate(tile_bounds(in_sizes)):
        out[t] = quantile_linear(cache[:, lo:hi], q).item()
    return out


# --------------------------------------------------------------------------------------------
# Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
# SC'11) in pure Python ints, to pin the device generator bit for bit.
_M0, _M1, _W0, _W1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85
_MASK = 0xFFFFFFFF


def philox4x32_10(ctr: Sequence[int], key: Sequence[int]) -> Tuple[int, int, int, int]:
    """Ten Philox rounds on a 4x32-bit counter with a 2x32-bit key."""
    c0, c1, c2, c3 = ctr
    k0, k1 = key
    for _ in range(10):
        p0, p1 = _M0 * c0, _M1 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & _MASK, p1 & _MASK, ((p0 >> 32) ^ c3 ^ k1) & _MASK, p0 & _MASK
        k0, k1 = (k0 + _W0) & _MASK, (k1 + _W1) & _MASK
    return c0, c1, c2, c3


def philox_counter(stream: int, tile: int, c0: int, c1: int, offset: int) -> Tuple[int, int, int, int]:
    """Counter layout of the device generator: (c0, c1, stream << 24 | tile, offset lo).
    Output noise: stream 0, c0 = n, c1 = (m // 16) * 2 + ((m // 4) % 2); the 8 normals of a call
    are rows 16 * (m // 16) + 4 * ((m // 4) % 2) + (j % 4) + 8 * (j // 4).
    Weight noise: stream 1, tile 0, c0 = k // 8, c1 = n; the 8 normals are k % 8 = 0..7."""
    return c0 & _MASK, c1 & _MASK, ((stream << 24) | tile) & _MASK, offset & _MASK
