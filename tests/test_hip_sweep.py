"""Seeded random sweeps of AnalogLinear and the convolutions against the CPU oracle: shapes that
fall on every kernel family (MFMA kernels on aligned, padded and channel-padded operands, sliced
contractions, predicated tails, the general kernels), all input-range modes, both resolution
conventions, clipping and on-the-fly weight quantisation. The hand-picked cases elsewhere pin
known corners; this net is for the combinations nobody thought of.

Left out on purpose: quantised weights together with an ADC (products of two integer grids land
exactly between two ADC levels for several per cent of the outputs, where the last bit of an
fp32 sum decides and a CPU and a GPU sum legitimately differ), and fast_mode (its range gradient
is the difference of two large bf16-rounded sums; the golden cases cover it).
"""
import math
import random

import pytest
import torch

from conv_cases import conv_case, make_conv_inputs, out_size
from golden_cases import DTYPES, case
from helpers import assert_close_lsb, case_input_range, oracle_cfg, oracle_fwd_bwd
from oracle import conv_mode as oc
from test_hip_linear import ROUNDING_STEP, check_against

pytestmark = pytest.mark.gpu

M_ROWS = [1, 3, 17, 64, 100, 130, 256, 300]
K_COLS = [8, 24, 64, 100, 128, 192, 256, 320, 384, 512, 520, 768, 1000, 1024]
N_OUT = [1, 5, 8, 10, 24, 64, 72, 100, 128, 200, 256, 520]
TILES = [-1, 64, 128, 256, 384, 512]


def linear_cases(seed, count):
    rng = random.Random(seed)
    cases = []
    for i in range(count):
        ir_mode = rng.choice(["none", "static", "static", "dynamic"])
        kw = dict(dtype=rng.choice(["bf16", "bf16", "f32"]), M=rng.choice(M_ROWS), K=rng.choice(K_COLS),
                  N=rng.choice(N_OUT), max_input_size=rng.choice(TILES), bias=rng.random() < 0.7,
                  ir_mode=ir_mode, w_scale=0.1, seed=100 + 1000 * seed + i)
        adc = False
        if ir_mode != "none":
            kw.update(inp_res=254, ir_init=rng.choice([1.0, 2.0, 3.0]), ir_decay=rng.choice([0.0, 0.01]))
            if rng.random() < 0.8:
                kw.update(out_res=rng.choice([254, 1 / 254, -1]),
                          out_bound=rng.choice([0.3, 0.6, 2.0, 10.0]))
                if kw["out_res"] == -1 and rng.random() < 0.5:
                    kw["out_bound"] = 0.0
                adc = kw["out_res"] != -1
            if rng.random() < 0.5:
                kw.update(clip="channel", clip_sigma=2.5)
        if not adc and rng.random() < 0.3:
            kw.update(weight_quant=rng.choice(["discretize", "discretize_per_channel"]),
                      modifier_res=rng.choice([30, 1 / 30]))
            if rng.random() < 0.4 and kw["weight_quant"] == "discretize_per_channel":
                kw.update(clip="learnable", lwc_scale=rng.choice([0.6, 1.0]))
        if rng.random() < 0.2:
            kw.update(training=False)
        cases.append(case(f"sweep_{seed}_{i}", **kw))
    return cases


LINEAR = linear_cases(0, 48) + linear_cases(1, 48)
# the same generator once more with every case in float16
LINEAR += [dict(c, dtype="f16", name=c["name"] + "_f16") for c in linear_cases(2, 32)]
# seed 3 holds float16 cases without an ADC in which a tile product lands on a rounding midpoint
LINEAR += [dict(c, dtype="f16", name=c["name"] + "_f16") for c in linear_cases(3, 48)]


def resolution_cases(seed, count):
    """DAC / ADC / weight-quantiser resolutions of every kind (numbers of states with few and with
    many significant bits, odd ones, relative resolutions) for the two 16-bit types: the quotient
    and step arithmetic of the kernels (products with reciprocals, a correction step, divisions)."""
    res = [2, 3, 5, 14, 30, 254, 255, 1000, 1022, 2046, 2047, 2048, 4094, 4095, 65534, 1 / 254, 1 / 30,
           0.37, 1 / 1022]
    rng = random.Random(seed)
    cases = []
    for i in range(count):
        kw = dict(M=rng.choice([17, 130, 256, 300]), K=rng.choice([64, 256, 512, 1024]),
                  N=rng.choice([8, 72, 128, 256]), max_input_size=rng.choice([-1, 64, 128, 256]),
                  ir_mode=rng.choice(["static", "dynamic"]), inp_res=rng.choice(res), out_res=rng.choice(res),
                  out_bound=rng.choice([0.3, 0.6, 2.0, 10.0]), ir_init=rng.choice([1.0, 2.0, 3.0]),
                  ir_decay=0.01, w_scale=0.1, seed=4000 + 100 * seed + i, clip=rng.choice(["none", "channel"]),
                  clip_sigma=2.5, bias=rng.random() < 0.5)
        if rng.random() < 0.3:
            kw.update(weight_quant=rng.choice(["discretize", "discretize_per_channel"]),
                      modifier_res=rng.choice(res))
        cases += [case(f"res_{seed}_{i}_{dt}", dtype=dt, **kw) for dt in ("f16", "bf16")]
    return cases


LINEAR += resolution_cases(1, 40)


def _named(gen, seed, count, name, dtype=None):
    found = [c for c in gen(seed, count) if c["name"] == name]
    assert len(found) == 1, name
    return dict(found[0], dtype=dtype, name=f"{name}_{dtype}") if dtype else found[0]


# Two configurations that longer runs of the generators above turned up, kept by name: in each the
# oracle itself places ONE tile output (row 151, tile 1 in the first; row 244, tile 8 among four
# candidates in the second) within the fp32 accumulation error of the step between the outermost
# ADC level and the first level beyond the bound. The GPU's sum falls on the other side: the output
# is the bound either way, the clamp mask differs, and with it that row's tile span of the input
# gradient (and that channel's span of the weight gradient) by g[m, n] * w[n, k] -- what
# check_against allows, and only there.
CLAMP_TIES = [
    _named(linear_cases, 41, 40, "sweep_41_31", "f16"),
    case("res_tie_f16", dtype="f16", M=300, K=1024, N=256, max_input_size=64, ir_mode="static", inp_res=2048,
         out_res=0.0009784735812133072, out_bound=0.6, ir_init=1.0, ir_decay=0.01, w_scale=0.1, seed=4090,
         clip="channel", clip_sigma=2.5, bias=True),
]
LINEAR += CLAMP_TIES
# float16 with ADC steps below the smallest normal float16 value (bounds of a few 1e-3: small
# weights): steps and quotients on the subnormal grid, where the kernels divide instead of
# multiplying with a reciprocal
LINEAR += [case(f"subnormal_step_{n}_f16", dtype="f16", M=130, K=256, N=72, max_input_size=128, ir_mode=mode,
                inp_res=254, out_res=n, out_bound=0.3, ir_init=1.0, ir_decay=0.01, w_scale=0.001, seed=4700 + i,
                clip="channel", clip_sigma=2.5, bias=False)
           for i, (n, mode) in enumerate([(14, "static"), (30, "dynamic"), (126, "static"), (254, "dynamic"),
                                          (510, "static"), (1000, "static"), (1022, "dynamic")])]


@pytest.fixture(autouse=True)
def _pad_channels_at_test_sizes(monkeypatch):
    """The host pads odd output widths only for large products; lower the threshold so that the
    sweep's sizes take that path too."""
    from aihwkit_lightning.nn.modules.hip_utils import hip_linear
    monkeypatch.setattr(hip_linear, "PAD_CHANNELS_MIN_WORK", 1 << 16)


def _summary(c):
    keys = ("dtype", "M", "K", "N", "max_input_size", "ir_mode", "out_res", "out_bound", "clip",
            "weight_quant", "training")
    return " ".join(f"{k}={c[k]}" for k in keys)


@pytest.mark.parametrize("c", LINEAR, ids=[c["name"] for c in LINEAR])
def test_random_linear_configurations(c):
    from hip_helpers import hip_fwd_bwd

    print(c["name"], _summary(c), flush=True)
    check_against(hip_fwd_bwd(c), oracle_fwd_bwd(c), c, c["name"])


def conv_cases(seed, count):
    rng = random.Random(seed)
    cases = []
    while len(cases) < count:
        ndim = rng.choice([1, 2, 2, 3])
        kernel = tuple(rng.choice([1, 2, 3, 5]) for _ in range(ndim))
        stride = tuple(rng.choice([1, 1, 2, 3]) for _ in range(ndim))
        # the reference (and this package) accept dilation only for two spatial dimensions
        dilation = tuple(rng.choice([1, 1, 2]) if ndim == 2 else 1 for _ in range(ndim))
        padding = tuple(rng.choice([0, 1, 2]) for _ in range(ndim))
        size = tuple(rng.choice([5, 7, 9, 12, 17, 30]) + dilation[d] * (kernel[d] - 1)
                     for d in range(ndim))
        if ndim == 3:
            size = tuple(min(s, 9 + dilation[d] * (kernel[d] - 1)) for d, s in enumerate(size))
        ir_mode = rng.choice(["none", "static", "dynamic"])
        kw = dict(dtype=rng.choice(["bf16", "f32"]), N=rng.choice([3, 8, 16, 40]),
                  max_input_size=rng.choice([-1, 9, 16, 64, 100]), ir_mode=ir_mode, w_scale=0.2,
                  seed=500 + len(cases), bias=rng.random() < 0.7)
        if ir_mode != "none":
            kw.update(inp_res=254, out_res=254, out_bound=rng.choice([1.0, 10.0]), ir_init=2.0,
                      ir_decay=0.01, clip=rng.choice(["none", "channel"]), clip_sigma=2.5)
        c = conv_case(f"conv_sweep_{seed}_{len(cases)}", ndim, rng.choice([0, 1, 2, 5]),
                      rng.choice([1, 3, 4, 8, 16, 24]), size, kernel, stride, padding, dilation, **kw)
        if min(out_size(c)) >= 1:
            cases.append(c)
    return cases


CONV = conv_cases(0, 48)
# a third of them once more in float16
CONV += [dict(c, dtype="f16", name=c["name"] + "_f16") for c in conv_cases(0, 48)[::3]]


@pytest.mark.parametrize("c", CONV, ids=[c["name"] for c in CONV])
def test_random_convolutions(c):
    from aihwkit_lightning.nn import AnalogConv1d, AnalogConv2d, AnalogConv3d
    from hip_helpers import rpu_config

    print(c["name"], {k: c[k] for k in ("ndim", "batch", "C", "N", "size", "kernel", "stride",
                                        "padding", "dilation", "dtype", "max_input_size",
                                        "ir_mode")}, flush=True)
    ndim, one = c["ndim"], c["ndim"] == 1
    x, w, b, g = make_conv_inputs(c)
    geo = {k: (c[k][0] if one else c[k]) for k in ("kernel", "stride", "padding", "dilation")}
    layer = {1: AnalogConv1d, 2: AnalogConv2d, 3: AnalogConv3d}[ndim](
        c["C"], c["N"], geo["kernel"], stride=geo["stride"], padding=geo["padding"],
        dilation=geo["dilation"], bias=b is not None, dtype=DTYPES[c["dtype"]],
        rpu_config=rpu_config(c))
    layer.set_weights_and_biases(w.unsqueeze(-2) if one else w, b)
    layer = layer.cuda().train(True)
    ir = case_input_range(c, len(layer.in_sizes))
    if ir is not None:
        layer.input_range.data = ir.cuda()
    xin = x.cuda().requires_grad_(True)
    out = layer(xin)
    out.backward(g.cuda())
    torch.cuda.synchronize()

    batched = c["batch"] > 0
    xb, gb = (x, g) if batched else (x.unsqueeze(0), g.unsqueeze(0))
    ref_out, saved = oc.conv_forward(xb, w, b, c["stride"], c["padding"], c["dilation"],
                                     oracle_cfg(c), ir, True)
    dx, dw, db, dir_ = oc.conv_backward(gb, saved)
    if not batched:
        ref_out, dx = ref_out[0], dx[0]
    rtol = {"f32": 1e-5, "bf16": 1e-2, "f16": 1e-3}[c["dtype"]]
    lsb = None
    if c["ir_mode"] == "static":  # an upper bound of the ADC step: 2 * range * out_bound * max|w| / 254
        lsb = 2 * 2.0 * c["out_bound"] * float(w.abs().max()) / 254 * 1.05
    elif c["ir_mode"] == "dynamic":  # the range is the patch's own abs-max
        lsb = 2 * float(x.abs().max()) * c["out_bound"] * float(w.abs().max()) / 254 * 1.05
    elif c["dtype"] in ROUNDING_STEP:
        # no ADC: a tile product on a rounding midpoint of the 16-bit type (see check_against)
        top = float(ref_out.abs().max())
        lsb = ROUNDING_STEP[c["dtype"]] * 2.0 ** math.ceil(math.log2(max(top, 1e-30)))
    def step16(ref):
        # float16 gradients: a per-tile partial on a rounding midpoint, as for the outputs
        if c["dtype"] != "f16":
            return None
        return ROUNDING_STEP["f16"] * 2.0 ** math.ceil(math.log2(max(float(ref.abs().max()), 1e-30)))

    assert_close_lsb(out.detach().cpu().float(), ref_out.float(), rtol, lsb, what="out")
    assert_close_lsb(xin.grad.cpu().float(), dx.float(), rtol, step16(dx), what="dx")
    wgrad = layer.weight.grad.cpu()
    assert_close_lsb((wgrad.squeeze(-2) if one else wgrad).float(), dw.float(), rtol, step16(dw), what="dw")
    if b is not None:
        assert_close_lsb(layer.bias.grad.cpu().float(), db.float(), rtol, step16(db), what="db")
    if dir_ is not None and layer.input_range.grad is not None:
        assert_close_lsb(layer.input_range.grad.cpu().float(), dir_.float(), rtol, None, what="dir")


@pytest.mark.parametrize("c", CLAMP_TIES, ids=[c["name"] for c in CLAMP_TIES])
def test_clamp_tie_cases_have_the_tie_in_the_oracle(c):
    """The two named cases differ from the oracle in the input gradient, and the oracle's own tie
    analysis names the place: a clamp decision within the accumulation error of the bound in
    exactly the row and tile span where the GPU's gradient differs, by no more than that one
    decision carries."""
    from hip_helpers import hip_fwd_bwd

    print(c["name"], _summary(c), flush=True)
    got, ref = hip_fwd_bwd(c), oracle_fwd_bwd(c)
    ties = ref["_ties"]
    assert 1 <= ties["n_keep"] <= 4
    diff = (got["dx"].double() - ref["dx"].double()).abs()
    rows = (diff > 1e-3 * float(ref["dx"].abs().max())).any(dim=1).nonzero().flatten().tolist()
    assert len(rows) <= 1
    for m in rows:
        cols = (diff[m] > 0).nonzero().flatten()
        span = [(lo, hi) for lo, hi in ties["spans"] if lo <= int(cols[0]) and int(cols[-1]) < hi]
        assert len(span) == 1, "the differences of a row lie within one tile"
        assert bool((diff[m] <= 1.01 * ties["dx"][m] + 1e-3 * ref["dx"][m].double().abs() + 1e-6).all())
        assert float(ties["dx"][m].max()) > 0
