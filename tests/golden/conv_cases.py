"""Convolution cases shared by the fixture writer (``make_golden_conv.py``) and the tests.

Every case is a golden-case dict of ``golden_cases.py`` (same configuration keys; ``M``, ``K``
unused) plus the geometry: ``ndim``, ``batch`` (0 = unbatched input), ``C`` input channels,
``size`` spatial input size, ``kernel``, ``stride``, ``padding``, ``dilation``. Inputs are
regenerated from seeds.
"""
import torch

from golden_cases import DEFAULTS, DTYPES

_ADC8 = dict(inp_res=254, out_res=254, out_bound=10.0)
_TIGHT = dict(inp_res=254, out_res=254, out_bound=1.5, clip="channel", clip_sigma=2.5,
              ir_decay=0.01, w_scale=0.3)


def conv_case(name, ndim, batch, C, size, kernel, stride, padding, dilation=None, **kw):
    out = dict(DEFAULTS)
    unknown = set(kw) - set(DEFAULTS)
    assert not unknown, unknown
    out.update(kw)
    out.update(name=name, ndim=ndim, batch=batch, C=C, size=tuple(size), kernel=tuple(kernel),
               stride=tuple(stride), padding=tuple(padding),
               dilation=tuple(dilation) if dilation is not None else (1,) * ndim)
    return out


CONV_CASES = [
    # no non-idealities: must equal torch's own convolution
    conv_case("conv2d_f32_plain", 2, 2, 3, (7, 6), (3, 3), (1, 1), (1, 1), N=5, seed=30),
    conv_case("conv1d_f32_plain", 1, 3, 4, (11,), (3,), (2,), (1,), N=6, seed=31),
    conv_case("conv3d_f32_plain", 3, 2, 2, (4, 7, 5), (2, 3, 2), (1, 2, 1), (1, 0, 1), N=4, seed=32),
    # 2-d: three tiles of nine patch entries, uneven stride/padding/dilation, learned input
    # range tight enough to clip, ADC with a bound tight enough to clamp
    conv_case("conv2d_f32_adc", 2, 2, 3, (9, 8), (3, 3), (2, 1), (1, 0), (1, 2), N=5,
              max_input_size=10, ir_mode="static", ir_values=[0.8, 2.5, 1.5], seed=33, **_TIGHT),
    conv_case("conv2d_bf16_adc", 2, 2, 3, (9, 8), (3, 3), (2, 1), (1, 0), (1, 2), N=5, dtype="bf16",
              max_input_size=10, ir_mode="static", ir_values=[0.8, 2.5, 1.5], seed=33, **_TIGHT),
    conv_case("conv2d_f32_dynamic", 2, 2, 3, (6, 7), (2, 3), (1, 2), (0, 1), N=6, max_input_size=9,
              ir_mode="dynamic", clip="channel", clip_sigma=2.5, w_scale=0.3, seed=34, **_ADC8),
    conv_case("conv2d_f32_unbatched", 2, 0, 3, (7, 6), (3, 2), (1, 1), (1, 1), N=4, max_input_size=9,
              ir_mode="static", ir_values=[1.0, 2.0], w_scale=0.3, seed=35, **_ADC8),
    conv_case("conv2d_f32_noise", 2, 2, 2, (5, 6), (3, 3), (1, 1), (1, 1), N=4, max_input_size=9,
              ir_mode="static", out_noise=0.1, weight_noise="add_normal_per_channel",
              modifier_std=0.05, w_scale=0.3, seed=36, **_ADC8),
    # 1-d: stored as a height-one 2-d kernel; three tiles of four
    conv_case("conv1d_f32_adc", 1, 3, 4, (11,), (3,), (2,), (1,), N=6, max_input_size=5,
              ir_mode="static", ir_values=[0.8, 2.5, 1.5], seed=37, **_TIGHT),
    conv_case("conv1d_bf16_adc", 1, 3, 4, (11,), (3,), (2,), (1,), N=6, dtype="bf16",
              max_input_size=5, ir_mode="static", ir_values=[0.8, 2.5, 1.5], seed=37, **_TIGHT),
    # 3-d: three tiles of eight
    conv_case("conv3d_f32_adc", 3, 2, 2, (4, 7, 5), (2, 3, 2), (1, 2, 1), (1, 0, 1), N=4,
              max_input_size=9, ir_mode="static", ir_values=[0.8, 2.5, 1.5], seed=38, **_TIGHT),
    conv_case("conv3d_bf16_adc", 3, 2, 2, (4, 7, 5), (2, 3, 2), (1, 2, 1), (1, 0, 1), N=4,
              dtype="bf16", max_input_size=9, ir_mode="static", ir_values=[0.8, 2.5, 1.5], seed=38,
              **_TIGHT),
    conv_case("conv3d_f32_unbatched", 3, 0, 2, (3, 5, 4), (2, 2, 2), (1, 1, 2), (0, 1, 1), N=3,
              max_input_size=8, ir_mode="dynamic", w_scale=0.3, seed=39, **_ADC8),
]

CONV_CASES_BY_NAME = {c["name"]: c for c in CONV_CASES}


def out_size(c):
    """Spatial output size of a case."""
    return tuple(
        (c["size"][d] + 2 * c["padding"][d] - c["dilation"][d] * (c["kernel"][d] - 1) - 1)
        // c["stride"][d] + 1
        for d in range(c["ndim"])
    )


def make_conv_inputs(c):
    """x [B, C, *size] (or [C, *size]), weight [N, C, *kernel], bias [N] or None, and the
    gradient of the output, in the case's dtype."""
    dtype = DTYPES[c["dtype"]]
    gen = torch.Generator().manual_seed(2000 + c["seed"])
    lead = (c["batch"],) if c["batch"] > 0 else ()
    x = (torch.randn(*lead, c["C"], *c["size"], generator=gen) * c["x_scale"]).to(dtype)
    w = (torch.randn(c["N"], c["C"], *c["kernel"], generator=gen) * c["w_scale"]).to(dtype)
    b = (torch.randn(c["N"], generator=gen) * 0.1).to(dtype) if c["bias"] else None
    g = torch.randn(*lead, c["N"], *out_size(c), generator=gen).to(dtype)
    return x, w, b, g
