"""GPU parity of the analog linear operator (through AnalogLinear -> custom ops -> C ABI)
against the CPU oracle and the reference's golden vectors.

Acceptance rule (the path's stated tolerance): noise disabled -> outputs and gradients within
1e-5 (fp32) / 1e-2 (bf16) / 1e-3 (fp16) relative to the tensor scale; elements outside that must
be at most one ADC LSB off (without an ADC: one step of the 16-bit type) and at most 0.1 % of the
tensor. Noise enabled -> mean and std of the injected noise
within 1 % of the configured values.
"""
import math

import pytest
import torch

from golden_cases import CASES, DTYPES, case, make_inputs
from helpers import (assert_close_lsb, assert_close_ties, golden, golden_tensor, oracle_fwd_bwd,
                     rel_scale_mismatch)
from oracle import torch_mode as om

pytestmark = pytest.mark.gpu

NOISELESS = [
    c for c in CASES
    if c["kind"] == "fwd_bwd" and c["out_noise"] == 0 and c["weight_noise"] == "none"
]
RTOL = {"f32": 1e-5, "bf16": 1e-2, "f16": 1e-3}
# spacing of the 16-bit values in [0.5, 1)
ROUNDING_STEP = {"bf16": 2.0 ** -8, "f16": 2.0 ** -11}


def adc_lsb(c, wmax_scale=None):
    """A generous upper bound of one ADC step for a case (None when the ADC is off)."""
    if c["out_res"] <= 0:
        return None
    n = c["out_res"] if c["out_res"] > 1 else 1.0 / c["out_res"]
    ir_max = max(c["ir_values"]) if c["ir_values"] else c["ir_init"]
    if c["ir_mode"] == "dynamic":
        ir_max = 6.0 * c["x_scale"]
    w_max = 6.0 * c["w_scale"] if wmax_scale is None else wmax_scale
    return 2.0 * ir_max * c["out_bound"] * w_max / n


def check_against(res, ref, c, tag, ties=None):
    """``ties``: the oracle's record of the decisions that hang on the accumulation order
    (``helpers.tie_allowances``; taken from ``ref["_ties"]`` when the oracle produced ``ref``)."""
    from hip_helpers import hip_fwd_bwd  # noqa: F401  (import checks the package loads)

    rtol = RTOL[c["dtype"]]
    ties = ref.get("_ties") if ties is None else ties
    lsb = adc_lsb(c)
    if c["dtype"] in ROUNDING_STEP:
        # Without an ADC (or with one finer than the type itself: 65534 states) the last rounding
        # is the tile product's own, to the 16-bit type. A product whose fp32 sum lies within a few
        # fp32 steps of the midpoint between two 16-bit values is rounded up or down by the order of
        # the summation, which differs between the MFMA kernels and the CPU: such an element may be
        # one 16-bit step (at the tensor's largest magnitude, the bound of a tile product) away,
        # under the same 0.1 % cap as the ADC's steps.
        top = float(ref["out"].abs().max())
        step16 = ROUNDING_STEP[c["dtype"]] * 2.0 ** math.ceil(math.log2(max(top, 1e-30)))
        lsb = step16 if lsb is None else torch.clamp_min(torch.as_tensor(lsb, dtype=torch.float64), step16)
    want = ref["out"].float().to(res["out"].dtype)
    assert_close_lsb(res["out"], want, rtol, lsb, what=f"{tag} out")
    if ties is not None:
        # an output may be a step off only where the oracle itself finds a tile product within the
        # accumulation error of a change of ADC level or clamp decision
        stray = rel_scale_mismatch(res["out"], want, rtol) & ~ties["near_out"]
        assert not bool(stray.any()), f"{tag} out: {int(stray.sum())} elements differ where no tile has a tie"
    # Gradients: a flipped ADC level never enters them (straight-through); a flipped clamp decision
    # of one (row, channel, tile) does, over the whole tile span of that row of dx and of that
    # channel of dw (and from there the input-range and learnable-clip gradients). The bias
    # gradient does not see the mask.
    for key in ("dx", "dw", "db", "dir", "dlwc"):
        if ref.get(key) is None:
            continue
        assert res.get(key) is not None, f"{tag}: no {key} from the HIP path"
        assert_close_ties(res[key].float(), ref[key].float(), rtol, ties, key, what=f"{tag} {key}")


@pytest.mark.parametrize("c", NOISELESS, ids=[c["name"] for c in NOISELESS])
def test_golden_cases_match_oracle_and_reference(c):
    from hip_helpers import hip_fwd_bwd

    res = hip_fwd_bwd(c)
    ref = oracle_fwd_bwd(c)
    check_against(res, ref, c, c["name"] + " vs oracle")
    gold = {k: golden_tensor(f"{c['name']}/{k}") if f"{c['name']}/{k}" in golden() else None
            for k in ("out", "dx", "dw", "db", "dir", "dlwc")}
    check_against(res, gold, c, c["name"] + " vs reference", ties=ref["_ties"])


SHAPES = [
    case("edge_f32", M=130, K=300, N=257, max_input_size=128, ir_mode="static", inp_res=254,
         out_res=254, out_bound=10.0, clip="channel", clip_sigma=2.5, ir_decay=0.01,
         ir_values=[2.0, 2.5, 3.0], seed=21),
    case("edge_bf16", dtype="bf16", M=130, K=304, N=257, max_input_size=128, ir_mode="static",
         inp_res=254, out_res=254, out_bound=10.0, clip="channel", clip_sigma=2.5, ir_decay=0.01,
         ir_values=[2.0, 2.5, 3.0], seed=21),
    case("vec_bf16_static", dtype="bf16", M=256, K=1024, N=384, max_input_size=256, ir_mode="static",
         inp_res=254, out_res=254, out_bound=10.0, clip="channel", clip_sigma=2.5, ir_decay=0.01,
         seed=22),
    case("vec_bf16_dynamic", dtype="bf16", M=256, K=1024, N=384, max_input_size=512,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=10.0, clip="channel", clip_sigma=2.5,
         seed=23),
    case("vec_f32_dynamic", M=192, K=512, N=256, max_input_size=256, ir_mode="dynamic", inp_res=254,
         out_res=254, out_bound=10.0, seed=24),
    case("vec_bf16_many_tiles", dtype="bf16", M=128, K=1152, N=128, max_input_size=64,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=25),
    case("fast_bf16_clamped", dtype="bf16", M=264, K=512, N=136, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=28),
    case("fast_bf16_dynamic_clamped", dtype="bf16", M=256, K=512, N=256, max_input_size=256,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.3, w_scale=0.1, seed=29),
    case("fast_bf16_plain", dtype="bf16", M=256, K=768, N=256, max_input_size=256, seed=30),
    case("vec_f32_plain", M=200, K=256, N=136, max_input_size=-1, seed=26),
    case("one_token_bf16", dtype="bf16", M=1, K=512, N=512, max_input_size=256, ir_mode="static",
         inp_res=254, out_res=254, out_bound=10.0, seed=27),
    # splits whose tiles do not start on 256-column boundaries: padded tile layout of xq / w_eff
    case("pad_bf16_uneven_clamped", dtype="bf16", M=256, K=1000, N=128, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=31),
    case("pad_bf16_extra_tiles", dtype="bf16", M=192, K=1003, N=64, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=10.0, clip="channel", clip_sigma=2.5,
         ir_decay=0.01, ir_values=[1.5, 2.0, 2.5, 3.0], seed=32),
    case("pad_bf16_576_dynamic", dtype="bf16", M=128, K=1152, N=192, max_input_size=576,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.3, w_scale=0.1, seed=33),
    case("pad_bf16_plain", dtype="bf16", M=64, K=300, N=64, max_input_size=128, seed=34),
    # equal tiles of a multiple of 8: padded operands, dense x / dx straight from the kernel
    case("pad_bf16_384_static_clamped", dtype="bf16", M=320, K=768, N=128, max_input_size=384,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01,
         ir_values=[1.5, 2.5], w_scale=0.1, seed=39),
    case("pad_bf16_fast_mode", dtype="bf16", M=128, K=520, N=64, max_input_size=256, ir_mode="fast",
         ir_values=[0.8, 2.5, 1.5], inp_res=254, out_res=254, out_bound=1.5, clip="channel",
         clip_sigma=2.5, w_scale=0.3, seed=35),
    # narrow layers with many rows: the weight-gradient kernel cuts the rows into slices
    case("sliced_dw_bf16_clamped", dtype="bf16", M=1536, K=512, N=128, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=37),
    case("pad_bf16_sliced_dw", dtype="bf16", M=1088, K=1000, N=64, max_input_size=256,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.3, w_scale=0.1, seed=38),
    # row counts and channel counts that are not multiples of 64: the MFMA backward ends its
    # contraction in one predicated chunk (N % 8 == 0 is what remains required)
    case("tail_bf16_rows_clamped", dtype="bf16", M=203, K=512, N=128, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=40),
    case("tail_bf16_channels_clamped", dtype="bf16", M=256, K=512, N=72, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=41),
    case("tail_bf16_both_dynamic", dtype="bf16", M=45, K=768, N=200, max_input_size=256,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.3, w_scale=0.1, seed=42),
    case("tail_bf16_one_row", dtype="bf16", M=1, K=512, N=8, max_input_size=256, ir_mode="static",
         inp_res=254, out_res=254, out_bound=10.0, seed=43),
    case("tail_pad_bf16_rows", dtype="bf16", M=1100, K=1000, N=40, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=44),
    case("tail_pad_bf16_384", dtype="bf16", M=130, K=768, N=24, max_input_size=384, ir_mode="static",
         inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_values=[1.5, 2.5], w_scale=0.1,
         seed=45),
    # few rows and many channels (a recurrent step, a small batch): the input-gradient kernel
    # cuts the channels into slices and a second kernel sums them and applies the epilogue
    case("sliced_dx_bf16_clamped", dtype="bf16", M=48, K=512, N=1024, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=46),
    case("sliced_dx_pad_bf16_384", dtype="bf16", M=70, K=768, N=640, max_input_size=384,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01,
         ir_values=[1.5, 2.5], w_scale=0.1, seed=47),
    case("sliced_dx_tail_bf16_dynamic", dtype="bf16", M=33, K=512, N=1000, max_input_size=256,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.3, w_scale=0.1, seed=48),
    case("sliced_dx_fast_mode", dtype="bf16", M=16, K=512, N=2048, max_input_size=256, ir_mode="fast",
         ir_values=[0.8, 2.5], inp_res=254, out_res=254, out_bound=1.5, clip="channel",
         clip_sigma=2.5, w_scale=0.05, seed=49),
    # uneven split: the element-wise epilogue stays unsliced
    case("pad_bf16_uneven_wide", dtype="bf16", M=40, K=1000, N=1024, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=50),
    # equal tiles of a multiple of 64 but an output width that is not a multiple of 8, too small
    # for channel padding: the general kernels
    case("bf16_aligned_tiles_odd_width", dtype="bf16", M=64, K=512, N=10, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=10.0, w_scale=0.1, seed=55),
    # output widths that are not a multiple of 8: zero channels are appended for the MFMA kernels
    case("padn_bf16_static_clamped", dtype="bf16", M=256, K=512, N=100, max_input_size=256,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=51),
    case("padn_bf16_384_dynamic", dtype="bf16", M=130, K=768, N=75, max_input_size=384,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.3, w_scale=0.1, seed=52),
    case("padn_bf16_pertensor_nobias", dtype="bf16", M=96, K=1000, N=61, max_input_size=256,
         bias=False, ir_mode="static", ir_init=2.0, inp_res=1 / 254, out_res=1 / 254, out_bound=2.0,
         w_scale=0.1, ir_decay=0.0, seed=53),
    # converter resolutions with more than 8 significant bits: the quantiser steps come from a
    # division (the product with 2 / n is only exact for n of up to 8 bits)
    case("bf16_10bit_static", dtype="bf16", M=200, K=512, N=136, max_input_size=256,
         ir_mode="static", inp_res=1022, out_res=1022, out_bound=0.6, ir_decay=0.01, ir_init=2.0,
         w_scale=0.1, seed=56),
    case("bf16_16bit_dynamic", dtype="bf16", M=130, K=512, N=72, max_input_size=256,
         ir_mode="dynamic", inp_res=65534, out_res=65534, out_bound=0.3, w_scale=0.1, seed=57),
    case("bf16_odd_states_static", dtype="bf16", M=96, K=768, N=64, max_input_size=384,
         ir_mode="static", inp_res=1001, out_res=1001, out_bound=0.6, ir_values=[1.5, 2.5],
         w_scale=0.1, seed=58),
    case("pad_bf16_lsq", dtype="bf16", M=64, K=200, N=64, max_input_size=100, ir_mode="static",
         clip="learnable", lwc_scale=0.7, weight_quant="discretize_per_channel", modifier_res=30,
         w_scale=0.3, inp_res=254, out_res=254, out_bound=10.0, seed=36),
]


# float16 has the same kernel set as bfloat16 (the forward for large grids excepted): a selection
# of the shapes above once more in float16, and two grids of a few hundred blocks
SHAPES += [dict(c, name=c["name"].replace("bf16", "f16"), dtype="f16") for c in SHAPES if c["name"] in (
    "edge_bf16", "vec_bf16_static", "vec_bf16_dynamic", "vec_bf16_many_tiles", "fast_bf16_clamped",
    "fast_bf16_dynamic_clamped", "one_token_bf16", "pad_bf16_uneven_clamped", "tail_bf16_both_dynamic",
    "bf16_10bit_static", "bf16_16bit_dynamic", "bf16_odd_states_static", "pad_bf16_lsq",
    "sliced_dw_bf16_clamped")]
# float16 takes the ADC step by a product for state counts of up to 11 significant bits (the
# twins above) and by a division beyond: 4095 states, learned and dynamic range
SHAPES += [
    case(f"f16_12bit_{mode}", dtype="f16", M=200, K=512, N=136, max_input_size=256, ir_mode=mode,
         inp_res=4095, out_res=4095, out_bound=0.6, ir_decay=0.01, ir_init=2.0, w_scale=0.1, seed=64)
    for mode in ("static", "dynamic")
]
# tiles narrower than the 8 inputs one thread of the weight kernels handles (several tiles per
# thread), with the on-the-fly weight quantiser per tile and channel
SHAPES += [
    case(f"narrow_tiles_{dt}_{ms}", dtype=dt, M=17, K=100, N=24, max_input_size=ms, ir_mode="static",
         inp_res=254, ir_init=2.0, ir_decay=0.01, weight_quant="discretize_per_channel", modifier_res=30,
         w_scale=0.1, seed=63)
    for dt in ("f32", "bf16", "f16") for ms in (1, 3, 6)
]
SHAPES += [
    case("grid_f16_static_clamped", dtype="f16", M=1536, K=1024, N=1024, max_input_size=512,
         ir_mode="static", inp_res=254, out_res=254, out_bound=0.9, clip="channel", clip_sigma=2.5,
         ir_decay=0.01, ir_init=3.0, w_scale=0.02, seed=61),
    case("grid_f16_dynamic_clamped", dtype="f16", M=1024, K=1024, N=1280, max_input_size=256,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.9, clip="channel", clip_sigma=2.5,
         w_scale=0.02, seed=62),
]


@pytest.mark.parametrize("c", SHAPES, ids=[c["name"] for c in SHAPES])
def test_seeded_shapes_match_oracle(c):
    from hip_helpers import hip_fwd_bwd

    res = hip_fwd_bwd(c)
    ref = oracle_fwd_bwd(c)
    check_against(res, ref, c, c["name"])


def test_leading_dims_and_1d_input():
    from hip_helpers import make_layer

    c = case("nd", M=24, K=64, N=48, max_input_size=32, ir_mode="static", inp_res=254, out_res=254,
             out_bound=10.0, seed=31)
    x, w, b, _ = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    flat = layer(x.cuda())
    nd = layer(x.cuda().view(2, 3, 4, 64))
    assert nd.shape == (2, 3, 4, 48)
    assert torch.equal(nd.reshape(24, 48), flat)
    one = layer(x[0].cuda())
    assert one.shape == (48,)
    assert torch.equal(one, flat[0])
    empty = layer(x[:0].cuda())
    assert empty.shape == (0, 48)
    # no rows, with gradients asked for: zeros for the input and every parameter
    x_empty = x[:0].cuda().requires_grad_(True)
    layer.zero_grad(set_to_none=True)
    layer(x_empty).sum().backward()
    assert x_empty.grad.shape == x_empty.shape
    for param in layer.parameters():
        if param.requires_grad:
            assert param.grad is not None and not bool(param.grad.any())


def _as_view(t, layout):
    """A device tensor equal to ``t`` [M, K] whose memory is laid out as ``layout`` says."""
    rows, cols = t.shape
    if layout == "offset_by_one_element":      # data pointer not on a 16-byte boundary
        buf = torch.empty(rows * cols + 3, dtype=t.dtype, device="cuda")
        view = buf[1:1 + rows * cols].view(rows, cols)
    elif layout == "columns_3_on_of_wider_rows":  # odd offset and a row stride larger than K
        view = torch.empty(rows, cols + 5, dtype=t.dtype, device="cuda")[:, 3:3 + cols]
    elif layout == "wider_rows":
        view = torch.empty(rows, cols + 8, dtype=t.dtype, device="cuda")[:, :cols]
    elif layout == "transposed":
        view = torch.empty(cols, rows, dtype=t.dtype, device="cuda").t()
    else:
        return t.cuda()
    view.copy_(t)
    return view


@pytest.mark.parametrize("layout", ["offset_by_one_element", "columns_3_on_of_wider_rows", "wider_rows",
                                    "transposed"])
@pytest.mark.parametrize("name", ["fast_bf16_clamped", "fast_f16_dynamic_clamped", "edge_f32",
                                  "pad_bf16_uneven_clamped"])
def test_inputs_and_gradients_that_are_views(name, layout):
    """The input and the incoming gradient as views of other storage (misaligned pointers, row
    strides that are not K, a transposed buffer): the same results, bit for bit, as with
    contiguous tensors."""
    from hip_helpers import hip_fwd_bwd, make_layer

    c = next(s for s in SHAPES if s["name"] == name)
    x, w, b, g = make_inputs(c)
    want = hip_fwd_bwd(c, inputs=(x, w, b, g))
    layer = make_layer(c, inputs=(x, w, b, g))
    xin = _as_view(x, layout).requires_grad_(True)
    torch.manual_seed(c["noise_seed"])
    out = layer(xin)
    out.backward(_as_view(g, layout))
    assert torch.equal(out.detach().cpu(), want["out"])
    assert torch.equal(xin.grad.cpu(), want["dx"])
    assert torch.equal(layer.weight.grad.cpu(), want["dw"])
    if want["db"] is not None:
        assert torch.equal(layer.bias.grad.cpu(), want["db"])
    if want["dir"] is not None:
        assert torch.equal(layer.input_range.grad.cpu(), want["dir"])


@pytest.mark.parametrize("name", ["sliced_dx_bf16_clamped", "pad_bf16_384_static_clamped",
                                  "pad_bf16_uneven_clamped"])
def test_no_grad_forward_equals_the_differentiable_forward(name):
    """Under no_grad the layer keeps nothing for a backward pass (and may take another operand
    layout); the output is the same, and the parameters' in-place state is untouched."""
    from hip_helpers import make_layer

    c = [s for s in SHAPES if s["name"] == name][0]
    x, w, b, _ = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    layer.eval()
    want = layer(x.cuda().requires_grad_(True))
    assert want.requires_grad
    with torch.no_grad():
        got = layer(x.cuda())
    assert not got.requires_grad
    assert torch.equal(got, want.detach())


@pytest.mark.parametrize("name", ["pad_bf16_uneven_clamped", "pad_bf16_384_static_clamped"])
def test_misaligned_gradient_with_padded_layout(name):
    """A gradient that starts 2 bytes off a 16-byte boundary (a slice of a larger buffer): with the
    operands in the padded tile layout the host copies it, as no other kernel reads that layout."""
    from hip_helpers import make_layer

    c = [s for s in SHAPES if s["name"] == name][0]
    x, w, b, g = make_inputs(c)
    ref = oracle_fwd_bwd(c)
    layer = make_layer(c, inputs=(x, w, b, g))
    buf = torch.zeros(g.numel() + 1, dtype=g.dtype, device="cuda")
    buf[1:] = g.cuda().reshape(-1)
    g_off = buf[1:].view(g.shape)
    assert g_off.data_ptr() % 16 != 0
    xin = x.cuda().requires_grad_(True)
    out = layer(xin)
    out.backward(g_off)
    res = dict(out=out.detach().cpu(), dx=xin.grad.cpu(), dw=layer.weight.grad.cpu(),
               db=layer.bias.grad.cpu() if layer.bias is not None else None,
               dir=None if layer.input_range is None or layer.input_range.grad is None
               else layer.input_range.grad.cpu())
    check_against(res, ref, c, name + " misaligned gradient")


@pytest.mark.parametrize("name", ["sliced_dx_bf16_clamped", "pad_bf16_uneven_clamped",
                                  "padn_bf16_static_clamped", "edge_f32"])
def test_frozen_weights_reuse_what_depends_on_the_weights(name):
    """Inside ``frozen_weights()`` the per-tile abs-max and the padded operand copies are computed
    by the first call only; results and gradients are those of ordinary calls, and a weight change
    after the block is seen again."""
    from hip_helpers import make_layer

    c = [s for s in SHAPES if s["name"] == name][0]
    x, w, b, g = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    xin = x.cuda().requires_grad_(True)
    want = layer(xin)
    want.backward(g.cuda())
    want_dx, want_dw = xin.grad.clone(), layer.weight.grad.clone()
    xin.grad = None
    layer.zero_grad(set_to_none=True)
    with layer.frozen_weights():
        first = layer(xin)
        assert layer._weight_cache, "nothing was kept for the next call"
        second = layer(xin)
        second.backward(g.cuda())
    assert layer._weight_cache is None
    assert torch.equal(first, want) and torch.equal(second, want)
    assert torch.equal(xin.grad, want_dx) and torch.equal(layer.weight.grad, want_dw)
    with torch.no_grad():
        layer.weight.mul_(0.5)
        changed = layer(x.cuda())
    assert not torch.equal(changed, want)


def test_padded_channels_with_noise_stay_finite():
    """Output noise scaled by the whole tile also lands on the appended channels; nothing of it
    may leak into the result."""
    from hip_helpers import make_layer

    c = case("padn_noise", dtype="bf16", M=256, K=512, N=100, max_input_size=256, ir_mode="static",
             inp_res=254, out_res=254, out_bound=10.0, out_noise=0.1, clip="channel", clip_sigma=2.5,
             weight_noise="add_normal_per_channel", modifier_std=0.02, w_scale=0.1, seed=54)
    x, w, b, g = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    xin = x.cuda().requires_grad_(True)
    out = layer(xin)
    assert out.shape == (256, 100) and torch.isfinite(out).all()
    out.backward(g.cuda())
    assert layer.weight.grad.shape == (100, 512) and torch.isfinite(layer.weight.grad).all()
    assert torch.isfinite(xin.grad).all() and torch.isfinite(layer.bias.grad).all()
    quiet = dict(c, out_noise=0.0, weight_noise="none")
    ref = make_layer(quiet, inputs=(x, w, b, None))(x.cuda())
    err = (out.float() - ref.float()).std() / ref.float().std()
    assert 0.0 < err < 0.2  # the noise is there, and it is noise-sized


def test_parameters_on_another_device_are_rejected():
    from hip_helpers import rpu_config
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.exceptions import HipBackendError

    c = case("cpu", M=4, K=16, N=8)
    layer = AnalogLinear(16, 8, rpu_config=rpu_config(c))  # parameters on the CPU
    with pytest.raises(HipBackendError, match="move the layer"):
        layer(torch.randn(4, 16).cuda())


def test_cpu_tensor_is_rejected():
    from hip_helpers import rpu_config
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.exceptions import HipBackendError

    c = case("cpu", M=4, K=16, N=8)
    layer = AnalogLinear(16, 8, rpu_config=rpu_config(c))
    with pytest.raises(HipBackendError):
        layer(torch.randn(4, 16))


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("per_channel", [False, True])
def test_output_noise_statistics(dtype, per_channel):
    """Per tile, the injected noise is N(0, out_noise/sqrt(T) * IR_t * wmax): mean and std of
    (noisy - clean) / expected_std within 1 %, measured with ADC and clamp off."""
    from hip_helpers import make_layer

    c = case("noise", dtype=dtype, M=1024, K=256, N=512, max_input_size=128, ir_mode="static",
             inp_res=254, out_noise=0.5, out_noise_per_channel=per_channel, ir_values=[2.0, 3.0],
             w_scale=0.05, seed=41, bias=False)
    x, w, b, _ = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    torch.manual_seed(7)
    noisy = layer(x.cuda()).float().cpu()
    layer.eval()
    clean = layer(x.cuda()).float().cpu()
    wmax = om.sliced_abs_max(w.float(), layer.in_sizes)  # [T, N]
    ir = torch.tensor(c["ir_values"])
    per_tile = (0.5 / 2 ** 0.5) * ir[:, None] * (wmax if per_channel else wmax.amax(1, keepdim=True))
    expected = per_tile.pow(2).sum(0).sqrt()  # [N] or [1]: tiles add independently
    z = (noisy - clean) / expected
    tol = 0.02 if dtype == "bf16" else 0.01  # bf16 rounding of the sum adds its own small variance
    assert abs(float(z.mean())) < 0.01
    assert abs(float(z.std()) - 1.0) < tol
    # successive calls draw fresh noise; the same torch seed replays it
    torch.manual_seed(7)
    layer.train()
    again = layer(x.cuda()).float().cpu()
    assert torch.equal(again, noisy)
    other = layer(x.cuda()).float().cpu()
    assert not torch.equal(other, noisy)


@pytest.mark.parametrize("kind", ["add_normal", "add_normal_per_channel"])
def test_weight_noise_statistics(kind):
    """dX = g @ W_eff exposes the noisy weights: with g = I the rows of dX are W_eff's rows."""
    from hip_helpers import make_layer

    c = case("wnoise", M=256, K=512, N=256, max_input_size=256, weight_noise=kind, modifier_std=0.1,
             w_scale=0.05, seed=42, bias=False)
    x, w, b, _ = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    xin = x.cuda().requires_grad_(True)
    torch.manual_seed(3)
    out = layer(xin)
    out.backward(torch.eye(256, device="cuda"))
    w_eff = xin.grad.cpu()  # [256 (= n), K]
    wmax = om.sliced_abs_max(w, layer.in_sizes)  # [T, N]
    for t, (lo, hi) in enumerate(om.tile_bounds(layer.in_sizes)):
        ref = wmax[t][:, None] if kind == "add_normal_per_channel" else wmax[t].max()
        z = (w_eff[:, lo:hi] - w[:, lo:hi]) / (0.1 * ref)
        assert abs(float(z.mean())) < 0.01
        assert abs(float(z.std()) - 1.0) < 0.01
    # the forward used the same noisy weights
    assert torch.allclose(out.detach().cpu(), x @ w_eff.T, atol=1e-4)


@pytest.mark.parametrize("c", [c for c in SHAPES if c["name"].startswith(("pad_", "tail_pad_"))],
                         ids=lambda c: c["name"])
def test_padded_layout_is_what_runs(c):
    """The pad_* shapes must actually take the padded tile layout (a non-zero stride from the
    library), or the cases above would only exercise the general kernels."""
    from aihwkit_lightning.nn.modules.hip_utils.ops import tile_stride

    n_tiles = len(om.split_sizes(c["K"], c["max_input_size"]))
    stride = tile_stride(c["K"], n_tiles, torch.bfloat16)
    assert stride > 0 and stride % 256 == 0 and stride * n_tiles <= 4 * c["K"]
    assert c["N"] % 8 == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("rows,k_in,max_size", [(5, 1003, 256), (64, 300, 128), (3, 7, 2), (130, 2304, 576)])
def test_pad_unpad_tiles_bit_exact(rows, k_in, max_size, dtype):
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS

    sizes = om.split_sizes(k_in, max_size)
    stride = (max(sizes) + 255) // 256 * 256
    x = torch.randn(rows, k_in, generator=torch.Generator().manual_seed(5)).to(dtype)
    want = torch.zeros(rows, len(sizes) * stride, dtype=dtype)
    for t, (lo, hi) in enumerate(om.tile_bounds(sizes)):
        want[:, t * stride:t * stride + hi - lo] = x[:, lo:hi]
    padded = OPS.pad_tiles(x.cuda(), sizes, stride)
    assert torch.equal(padded.cpu(), want)
    assert torch.equal(OPS.unpad_tiles(padded, sizes, stride).cpu(), x)


def test_misaligned_input_with_padded_layout():
    """An input whose storage does not start on a 16-byte boundary (a view into a larger buffer)
    through the padded-layout path: the input-gradient kernel wants x aligned like dx, the op
    makes the copy."""
    from hip_helpers import make_layer

    c = [s for s in SHAPES if s["name"] == "pad_bf16_extra_tiles"][0]
    x, w, b, g = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, g))
    flat = torch.zeros(x.numel() + 8, dtype=x.dtype, device="cuda")
    flat[3:3 + x.numel()] = x.cuda().reshape(-1)
    xin = flat[3:3 + x.numel()].view_as(x).requires_grad_(True)
    assert xin.data_ptr() % 16 != 0
    out = layer(xin)
    out.backward(g.cuda())
    ref = oracle_fwd_bwd(c)
    res = dict(out=out.detach().cpu(), dx=xin.grad.cpu(), dw=layer.weight.grad.cpu(),
               db=layer.bias.grad.cpu(), dir=layer.input_range.grad.cpu())
    check_against(res, ref, c, "misaligned x")


@pytest.mark.parametrize("rows", [1, 48, 130])
@pytest.mark.parametrize("ir_mode", ["static", "dynamic"])
def test_few_row_forward_with_one_tile_per_block_is_bit_identical(rows, ir_mode):
    """Few rows: every K-tile of an output block goes to a block of its own and the per-tile
    results are added in tile order by a second kernel. Output (noise on: the normals are keyed
    by tile, row and column, not by block), clamp mask and gradients equal the one-block-per-
    output-block forward bit for bit."""
    from hip_helpers import make_layer
    from aihwkit_lightning.nn.modules.hip_utils import ops

    c = case(f"few_rows_{rows}_{ir_mode}", dtype="bf16", M=rows, K=1536, N=1024, max_input_size=512,
             ir_mode=ir_mode, inp_res=254, out_res=254, out_bound=0.4, out_noise=0.05,
             ir_decay=0.01, ir_init=2.0, w_scale=0.1, training=True, seed=61)
    x, w, b, g = make_inputs(c)
    results = []
    for split in (True, False):
        ops.SPLIT_FEW_ROW_FORWARD = split
        try:
            layer = make_layer(c, inputs=(x, w, b, g))
            torch.manual_seed(11)   # the Philox seed of the call comes from torch's generator
            inp = x.cuda().requires_grad_()
            out = layer(inp)
            out.backward(g.cuda())
            results.append((out.detach().clone(), inp.grad.clone(), layer.weight.grad.clone(),
                            layer.bias.grad.clone()))
        finally:
            ops.SPLIT_FEW_ROW_FORWARD = True
    for got, want, what in zip(results[0], results[1], ("out", "dx", "dw", "db")):
        assert torch.equal(got, want), what
    assert results[0][0].abs().max() > 0


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_counter_left_at_minus_infinity_means_the_ranges_are_set(dtype):
    """Calibration leaves ``input_range_update_idx`` at -inf (reference calibration.py:159). A
    training forward of such a layer with ``init_from_data > 0`` -- e.g. after its state was
    loaded into a fresh layer -- must treat the initialisation as finished: the ranges stay."""
    from hip_helpers import make_layer

    c = case("minus_inf", dtype=dtype, M=32, K=64, N=16, max_input_size=32, ir_mode="static",
             init_from_data=10, inp_res=254, seed=33)
    x, w, b, _ = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    layer.input_range.data.fill_(1.5)
    layer.input_range_update_idx.data.fill_(float("-inf"))
    state = {k: v.clone() for k, v in layer.state_dict().items()}
    fresh = make_layer(c, inputs=(x, w, b, None))
    fresh.load_state_dict(state)
    fresh.train()
    out = fresh(x.cuda())
    assert bool(torch.isfinite(out.float()).all())
    assert torch.equal(fresh.input_range.data.cpu().float(), torch.full((2,), 1.5))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("clamps", [False, True], ids=["nothing_clamped", "some_clamped"])
def test_clamp_flag_token_and_a_stale_match(dtype, clamps):
    """The forward's one-word "something was clamped" flag in its two forms: cleared by the
    library and set non-zero (token 0), or the caller's per-call token stored into a word that
    nobody cleared. Both give the backward the same answer; and a word that holds the token
    although nothing was clamped (a stale value in reused memory) only makes the backward apply
    a mask without bits: the same gradients, bit for bit."""
    from aihwkit_lightning.nn.modules.hip_utils import library as L
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS

    gen = torch.Generator().manual_seed(21)
    m_rows, k_in, n_out, tile = 256, 512, 256, 256
    in_sizes = [tile] * (k_in // tile)
    x = torch.randn(m_rows, k_in, generator=gen).to(dtype).cuda()
    w = (0.05 * torch.randn(n_out, k_in, generator=gen)).to(dtype).cuda()
    g = torch.randn(m_rows, n_out, generator=gen).to(dtype).cuda()
    ir = torch.full((len(in_sizes),), 3.0).to(dtype).cuda()
    out_bound = 1.0 if clamps else 1000.0
    fcfg = [254.0, 254.0, out_bound, 0.0, 0.01, 0.95]
    wmax, tile_max, _, _ = OPS.weight_prep(w, in_sizes, 0, 0, 1.0, 0.0, 0, 0, False, False)

    def run(token, overwrite_flag=None):
        icfg = [L.AHL_IR_STATIC, 0, 1, 1, 0, 0, 0, L.AHL_IR_GRAD_LEARNED, 0, 0, token]
        xq, _ = OPS.dac(x, ir, in_sizes, icfg, fcfg)
        y, keep, flag = OPS.linear_fwd(x, xq, w, None, ir, wmax, tile_max, in_sizes, icfg, fcfg, True)
        if overwrite_flag is not None:
            flag.fill_(overwrite_flag)
        dx, ir_grad = OPS.linear_bwd_dx(g, keep, flag, w, x, ir, in_sizes, icfg, fcfg)
        dw, dbias = OPS.linear_bwd_dw(g, keep, flag, None, xq, ir, in_sizes, icfg, fcfg, True)
        return y, keep, int(flag.item()), dx, ir_grad, dw, dbias

    classic = run(0)
    token = 0x5EED1234
    tokened = run(token)
    if dtype == torch.bfloat16:   # the MFMA kernels of the bf16 path track clamping; the general
        assert (classic[2] != 0) == clamps   # kernels always tell the backward to honour the mask
    assert (tokened[2] == token) or not clamps
    if clamps:
        assert bool((classic[1] != 0).any())
    stale = run(token, overwrite_flag=token)   # the word says "clamped" whatever happened
    for a, b, c in zip(classic, tokened, stale):
        if isinstance(a, torch.Tensor):
            assert torch.equal(a, b) and torch.equal(a, c)
