"""GPU parity of the analog convolutions (AnalogConv1d/2d/3d -> custom ops -> C ABI) against the
CPU oracle and the reference's golden vectors, and of the three data-movement entry points
(ahl_im2col, ahl_col2im, ahl_transpose_batched), which are pure copies / fixed-order sums and
therefore compared bit for bit.

Layer acceptance rule as for the linear operator: 1e-5 (fp32) / 1e-2 (bf16) relative to the
tensor scale, elements outside that at most one ADC LSB off and at most 0.1 % of the tensor.
"""
import os

import numpy as np
import pytest
import torch

from conv_cases import CONV_CASES, conv_case, make_conv_inputs
from golden_cases import DTYPES
from helpers import assert_close_lsb, case_input_range, oracle_cfg
from oracle import conv_mode as oc
from oracle import torch_mode as om

pytestmark = pytest.mark.gpu

CONV_GOLDEN = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                        "conv_cases.npz")))
RTOL = {"f32": 1e-5, "bf16": 1e-2, "f16": 1e-3}

GEOMS = [
    # batch, C, size(3), kernel(3), stride(3), padding(3), dilation(3)
    (2, 3, (1, 9, 8), (1, 3, 3), (1, 2, 1), (0, 1, 0), (1, 1, 2)),   # K = 27: scalar stores
    (3, 8, (1, 1, 37), (1, 1, 5), (1, 1, 2), (0, 0, 2), (1, 1, 1)),  # 1-d, K = 40: vector stores
    (2, 4, (5, 6, 7), (2, 3, 2), (1, 2, 1), (1, 0, 1), (1, 1, 1)),   # 3-d, K = 48
    (1, 16, (1, 33, 29), (1, 3, 3), (1, 1, 1), (0, 1, 1), (1, 1, 1)),  # K = 144, odd sizes
    (2, 2, (3, 4, 5), (3, 4, 5), (1, 1, 1), (0, 0, 0), (1, 1, 1)),   # kernel == input
    # channel counts that are multiples of 8: the tiled fold kernel
    (2, 8, (4, 9, 70), (2, 3, 3), (1, 2, 1), (1, 1, 1), (1, 1, 1)),   # 3-d, two column tiles
    (2, 16, (1, 17, 131), (1, 3, 5), (1, 2, 3), (0, 1, 2), (1, 2, 2)),  # strides and dilations
    (1, 8, (1, 5, 200), (1, 1, 7), (1, 1, 4), (0, 0, 0), (1, 1, 1)),   # stride > 1 along the row
    (3, 24, (1, 12, 12), (1, 1, 1), (1, 1, 1), (0, 0, 0), (1, 1, 1)),   # 1 x 1 kernel
    (2, 8, (1, 9, 7), (1, 3, 3), (1, 2, 1), (0, 1, 1), (1, 1, 1)),     # narrow image: 8 x 8 pixel patches
    (1, 8, (2, 30, 28), (2, 5, 3), (1, 3, 2), (0, 2, 1), (1, 1, 1)),   # 2 x 32 patches, strides, 3-d
    (2, 16, (1, 14, 14), (1, 3, 3), (1, 1, 1), (0, 1, 1), (1, 2, 2)),  # 4 x 16 patches, dilation
    # 5 x 5 kernel on a 40-wide image: the 256-pixel fold kernel's staging area does not fit,
    # the 64-pixel one's does
    (2, 8, (1, 12, 40), (1, 5, 5), (1, 1, 1), (0, 2, 2), (1, 1, 1)),
    (1, 16, (1, 28, 28), (1, 3, 3), (1, 1, 1), (0, 1, 1), (1, 1, 1)),  # 8 x 32 patches of the 256-pixel kernel
    (1, 8, (3, 10, 18), (2, 3, 3), (2, 2, 1), (1, 0, 1), (1, 1, 1)),   # 3-d, strides, 256 pixels
]


def _geom_list(geom):
    batch, chan, size, kernel, stride, padding, dilation = geom
    return [batch, chan, *size, *kernel, *stride, *padding, *dilation]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("geom", GEOMS, ids=[f"geom{i}" for i in range(len(GEOMS))])
def test_patch_kernels_bit_exact(geom, dtype):
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS, conv_out_size

    batch, chan, size, kernel, stride, padding, dilation = geom
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(batch, chan, *size, generator=gen).to(dtype)
    want_cols, out = oc.conv_patches(x, kernel, stride, padding, dilation)
    assert conv_out_size(_geom_list(geom)) == out
    cols = OPS.im2col(x.cuda(), _geom_list(geom))
    assert torch.equal(cols.cpu(), want_cols)
    g = torch.randn(want_cols.shape, generator=gen).to(dtype)
    want_dx = oc.conv_fold(g, x.shape, kernel, stride, padding, dilation)
    dx = OPS.col2im(g.cuda(), _geom_list(geom))
    assert torch.equal(dx.cpu(), want_dx)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 33, 65), (2, 64, 32), (5, 7, 130), (1, 300, 17),
                                   # whole 16-byte vectors on both sides: the vector kernel,
                                   # full and partial 64 x 64 tiles
                                   (3, 784, 256), (2, 72, 200), (1, 8, 8), (4, 136, 24)])
def test_transpose_batched_bit_exact(shape, dtype):
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS

    src = torch.randn(*shape, generator=torch.Generator().manual_seed(8)).to(dtype)
    got = OPS.transpose_batched(src.cuda())
    assert got.is_contiguous() and torch.equal(got.cpu(), src.transpose(1, 2).contiguous())


@pytest.mark.gpu
def test_unfold3d_is_the_unfold_of_a_volume():
    """Two anchors that do not go through the oracle: a volume of depth 1 with a depth-1 kernel
    is ``torch.nn.functional.unfold``'s 2-D case bit for bit, and for a real volume
    ``weight.view(O, -1) @ unfold3d(x)`` is ``conv3d(x, weight)``; the gradient is the adjoint."""
    from aihwkit_lightning.nn.modules.conv import unfold3d

    gen = torch.Generator().manual_seed(31)
    flat = torch.randn(2, 3, 1, 9, 11, generator=gen)
    got = unfold3d(flat.cuda(), (1, 3, 2), padding=(0, 1, 2), stride=(1, 2, 1))
    want = torch.nn.functional.unfold(flat[:, :, 0], (3, 2), padding=(1, 2), stride=(2, 1))
    assert torch.equal(got.cpu(), want)
    assert torch.equal(unfold3d(flat[0].cuda(), (1, 3, 2), (0, 1, 2), (1, 2, 1)).cpu(), want[0])

    vol = torch.randn(2, 4, 6, 7, 5, generator=gen, dtype=torch.float64).float()
    weight = torch.randn(5, 4, 3, 2, 3, generator=gen)
    x = vol.cuda().requires_grad_()
    cols = unfold3d(x, (3, 2, 3), padding=(1, 0, 2), stride=(2, 1, 1))
    ref_in = vol.clone().requires_grad_()
    ref = torch.nn.functional.conv3d(ref_in, weight, padding=(1, 0, 2), stride=(2, 1, 1))
    out = (weight.view(5, -1).cuda() @ cols).view(ref.shape)
    assert torch.allclose(out.cpu(), ref, rtol=1e-5, atol=1e-5)
    g = torch.randn(ref.shape, generator=gen)
    out.backward(g.cuda())
    ref.backward(g)
    assert torch.allclose(x.grad.cpu(), ref_in.grad, rtol=1e-5, atol=1e-5)


def make_conv_layer(c, w, b):
    from hip_helpers import rpu_config
    from aihwkit_lightning.nn import AnalogConv1d, AnalogConv2d, AnalogConv3d

    cls = {1: AnalogConv1d, 2: AnalogConv2d, 3: AnalogConv3d}[c["ndim"]]
    one = c["ndim"] == 1
    pick = (lambda v: v[0]) if one else (lambda v: v)
    layer = cls(c["C"], c["N"], pick(c["kernel"]), stride=pick(c["stride"]),
                padding=pick(c["padding"]), dilation=pick(c["dilation"]), bias=b is not None,
                dtype=DTYPES[c["dtype"]], rpu_config=rpu_config(c))
    layer.set_weights_and_biases(w.unsqueeze(-2) if one else w, b)
    layer = layer.cuda()
    ir = case_input_range(c, len(layer.in_sizes))
    if ir is not None:
        layer.input_range.data = ir.cuda()
    layer.train(c["training"])
    return layer


def hip_conv_fwd_bwd(c, inputs):
    x, w, b, g = inputs
    layer = make_conv_layer(c, w, b)
    xin = x.cuda().requires_grad_(True)
    torch.manual_seed(c["noise_seed"])
    out = layer(xin)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    wgrad = layer.weight.grad.cpu()
    res = dict(out=out.detach().cpu(), dx=xin.grad.cpu(),
               dw=wgrad.squeeze(-2) if c["ndim"] == 1 else wgrad, db=None, dir=None)
    if b is not None:
        res["db"] = layer.bias.grad.cpu()
    if layer.input_range is not None and layer.input_range.grad is not None:
        res["dir"] = layer.input_range.grad.cpu()
    return res


def oracle_conv_fwd_bwd(c, inputs):
    x, w, b, g = inputs
    batched = c["batch"] > 0
    xb, gb = (x, g) if batched else (x.unsqueeze(0), g.unsqueeze(0))
    ir = case_input_range(c, len(om.split_sizes(w[0].numel(), c["max_input_size"])))
    torch.manual_seed(c["noise_seed"])
    out, saved = oc.conv_forward(xb, w, b, c["stride"], c["padding"], c["dilation"], oracle_cfg(c),
                                 ir, c["training"])
    dx, dw, db, dir_ = oc.conv_backward(gb, saved)
    if not batched:
        out, dx = out.squeeze(0), dx.squeeze(0)
    return dict(out=out, dx=dx, dw=dw, db=db if b is not None else None, dir=dir_)


def check(res, ref, c, tag):
    from test_hip_linear import adc_lsb

    rtol = RTOL[c["dtype"]]
    assert_close_lsb(res["out"].float(), ref["out"].float(), rtol, adc_lsb(c), what=f"{tag} out")
    for key in ("dx", "dw", "db", "dir"):
        if ref.get(key) is None:
            continue
        assert res.get(key) is not None, f"{tag}: no {key} from the HIP path"
        assert_close_lsb(res[key].float(), ref[key].float(), rtol, None, what=f"{tag} {key}")


NOISELESS = [c for c in CONV_CASES if c["out_noise"] == 0 and c["weight_noise"] == "none"]


@pytest.mark.parametrize("c", NOISELESS, ids=[c["name"] for c in NOISELESS])
def test_golden_convolutions_match_oracle_and_reference(c):
    inputs = make_conv_inputs(c)
    res = hip_conv_fwd_bwd(c, inputs)
    check(res, oracle_conv_fwd_bwd(c, inputs), c, c["name"] + " vs oracle")
    gold = {k: torch.from_numpy(CONV_GOLDEN[f"{c['name']}/{k}"])
            if f"{c['name']}/{k}" in CONV_GOLDEN else None for k in ("out", "dx", "dw", "db", "dir")}
    check(res, gold, c, c["name"] + " vs reference")


_ADC = dict(inp_res=254, out_res=254, out_bound=10.0, clip="channel", clip_sigma=2.5, ir_decay=0.01)
SHAPES = [
    # ResNet-like 3x3 layer: K = 576 in three tiles of 192, 1568 patches
    conv_case("conv2d_bf16_resnet", 2, 2, 64, (28, 28), (3, 3), (1, 1), (1, 1), N=128, dtype="bf16",
              max_input_size=256, ir_mode="static", ir_init=3.0, seed=50, **_ADC),
    conv_case("conv2d_f32_strided", 2, 3, 16, (19, 17), (5, 3), (2, 2), (2, 1), N=40,
              max_input_size=128, ir_mode="static", ir_init=3.0, seed=51, **_ADC),
    conv_case("conv1d_bf16_long", 1, 4, 32, (200,), (7,), (3,), (3,), N=64, dtype="bf16",
              max_input_size=128, ir_mode="dynamic", seed=52, **_ADC),
    conv_case("conv3d_bf16_video", 3, 2, 8, (6, 14, 14), (3, 3, 3), (1, 2, 2), (1, 1, 1), N=32,
              dtype="bf16", max_input_size=128, ir_mode="static", ir_init=3.0, seed=53, **_ADC),
]


@pytest.mark.parametrize("c", SHAPES, ids=[c["name"] for c in SHAPES])
def test_seeded_convolutions_match_oracle(c):
    inputs = make_conv_inputs(c)
    check(hip_conv_fwd_bwd(c, inputs), oracle_conv_fwd_bwd(c, inputs), c, c["name"])


# Convolutions the layer runs WITHOUT the patch matrix (16-bit, stride 1, dilation 1, a learned
# static range or none, K-tiles of whole channels in multiples of 64, out_channels a multiple of
# 64): against the oracle (the reference's unfold + linear model) and against the patch path.
_IMG = dict(inp_res=254, out_res=254, clip="channel", clip_sigma=2.5, ir_decay=0.01, ir_mode="static")
DIRECT = [
    # three tiles of 64 channels x 9 taps, ranges that clip some inputs, no output clamps
    conv_case("direct_bf16_three_tiles", 2, 2, 192, (9, 11), (3, 3), (1, 1), (1, 1), N=64, dtype="bf16",
              max_input_size=576, ir_values=[1.5, 3.0, 2.0], out_bound=12.0, seed=60, **_IMG),
    # one tile of 128 channels (the 128-wide input-gradient blocks), 5 x 3 kernel, uneven padding,
    # a bound that clamps, 300 output channels would not do: 128
    conv_case("direct_bf16_clamped", 2, 3, 128, (8, 7), (5, 3), (1, 1), (2, 0), N=128, dtype="bf16",
              max_input_size=-1, ir_values=[2.0], out_bound=3.0, w_scale=0.05, seed=61, **_IMG),
    conv_case("direct_f16_two_tiles", 2, 2, 128, (10, 10), (3, 3), (1, 1), (1, 1), N=64, dtype="f16",
              max_input_size=600, ir_values=[2.5, 1.5], out_bound=12.0, seed=62, **_IMG),
    # no padding, 1 x 1 kernel: the image rows ARE the patch rows
    conv_case("direct_bf16_pointwise", 2, 2, 64, (6, 5), (1, 1), (1, 1), (0, 0), N=64, dtype="bf16",
              ir_values=[2.0], out_bound=12.0, seed=63, **_IMG),
    # volumes and sequences
    conv_case("direct_bf16_volume", 3, 2, 64, (4, 6, 5), (2, 3, 3), (1, 1, 1), (1, 1, 0), N=64, dtype="bf16",
              ir_values=[2.0], out_bound=12.0, seed=64, **_IMG),
    conv_case("direct_bf16_sequence", 1, 3, 128, (70,), (5,), (1,), (2,), N=64, dtype="bf16",
              max_input_size=320, ir_values=[2.0, 1.0], out_bound=12.0, seed=65, **_IMG),
    # no converters at all: the plain convolution in 16-bit arithmetic
    conv_case("direct_bf16_plain", 2, 2, 64, (9, 9), (3, 3), (1, 1), (1, 1), N=64, dtype="bf16", seed=66),
    # evaluation mode (no input-range gradient, nothing kept for a backward pass of the range)
    conv_case("direct_bf16_eval", 2, 2, 64, (9, 9), (3, 3), (1, 1), (1, 1), N=64, dtype="bf16",
              ir_values=[2.0], out_bound=12.0, seed=67, training=False, **_IMG),
    # an unbatched image
    conv_case("direct_bf16_unbatched", 2, 0, 64, (12, 9), (3, 3), (1, 1), (1, 1), N=64, dtype="bf16",
              ir_values=[2.0], out_bound=12.0, seed=68, **_IMG),
]


@pytest.mark.parametrize("c", DIRECT, ids=[c["name"] for c in DIRECT])
def test_convolutions_read_off_the_image(c, monkeypatch):
    from aihwkit_lightning.nn.modules.hip_utils import hip_conv

    inputs = make_conv_inputs(c)
    calls = []
    real = hip_conv.HipConv.forward
    monkeypatch.setattr(hip_conv.HipConv, "forward",
                        staticmethod(lambda *a: calls.append(1) or real(*a)))
    res = hip_conv_fwd_bwd(c, inputs)
    assert calls, "the layer did not call the image path"
    check(res, oracle_conv_fwd_bwd(c, inputs), c, c["name"] + " vs oracle")
    monkeypatch.setattr(hip_conv, "ENABLED", False)
    del calls[:]
    patches = hip_conv_fwd_bwd(c, inputs)
    assert not calls
    check(res, patches, c, c["name"] + " vs the patch path")


_SWEEP = [
    # ndim, batch, C, size, kernel, padding, N, channels per tile (0: one tile), dtype
    (2, 1, 64, (5, 40), (3, 5), (1, 2), 64, 0, "bf16"),          # one image, wide kernel
    (2, 3, 128, (13, 6), (7, 3), (3, 1), 192, 64, "bf16"),       # 7-tall kernel, N = 3 x 64
    (2, 2, 256, (6, 6), (1, 1), (1, 1), 128, 128, "f16"),        # 1 x 1 kernel WITH padding
    (2, 2, 64, (4, 4), (4, 4), (0, 0), 64, 0, "bf16"),           # kernel == image: one output per image
    (2, 5, 64, (17, 3), (3, 3), (0, 1), 64, 0, "f16"),           # padding in one dimension only
    (3, 1, 64, (5, 5, 5), (3, 3, 3), (1, 1, 1), 64, 0, "bf16"),  # 27 taps
    (3, 2, 128, (3, 8, 4), (1, 3, 2), (0, 1, 1), 64, 64, "bf16"),  # even kernel extent, two tiles
    (1, 2, 64, (300,), (9,), (4,), 128, 0, "bf16"),              # long sequence, 9 taps
    (1, 4, 192, (33,), (3,), (0,), 64, 64, "f16"),               # three tiles, no padding
    (2, 0, 128, (9, 10), (3, 3), (2, 2), 64, 64, "bf16"),        # unbatched, padding wider than the kernel needs
    # enough pixels for a sliced weight gradient, K-tiles of 3 x 192 columns (the 192-wide blocks):
    # 4 x 16 x 16 = 1024 padded pixels (whole chunks of 64), 4 x 18 x 18 (a partial last chunk),
    # 6 x 192 columns in f16, 9 x 192 columns from 27 taps, and N beyond one row of blocks
    (2, 4, 128, (14, 14), (3, 3), (1, 1), 64, 64, "bf16"),
    (2, 4, 192, (16, 16), (3, 3), (1, 1), 128, 64, "bf16"),
    (2, 4, 128, (16, 15), (3, 3), (1, 1), 64, 0, "f16"),
    (3, 2, 64, (8, 9, 8), (3, 3, 3), (1, 1, 1), 64, 0, "bf16"),
    (2, 4, 64, (16, 16), (3, 3), (1, 1), 320, 0, "bf16"),
]


@pytest.mark.parametrize("spec", _SWEEP, ids=[f"geom{i}" for i in range(len(_SWEEP))])
def test_image_path_equals_patch_path_over_geometries(spec, monkeypatch):
    """Index arithmetic of the image path (padded grid, tap offsets, lead rows, layouts) over kernel
    shapes, paddings and tilings: outputs and every gradient against the patch path on the same
    layer and inputs (the patch path is the one compared with the reference's goldens)."""
    from aihwkit_lightning.nn.modules.hip_utils import hip_conv

    ndim, batch, chan, size, kernel, padding, n_out, ct, dtype = spec
    kvol = 1
    for k in kernel:
        kvol *= k
    tiles = 1 if ct == 0 else chan // ct
    c = conv_case("sweep", ndim, batch, chan, size, kernel, (1,) * ndim, padding, N=n_out, dtype=dtype,
                  max_input_size=-1 if ct == 0 else ct * kvol, ir_values=[1.5 + 0.5 * t for t in range(tiles)],
                  out_bound=2.0, w_scale=0.05, seed=70 + len(size) + chan, **_IMG)
    inputs = make_conv_inputs(c)
    calls = []
    real = hip_conv.HipConv.forward
    monkeypatch.setattr(hip_conv.HipConv, "forward", staticmethod(lambda *a: calls.append(1) or real(*a)))
    res = hip_conv_fwd_bwd(c, inputs)
    assert calls, "the layer did not call the image path"
    monkeypatch.setattr(hip_conv, "ENABLED", False)
    check(res, hip_conv_fwd_bwd(c, inputs), c, f"{spec} vs the patch path")


def test_image_path_declines_what_it_does_not_cover():
    from aihwkit_lightning.nn.modules.hip_utils import hip_conv

    base = dict(N=64, dtype="bf16", ir_values=[2.0], out_bound=12.0, **_IMG)
    declined = [
        conv_case("strided", 2, 2, 64, (9, 9), (3, 3), (2, 1), (1, 1), **base),
        conv_case("dilated", 2, 2, 64, (9, 9), (3, 3), (1, 1), (1, 1), (1, 2), **base),
        conv_case("odd_channels", 2, 2, 48, (9, 9), (3, 3), (1, 1), (1, 1), **base),
        conv_case("odd_outputs", 2, 2, 64, (9, 9), (3, 3), (1, 1), (1, 1), **{**base, "N": 40}),
        conv_case("split_taps", 2, 2, 64, (9, 9), (3, 3), (1, 1), (1, 1),
                  **{**base, "max_input_size": 300, "ir_values": [2.0, 2.0]}),
        conv_case("dynamic", 2, 2, 64, (9, 9), (3, 3), (1, 1), (1, 1),
                  **{**base, "ir_mode": "dynamic", "ir_values": None}),
        conv_case("fp32", 2, 2, 64, (9, 9), (3, 3), (1, 1), (1, 1), **{**base, "dtype": "f32"}),
    ]
    for c in declined:
        x, w, b, _ = make_conv_inputs(c)
        layer = make_conv_layer(c, w, b)
        assert not hip_conv.direct_conv_applies(layer, x.cuda(), layer.geometry(tuple(x.shape)), False), c["name"]


def test_conv1d_state_dict_round_trip_with_torch():
    """An AnalogConv1d saves and loads nn.Conv1d-shaped weights (reference conv.py:497-512)."""
    from hip_helpers import rpu_config
    from aihwkit_lightning.nn import AnalogConv1d

    c = CONV_CASES[1]
    digital = torch.nn.Conv1d(4, 6, 3, stride=2, padding=1).cuda()
    analog = AnalogConv1d.from_digital(digital, rpu_config(c))
    assert analog.weight.shape == (6, 4, 1, 3) and analog.state_dict()["weight"].shape == (6, 4, 3)
    x = torch.randn(3, 4, 11, device="cuda")
    assert torch.allclose(analog(x), digital(x), rtol=1e-5, atol=1e-5)
    other = AnalogConv1d(4, 6, 3, stride=2, padding=1, rpu_config=rpu_config(c)).cuda()
    other.load_state_dict(analog.state_dict())
    assert torch.equal(other.weight, analog.weight)
    back = AnalogConv1d.to_digital(other)
    assert torch.equal(back.weight, digital.weight)


def test_calibration_max_sees_patches():
    """reference tests/test_calibration.py:139-158 for AnalogConv2d: after MAX calibration the
    range of tile t is the abs-max of the unfolded input over that tile's patch entries."""
    from aihwkit_lightning.inference import calibrate_input_ranges, InputRangeCalibrationType
    from aihwkit_lightning.nn import AnalogConv2d
    from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig

    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 10
    layer = AnalogConv2d(3, 4, 3, stride=2, padding=1, rpu_config=cfg).cuda().eval()
    gen = torch.Generator().manual_seed(9)
    batches = [torch.randn(2, 3, 9, 8, generator=gen) for _ in range(4)]
    calibrate_input_ranges(layer, InputRangeCalibrationType.MAX,
                           iter([((b.cuda(),), {}) for b in batches]), verbose=False)
    rows = [oc.conv_patches(b.unsqueeze(2), [1, 3, 3], [1, 2, 2], [0, 1, 1], [1, 1, 1])[0]
            .reshape(-1, 27) for b in batches]
    assert torch.equal(layer.input_range.data.cpu(), om.calibrate_max(rows, layer.in_sizes))
    assert layer(batches[0].cuda()).shape == (2, 4, 5, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_weight_layouts_through_the_c_abi(dtype):
    """ahl_conv_weight_layout modes 0, 1, 2 against index arithmetic on the host, mode 1 with tiles
    that start every `stride` columns, and ahl_conv_weight_layouts (modes 0 and 2 in one launch)
    against the two single launches, bit for bit."""
    from ctypes import byref
    from aihwkit_lightning.nn.modules.hip_utils import library as L, ops

    lib = L.load()
    n_out, chan, kern, ct = 64, 128, (3, 2), 64
    kvol, n_tiles = kern[0] * kern[1], chan // ct
    k_in = chan * kvol
    geom = [2, chan, 7, 6, 1, kern[0], kern[1], 1, 1, 1, 1, 1, 1, 1, 1, 1, 1]
    cgeom = ops.conv_geom(geom)
    ends = L.tile_ends_array([ct * kvol] * n_tiles)
    dt = L.AHL_BF16 if dtype == torch.bfloat16 else L.AHL_F16
    stream = ops.current_stream()
    gen = torch.Generator().manual_seed(5)
    w = torch.randn(n_out, k_in, generator=gen).to(dtype).cuda()

    def layout(src, ld_src, mode, stride, shape):
        dst = torch.zeros(shape, dtype=dtype, device="cuda")
        rc = lib.ahl_conv_weight_layout(ops.ptr(src), ld_src, dt, n_out, byref(cgeom), ends, n_tiles, mode, stride,
                                        ops.ptr(dst), dst.size(1), stream)
        assert rc == 0
        return dst

    # the layer's order: column (channel, tap); the forward's: per tile (tap, channel in the tile)
    w4 = w.view(n_out, n_tiles, ct, kvol)
    want_taps = w4.permute(0, 1, 3, 2).reshape(n_out, k_in)
    want_dx = w.view(n_out, chan, kvol).permute(1, 2, 0).reshape(chan, kvol * n_out)
    taps = layout(w, k_in, 0, 0, (n_out, k_in))
    w_dx = layout(w, k_in, 2, 0, (chan, kvol * n_out))
    assert torch.equal(taps, want_taps) and torch.equal(w_dx, want_dx)
    # mode 1 from tiles that start every 448 columns (384 of them data)
    stride = 448
    spaced = torch.full((n_out, n_tiles * stride), float("nan"), dtype=dtype, device="cuda")
    for t in range(n_tiles):
        spaced[:, t * stride:t * stride + ct * kvol] = taps[:, t * ct * kvol:(t + 1) * ct * kvol]
    assert torch.equal(layout(spaced, spaced.size(1), 1, stride, (n_out, k_in)), w)
    both_taps = torch.zeros_like(taps)
    both_dx = torch.zeros_like(w_dx)
    rc = lib.ahl_conv_weight_layouts(ops.ptr(w), k_in, dt, n_out, byref(cgeom), ends, n_tiles, ops.ptr(both_taps), k_in,
                                     ops.ptr(both_dx), both_dx.size(1), stream)
    assert rc == 0
    assert torch.equal(both_taps, taps) and torch.equal(both_dx, w_dx)
    # refusals: a missing destination, tiles that split a channel's taps
    assert lib.ahl_conv_weight_layouts(ops.ptr(w), k_in, dt, n_out, byref(cgeom), ends, n_tiles, ops.ptr(both_taps), k_in,
                                       None, 0, stream) == 1   # AHL_ERR_ARG
    odd = L.tile_ends_array([100, k_in - 100])
    assert lib.ahl_conv_weight_layouts(ops.ptr(w), k_in, dt, n_out, byref(cgeom), odd, 2, ops.ptr(both_taps), k_in,
                                       ops.ptr(both_dx), both_dx.size(1), stream) != 0
