"""GPU parity of the memory-bound kernels (abs-max, std, clipping, quantisation, calibration,
input-range initialisation, column sums, DAC pre-pass) against the oracle, the reference's
golden vectors and closed forms. All calls go through the torch custom ops over the C ABI."""
import warnings

import pytest
import torch

from golden_cases import CASES_BY_NAME, DTYPES, case, make_inputs
from helpers import golden_tensor
from oracle import torch_mode as om

pytestmark = pytest.mark.gpu


def ops():
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS
    return OPS


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("n", [1, 10, 25, 255, 257, 1023, 1025])
def test_sliced_absmax_brute_force(n, dtype):
    # sizes and tile width of the reference's self-check (triton_abs_max.py:405-419); bit exact
    torch.manual_seed(n)
    w = torch.randn(n, n).to(dtype)
    sizes = om.split_sizes(n, 128)
    out, tmax, tmin = ops().sliced_absmax(w.cuda(), sizes, True)
    ref = om.sliced_abs_max(w, sizes)
    assert torch.equal(out.cpu(), ref)
    assert torch.equal(tmax.cpu(), ref.float().amax(1))
    assert torch.equal(tmin.cpu(), ref.float().amin(1))


def test_sliced_absmax_strided_rows_and_activation_shape():
    torch.manual_seed(0)
    big = torch.randn(300, 1100).to(torch.bfloat16).cuda()
    view = big[:, 7:1031]  # unaligned start, row stride 1100
    sizes = om.split_sizes(1024, 512)
    out, _, _ = ops().sliced_absmax(view, sizes, False)
    assert torch.equal(out.cpu(), om.sliced_abs_max(view.cpu(), sizes))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape,max_size", [((1, 63), 11), ((64, 512), 256), ((333, 1030), 128)])
def test_sliced_std(shape, max_size, dtype):
    torch.manual_seed(1)
    x = (torch.randn(*shape) * 1.7 + 0.3).to(dtype)
    sizes = om.split_sizes(shape[1], max_size)
    got = ops().sliced_std(x.cuda(), sizes).cpu()
    ref = torch.stack([x[:, lo:hi].double().std() for lo, hi in om.tile_bounds(sizes)]).float()
    assert torch.allclose(got, ref, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("name", ["f32_ir_init", "bf16_ir_init"])
def test_input_range_initialisation_matches_reference(name):
    """Training forwards during the data-initialisation phase: input_range, the update counter
    and the outputs after every step against the reference's recorded sequence."""
    from hip_helpers import make_layer

    c = CASES_BY_NAME[name]
    dtype = DTYPES[c["dtype"]]
    layer = make_layer(c)
    rtol = 1e-5 if c["dtype"] == "f32" else 1e-2
    for step in range(c["steps"]):
        xs = golden_tensor(f"{name}/x{step}", dtype).cuda()
        out = layer(xs)
        ir_ref = golden_tensor(f"{name}/ir{step}")
        assert torch.allclose(layer.input_range.data.float().cpu(), ir_ref, rtol=rtol, atol=0), step
        assert torch.equal(layer.input_range_update_idx.float().cpu(), golden_tensor(f"{name}/idx{step}"))
        ref = golden_tensor(f"{name}/out{step}")
        err = (out.float().cpu() - ref).abs().max() / ref.abs().mean()
        assert err < (1e-4 if c["dtype"] == "f32" else 6e-2), (step, float(err))
    # the host-side phase tracking switched the initialisation off without being told
    assert layer._ir_init_active is False or layer._ir_init_calls >= c["init_from_data"]


@pytest.mark.parametrize("name", ["f32_fast_init", "bf16_fast_init", "f32_fast_init_minmax"])
def test_fast_mode_range_sequence_matches_reference(name):
    """fast_mode training forwards: running min / max, the step counter, the range and the outputs
    after every step against the reference's recorded sequence. The state is bit-exact: it is a
    few dtype-rounded operations on exact minima and maxima."""
    from hip_helpers import make_layer

    c = CASES_BY_NAME[name]
    dtype = DTYPES[c["dtype"]]
    layer = make_layer(c)
    for step in range(c["steps"]):
        xs = golden_tensor(f"{name}/x{step}", dtype).cuda()
        out = layer(xs)
        for key, buf in (("ir", layer.input_range.data), ("idx", layer.input_range_update_idx),
                         ("xmin", layer.x_min), ("xmax", layer.x_max)):
            assert torch.equal(buf.float().cpu(), golden_tensor(f"{name}/{key}{step}")), (key, step)
        ref = golden_tensor(f"{name}/out{step}")
        err = (out.float().cpu() - ref).abs().max() / ref.abs().mean()
        assert err < (1e-4 if c["dtype"] == "f32" else 6e-2), (step, float(err))
    assert layer._ir_init_active is False or layer._ir_init_calls >= c["init_from_data"]


@pytest.mark.parametrize("name", ["f32_clip_layer", "f32_clip_channel", "bf16_clip_channel"])
def test_clip_weights_via_optimizer_matches_reference(name):
    from hip_helpers import make_layer
    from aihwkit_lightning.optim import AnalogOptimizer

    c = CASES_BY_NAME[name]
    x, w, b, _ = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    optim = AnalogOptimizer(torch.optim.SGD, layer.analog_layers, layer.parameters(), lr=0.0)
    layer(x.cuda()).sum().backward()
    optim.step()
    got = layer.weight.data.float().cpu()
    ref = golden_tensor(f"{name}/w_clipped")
    if c["dtype"] == "bf16":
        assert torch.equal(got, ref)
    else:
        assert torch.allclose(got, ref, rtol=1e-6, atol=0)
    assert not torch.equal(got, w.float())


@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_clip_weights_closed_form(dtype, per_channel):
    # the reference's test_clipping: W == W0.clamp(+-sigma * std)
    torch.manual_seed(2)
    w = torch.randn(100, 3072 if per_channel else 771).to(dtype)
    dev = w.cuda().clone()
    ops().clip_weights(dev, 2.0, 1 if per_channel else 0)
    ref = om.clip_weights(w, 2.0, per_channel)
    if dtype == torch.float32:
        assert torch.allclose(dev.cpu(), ref, rtol=2e-6, atol=0)
    else:
        # a bf16 bound may round differently for a row whose std sits on a rounding boundary
        mism = (dev.cpu() != ref).float().mean()
        assert mism < 2e-3


@pytest.mark.parametrize("per_channel", [False, True])
def test_clip_weights_of_a_single_weight_is_left_alone(per_channel):
    """The unbiased std of one value is NaN; the reference's clamp at +-NaN then turns the weight
    into NaN. Here such a row (or one-weight matrix) stays as it is -- a stated difference."""
    w = torch.tensor([[0.7], [-1.2], [0.0]]) if per_channel else torch.tensor([[0.7]])
    dev = w.cuda().clone()
    ops().clip_weights(dev, 2.0, 1 if per_channel else 0)
    assert torch.equal(dev.cpu(), w)
    assert torch.isnan(om.clip_weights(w, 2.0, per_channel)).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("vectors", [1, 63, 256, 257, 768, 1024, 2048, 2049],
                         ids=lambda v: f"{v}_vectors")
def test_clip_weights_per_channel_row_lengths(vectors, dtype):
    """Rows of 1 .. 2049 16-byte vectors: the kernels that keep a row in registers (up to 4, 8, 16,
    32 vectors per lane, with full and partly filled last rounds) and the one that reads it twice
    (2049 vectors); a clamped row's values may only be the row's own values or +-bound."""
    cols = vectors * (4 if dtype == torch.float32 else 8)
    gen = torch.Generator().manual_seed(vectors)
    w = torch.randn(37, cols, generator=gen)
    w = (w * (1.0 + 4.0 * (torch.rand(37, cols, generator=gen) < 0.02))).to(dtype)
    dev = w.cuda().clone()
    ops().clip_weights(dev, 2.0, 1)
    got, ref = dev.cpu(), om.clip_weights(w, 2.0, True)
    if dtype == torch.float32:
        assert torch.allclose(got, ref, rtol=2e-6, atol=0)
    else:
        assert float((got != ref).float().mean()) < 2e-3
    changed = got != w
    assert bool(changed.any()) or cols < 64
    bound = got.abs().amax(dim=1, keepdim=True)
    assert torch.equal(got[changed].abs(), bound.expand_as(got)[changed])


@pytest.mark.parametrize("name", ["f32_quantize_channel", "f32_quantize_odd", "bf16_quantize_tensor",
                                  "f32_quantize_lsq_clip", "bf16_quantize_lsq_clip",
                                  "f32_quantize_lsq_quant", "bf16_quantize_lsq_quant",
                                  "f32_quantize_lsq_clip_big"])
def test_quantize_weights_matches_reference(name):
    from hip_helpers import make_layer
    from aihwkit_lightning.simulator.configs import WeightQuantizationType, WeightClipType

    c = CASES_BY_NAME[name]
    x, w, b, _ = make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, None))
    layer.eval()
    before = layer(x.cuda()).float().cpu()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        layer.quantize_weights()
    got = layer.weight.data.float().cpu()
    ref = golden_tensor(f"{name}/w_quantized")
    if c["dtype"] == "bf16":
        assert torch.equal(got, ref)
    else:
        assert torch.allclose(got, ref, rtol=1e-6, atol=1e-9)
    assert layer.rpu_config.modifier.quantization_type == WeightQuantizationType.NONE
    assert layer.rpu_config.clip.type == WeightClipType.NONE
    after = layer(x.cuda()).float().cpu()
    ref_out = golden_tensor(f"{name}/out")
    tol = 1e-5 if c["dtype"] == "f32" else 2e-2
    assert torch.allclose(after, ref_out, rtol=tol, atol=tol * float(ref_out.abs().mean()))
    # invariant of tests/test_post_training_weight_quantization.py: same outputs before/after
    assert torch.allclose(before, after, rtol=tol, atol=tol * float(ref_out.abs().mean()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("scales", ["small", "all_large", "mixed"])
@pytest.mark.parametrize("cols,tile", [(512, 256), (2560, 1280), (300, 100), (100, 3), (26, 1)],
                         ids=["held", "long_segments", "unaligned_tiles", "tiles_of_3", "tiles_of_1"])
@pytest.mark.parametrize("rows", [24, 700])
def test_quantize_weights_per_channel_scale_switch(rows, cols, tile, scales, dtype):
    """The per-channel quantiser against the oracle where the reference's resolution convention
    matters: it reads the scales as numbers of states only if EVERY scale of a tile exceeds one.
    `small`: none does (the one-pass kernel alone); `all_large`: all do; `mixed`: some channels do,
    so the switch stays off but their segments wait for the tile minimum. Segments held in
    registers, segments longer than that, a split the one-pass kernel does not take, and tiles
    narrower than the 8 inputs a thread of the general kernel handles (several tiles per thread);
    a handful of channels and more than one block's worth of them."""
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    gen = torch.Generator().manual_seed(cols + len(scales))
    w = torch.randn(rows, cols, generator=gen)
    if scales == "all_large":
        w = w * 400.0
    elif scales == "mixed":
        w[::3] = w[::3] * 400.0
    w = w.to(dtype)
    sizes = om.split_sizes(cols, tile)
    dev = w.cuda().clone()
    ops().quantize_weights(dev, sizes, L.AHL_QUANT_DISCRETIZE_PER_CHANNEL, 30.0)
    ref = om.quantize_weights(w, sizes, om.DISCRETIZE_PER_CHANNEL, 30.0)
    got = dev.cpu()
    if dtype == torch.bfloat16:
        assert torch.equal(got, ref)
    else:
        assert torch.allclose(got, ref, rtol=1e-6, atol=1e-9)
    assert not torch.equal(got, w)


@pytest.mark.parametrize("in_size", [10, 255, 257])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_calibration_max(in_size, dtype):
    # tests/test_calibration.py:155-158: input_range[t] == |x[:, tile]|.max()
    from aihwkit_lightning.inference import calibrate_input_ranges, InputRangeCalibrationType
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig

    torch.manual_seed(3)
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 256
    layer = AnalogLinear(in_size, 7, dtype=dtype, rpu_config=cfg).cuda().eval()
    batches = [torch.randn(2, 3, in_size).to(dtype) for _ in range(5)]
    loader = [((b.cuda(),), {}) for b in batches]
    calibrate_input_ranges(layer, InputRangeCalibrationType.MAX, iter(loader), verbose=False)
    assert layer.rpu_config.pre_post.input_range.enable
    ref = om.calibrate_max(batches, layer.in_sizes)
    assert torch.equal(layer.input_range.data.cpu(), ref)
    assert layer.input_range.dtype == dtype
    out = layer(batches[0].cuda())  # the calibrated layer runs with the input range on
    assert out.shape == (2, 3, 7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_col_sum(dtype):
    torch.manual_seed(4)
    g = torch.randn(1000, 517).to(dtype)
    got = ops().col_sum(g.cuda()).float().cpu()
    ref = g.double().sum(0)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(got, ref.float(), rtol=tol, atol=tol * float(ref.abs().mean()))


@pytest.mark.parametrize("mode", ["static", "dynamic"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_dac_prepass_bit_exact(dtype, mode):
    """The clamp + DAC (+ dynamic abs-max) pass against the oracle's quantiser, bit for bit."""
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    torch.manual_seed(5)
    x = (torch.randn(130, 512) * 1.3).to(dtype)
    sizes = om.split_sizes(512, 128)
    ir = torch.tensor([0.9, 1.7, 2.5, 3.3]).to(dtype)
    icfg = [L.AHL_IR_STATIC if mode == "static" else L.AHL_IR_DYNAMIC, 0, 0, 0, 0, 0, 0]
    fcfg = [254.0, -1.0, 0.0, 0.0, 0.0, 0.0]
    xq, ir_dyn = ops().dac(x.cuda(), ir.cuda() if mode == "static" else None, sizes, icfg, fcfg)
    for t, (lo, hi) in enumerate(om.tile_bounds(sizes)):
        x_t = x[:, lo:hi]
        if mode == "static":
            ref = om.quantize(torch.clamp(x_t, -ir[t], ir[t]), om.quant_step(ir[t], 254))
        else:
            ir_t = x_t.abs().max(dim=-1, keepdim=True)[0]
            assert torch.equal(ir_dyn[t].cpu(), ir_t.view(-1))
            ref = om.quantize(x_t, om.quant_step(ir_t, 254))
        got = xq[:, lo:hi].cpu()
        if dtype == torch.bfloat16:
            assert torch.equal(got, ref)
        else:
            assert torch.allclose(got, ref, rtol=1e-6, atol=1e-7)


def test_reduction_bound_pipeline_one_matrix():
    """One 8192 x 3072 fp32 weight matrix of the post-training configuration: per-tile abs-max,
    clip at 3 sigma per channel, quantise per channel to 254 states; then running abs-max
    calibration over Laplace activations. Compared with the oracle at full size."""
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    gen = torch.Generator().manual_seed(4)
    w = 0.02 * torch.randn(8192, 3072, generator=gen)
    w = torch.where(torch.rand(8192, 3072, generator=gen) < 1e-3, w * 20, w)
    sizes = om.split_sizes(3072, 512)
    dev = w.cuda().clone()
    wmax, _, _ = ops().sliced_absmax(dev, sizes, True)
    assert torch.equal(wmax.cpu(), om.sliced_abs_max(w, sizes))
    ops().clip_weights(dev, 3.0, L.AHL_CLIP_PER_CHANNEL)
    ref = om.clip_weights(w, 3.0, True)
    assert torch.allclose(dev.cpu(), ref, rtol=2e-6, atol=0)
    ops().quantize_weights(dev, sizes, L.AHL_QUANT_DISCRETIZE_PER_CHANNEL, 254.0)
    ref_q = om.quantize_weights(dev.cpu() * 0 + ref, sizes, om.DISCRETIZE_PER_CHANNEL, 254.0)
    diff = (dev.cpu() - ref_q).abs()
    lsb = 2 * ref.abs().amax() / 254
    assert float((diff > 1e-6).float().mean()) < 1e-3 and float(diff.max()) <= float(lsb) * 1.01
    lap = torch.distributions.Laplace(0.0, 1.0)
    cache = torch.full((len(sizes),), float("-inf"), device="cuda")
    batches = []
    for i in range(4):
        torch.manual_seed(100 + i)
        b = lap.sample((2048, 3072))
        batches.append(b)
        ops().running_absmax(b.cuda(), sizes, cache)
    assert torch.equal(cache.cpu(), om.calibrate_max(batches, sizes))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("k_in,max_size", [(1024, 512), (2304, 1152), (640, 128)])
def test_one_pass_weight_prep_matches_two_pass(k_in, max_size, dtype):
    """Abs-max + per-channel weight noise in one kernel (aligned rows) must give the bits of the
    separate abs-max and modifier kernels (taken for a row stride that is not a multiple of 8)."""
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    sizes = om.split_sizes(k_in, max_size)
    w = (0.05 * torch.randn(96, k_in, generator=torch.Generator().manual_seed(6))).to(dtype).cuda()
    padded = torch.zeros(96, k_in + 3, dtype=dtype, device="cuda")
    padded[:, :k_in] = w
    args = (sizes, L.AHL_QUANT_NONE, L.AHL_NOISE_ADD_NORMAL_PER_CHANNEL, 1.0, 0.05, 77, 1, True)
    one = ops().weight_prep(w, *args)
    two = ops().weight_prep(padded[:, :k_in], *args)
    for a, b, what in zip(one, two, ("wmax", "tile_max", "tile_min", "w_eff")):
        assert torch.equal(a, b), what
    assert not torch.equal(one[3], w), "the noise must change the weights"
    skipped = ops().weight_prep(w, *args, True)
    assert torch.equal(skipped[0], one[0]) and torch.equal(skipped[3], one[3])
