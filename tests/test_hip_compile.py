"""The custom ops under torch's own checks (schema, fake kernels, functionalisation), and
``torch.compile`` of models that hold analog layers (the reference smoke-tests compilation in
``tests/test_speed.py:98-99``)."""
import pytest
import torch

from golden_cases import case, make_inputs

pytestmark = pytest.mark.gpu


def _ops():
    from aihwkit_lightning.nn.modules.hip_utils import library as L
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS

    return OPS, L


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_opcheck_linear_ops(dtype):
    OPS, L = _ops()
    gen = torch.Generator().manual_seed(5)
    m, k, n, in_sizes = 96, 512, 128, [256, 256]
    x = torch.randn(m, k, generator=gen).to(dtype).cuda()
    w = (0.05 * torch.randn(n, k, generator=gen)).to(dtype).cuda()
    b = torch.zeros(n, dtype=dtype, device="cuda")
    g = torch.randn(m, n, generator=gen).to(dtype).cuda()
    ir = torch.full((2,), 3.0, dtype=dtype, device="cuda")
    icfg = [L.AHL_IR_STATIC, 0, 1, 0, 0, 0, 0]
    fcfg = [254.0, 254.0, 0.5, 0.0, 0.01, 0.95]
    checks = ("test_schema", "test_faketensor", "test_aot_dispatch_dynamic")
    opcheck = torch.library.opcheck
    opcheck(OPS.weight_prep.default, (w, in_sizes, L.AHL_QUANT_NONE, L.AHL_NOISE_NONE, 1.0, 0.0, 0, 0, False),
            test_utils=checks)
    wmax, tile_max, _, _ = OPS.weight_prep(w, in_sizes, L.AHL_QUANT_NONE, L.AHL_NOISE_NONE, 1.0, 0.0, 0, 0, False)
    opcheck(OPS.dac.default, (x, ir, in_sizes, icfg, fcfg), test_utils=checks)
    xq, _ = OPS.dac(x, ir, in_sizes, icfg, fcfg)
    args = (x, xq, w, b, ir, wmax, tile_max, in_sizes, icfg, fcfg, True)
    opcheck(OPS.linear_fwd.default, args, test_utils=checks)
    _, keep, flag = OPS.linear_fwd(*args)
    opcheck(OPS.linear_bwd_dx.default, (g, keep, flag, w, x, ir, in_sizes, icfg, fcfg), test_utils=checks)
    opcheck(OPS.linear_bwd_dw.default, (g, keep, flag, x, xq, ir, in_sizes, icfg, fcfg, True),
            test_utils=checks)


def test_opcheck_reductions_and_weight_ops():
    OPS, L = _ops()
    gen = torch.Generator().manual_seed(6)
    in_sizes = [192, 192]
    x = torch.randn(300, 384, generator=gen).cuda()
    w = (0.05 * torch.randn(64, 384, generator=gen)).cuda()
    checks = ("test_schema", "test_faketensor", "test_aot_dispatch_dynamic")
    opcheck = torch.library.opcheck
    opcheck(OPS.sliced_absmax.default, (x, in_sizes, True), test_utils=checks)
    opcheck(OPS.sliced_std.default, (x, in_sizes), test_utils=checks)
    opcheck(OPS.sliced_std_kept.default, (x, in_sizes), test_utils=checks)
    opcheck(OPS.sliced_quantile.default, (x, in_sizes, 0.999), test_utils=checks)
    opcheck(OPS.row_nonzero.default, (x,), test_utils=checks)
    opcheck(OPS.col_sum.default, (x,), test_utils=checks)
    cache = torch.zeros(2, device="cuda")
    opcheck(OPS.running_absmax.default, (x, in_sizes, cache), test_utils=checks)
    opcheck(OPS.clip_weights.default, (w.clone(), 2.0, L.AHL_CLIP_PER_CHANNEL), test_utils=checks)
    opcheck(OPS.quantize_weights.default, (w.clone(), in_sizes, L.AHL_QUANT_DISCRETIZE_PER_CHANNEL, 30.0),
            test_utils=checks)
    opcheck(OPS.pad_tiles.default, (x, in_sizes, 256), test_utils=checks)
    geom = [2, 8, 1, 12, 12, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1]
    img = torch.randn(2, 8, 1, 12, 12, generator=gen).cuda()
    opcheck(OPS.im2col.default, (img, geom), test_utils=checks)
    opcheck(OPS.col2im.default, (OPS.im2col(img, geom), geom), test_utils=checks)
    opcheck(OPS.transpose_batched.default, (torch.randn(3, 5, 7, generator=gen).cuda(),), test_utils=checks)


def test_traced_op_matches_eager():
    """A function made of the custom ops alone compiles as ONE graph (the fake kernels give
    the tracer every shape) and returns what the eager calls return."""
    OPS, L = _ops()
    gen = torch.Generator().manual_seed(7)
    in_sizes = [256, 256]
    x = torch.randn(64, 512, generator=gen).cuda()
    w = (0.05 * torch.randn(96, 512, generator=gen)).cuda()
    ir = torch.full((2,), 3.0, device="cuda")
    icfg = [L.AHL_IR_STATIC, 0, 1, 0, 0, 0, 0]
    fcfg = [254.0, 254.0, 0.5, 0.0, 0.01, 0.95]

    def fwd(inp, weight):
        wmax, tile_max, _, _ = OPS.weight_prep(weight, in_sizes, L.AHL_QUANT_NONE, L.AHL_NOISE_NONE, 1.0,
                                               0.0, 0, 0, False)
        xq, _ = OPS.dac(inp, ir, in_sizes, icfg, fcfg)
        return OPS.linear_fwd(inp, xq, weight, None, ir, wmax, tile_max, in_sizes, icfg, fcfg, False)[0] * 2.0

    compiled = torch.compile(fwd, fullgraph=True, backend="aot_eager")
    assert torch.equal(compiled(x, w), fwd(x, w))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_compiled_model_with_analog_layers(dtype):
    """torch.compile of a small model: the analog layers run as opaque calls between the compiled
    parts; outputs and gradients equal the eager model's."""
    from hip_helpers import make_layer

    c = case("compile", dtype=dtype, M=64, K=512, N=256, max_input_size=256, ir_mode="static",
             inp_res=254, out_res=254, out_bound=0.6, clip="channel", clip_sigma=2.5, ir_decay=0.01,
             w_scale=0.05, seed=91)
    x, w, b, g = make_inputs(c)

    def model_of():
        layer = make_layer(c, inputs=(None, w, b, None))
        return torch.nn.Sequential(torch.nn.LayerNorm(512, device="cuda", dtype=x.dtype), layer,
                                   torch.nn.GELU())

    eager, other = model_of(), model_of()
    compiled = torch.compile(other, backend="aot_eager")
    xe, xc = x.cuda().requires_grad_(True), x.cuda().requires_grad_(True)
    out_e = eager(xe)
    out_e.backward(g.cuda())
    for _ in range(2):   # the second call runs the cached compilation
        xc.grad = None
        other.zero_grad(set_to_none=True)
        out_c = compiled(xc)
        out_c.backward(g.cuda())
    torch.cuda.synchronize()
    assert torch.equal(out_c, out_e)
    assert torch.equal(xc.grad, xe.grad)
    assert torch.equal(other[1].weight.grad, eager[1].weight.grad)
    assert torch.equal(other[1].input_range.grad, eager[1].input_range.grad)
