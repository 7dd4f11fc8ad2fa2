"""GPU parity at the full benchmark sizes (4096 -> 4096, 8192 tokens, 8 tiles of 512, bf16 and float16).

The small-shape tests never launch more than a handful of blocks; these cases run the MFMA
kernels with their real grids (2048 / 512 / 256 blocks: XCD remap, band-swizzled tile order,
two passes over the CUs) and check them two ways:

* plain product (no input range, no DAC/ADC): forward and both gradients reduce to library
  matrix products (y = x W^T, dX = g W, dW = g^T x), checked against torch on the same device;
* the full analog configuration with the noise off: against the CPU oracle on the whole problem
  (a few seconds per pass), to the stated tolerance of the path.
"""
import pytest
import torch

from golden_cases import case, make_inputs
from helpers import assert_close_lsb, oracle_fwd_bwd

pytestmark = pytest.mark.gpu

FULL = dict(dtype="bf16", M=8192, K=4096, N=4096, max_input_size=512)


def test_full_size_plain_product_matches_library_gemm():
    from hip_helpers import hip_fwd_bwd

    c = case("full_plain", seed=41, **FULL)
    x, w, b, g = make_inputs(c)
    res = hip_fwd_bwd(c, inputs=(x, w, b, g))
    xd, wd, gd = x.cuda().float(), w.cuda().float(), g.cuda().float()
    # fp32 products of the bf16 operands, rounded to bf16 once per K-tile and summed in bf16 in
    # tile order, as the path (and the reference on bf16 tensors) does
    out = torch.zeros(c["M"], c["N"], dtype=torch.bfloat16, device="cuda")
    for t in range(c["K"] // 512):
        sl = slice(512 * t, 512 * (t + 1))
        out = out + (xd[:, sl] @ wd[:, sl].t()).to(torch.bfloat16)
    if b is not None:
        out = out + b.cuda()
    out_ref = out.float().cpu()
    dx_ref = (gd @ wd).cpu()
    dw_ref = (gd.t() @ xd).cpu()
    db_ref = gd.sum(0).cpu()
    # a tile's partial product may round to the neighbouring bf16 value when the two fp32
    # accumulation orders differ in the last bit; one bf16 step of a partial of magnitude < 8
    assert_close_lsb(res["out"].float(), out_ref, 1e-2, 2.0 ** -5, max_frac=1e-5, what="full plain out")
    assert_close_lsb(res["dx"].float(), dx_ref, 1e-2, None, what="full plain dx")
    assert_close_lsb(res["dw"].float(), dw_ref, 1e-2, None, what="full plain dw")
    assert_close_lsb(res["db"].float(), db_ref, 1e-2, None, what="full plain db")


@pytest.mark.parametrize("ir_mode,dtype", [("static", "bf16"), ("dynamic", "bf16"), ("static", "f16")])
def test_full_size_analog_matches_oracle(ir_mode, dtype):
    from hip_helpers import hip_fwd_bwd

    # out_bound 0.9 clamps a visible fraction of the tile outputs, so the clamp mask and the
    # "anything clamped" flag are exercised at the full grid as well
    c = case(f"full_{ir_mode}_{dtype}", ir_mode=ir_mode, inp_res=254, out_res=254, out_bound=0.9,
             clip="channel", clip_sigma=2.5, ir_decay=0.01, ir_init=3.0, w_scale=0.02, seed=42,
             **dict(FULL, dtype=dtype))
    inputs = make_inputs(c)
    res = hip_fwd_bwd(c, inputs=inputs)
    torch.set_num_threads(16)
    ref = oracle_fwd_bwd(c, ties=False)   # the float64 tie analysis is for small cases; the rule is stated below
    # An ADC level that flips in one tile (rounding-boundary tie, from the different fp32
    # accumulation order of the two GEMMs) moves that tile's output by one ADC step; the bf16
    # running sum over the 8 tiles can then land on the neighbouring bf16 value of a partial sum
    # of magnitude < 2, i.e. 2^-7, which is larger than the ADC step itself. Allowed on at most
    # 0.001 % of the elements.
    # float16 (spacing 2^-10 below 2) keeps the flipped ADC step itself: 2 * 0.9 * 3 * max|w| / 254.
    rtol = 1e-2 if dtype == "bf16" else 1e-3
    lsb = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10 + 5.4 * float(inputs[1].abs().max()) / 254
    # In bf16 a flipped level shows only where the running sum changes (at most 0.001 % of the
    # elements); in float16 every flipped level is visible (0.012 % measured), under the path's
    # own cap of 0.1 %.
    assert_close_lsb(res["out"].float(), ref["out"].float(), rtol, lsb,
                     max_frac=1e-5 if dtype == "bf16" else 1e-3, what=f"{c['name']} out")
    # Gradients see such a tie only where the flipped level is the outermost one: the value is
    # then clamped in one computation and kept at +-bound in the other, and the clamp mask of
    # that (row, column, tile) differs. One flipped mask bit changes 512 entries of dX by
    # g[m, n] * W[n, k] and 512 entries of dW by g[m, n] * xq[m, k].
    x, w, _, g = inputs
    flip = {"dx": float(g.abs().max() * w.abs().max()), "dw": float(g.abs().max() * x.abs().max()),
            "db": None, "dir": None}
    for key in ("dx", "dw", "db", "dir"):
        if ref.get(key) is None:
            continue
        assert_close_lsb(res[key].float(), ref[key].float(), rtol, flip[key], max_frac=1e-3,
                         what=f"{c['name']} {key}")


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("out_bound", [10.0, 0.9], ids=["rare_clamps", "frequent_clamps"])
def test_the_two_forward_kernels_agree_bit_for_bit(dtype, out_bound, monkeypatch):
    """Large grids with a learned range run the kernel that works a tile's epilogue off inside the
    next tile's product loop; AHL_FORWARD_KERNEL=blocks in the environment keeps them on the kernel
    for small grids. Same seed, output noise, ADC and clamp on: outputs (noise draws included),
    clamp-dependent gradients and all, bit for bit."""
    from hip_helpers import hip_fwd_bwd

    c = case(f"two_kernels_{dtype}", ir_mode="static", inp_res=254, out_res=254, out_bound=out_bound,
             out_noise=0.04, clip="channel", clip_sigma=2.5, ir_decay=0.01, ir_init=3.0, w_scale=0.02,
             seed=43, **dict(FULL, dtype=dtype))
    inputs = make_inputs(c)
    monkeypatch.delenv("AHL_FORWARD_KERNEL", raising=False)
    piped = hip_fwd_bwd(c, inputs=inputs)
    monkeypatch.setenv("AHL_FORWARD_KERNEL", "blocks")
    blocks = hip_fwd_bwd(c, inputs=inputs)
    for key in ("out", "dx", "dw", "db", "dir"):
        if piped.get(key) is not None:
            assert torch.equal(piped[key], blocks[key]), key
    assert bool(piped["out"].float().std() > 0)


@pytest.mark.parametrize("dtype,tile,noise", [("bf16", 576, 0.04), ("f16", 640, 0.04), ("bf16", 1088, 0.0)])
def test_the_two_forward_kernels_agree_on_longer_tiles(dtype, tile, noise, monkeypatch):
    """K-tiles of more than 512 columns (any multiple of 64): the first eight chunks of a tile carry
    the epilogue of the tile before, the others are product only. Same results as the kernel for
    small grids, bit for bit, with noise, ADC and clamps."""
    from hip_helpers import hip_fwd_bwd

    c = case(f"long_tiles_{dtype}_{tile}", dtype=dtype, M=4096, K=2 * tile, N=2048, max_input_size=tile,
             ir_mode="static", inp_res=254, out_res=254, out_bound=0.9, out_noise=noise, clip="channel",
             clip_sigma=2.5, ir_decay=0.01, ir_init=3.0, w_scale=0.02, seed=47)
    inputs = make_inputs(c)
    monkeypatch.delenv("AHL_FORWARD_KERNEL", raising=False)
    piped = hip_fwd_bwd(c, inputs=inputs)
    monkeypatch.setenv("AHL_FORWARD_KERNEL", "blocks")
    blocks = hip_fwd_bwd(c, inputs=inputs)
    for key in ("out", "dx", "dw", "db", "dir"):
        if piped.get(key) is not None:
            assert torch.equal(piped[key], blocks[key]), key
    assert bool(piped["out"].float().std() > 0)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_the_two_forward_kernels_agree_on_an_image(dtype, monkeypatch):
    """A convolution read off the image with enough pixels for the large-grid forward kernel (its A
    operand's chunk offsets come from the tap map): same outputs and gradients as with the kernel
    for small grids, bit for bit, noise included."""
    from conv_cases import conv_case, make_conv_inputs
    from test_hip_conv import hip_conv_fwd_bwd

    c = conv_case(f"image_two_kernels_{dtype}", 2, 64, 128, (28, 28), (3, 3), (1, 1), (1, 1), N=256, dtype=dtype,
                  max_input_size=576, ir_mode="static", ir_values=[2.0, 1.5], inp_res=254, out_res=254,
                  out_bound=1.5, out_noise=0.04, clip="channel", clip_sigma=2.5, ir_decay=0.01,
                  w_scale=0.02, seed=48)
    inputs = make_conv_inputs(c)
    monkeypatch.delenv("AHL_FORWARD_KERNEL", raising=False)
    piped = hip_conv_fwd_bwd(c, inputs)
    monkeypatch.setenv("AHL_FORWARD_KERNEL", "blocks")
    blocks = hip_conv_fwd_bwd(c, inputs)
    for key in ("out", "dx", "dw", "db", "dir"):
        if piped.get(key) is not None:
            assert torch.equal(piped[key], blocks[key]), key
    assert bool(piped["out"].float().std() > 0)


@pytest.mark.parametrize("n_out,k_in", [(8192, 3072), (3072, 8192), (2048, 4096)],
                         ids=["cut_along_columns", "cut_along_rows", "one_launch"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_weight_gradient_whose_tiles_do_not_fill_whole_rounds(n_out, k_in, dtype):
    """384 output tiles of 256 x 256 are 1.5 rounds of the 256 CUs: the weight gradient then runs as
    two launches (the tiles of the full round; the rest with its contraction sliced). Through the
    operators, with a bound that clamps 5 % of the outputs: dW against (g without the clamped
    outputs of the column's K-tile)^T xq computed with torch from the kernel's own clamp mask, the
    bias gradient against the column sums of g."""
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    m_rows, tile = 1024, 512
    gen = torch.Generator().manual_seed(52)
    x = torch.randn(m_rows, k_in, generator=gen).to(dtype).cuda()
    g = torch.randn(m_rows, n_out, generator=gen).to(dtype).cuda()
    w = (0.02 * torch.randn(n_out, k_in, generator=gen)).to(dtype).cuda()
    bias = torch.zeros(n_out, dtype=dtype, device="cuda")
    in_sizes = [tile] * (k_in // tile)
    ir = torch.full((len(in_sizes),), 3.0, dtype=dtype, device="cuda")
    wmax, tile_max, _, _ = OPS.weight_prep(w, in_sizes, L.AHL_QUANT_NONE, L.AHL_NOISE_NONE, 1.0, 0.0, 0, 1, False)
    icfg = [L.AHL_IR_STATIC, 0, 1, 1, 0, 0, 0]
    fcfg = [254.0, 254.0, 3.6, 0.0, 0.01, 0.95]
    xq, _ = OPS.dac(x, ir, in_sizes, icfg, fcfg)
    _, keep, flag = OPS.linear_fwd(None, xq, w, bias, ir, wmax, tile_max, in_sizes, icfg, fcfg, True)
    dw, db = OPS.linear_bwd_dw(g, keep, flag, None, xq, ir, in_sizes, icfg, fcfg, True)
    torch.cuda.synchronize()
    # keep: [T, ceil(N / 32), rows64(M)] words, bit n % 32 of word (n / 32, m) set where clamped
    words = keep.view(torch.int32)[:, :, :m_rows].to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(32, device="cuda", dtype=torch.int64).view(1, 1, 32, 1)
    clamped = ((words.unsqueeze(2) >> shifts) & 1).reshape(len(in_sizes), -1, m_rows)[:, :n_out]   # [T, N, M]
    frac = float(clamped.float().mean())
    assert 0.01 < frac < 0.2, frac
    want = torch.empty(n_out, k_in, dtype=torch.float32, device="cuda")
    for t in range(len(in_sizes)):
        gm = g.float() * (1.0 - clamped[t].t().float())
        want[:, t * tile:(t + 1) * tile] = gm.t() @ xq[:, t * tile:(t + 1) * tile].float()
    scale = float(want.abs().max())
    tol = 4e-3 if dtype == torch.bfloat16 else 1e-3    # one rounding of the fp32 sum to the dtype
    assert float((dw.float() - want).abs().max()) <= tol * scale
    want_db = g.float().sum(0)
    assert float((db.float() - want_db).abs().max()) <= tol * float(want_db.abs().max())


def test_llama_mlp_block_matches_oracle():
    """Configuration 4 of the baseline: a LLaMA-style MLP block (hidden 3072, intermediate 8192,
    SiLU gating: down(silu(gate(x)) * up(x))), bf16, 4096 tokens, tiles of 512, 8-bit DAC/ADC,
    forward + backward through three analog layers, noise off for a deterministic comparison.

    The block composes three layers, so a rounding-boundary tie in one layer's ADC reaches the
    next layer's input: element-wise bounds do not compose. Compared instead: every layer on the
    oracle's own input for that layer (element-wise, the path's tolerance), and the block's
    output and input gradient against the oracle's in the mean (1 % of the mean magnitude).
    """
    import torch.nn.functional as F
    from hip_helpers import make_layer
    from helpers import oracle_cfg
    from oracle import torch_mode as om

    hidden, inter, tokens = 3072, 8192, 4096
    common = dict(dtype="bf16", max_input_size=512, ir_mode="static", inp_res=254, out_res=254,
                  out_bound=10.0, clip="channel", clip_sigma=2.5, ir_decay=0.01, bias=False)
    cases = {
        "gate": case("mlp_gate", M=tokens, K=hidden, N=inter, ir_init=3.0, w_scale=0.02, seed=43, **common),
        "up": case("mlp_up", M=tokens, K=hidden, N=inter, ir_init=3.0, w_scale=0.02, seed=44, **common),
        "down": case("mlp_down", M=tokens, K=inter, N=hidden, ir_init=1.0, w_scale=0.02, seed=45, **common),
    }
    weights = {k: make_inputs(c)[1] for k, c in cases.items()}
    x = make_inputs(cases["gate"])[0]
    g = make_inputs(cases["down"])[3]
    layers = {k: make_layer(c, inputs=(None, weights[k], None, None)) for k, c in cases.items()}

    # ---- HIP block ----
    xd = x.cuda().requires_grad_(True)
    gate, up = layers["gate"](xd), layers["up"](xd)
    act = F.silu(gate) * up
    out = layers["down"](act)
    out.backward(g.cuda())
    torch.cuda.synchronize()

    # ---- oracle block (explicit backward per layer, torch autograd for the gating) ----
    torch.set_num_threads(16)
    ir3 = lambda c: torch.full((len(om.split_sizes(c["K"], 512)),), c["ir_init"], dtype=torch.bfloat16)  # noqa: E731
    o_gate, s_gate = om.linear_forward(x, weights["gate"], None, oracle_cfg(cases["gate"]), ir3(cases["gate"]), True)
    o_up, s_up = om.linear_forward(x, weights["up"], None, oracle_cfg(cases["up"]), ir3(cases["up"]), True)
    gate_r, up_r = o_gate.clone().requires_grad_(True), o_up.clone().requires_grad_(True)
    act_r = F.silu(gate_r) * up_r
    o_out, s_down = om.linear_forward(act_r.detach(), weights["down"], None, oracle_cfg(cases["down"]),
                                      ir3(cases["down"]), True)
    d_act, dw_down, _, _ = om.linear_backward(g, s_down)
    act_r.backward(d_act)
    dx_gate, dw_gate, _, _ = om.linear_backward(gate_r.grad, s_gate)
    dx_up, dw_up, _, _ = om.linear_backward(up_r.grad, s_up)
    dx_ref = dx_gate + dx_up

    def mean_close(got, ref, what):
        got, ref = got.float().cpu(), ref.float()
        err = float((got - ref).abs().mean()) / float(ref.abs().mean())
        assert err < 1e-2, f"{what}: mean error {err:.3e} of the mean magnitude"

    # one ADC step of one tile (0.02) moves the bf16 running sum to the neighbouring bf16 value:
    # 2^-5 for the largest outputs here (magnitude 4 to 8)
    lsb = 2.0 ** -5
    assert_close_lsb(gate.detach().float().cpu(), o_gate.float(), 1e-2, lsb, max_frac=1e-4, what="gate out")
    assert_close_lsb(up.detach().float().cpu(), o_up.float(), 1e-2, lsb, max_frac=1e-4, what="up out")
    mean_close(out.detach(), o_out, "block output")
    mean_close(xd.grad, dx_ref, "block input gradient")
    mean_close(layers["down"].weight.grad, dw_down, "down-projection weight gradient")
    mean_close(layers["gate"].weight.grad, dw_gate, "gate-projection weight gradient")
    mean_close(layers["up"].weight.grad, dw_up, "up-projection weight gradient")
    # the down projection on the oracle's own activations: element-wise
    down_on_ref = layers["down"](act_r.detach().cuda())
    assert_close_lsb(down_on_ref.detach().float().cpu(), o_out.float(), 1e-2, lsb, max_frac=1e-4,
                     what="down out on the oracle's activations")


def _tail_reproduces(layer, x, g_shape, tail, chunk, what):
    """Rows (images) are independent of each other: the last `tail` of a large batch must come out
    bit for bit as they do on their own (a wrong 64-bit offset anywhere moves them), and the
    weight / bias gradients must be the sum of the gradients of the batch's chunks."""
    gen = torch.Generator(device="cuda").manual_seed(9)
    xs = x[-tail:].clone().requires_grad_()
    x.requires_grad_()
    y = layer(x)
    assert tuple(y.shape) == tuple(g_shape)
    g = torch.randn(g_shape, device="cuda", generator=gen, dtype=x.dtype)
    y.backward(g)
    dw, db = layer.weight.grad.float(), layer.bias.grad.float()
    layer.zero_grad(set_to_none=True)
    ys = layer(xs)
    ys.backward(g[-tail:].clone())
    assert torch.equal(y[-tail:], ys), f"{what}: output of the last rows"
    assert torch.equal(x.grad[-tail:], xs.grad), f"{what}: input gradient of the last rows"
    acc_w, acc_b = torch.zeros_like(dw), torch.zeros_like(db)
    for r0 in range(0, x.shape[0], chunk):
        layer.zero_grad(set_to_none=True)
        layer(x.detach()[r0:r0 + chunk]).backward(g[r0:r0 + chunk])
        acc_w += layer.weight.grad.float()
        acc_b += layer.bias.grad.float()
    # every chunk's gradient is rounded to bf16 (2^-9 relative, 2.3e-3 in the mean); rows that
    # went missing or were read from a wrapped offset would show as 2e-2 and more
    assert float((dw - acc_w).norm() / acc_w.norm()) < 5e-3, f"{what}: weight gradient"
    assert float((db - acc_b).norm() / acc_b.norm()) < 5e-3, f"{what}: bias gradient"


def _big_case(K, N):
    return case("big_index", dtype="bf16", M=1, K=K, N=N, max_input_size=512, ir_mode="static",
                inp_res=254, out_res=254, out_bound=0.9, clip="channel", clip_sigma=2.5,
                ir_decay=0.01, ir_init=3.0, w_scale=0.02, seed=5)


@pytest.mark.parametrize("shape", [(2 ** 19 + 192, 4096, 4096, 512, 2112),
                                   (2 ** 22 + 40, 520, 520, 260, 200)],
                         ids=["4096x4096", "520x520_padded_tiles"])
def test_more_than_2_31_elements_per_tensor(shape):
    """Activations, gradients and clamp masks with more than 2^31 elements: the MFMA kernels, the
    DAC pass and the mask addressing in 64-bit offsets."""
    from hip_helpers import rpu_config
    from aihwkit_lightning.nn import AnalogLinear

    rows, k_in, n_out, tile, tail = shape
    assert rows * min(k_in, n_out) > 2 ** 31
    c = _big_case(k_in, n_out)
    c["max_input_size"] = tile
    gen = torch.Generator(device="cuda").manual_seed(3)
    layer = AnalogLinear(k_in, n_out, bias=True, dtype=torch.bfloat16, rpu_config=rpu_config(c)).cuda()
    with torch.no_grad():
        layer.weight.copy_(0.02 * torch.randn(n_out, k_in, device="cuda", generator=gen))
        layer.bias.copy_(0.1 * torch.randn(n_out, device="cuda", generator=gen))
    layer.train()
    x = torch.randn(rows, k_in, device="cuda", generator=gen, dtype=torch.bfloat16)
    _tail_reproduces(layer, x, (rows, n_out), tail, 65536, f"{rows} x {k_in} -> {n_out}")


@pytest.mark.parametrize("geom", [(3700, 64, 64, 96, 2, 2, 0), (520, 64, 64, 96, 3, 1, 1)],
                         ids=["input_2e9", "patches_2.7e9"])
def test_convolution_with_more_than_2_31_elements(geom):
    """Patch extraction, its adjoint and the layout change at more than 2^31 elements: once in the
    input itself (non-overlapping 2x2 patches), once in the patch matrix only (3x3, pad 1)."""
    from hip_helpers import rpu_config
    from aihwkit_lightning.nn import AnalogConv2d

    batch, chan, n_out, size, kernel, stride, pad = geom
    out = (size + 2 * pad - kernel) // stride + 1
    assert batch * out * out * chan * kernel * kernel > 2 ** 31
    c = _big_case(chan * kernel * kernel, n_out)
    gen = torch.Generator(device="cuda").manual_seed(3)
    layer = AnalogConv2d(chan, n_out, kernel, stride=stride, padding=pad, bias=True,
                         dtype=torch.bfloat16, rpu_config=rpu_config(c)).cuda()
    with torch.no_grad():
        layer.weight.copy_(0.05 * torch.randn(layer.weight.shape, device="cuda", generator=gen))
        layer.bias.copy_(0.1 * torch.randn(n_out, device="cuda", generator=gen))
    layer.train()
    x = torch.randn(batch, chan, size, size, device="cuda", generator=gen, dtype=torch.bfloat16)
    _tail_reproduces(layer, x, (batch, n_out, out, out), 16, max(16, batch // 8), f"conv {geom}")
    del x
    torch.cuda.empty_cache()
