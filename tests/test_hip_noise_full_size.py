"""Noise-on GPU tests at the full benchmark grids (4096 -> 4096 with 8192 tokens, the MLP block's
3072 -> 8192 with 4096 tokens): the kernel instantiations that a training step of the benchmark
configurations launches, with thousands of blocks.

Every K-tile injects its own noise N(0, out_noise / sqrt(T) * IR_t * max|W_tile|) before its ADC
(reference torch_utils/torch_linear.py:255-283); weight noise is N(0, std_dev * max|W_tile[n, :]|)
per tile and channel (:444-460). To see ONE tile's noise in the layer output, the other tiles are
switched off: a static input range of 0 (or, for the dynamic range, all-zero input columns) makes
a tile's quantised input, its noise scale and its ADC bound exactly zero, so the layer output is
that single tile's result bit for bit.

bf16: the clean value lies on the bf16 grid and the noisy one is rounded onto it, so the noise
arrives in whole grid steps; its variance is ulp^2 * sum_k k^2 P(k - 1/2 < n / ulp < k + 1/2) per
element (= sigma^2 + ulp^2 / 12 once sigma exceeds the step), in closed form, and the 1 % bar is
held against that.
"""
import math

import numpy as np
import pytest
import torch

from golden_cases import case, make_inputs
from helpers import assert_close_lsb

pytestmark = pytest.mark.gpu

T_DTYPE = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
SIXTEEN_BIT = ("bf16", "f16")


def _layer(c, w, ir=None):
    from hip_helpers import make_layer

    layer = make_layer(c, inputs=(None, w, None, None))
    if ir is not None:
        layer.input_range.data = ir.to("cuda", T_DTYPE[c["dtype"]])
    return layer


def _wmax(w, n_tiles):
    """[T, N] per-tile per-channel abs-max of w[N, K] (equal tiles), float32 on the GPU."""
    n_out, k_in = w.shape
    return w.cuda().float().abs().view(n_out, n_tiles, k_in // n_tiles).amax(2).t().contiguous()


def _rd(t, dtype):
    """Round an fp32 tensor to the layer dtype and back (the reference's per-op rounding)."""
    return t.to(T_DTYPE[dtype]).float()


def _ulp16(v, dtype):
    """Spacing of the 16-bit type's numbers at the magnitude of v (fp32 tensor; normal range)."""
    _, e = torch.frexp(v.abs().clamp_min(2.0 ** -14))
    return torch.ldexp(torch.ones_like(v), e - (8 if dtype == "bf16" else 11))


def _rounded_noise_var(sigma, ulp):
    """Variance of rd(y + n) - y for a value y on the bf16 grid of spacing `ulp` and n ~ N(0, sigma):
    the noise is rounded to whole grid steps, Var = ulp^2 * sum_k k^2 P(k - 1/2 < n / ulp < k + 1/2).
    For sigma >= 1.5 ulp this is sigma^2 + ulp^2 / 12 to better than 1e-9 (relative); below, the
    sum is evaluated term by term (it falls below sigma^2 once sigma < ulp / 2: small noise is
    mostly rounded away)."""
    sigma, ulp = torch.broadcast_tensors(sigma, ulp)
    s = (sigma / ulp).double()
    var = (s ** 2 + 1.0 / 12.0)
    small = s < 1.5
    ss = s[small].clamp_min(1e-6)
    acc = torch.zeros_like(ss)
    for k in range(1, 10):
        acc += 2.0 * k * k * (torch.special.ndtr((k + 0.5) / ss) - torch.special.ndtr((k - 0.5) / ss))
    var[small] = acc
    return (var * ulp.double() ** 2).float()


def _noise_scale(c, ir, wmax_t, n_tiles):
    """sigma[m or 1, N] of one tile with the path's own roundings:
    rd(wmax_red * rd(out_noise / sqrt(T) * IR))."""
    s = c["out_noise"] / math.sqrt(n_tiles)
    wr = wmax_t if c["out_noise_per_channel"] else wmax_t.max().expand_as(wmax_t)
    return _rd(wr[None, :] * _rd(s * ir, c["dtype"]), c["dtype"])


def _adc(c, ir, wmax_t):
    """Bound B and step r [m or 1, N] of one tile's ADC with the path's roundings."""
    per_channel = c["clip"] in ("channel", "learnable")
    wb = wmax_t if per_channel else wmax_t.max().expand_as(wmax_t)
    bound = _rd(_rd(ir * c["out_bound"], c["dtype"]) * wb[None, :], c["dtype"])
    step = _rd(_rd(2.0 * bound, c["dtype"]) / c["out_res"], c["dtype"])
    return bound, step


def _moments(z):
    z = z.double()
    return float(z.mean()), float(z.std())


FULL = dict(M=8192, K=4096, N=4096, max_input_size=512)
MLP_UP = dict(M=4096, K=3072, N=8192, max_input_size=512)


# ---------------------------------------------------------------------------------------------
# (i) / (ii) output noise per tile, ADC off
@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("per_channel", [False, True], ids=["per_tile_max", "per_channel"])
@pytest.mark.parametrize("ir_mode", ["static", "dynamic"])
def test_output_noise_per_tile_statistics(dtype, per_channel, ir_mode):
    """Mean and std of (noisy - clean) / sigma_t within 1 %, for every tile on its own, at the
    benchmark grid, sigma_t = out_noise / sqrt(T) * IR_t * wmax_t (per channel or the tile's max).
    The tiles carry different ranges, so a mix-up of tiles' scales would show."""
    c = case(f"noise_full_{ir_mode}", dtype=dtype, ir_mode=ir_mode, inp_res=254, out_noise=0.04,
             out_noise_per_channel=per_channel, w_scale=0.02, seed=71, bias=False, **FULL)
    x, w, _, _ = make_inputs(c)
    n_tiles, kt = 8, 512
    wmax = _wmax(w, n_tiles)
    xd = x.cuda()
    ranges = [3.0, 2.0, 2.5, 3.5, 1.5, 3.0, 2.75, 2.25]
    # fp32 runs on the general kernels (~12 ms per forward): three tiles are enough there
    tiles = range(n_tiles) if dtype in SIXTEEN_BIT else (0, 3, 7)
    for t in tiles:
        if ir_mode == "static":
            ir = torch.zeros(n_tiles)
            ir[t] = ranges[t]
            layer = _layer(c, w, ir)
            xin = xd
            ir_rows = torch.full((1, 1), ranges[t], device="cuda")
        else:
            layer = _layer(c, w)
            xin = torch.zeros_like(xd)
            xin[:, t * kt:(t + 1) * kt] = xd[:, t * kt:(t + 1) * kt] * (ranges[t] / 3.0)
            ir_rows = xin[:, t * kt:(t + 1) * kt].float().abs().amax(1, keepdim=True)
        torch.manual_seed(100 + t)
        noisy = layer(xin).float()
        layer.eval()
        clean = layer(xin).float()
        sigma = _noise_scale(c, ir_rows, wmax[t], n_tiles)
        var = sigma ** 2
        if dtype in SIXTEEN_BIT:
            var = _rounded_noise_var(sigma, _ulp16(clean, dtype))
        z = (noisy - clean).detach() / var.sqrt()
        mean, std = _moments(z)
        assert abs(mean) < 0.01, f"tile {t}: mean {mean}"
        assert abs(std - 1.0) < 0.01, f"tile {t}: std {std}"
        # against the wrong tile's scale the same statistic is far off: the test can tell tiles apart
        other = (t + 1) % n_tiles
        if ir_mode == "static":
            wrong = _noise_scale(c, torch.full((1, 1), ranges[other], device="cuda"), wmax[other], n_tiles)
            assert abs(_moments((noisy - clean).detach() / wrong)[1] - 1.0) > 0.03


# ---------------------------------------------------------------------------------------------
# (iii) noise together with the ADC and the clamp
def _emulate_levels(c, acc, sigma, bound, step, gen):
    """ADC levels of rd(acc + sigma * xi) for fresh normals xi, with the path's roundings."""
    xi = torch.randn(acc.shape, device="cuda", generator=gen)
    y = _rd(acc + sigma * xi, c["dtype"])
    rcp = 1.0 / step.clamp_min(1.17549435e-38)
    q = torch.round(_rd(y * rcp, c["dtype"]))
    yq = _rd(q * step, c["dtype"])
    yq = torch.minimum(torch.maximum(yq, -bound), bound)
    return torch.round(yq / step)


@pytest.mark.parametrize("shape,ir_mode,out_noise", [
    (FULL, "static", 0.04), (FULL, "static", 0.4), (FULL, "dynamic", 0.04), (FULL, "dynamic", 0.4),
    (MLP_UP, "static", 0.067), (MLP_UP, "static", 0.67),
], ids=["c3", "c3_x10", "c2", "c2_x10", "c4", "c4_x10"])
@pytest.mark.parametrize("dtype", ["bf16", "f32", "f16"])
def test_output_noise_with_adc_and_clamp(shape, ir_mode, out_noise, dtype):
    """Noise, ADC and clamp together at the benchmark shapes (learned range: the forward of
    configuration 3 and of the MLP block; dynamic range: configuration 2), one tile at a time:
    * every output is a multiple of its ADC step and within the bound;
    * the mean of (noisy - clean) is within 1 % of the standard deviation of that difference;
    * the distribution of the level differences (noisy - clean) / step equals, bin by bin, the one
      obtained by adding torch's own normals of the configured scale to the same pre-ADC values and
      quantising with the path's arithmetic (Monte Carlo with as many samples as outputs).
    The x10 variants put the noise at about the ADC step, where its scale moves every bin."""
    if dtype == "f32" and (out_noise > 0.1 or shape is MLP_UP):
        pytest.skip("fp32 runs the general kernels; one case per range mode is enough")
    c = case("noise_adc", dtype=dtype, ir_mode=ir_mode, inp_res=254, out_res=254, out_bound=10.0,
             out_noise=out_noise, out_noise_per_channel=True, clip="channel", clip_sigma=2.5,
             w_scale=0.02, seed=72, bias=False, **shape)
    x, w, _, _ = make_inputs(c)
    kt = 512
    n_tiles = c["K"] // kt
    wmax = _wmax(w, n_tiles)
    xd = x.cuda()
    gen = torch.Generator(device="cuda").manual_seed(5)
    for t in (0, n_tiles - 1):
        if ir_mode == "static":
            ir = torch.zeros(n_tiles)
            ir[t] = 3.0
            xin = xd
            ir_rows = torch.full((1, 1), 3.0, device="cuda")
        else:
            ir = None
            xin = torch.zeros_like(xd)
            xin[:, t * kt:(t + 1) * kt] = xd[:, t * kt:(t + 1) * kt]
            ir_rows = xin[:, t * kt:(t + 1) * kt].float().abs().amax(1, keepdim=True)
        layer = _layer(c, w, ir)
        torch.manual_seed(200 + t)
        noisy = layer(xin).float()
        layer.eval()
        clean = layer(xin).float()
        # the tile's product before noise and ADC: the same layer without output stage
        plain = _layer(dict(c, out_res=-1.0, out_bound=0.0, out_noise=0.0), w, ir)
        plain.eval()
        acc = plain(xin).float()
        sigma = _noise_scale(c, ir_rows, wmax[t], n_tiles)
        bound, step = _adc(c, ir_rows, wmax[t])
        levels = torch.round(noisy / step)
        on_grid = _rd(levels * step, dtype)
        if dtype in SIXTEEN_BIT:   # exactly a level, or clamped to the bound itself
            assert bool(((on_grid == noisy) | (noisy.abs() == bound)).all())
        else:
            assert float((on_grid - noisy).abs().max()) <= 1e-6 * float(bound.max())
        assert bool((noisy.abs() <= bound).all())
        assert float(levels.abs().max()) <= 127
        d_levels = levels - torch.round(clean / step)
        diff = noisy - clean
        assert abs(float(diff.double().mean())) < 0.01 * float(diff.double().std())
        want = _emulate_levels(c, acc, sigma, bound, step, gen) - torch.round(clean / step)
        lo, hi = int(min(d_levels.min(), want.min())), int(max(d_levels.max(), want.max()))
        assert hi - lo < 64
        got_h = torch.bincount((d_levels - lo).long().flatten(), minlength=hi - lo + 1).double()
        want_h = torch.bincount((want - lo).long().flatten(), minlength=hi - lo + 1).double()
        n = float(got_h.sum())
        for k in range(hi - lo + 1):
            p = float(want_h[k]) / n
            if p < 1e-4:
                continue
            # 1 % of the bin, plus five standard deviations of the two binomial counts
            tol = 0.01 * p + 5.0 * math.sqrt(2.0 * p * (1.0 - p) / n)
            assert abs(float(got_h[k]) / n - p) < tol, f"tile {t} level difference {k + lo}: " \
                f"{float(got_h[k]) / n:.6f} vs {p:.6f}"
        # second moment of the level difference within 1 %
        m2_got = float((d_levels.double() ** 2).mean())
        m2_want = float((want.double() ** 2).mean())
        assert abs(m2_got / m2_want - 1.0) < 0.01 + 5.0 / math.sqrt(m2_want * n)


# ---------------------------------------------------------------------------------------------
# (iv) weight noise at 4096 x 4096
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("kind", ["add_normal_per_channel", "add_normal"])
def test_weight_noise_statistics_at_full_size(dtype, kind):
    """With g = I the rows of dX = g @ W_eff are the noisy weights themselves (no input range, so
    nothing masks dX): per tile, (W_eff - W) / (std_dev * wmax_t) has mean 0 and std 1 within 1 %,
    at 4096 x 4096 with the benchmark's std_dev 0.02; and the forward used the same W_eff."""
    n = 4096
    c = case("wnoise_full", dtype=dtype, M=n, K=n, N=n, max_input_size=512, weight_noise=kind,
             modifier_std=0.02, w_scale=0.02, seed=73, bias=False)
    x, w, _, _ = make_inputs(c)
    layer = _layer(c, w)
    xin = x.cuda().requires_grad_(True)
    torch.manual_seed(9)
    out = layer(xin)
    out.backward(torch.eye(n, device="cuda", dtype=T_DTYPE[dtype]))
    w_eff = xin.grad.float()
    wd = w.cuda().float()
    wmax = _wmax(w, 8)
    for t in range(8):
        sl = slice(512 * t, 512 * (t + 1))
        ref = wmax[t][:, None] if kind == "add_normal_per_channel" else wmax[t].max()
        sigma = _rd(0.02 * ref, dtype)
        var = (sigma ** 2).expand(n, 512)
        if dtype == "bf16":
            var = _rounded_noise_var(sigma.expand(n, 512), _ulp16(wd[:, sl], dtype))
        mean, std = _moments((w_eff[:, sl] - wd[:, sl]) / var.sqrt())
        assert abs(mean) < 0.01, f"tile {t}: mean {mean}"
        assert abs(std - 1.0) < 0.01, f"tile {t}: std {std}"
    # tiles are independent draws
    za = (w_eff[:, :512] - wd[:, :512]).flatten()
    zb = (w_eff[:, 512:1024] - wd[:, 512:1024]).flatten()
    assert abs(float(torch.corrcoef(torch.stack([za, zb]))[0, 1])) < 1e-3
    # the forward multiplied by the same noisy weights: per K-tile product rounded to the dtype
    # and summed in tile order
    want = torch.zeros(n, n, device="cuda", dtype=T_DTYPE[dtype])
    for t in range(8):
        sl = slice(512 * t, 512 * (t + 1))
        want = want + (x.cuda().float()[:, sl] @ w_eff[:, sl].t()).to(T_DTYPE[dtype])
    # (a partial product may round to the neighbouring value when the fp32 summation orders of
    # the two products differ in the last bit: one step of a running total of magnitude < 8)
    assert_close_lsb(out.detach().float().cpu(), want.float().cpu(), 1e-2 if dtype == "bf16" else 1e-5,
                     2.0 ** -5 if dtype == "bf16" else None, max_frac=1e-3, what="forward with noisy weights")


# ---------------------------------------------------------------------------------------------
# (v) shape of the in-kernel normals
def _model_tail_mass(thresholds):
    """P(|r cos(theta)| > c) for the device transform: r^2 = (16 - log2(a)) * 2 ln 2 over the
    65536 values a = i + 0.5, theta uniform."""
    a = np.arange(65536, dtype=np.float64) + 0.5
    r = np.sqrt((16.0 - np.log2(a)) * 2.0 * math.log(2.0))
    out = []
    for c in thresholds:
        ratio = np.clip(c / r, 0.0, 1.0)
        out.append(float(np.mean(np.where(r > c, 2.0 / math.pi * np.arccos(ratio), 0.0))))
    return out, float(np.mean(r ** 4) * 3.0 / 8.0)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_in_kernel_normals_have_a_normal_shape(dtype):
    """The normals the forward kernels draw (Philox4x32-10, Box-Muller on two 16-bit uniforms,
    radius limited to 4.85 sigma), sampled through the layer itself: all-zero input, one active
    tile, no ADC, so that output = sigma * xi. Kurtosis and the mass beyond 2, 3 and 4 sigma agree
    with the transform's own distribution (enumerated on the host) and with the normal
    distribution to the stated deficits; nothing lies beyond the radius limit."""
    c = case("normal_shape", dtype=dtype, ir_mode="static", inp_res=254, out_noise=0.04,
             out_noise_per_channel=True, w_scale=0.02, seed=74, bias=False, **FULL)
    _, w, _, _ = make_inputs(c)
    wmax = _wmax(w, 8)
    zeros = torch.zeros(c["M"], c["K"], device="cuda", dtype=T_DTYPE[dtype])
    samples = []
    for t in (1, 6):
        ir = torch.zeros(8)
        ir[t] = 3.0
        layer = _layer(c, w, ir)
        torch.manual_seed(300 + t)
        out = layer(zeros).float()
        sigma = _noise_scale(c, torch.full((1, 1), 3.0, device="cuda"), wmax[t], 8)
        samples.append((out / sigma).flatten())
    z = torch.cat(samples).double()
    n = z.numel()
    (p2, p3, p4), kurt_model = _model_tail_mass([2.0, 3.0, 4.0])
    exact = [math.erfc(v / math.sqrt(2.0)) for v in (2.0, 3.0, 4.0)]
    # the transform against the normal distribution (host enumeration, no sampling error)
    assert abs(p2 / exact[0] - 1.0) < 2e-3 and abs(p3 / exact[1] - 1.0) < 5e-3
    assert abs(p4 / exact[2] - 1.0) < 5e-3        # the 4.85 sigma radius limit costs 0.2 % of this tail
    assert abs(kurt_model - 3.0) < 5e-3
    # the kernel's samples against the transform; bf16 outputs carry a rounding of 2^-9 relative
    slack = 0.01 if dtype == "bf16" else 0.0
    assert abs(float(z.mean())) < 5.0 / math.sqrt(n)
    assert abs(float(z.std()) - 1.0) < 2e-3
    kurt = float((z ** 4).mean() / (z ** 2).mean() ** 2)
    assert abs(kurt - kurt_model) < 0.01
    for thr, p in ((2.0, p2), (3.0, p3), (4.0, p4)):
        got = float((z.abs() > thr).double().mean())
        assert abs(got / p - 1.0) < slack + 0.01 + 5.0 / math.sqrt(p * n), f"mass beyond {thr}: {got} vs {p}"
    assert float(z.abs().max()) < 4.9
