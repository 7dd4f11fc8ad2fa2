"""Case definitions shared by the fixture writer (``make_golden.py``) and the tests.

Inputs are regenerated from seeds with torch's CPU generator (bit-reproducible), so the fixture
file holds only the reference's outputs plus input checksums.
"""
import torch

DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}

DEFAULTS = dict(
    dtype="f32", M=8, K=16, N=8, bias=True, max_input_size=-1,
    inp_res=-1.0, out_res=-1.0, out_bound=0.0, out_noise=0.0, out_noise_per_channel=False,
    clip="none", clip_sigma=-1.0, weight_quant="none", weight_noise="none", modifier_res=0.0,
    modifier_std=0.0, ir_mode="none", ir_init=3.0, init_from_data=0, init_std_alpha=3.0,
    ir_decay=0.001, ir_min_pct=0.95, ir_values=None, training=True, kind="fwd_bwd",
    seed=0, noise_seed=1234, x_scale=1.0, w_scale=0.02, steps=0, act_range_momentum=0.95, lwc_scale=1.0,
)


def case(name, **kw):
    out = dict(DEFAULTS)
    unknown = set(kw) - set(DEFAULTS)
    assert not unknown, unknown
    out.update(kw)
    out["name"] = name
    return out


_ADC8 = dict(inp_res=254, out_res=254, out_bound=10.0)

CASES = [
    # configuration 1 of the baseline: 512 -> 512 fp32, 64 tokens, 2 tiles of 256, learned range
    # 3.0, 8-bit DAC/ADC with bound 10, per-channel clip (=> per-channel ADC bound), noise off
    case("c1_fp32", M=64, K=512, N=512, max_input_size=256, ir_mode="static", clip="channel",
         clip_sigma=2.5, ir_decay=0.01, **_ADC8),
    # the same with the output noise on, replayed through the seeded torch generator
    case("c1_fp32_noise", M=64, K=512, N=512, max_input_size=256, ir_mode="static", clip="channel",
         clip_sigma=2.5, ir_decay=0.01, out_noise=0.04, seed=1, **_ADC8),
    # small bf16 layer, 3 uneven tiles (9, 9, 8), ranges tight enough to clip inputs and a bound
    # tight enough to clamp outputs, decay switch exercised by per-tile ranges
    case("bf16_static_clip", dtype="bf16", M=12, K=26, N=16, max_input_size=9, ir_mode="static",
         ir_values=[0.8, 2.5, 1.5], inp_res=254, out_res=254, out_bound=1.5, clip="channel",
         clip_sigma=2.5, ir_decay=0.01, w_scale=0.3, seed=2),
    case("f32_static_clip", M=12, K=26, N=16, max_input_size=9, ir_mode="static",
         ir_values=[0.8, 2.5, 1.5], inp_res=254, out_res=254, out_bound=1.5, clip="channel",
         clip_sigma=2.5, ir_decay=0.01, w_scale=0.3, seed=2),
    # per-tensor ADC bound (clip type not per channel), resolutions given as inverses
    case("f32_static_pertensor", M=9, K=20, N=12, max_input_size=10, ir_mode="static",
         ir_values=[1.0, 2.0], inp_res=1 / 254, out_res=1 / 254, out_bound=2.0, w_scale=0.3,
         ir_decay=0.0, seed=3),
    case("bf16_static_pertensor", dtype="bf16", M=9, K=20, N=12, max_input_size=10,
         ir_mode="static", ir_values=[1.0, 2.0], inp_res=1 / 254, out_res=1 / 254, out_bound=2.0,
         w_scale=0.3, ir_decay=0.0, seed=3),
    # dynamic input range (per token, per tile), with and without per-channel bound
    case("f32_dynamic", M=10, K=24, N=12, max_input_size=12, ir_mode="dynamic", clip="channel",
         clip_sigma=2.5, w_scale=0.3, seed=4, **_ADC8),
    case("bf16_dynamic", dtype="bf16", M=10, K=24, N=12, max_input_size=12, ir_mode="dynamic",
         clip="channel", clip_sigma=2.5, w_scale=0.3, seed=4, **_ADC8),
    case("bf16_dynamic_tight", dtype="bf16", M=10, K=24, N=12, max_input_size=12,
         ir_mode="dynamic", inp_res=254, out_res=254, out_bound=0.3, w_scale=0.3, seed=5),
    # noise paths, replayed bit for bit through torch's generator
    case("f32_outnoise_channel", M=8, K=20, N=10, max_input_size=10, ir_mode="static",
         out_noise=0.1, out_noise_per_channel=True, w_scale=0.3, seed=6, **_ADC8),
    case("bf16_outnoise", dtype="bf16", M=8, K=20, N=10, max_input_size=10, ir_mode="static",
         out_noise=0.1, w_scale=0.3, seed=6, **_ADC8),
    case("f32_wnoise_channel", M=8, K=20, N=10, max_input_size=10, ir_mode="static",
         weight_noise="add_normal_per_channel", modifier_std=0.05, w_scale=0.3, seed=7, **_ADC8),
    case("bf16_wnoise_tensor", dtype="bf16", M=8, K=20, N=10, max_input_size=10, ir_mode="static",
         weight_noise="add_normal", modifier_std=0.05, out_noise=0.05, w_scale=0.3, seed=7, **_ADC8),
    # on-the-fly weight quantisation (straight-through), both scale kinds, both res conventions
    case("f32_wquant_channel", M=8, K=20, N=10, max_input_size=10, weight_quant="discretize_per_channel",
         modifier_res=30, w_scale=0.3, seed=8),
    case("bf16_wquant_tensor", dtype="bf16", M=8, K=20, N=10, max_input_size=10,
         weight_quant="discretize", modifier_res=1 / 30, w_scale=0.3, seed=8),
    case("f32_wquant_noise", M=8, K=20, N=10, max_input_size=10, ir_mode="static",
         weight_quant="discretize_per_channel", modifier_res=14, weight_noise="add_normal_per_channel",
         modifier_std=0.05, w_scale=0.3, seed=9, **_ADC8),
    # plain: no input range, eval mode, no bias
    case("f32_plain_eval", M=7, K=33, N=5, bias=False, training=False, seed=10),
    case("bf16_plain_tiles", dtype="bf16", M=7, K=33, N=5, max_input_size=16, seed=10),
    # DAC only (no output stage), static range without learning data
    case("bf16_dac_only", dtype="bf16", M=16, K=32, N=8, max_input_size=16, ir_mode="static",
         ir_values=[1.0, 3.0], inp_res=254, w_scale=0.3, seed=11),
    # input-range initialisation from data over several training steps
    case("f32_ir_init", kind="ir_init", steps=4, M=16, K=24, N=8, max_input_size=12,
         ir_mode="static", init_from_data=3, inp_res=254, seed=12),
    case("bf16_ir_init", dtype="bf16", kind="ir_init", steps=4, M=16, K=24, N=8, max_input_size=12,
         ir_mode="static", init_from_data=3, inp_res=254, seed=12),
    # fast_mode input range: plain clamp to a range that follows the running min / max of the
    # data; gradients are those of torch.clamp with tensor bounds
    case("f32_fast_clip", M=12, K=26, N=16, max_input_size=9, ir_mode="fast",
         ir_values=[0.8, 2.5, 1.5], inp_res=254, out_res=254, out_bound=1.5, clip="channel",
         clip_sigma=2.5, w_scale=0.3, seed=15),
    case("bf16_fast_clip", dtype="bf16", M=12, K=26, N=16, max_input_size=9, ir_mode="fast",
         ir_values=[0.8, 2.5, 1.5], inp_res=254, out_res=254, out_bound=1.5, clip="channel",
         clip_sigma=2.5, w_scale=0.3, seed=15),
    case("f32_fast_init", kind="ir_fast_init", steps=5, M=16, K=24, N=8, max_input_size=12,
         ir_mode="fast", init_from_data=4, inp_res=254, seed=16),
    case("bf16_fast_init", dtype="bf16", kind="ir_fast_init", steps=5, M=16, K=24, N=8,
         max_input_size=12, ir_mode="fast", init_from_data=4, inp_res=254, seed=16),
    case("f32_fast_init_minmax", kind="ir_fast_init", steps=4, M=16, K=24, N=8, max_input_size=12,
         ir_mode="fast", init_from_data=3, act_range_momentum=-1, inp_res=254, seed=17),
    # learnable per-channel weight clip (LSQ): clip only, clip + on-the-fly quantisation, and clip
    # + weight noise (whose scale is then the learned clip); the clip values start at lwc_scale
    # times the per-tile per-channel abs-max so that some weights are actually clipped
    case("f32_lsq_clip", M=10, K=24, N=12, max_input_size=12, ir_mode="static", clip="learnable",
         lwc_scale=0.6, w_scale=0.3, seed=18, **_ADC8),
    case("bf16_lsq_clip", dtype="bf16", M=10, K=24, N=12, max_input_size=12, ir_mode="static",
         clip="learnable", lwc_scale=0.6, w_scale=0.3, seed=18, **_ADC8),
    case("f32_lsq_quant", M=10, K=24, N=12, max_input_size=12, ir_mode="static", clip="learnable",
         lwc_scale=0.7, weight_quant="discretize_per_channel", modifier_res=30, w_scale=0.3, seed=19,
         **_ADC8),
    case("bf16_lsq_quant", dtype="bf16", M=10, K=24, N=12, max_input_size=12, ir_mode="static",
         clip="learnable", lwc_scale=0.7, weight_quant="discretize_per_channel", modifier_res=30,
         w_scale=0.3, seed=19, **_ADC8),
    case("f32_lsq_clip_wnoise", M=10, K=24, N=12, max_input_size=12, ir_mode="static",
         clip="learnable", lwc_scale=0.6, weight_noise="add_normal_per_channel", modifier_std=0.05,
         w_scale=0.3, seed=20, **_ADC8),
    case("f32_lsq_clip_big", M=6, K=16, N=8, max_input_size=8, clip="learnable", lwc_scale=0.6,
         w_scale=4.0, seed=21),
    # the clip at its initial value (the per-channel abs-max: every channel has a weight exactly on
    # the boundary) and the resolution given as an inverse: the number of states is
    # max(res, 1 / res) in Python's double arithmetic (exactly 30), and whether the boundary weight
    # counts as clipped hangs on the last bit of w / (2 clip / 30)
    case("f32_lsq_quant_boundary", M=1, K=512, N=8, max_input_size=512, ir_mode="static", ir_init=1.0,
         ir_decay=0.0, clip="learnable", lwc_scale=1.0, weight_quant="discretize_per_channel",
         modifier_res=1 / 30, w_scale=0.1, seed=156, **_ADC8),
    # optimizer-step clipping
    case("f32_clip_layer", kind="clip", M=4, K=40, N=24, clip="layer", clip_sigma=2.0, w_scale=1.0,
         seed=13),
    case("f32_clip_channel", kind="clip", M=4, K=40, N=24, clip="channel", clip_sigma=2.0,
         w_scale=1.0, seed=13),
    case("bf16_clip_channel", dtype="bf16", kind="clip", M=4, K=40, N=24, clip="channel",
         clip_sigma=2.0, w_scale=1.0, seed=13),
    # post-training quantisation, including an odd number of states
    case("f32_quantize_channel", kind="quantize", M=4, K=40, N=24, max_input_size=16,
         weight_quant="discretize_per_channel", modifier_res=254, w_scale=0.5, seed=14),
    case("f32_quantize_odd", kind="quantize", M=4, K=40, N=24, max_input_size=16,
         weight_quant="discretize_per_channel", modifier_res=31, w_scale=0.5, seed=14),
    case("bf16_quantize_tensor", dtype="bf16", kind="quantize", M=4, K=40, N=24, max_input_size=16,
         weight_quant="discretize", modifier_res=62, w_scale=0.5, seed=14),
    # post-training quantisation under a learned per-channel clip: the clip alone (the weights
    # are clamped in place), the clip as the quantiser's range, and clip values above one (the
    # "all scales above one" switch of the resolution convention)
    case("f32_quantize_lsq_clip", kind="quantize", M=4, K=40, N=24, max_input_size=16,
         clip="learnable", lwc_scale=0.6, w_scale=0.5, seed=22),
    case("bf16_quantize_lsq_clip", dtype="bf16", kind="quantize", M=4, K=40, N=24, max_input_size=16,
         clip="learnable", lwc_scale=0.6, w_scale=0.5, seed=22),
    case("f32_quantize_lsq_quant", kind="quantize", M=4, K=40, N=24, max_input_size=16,
         clip="learnable", lwc_scale=0.7, weight_quant="discretize_per_channel", modifier_res=30,
         w_scale=0.5, seed=23),
    case("bf16_quantize_lsq_quant", dtype="bf16", kind="quantize", M=4, K=40, N=24,
         max_input_size=16, clip="learnable", lwc_scale=0.7, weight_quant="discretize_per_channel",
         modifier_res=30, w_scale=0.5, seed=23),
    case("f32_quantize_lsq_clip_big", kind="quantize", M=4, K=32, N=8, max_input_size=16,
         clip="learnable", lwc_scale=0.6, w_scale=6.0, seed=24),
]

# float16 (the dtype of the reference's accelerated path and speed scripts): every bfloat16 case
# once more in float16
CASES += [dict(c, name=c["name"].replace("bf16", "f16"), dtype="f16") for c in CASES
          if c["dtype"] == "bf16"]

CASES_BY_NAME = {c["name"]: c for c in CASES}


def make_learnable_clip(c, w):
    """Initial learnable_weight_clip [T, N] of a case: lwc_scale x per-tile per-channel abs-max."""
    k, mx = c["K"], c["max_input_size"]
    n_tiles = 1 if mx <= 0 else -(-k // mx)
    base, extra = divmod(k, n_tiles)
    sizes = [base + 1 if i < extra else base for i in range(n_tiles)]
    parts = torch.split(w.abs().float(), sizes, dim=1)
    return (torch.stack([p.amax(dim=1) for p in parts]) * c["lwc_scale"]).to(w.dtype)


def make_inputs(c):
    """x[M, K], W[N, K], bias[N] or None, grad_out[M, N] for a case, in its dtype."""
    dtype = DTYPES[c["dtype"]]
    gen = torch.Generator().manual_seed(1000 + c["seed"])
    x = (torch.randn(c["M"], c["K"], generator=gen) * c["x_scale"]).to(dtype)
    w = (torch.randn(c["N"], c["K"], generator=gen) * c["w_scale"]).to(dtype)
    b = (torch.randn(c["N"], generator=gen) * 0.1).to(dtype) if c["bias"] else None
    g = torch.randn(c["M"], c["N"], generator=gen).to(dtype)
    return x, w, b, g
