"""Pins the oracle against what the mathematics and the reference's own tests fix (no GPU):
closed forms, reductions to library routines, brute force, known-answer vectors."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import torch_mode as om


def test_split_rule_matches_reference_examples():
    # nn/modules/linear.py:155-170; 257/128 -> [86, 86, 85] (the code, not the stale docstring)
    assert om.split_sizes(257, 128) == [86, 86, 85]
    assert om.split_sizes(512, 256) == [256, 256]
    assert om.split_sizes(10, -1) == [10]
    assert om.split_sizes(10, 11) == [10]
    assert om.split_sizes(10, 9) == [5, 5]
    for size in range(1, 200):
        for mx in (1, 3, 7, 64, 128):
            sizes = om.split_sizes(size, mx)
            assert sum(sizes) == size and max(sizes) <= mx and max(sizes) - min(sizes) <= 1
            assert len(sizes) == math.ceil(size / mx) and sizes == sorted(sizes, reverse=True)


def test_plain_config_reduces_to_f_linear():
    torch.manual_seed(0)
    x, w, b = torch.randn(9, 37), torch.randn(11, 37), torch.randn(11)
    for max_size in (-1, 8, 37):
        out, _ = om.linear_forward(x, w, b, om.OracleCfg(max_input_size=max_size), None, True)
        assert torch.allclose(out, F.linear(x, w, b), atol=1e-5)


def test_dac_closed_form():
    # user guide: x_q = IR/127 * round(clamp(x, -IR, IR) * 127 / IR) for 254 states
    torch.manual_seed(1)
    x = torch.randn(64, 16, dtype=torch.float64) * 2
    ir = torch.tensor([1.5], dtype=torch.float64)
    cfg = om.OracleCfg(inp_res=254, ir_mode=om.IR_STATIC)
    w = torch.eye(16, dtype=torch.float64)
    out, _ = om.linear_forward(x, w, None, cfg, ir, False)
    expect = torch.round(x.clamp(-1.5, 1.5) * 127 / 1.5) * 1.5 / 127
    assert torch.allclose(out, expect, atol=1e-12)
    # resolution given as 1/states is the same quantiser
    cfg2 = om.OracleCfg(inp_res=1 / 254, ir_mode=om.IR_STATIC)
    out2, _ = om.linear_forward(x, w, None, cfg2, ir, False)
    assert torch.allclose(out2, expect, atol=1e-12)


def test_adc_and_clamp_closed_form_single_tile():
    torch.manual_seed(2)
    x = torch.randn(32, 8, dtype=torch.float64)
    w = torch.randn(5, 8, dtype=torch.float64)
    ir = torch.tensor([10.0], dtype=torch.float64)
    cfg = om.OracleCfg(out_res=254, out_bound=0.05, ir_mode=om.IR_STATIC)
    out, saved = om.linear_forward(x, w, None, cfg, ir, False)
    bound = 10.0 * 0.05 * w.abs().max()
    y = x @ w.T
    step = 2 * bound / 254
    expect = (torch.round(y / step) * step).clamp(-bound, bound)
    assert torch.allclose(out, expect, atol=1e-12)
    assert (~saved["tiles"][0]["keep"]).any(), "the case must clamp something"


def test_output_noise_std_closed_form():
    # docs: sigma_out / sqrt(T) * IR * max|W_tile| per tile, tiles add independently
    x = torch.zeros(4000, 8)
    w = torch.randn(6, 8)
    ir = torch.tensor([2.0, 3.0])
    cfg = om.OracleCfg(max_input_size=4, out_noise=0.3, ir_mode=om.IR_STATIC)
    torch.manual_seed(3)
    out, _ = om.linear_forward(x, w, None, cfg, ir, True)
    wmax = om.sliced_abs_max(w, [4, 4]).amax(1)
    expect = math.sqrt(sum((0.3 / math.sqrt(2) * float(ir[t]) * float(wmax[t])) ** 2 for t in range(2)))
    assert abs(float(out.std()) / expect - 1) < 0.02
    out_eval, _ = om.linear_forward(x, w, None, cfg, ir, False)
    assert float(out_eval.abs().max()) == 0.0


def test_weight_noise_and_quantiser_closed_form():
    # re-derivation in the reference's test_weight_modifier (tests/...against_aihwkit.py:934-965)
    torch.manual_seed(0)
    w = torch.randn(1, 10)
    inp = torch.randn(10, 10)
    for res in (30, 1 / 30):
        n_states = res / 2 if res > 1 else 1 / (2 * res)
        for kind, wmax in ((om.DISCRETIZE_PER_CHANNEL, w.abs().amax(1, keepdim=True)),
                           (om.DISCRETIZE, w.abs().max())):
            step = wmax / n_states
            w_q = (w / step).round() * step
            for noise in (om.NONE, om.ADD_NORMAL, om.ADD_NORMAL_PER_CHANNEL):
                cfg = om.OracleCfg(weight_quant=kind, modifier_res=res, weight_noise=noise,
                                   modifier_std=0.05)
                torch.manual_seed(0)
                out, _ = om.linear_forward(inp, w, None, cfg, None, True)
                torch.manual_seed(0)
                w_eff = w_q if noise == om.NONE else w_q + 0.05 * w.abs().max() * torch.randn_like(w_q)
                assert torch.allclose(out, inp @ w_eff.T, atol=1e-5)


def test_clip_closed_form():
    torch.manual_seed(4)
    w = torch.randn(20, 10)
    for sigma in (2.0, 3.0):
        b = w.std() * sigma
        assert torch.equal(om.clip_weights(w, sigma, False), w.clamp(-b, b))
        b = w.std(1, keepdim=True) * sigma
        assert torch.equal(om.clip_weights(w, sigma, True), w.clamp(-b, b))


def test_quantize_weights_is_idempotent_on_outputs():
    # tests/test_post_training_weight_quantization.py:117-125: the loss of the on-the-fly
    # quantised layer equals the loss after quantising the weights in place
    torch.manual_seed(5)
    x, w = torch.randn(16, 64), torch.randn(24, 64) * 0.2
    for kind in (om.DISCRETIZE, om.DISCRETIZE_PER_CHANNEL):
        for bits in (2, 4, 8):
            res = 2 ** bits - 2
            for max_size in (16, 64):
                cfg = om.OracleCfg(max_input_size=max_size, weight_quant=kind, modifier_res=res)
                before, _ = om.linear_forward(x, w, None, cfg, None, False)
                w_q = om.quantize_weights(w, om.split_sizes(64, max_size), kind, res)
                plain = om.OracleCfg(max_input_size=max_size)
                after, _ = om.linear_forward(x, w_q, None, plain, None, False)
                assert torch.allclose(before, after, atol=1e-6)
                again = om.quantize_weights(w_q, om.split_sizes(64, max_size), kind, res)
                assert torch.allclose(again, w_q, atol=1e-7)


@pytest.mark.parametrize("in_size", [10, 255, 257])
def test_calibration_max_closed_form(in_size):
    # tests/test_calibration.py:155-158
    torch.manual_seed(6)
    batches = [torch.randn(3, 5, in_size) for _ in range(4)]
    in_sizes = om.split_sizes(in_size, 256)
    got = om.calibrate_max(batches, in_sizes)
    allx = torch.cat([b.reshape(-1, in_size) for b in batches])
    for t, (lo, hi) in enumerate(om.tile_bounds(in_sizes)):
        assert float(got[t]) == float(allx[:, lo:hi].abs().max())


def test_sliced_reductions_brute_force():
    # the self-checks at triton_abs_max.py:405-419 and triton_std.py:277-291
    torch.manual_seed(7)
    for n in (1, 10, 25, 255, 257):
        w = torch.randn(n, n)
        sizes = om.split_sizes(n, 128)
        got = om.sliced_abs_max(w, sizes)
        lo = 0
        for t, s in enumerate(sizes):
            for r in range(0, n, max(1, n // 7)):
                assert float(got[t, r]) == max(abs(float(v)) for v in w[r, lo:lo + s])
            lo += s
    x = torch.randn(5, 63)
    sizes = om.split_sizes(63, 11)
    got = om.sliced_std(x, sizes)
    lo = 0
    for t, s in enumerate(sizes):
        vals = x[:, lo:lo + s].reshape(-1).double()
        var = ((vals - vals.mean()) ** 2).sum() / (vals.numel() - 1)
        assert abs(float(got[t]) - math.sqrt(float(var))) < 1e-6
        lo += s


def test_backward_rules_brute_force():
    """The explicit backward against a literal, element-by-element evaluation of the rules:
    clamp mask, straight-through quantisers, input-range gradient with decay switch."""
    torch.manual_seed(8)
    M, K, N = 5, 6, 4
    x = torch.randn(M, K, dtype=torch.float64) * 1.5
    w = torch.randn(N, K, dtype=torch.float64) * 0.4
    g = torch.randn(M, N, dtype=torch.float64)
    ir = torch.tensor([1.0, 2.0], dtype=torch.float64)
    cfg = om.OracleCfg(max_input_size=3, inp_res=14, out_res=14, out_bound=1.2, ir_mode=om.IR_STATIC,
                       ir_decay=0.1, ir_input_min_percentage=0.5)
    out, saved = om.linear_forward(x, w, None, cfg, ir, True)
    dx, dw, db, dir_ = om.linear_backward(g, saved)
    for t, (lo, hi) in enumerate(om.tile_bounds([3, 3])):
        rec = saved["tiles"][t]
        s_up = s_lo = 0.0
        clipped = 0
        for m in range(M):
            for k in range(lo, hi):
                d = sum(float(g[m, n]) * float(rec["keep"][m, n]) * float(w[n, k]) for n in range(N))
                xv, irv = float(x[m, k]), float(ir[t])
                if xv >= irv:
                    s_up += min(d, 0.0)
                if xv <= -irv:
                    s_lo += max(d, 0.0)
                clipped += int(xv >= irv or xv <= -irv)
                expect = 0.0 if abs(xv) > irv else d
                assert abs(float(dx[m, k]) - expect) < 1e-12
        grad = (s_up - s_lo) * float(ir[t])
        if 1.0 - clipped / (M * 3) > 0.5:
            grad += 0.1 * float(ir[t])
        assert abs(float(dir_[t]) - grad) < 1e-12
        for n in range(N):
            for k in range(lo, hi):
                e = sum(float(g[m, n]) * float(rec["keep"][m, n]) * float(rec["xq"][m, k - lo]) for m in range(M))
                assert abs(float(dw[n, k]) - e) < 1e-12
    assert torch.allclose(db, g.sum(0))


def test_philox_known_answers():
    # Random123 known-answer vectors for philox4x32-10
    assert om.philox4x32_10((0, 0, 0, 0), (0, 0)) == (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)
    f = 0xFFFFFFFF
    assert om.philox4x32_10((f, f, f, f), (f, f)) == (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)
    assert om.philox4x32_10((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344),
                            (0xA4093822, 0x299F31D0)) == (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)


def test_bf16_division_by_reciprocal_is_exact():
    """The kernels compute bf16(x / d) as bf16(x * fl32(1/d)) for bf16 operands. Exhaustive over
    all pairs of 8-bit significands (exponents do not matter)."""
    sig = torch.arange(128, 256, dtype=torch.float32)
    x = sig.view(-1, 1).expand(128, 128)
    d = sig.view(1, -1).expand(128, 128)
    exact = (x / d).to(torch.bfloat16)
    via_rcp = (x * (1.0 / d)).to(torch.bfloat16)
    assert torch.equal(exact, via_rcp)
    # and with a reciprocal that is off by one fp32 ulp (v_rcp_f32 accuracy)
    rcp = 1.0 / d
    for delta in (-1, 1):
        bumped = (rcp.view(torch.int32) + delta).view(torch.float32)
        assert torch.equal((x * bumped).to(torch.bfloat16), exact)


def test_float16_division_through_the_reciprocal():
    """How the kernels divide float16 values x / d (both exact in fp32), exhaustive over all pairs
    of 11-bit significands (the significands decide; a few exponent pairs on top):
    * with the correctly rounded fp32 reciprocal, float16(x * rcp) == float16(x / d) -- what the
      paths whose reciprocal comes from an IEEE division use, and the ADC step rd(2B) / n for
      state counts n of up to 11 significant bits (n is then a float16 value like d);
    * with a reciprocal one fp32 step off (the hardware's approximate reciprocal) that fails for a
      few pairs, and one correction step, q0 = x * rcp, r = fma(-d, q0, x), q1 = fma(r, rcp, q0),
      gives the IEEE fp32 quotient bit for bit."""
    def fma32(a, b, c):  # the products below are exact in float64 (at most 11 + 24 bits)
        return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)

    sig = (1024 + np.arange(1024)).astype(np.float32)
    x0, d0 = np.repeat(sig, 1024), np.tile(sig, 1024)
    off_by_one_fails = 0
    for ex, ed in ((0, 0), (-14, 15), (15, -14), (3, -2)):
        x = np.ldexp(x0, ex - 10).astype(np.float32)
        d = np.ldexp(d0, ed - 10).astype(np.float32)
        want = (x / d).astype(np.float32)
        exact_rcp = (np.float32(1.0) / d).astype(np.float32)
        assert np.array_equal((x * exact_rcp).astype(np.float16), want.astype(np.float16)), (ex, ed)
        for towards in (None, np.inf, -np.inf):
            rcp = exact_rcp if towards is None else np.nextafter(exact_rcp, np.float32(towards))
            q0 = (x * rcp).astype(np.float32)
            if towards is not None:
                off_by_one_fails += int((q0.astype(np.float16) != want.astype(np.float16)).sum())
            q1 = fma32(fma32(-d, q0, x), rcp, q0)
            assert np.array_equal(q1, want), (ex, ed, towards)
    assert off_by_one_fails > 0


def test_float16_quotients_below_the_smallest_normal_value():
    """A quotient below 2^-14 is rounded on float16's subnormal grid, where the exact quotient can be
    a tie that the rounded reciprocal tips: float16(x * fl32(1 / d)) differs from float16(x / d) for
    some pairs (x = 5.424e-6, d = 14 among them). The kernels therefore take the corrected quotient
    q1 = fma(fma(-d, q0, x), rcp, q0) whenever |q0| < 6.2e-5 (F16::div_exact_rcp), and divide for an
    ADC step that small (adc_step). Exhaustive over every finite float16 x, for the state counts the
    resolution sweeps use and a few float16 steps as divisors: the guarded quotient equals the IEEE
    fp32 quotient wherever the guard applies, and float16-rounds like it everywhere."""
    def fma32(a, b, c):
        return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)

    bits = np.arange(65536, dtype=np.uint16)
    x = bits.view(np.float16).astype(np.float32)
    x = x[np.isfinite(x)]
    divisors = [14.0, 30.0, 126.0, 254.0, 510.0, 1000.0, 1022.0, 2046.0, 3.0, 5.0,
                float(np.float16(0.0189)), float(np.float16(3.3e-3)), float(np.float16(1.7)), float(np.float16(6.5e-5))]
    plain_fails = 0
    for dv in divisors:
        d = np.full_like(x, np.float32(dv))
        want32 = (x / d).astype(np.float32)
        rcp = (np.float32(1.0) / d).astype(np.float32)
        q0 = (x * rcp).astype(np.float32)
        q1 = fma32(fma32(-d, q0, x), rcp, q0)
        q1 = np.where((x == 0) | ~np.isfinite(q0), q0, q1)   # zero keeps its sign (the device's class test)
        small = np.abs(q0) < np.float32(6.2e-5)
        with np.errstate(over="ignore"):
            plain_fails += int((q0.astype(np.float16) != want32.astype(np.float16)).sum())
            guarded = np.where(small, q1, q0)
            assert np.array_equal(q1[small], want32[small]), dv
            assert np.array_equal(guarded.astype(np.float16), want32.astype(np.float16)), dv
            # the plain product is wrong only where the guard applies ...
            wrong = q0.astype(np.float16) != want32.astype(np.float16)
            assert not bool((wrong & ~small).any()), dv
            # ... and rounding to an integer hides it (F16::div_to_round)
            assert np.array_equal(np.rint(q0.astype(np.float16).astype(np.float32)),
                                  np.rint(want32.astype(np.float16).astype(np.float32))), dv
    assert plain_fails > 0


def test_box_muller16_statistics():
    """The device transform (two 16-bit uniforms per pair) has mean 0 and variance 1 to 1e-3
    when enumerated over a full grid of its inputs."""
    a = np.arange(65536, dtype=np.float64) + 0.5
    r = np.sqrt((16.0 - np.log2(a)) * 2.0 * math.log(2.0))
    assert abs(np.mean(r ** 2) / 2.0 - 1.0) < 1e-3  # E[r^2] = 2 for a unit normal pair
    b = 1.0 + np.arange(65536, dtype=np.float64) / 65536.0  # revolutions, mantissa of a float in [1, 2)
    c, s_ = np.cos(2 * np.pi * b), np.sin(2 * np.pi * b)
    # radius and angle are independent: moments factorise over the grid
    assert abs(c.mean()) < 1e-12 and abs(s_.mean()) < 1e-12
    assert abs(np.mean(r ** 2) * np.mean(c ** 2) - 1.0) < 1e-4
    assert abs(np.mean(r ** 2) * np.mean(s_ ** 2) - 1.0) < 1e-4
    assert abs(np.mean(c * s_)) < 1e-12
    assert 4.8 < r.max() < 4.9  # the stated tail limit
