"""GPU parity at the full benchmark sizes (4096 -> 4096, 8192 tokens, 8 tiles of 512, bf16).

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


@pytest.mark.parametrize("ir_mode", ["static", "dynamic"])
def test_full_size_analog_matches_oracle(ir_mode):
    from hip_helpers import hip_fwd_bwd

    # out_bound 0.9 clamps a visible fraction of the tile outputs, so the clamp mask and the
    # "anything clamped" flag are exercised at the full grid as well
    c = case(f"full_{ir_mode}", ir_mode=ir_mode, inp_res=254, out_res=254, out_bound=0.9,
             clip="channel", clip_sigma=2.5, ir_decay=0.01, ir_init=3.0, w_scale=0.02, seed=42, **FULL)
    inputs = make_inputs(c)
    res = hip_fwd_bwd(c, inputs=inputs)
    torch.set_num_threads(16)
    ref = oracle_fwd_bwd(c)
    # An ADC level that flips in one tile (rounding-boundary tie, from the different fp32
    # accumulation order of the two GEMMs) moves that tile's output by one ADC step; the bf16
    # running sum over the 8 tiles can then land on the neighbouring bf16 value of a partial sum
    # of magnitude < 2, i.e. 2^-7, which is larger than the ADC step itself. Allowed on at most
    # 0.001 % of the elements.
    lsb = 2.0 ** -7
    assert_close_lsb(res["out"].float(), ref["out"].float(), 1e-2, lsb, max_frac=1e-5,
                     what=f"{c['name']} out")
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
        assert_close_lsb(res[key].float(), ref[key].float(), 1e-2, flip[key], max_frac=1e-3,
                         what=f"{c['name']} {key}")
