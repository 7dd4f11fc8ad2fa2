"""The allocation-free input-gradient entry point (``ahl_linear_bwd_dx_static``, workspace in a
static device array) against ``ahl_linear_bwd_dx`` with a caller workspace, called through the
C ABI directly: same kernels, so outputs must be equal bit for bit. Each case makes two calls in
a row, the second on a smaller problem (the static array still holds the first call's contents).
"""
from ctypes import byref, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _cfg(L, dtype, ir_mode, tile_stride=0):
    cfg = L.AhlLinearCfg()
    cfg.dtype = {torch.bfloat16: L.AHL_BF16, torch.float16: L.AHL_F16, torch.float32: L.AHL_F32}[dtype]
    cfg.ir_mode = ir_mode
    cfg.inp_res, cfg.out_res, cfg.out_bound, cfg.out_noise = 254.0, 254.0, 10.0, 0.0
    cfg.bound_per_channel, cfg.training = 1, 1
    cfg.ir_decay, cfg.ir_input_min_percentage = 0.01, 0.95
    cfg.ir_grad_rule = L.AHL_IR_GRAD_LEARNED
    cfg.tile_stride = tile_stride
    return cfg


def _ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


def _both(L, lib, dtype, m_rows, k_in, n_out, tile, seed, with_mask):
    """dx / ir_grad of the workspace entry point and of the static one on the same operands."""
    gen = torch.Generator().manual_seed(seed)
    g = torch.randn(m_rows, n_out, generator=gen).to(dtype).cuda()
    w = (torch.randn(n_out, k_in, generator=gen) * 0.05).to(dtype).cuda()
    x = (torch.randn(m_rows, k_in, generator=gen) * 1.5).to(dtype).cuda()
    n_tiles = k_in // tile
    ir = torch.linspace(1.0, 3.0, n_tiles).to(dtype).cuda()
    ends = L.tile_ends_array([tile] * n_tiles)
    # tiles that do not start on 256-column boundaries: the weights come in the padded tile layout
    # (tile t at column t * stride, zeros up to the next tile), x and dx stay dense
    cfg = _cfg(L, dtype, L.AHL_IR_STATIC)
    stride = int(lib.ahl_tile_stride(k_in, n_tiles, cfg.dtype))
    ldw = k_in
    if stride > 0:
        padded = torch.zeros(n_out, n_tiles * stride, dtype=dtype, device="cuda")
        for t in range(n_tiles):
            padded[:, t * stride:t * stride + tile] = w[:, t * tile:(t + 1) * tile]
        w, ldw = padded, n_tiles * stride
    keep = flag = None
    if with_mask:
        rows = (m_rows + 63) // 64 * 64
        keep = (torch.rand(n_tiles, (n_out + 31) // 32, rows, generator=gen) < 0.1).to(torch.int32)
        keep = (keep * torch.randint(1, 2 ** 31 - 1, keep.shape, generator=gen, dtype=torch.int32)).cuda()
        flag = torch.ones(1, dtype=torch.int32, device="cuda")
    cfg = _cfg(L, dtype, L.AHL_IR_STATIC, stride)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    need = lib.ahl_linear_bwd_dx_ws_bytes(m_rows, k_in, n_out, n_tiles, cfg.dtype, stride)
    assert 0 < need <= L.STATIC_DX_SCRATCH_BYTES
    out = []
    for static in (False, True):
        dx = torch.full((m_rows, k_in), float("nan"), dtype=dtype, device="cuda")
        ir_grad = torch.full((n_tiles,), float("nan"), dtype=dtype, device="cuda")
        head = [_ptr(g), n_out, _ptr(keep), _ptr(flag), _ptr(w), ldw, _ptr(x), k_in, _ptr(ir), _ptr(dx),
                k_in, _ptr(ir_grad), m_rows, k_in, n_out, ends, n_tiles, byref(cfg)]
        if static:
            rc = lib.ahl_linear_bwd_dx_static(*head, stream)
        else:
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            rc = lib.ahl_linear_bwd_dx(*head, _ptr(ws), stream)
        torch.cuda.synchronize()
        assert rc == 0, (static, rc, lib.ahl_last_hip_error())
        out.append((dx.cpu(), ir_grad.cpu()))
    return out


@pytest.mark.parametrize("dtype,first,second", [
    # bf16 MFMA kernel, few rows: the channels are cut into slices (fp32 partial results in the
    # workspace) -- then a smaller sliced problem
    (torch.bfloat16, (64, 4096, 1024, 512), (32, 1024, 512, 256)),
    # bf16 MFMA kernel, one slice (only the input-range partial sums use the workspace)
    (torch.bfloat16, (1024, 2048, 448, 512), (300, 512, 264, 256)),
    # fp32 general kernels: transposed weights + partial sums in the workspace
    (torch.float32, (96, 768, 640, 256), (17, 60, 24, 20)),
    # the float16 instantiations of the MFMA kernel, sliced and not
    (torch.float16, (64, 4096, 1024, 512), (300, 512, 264, 256)),
    # padded tile layout (2304 inputs in tiles of 576, stride 768; then 1152 in tiles of 384,
    # stride 512): the workspace size follows the padded width
    (torch.bfloat16, (64, 2304, 1024, 576), (200, 1152, 128, 384)),
    (torch.float16, (1024, 2304, 256, 576), (64, 1152, 512, 384)),
], ids=["bf16_sliced", "bf16_one_slice", "f32_general", "f16", "bf16_padded", "f16_padded"])
@pytest.mark.parametrize("with_mask", [False, True], ids=["no_mask", "mask"])
def test_static_scratch_dx_equals_workspace_dx(dtype, first, second, with_mask):
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    lib = L.load()
    for i, (m_rows, k_in, n_out, tile) in enumerate((first, second)):
        (dx_ws, ig_ws), (dx_st, ig_st) = _both(L, lib, dtype, m_rows, k_in, n_out, tile, 90 + i, with_mask)
        assert not torch.isnan(dx_ws.float()).any() and not torch.isnan(ig_ws.float()).any()
        assert float(dx_ws.float().abs().max()) > 0
        assert torch.equal(dx_st, dx_ws), f"dx differs (call {i})"
        assert torch.equal(ig_st, ig_ws), f"input-range gradient differs (call {i})"


def test_static_scratch_rejects_shapes_beyond_its_size():
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    lib = L.load()
    m_rows, k_in, n_out, tile = 64, 4096, 4096, 512   # fp32: 64 MiB of transposed weights
    cfg = _cfg(L, torch.float32, L.AHL_IR_NONE)
    assert lib.ahl_linear_bwd_dx_ws_bytes(m_rows, k_in, n_out, 8, cfg.dtype, 0) > L.STATIC_DX_SCRATCH_BYTES
    g = torch.zeros(m_rows, n_out, device="cuda")
    w = torch.zeros(n_out, k_in, device="cuda")
    dx = torch.full((m_rows, k_in), 7.0, device="cuda")
    rc = lib.ahl_linear_bwd_dx_static(
        _ptr(g), n_out, None, None, _ptr(w), k_in, None, 0, None, _ptr(dx), k_in, None, m_rows, k_in,
        n_out, L.tile_ends_array([tile] * 8), 8, byref(cfg), c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == 5   # AHL_ERR_WORKSPACE
    assert bool((dx == 7.0).all())   # nothing was launched
