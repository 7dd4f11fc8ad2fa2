"""Torch custom ops (namespace ``aihwkit_hip``) over the C ABI of ``libanalog_hip.so``.

Each op allocates its outputs and scratch with torch (device memory plumbing only), passes raw
device pointers, sizes and the current HIP stream to one C entry point, and returns. The ops are
registered for the CUDA (= ROCm/HIP) dispatch key only: calling them on CPU tensors raises.
"""
import os
import sys
import threading
from ctypes import byref, c_void_p
from functools import lru_cache
from typing import List, Optional, Tuple

import torch
from torch import Tensor

from . import library as L
from ....exceptions import HipBackendError

_DTYPES = {torch.float32: L.AHL_F32, torch.bfloat16: L.AHL_BF16, torch.float16: L.AHL_F16}


def dtype_id(dtype: torch.dtype) -> int:
    """Map a torch dtype onto the ABI's dtype enum."""
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise HipBackendError(
            f"dtype {dtype} is not supported by the HIP backend (float32, bfloat16 and float16 are)"
        ) from None


# Shape inference ("fake" / meta kernels, what torch.compile and torch.library.opcheck ask an
# op for) runs the op's own Python with the launches left out: inside `_shapes_only()` pointers
# and the stream are null, every entry point returns 0 (the OK status; as a workspace size: no
# workspace) without being called, and sizes may be symbolic. The switch is per thread: while one
# thread traces, the autograd engine's device thread (which runs the backward ops) must go on
# launching.
class _ShapesOnly(threading.local):
    depth = 0


_SHAPES_ONLY = _ShapesOnly()


class _NoLaunch:
    """Stands in for the library while shapes are inferred: every entry point is ``lambda *a: 0``."""

    def __getattr__(self, name):
        return lambda *args: 0


def _lib():
    return _NoLaunch() if _SHAPES_ONLY.depth else L.load()


def _shapes_only(fn):
    """``fn`` as a fake kernel: same outputs (shapes, dtypes, devices), nothing launched."""
    def fake(*args, **kwargs):
        _SHAPES_ONLY.depth += 1
        try:
            return fn(*args, **kwargs)
        finally:
            _SHAPES_ONLY.depth -= 1
    return fake


def _ptr(tensor: Optional[Tensor]):
    if tensor is None or _SHAPES_ONLY.depth:
        return None
    return c_void_p(tensor.data_ptr())


def _ref(struct):
    return None if struct is None else byref(struct)


def _aligned16(tensor: Tensor) -> bool:
    return bool(_SHAPES_ONLY.depth) or tensor.data_ptr() % 16 == 0


_raw_stream = torch._C._cuda_getCurrentRawStream  # pylint: disable=protected-access
_current_device = torch._C._cuda_getDevice if hasattr(torch._C, "_cuda_getDevice") else torch.cuda.current_device  # pylint: disable=protected-access


def _stream():
    if _SHAPES_ONLY.depth:
        return None
    # the raw handle of torch's current stream, without building a Stream object per launch
    return c_void_p(_raw_stream(_current_device()))


def _rows2d(tensor: Tensor, name: str) -> Tensor:
    if tensor.dim() != 2:
        raise HipBackendError(f"{name} must be 2-D, got shape {tuple(tensor.shape)}")
    if tensor.stride(1) != 1 and tensor.size(1) != 1:
        tensor = tensor.contiguous()
    if tensor.size(0) > 1 and tensor.stride(0) < tensor.size(1):
        tensor = tensor.contiguous()
    return tensor


def _vector_aligned(tensor: Tensor) -> Tensor:
    """``tensor`` itself if its rows start on 16-byte boundaries, else a fresh contiguous copy (the
    MFMA kernels load whole 16-byte vectors; with operands in the padded tile layout there is no
    other kernel to fall back to)."""
    if _aligned16(tensor) and (_ld(tensor) * tensor.element_size()) % 16 == 0:
        return tensor
    return tensor.clone(memory_format=torch.contiguous_format)


def _ld(tensor: Tensor) -> int:
    return tensor.stride(0) if tensor.size(0) > 1 else max(tensor.size(1), tensor.stride(0))


def _linear_cfg(dtype: torch.dtype, icfg: List[int], fcfg: List[float]) -> L.AhlLinearCfg:
    cfg = L.AhlLinearCfg()
    cfg.dtype = dtype_id(dtype)
    (cfg.ir_mode, cfg.out_noise_per_channel, cfg.bound_per_channel, cfg.training,
     cfg.skip_rounding, seed, offset) = icfg[:7]
    cfg.ir_grad_rule = icfg[7] if len(icfg) > 7 else L.AHL_IR_GRAD_LEARNED
    cfg.tile_stride = icfg[8] if len(icfg) > 8 else 0
    # device address of the noise state {key, call counter} (0: the seed comes by value)
    cfg.seed_state = (icfg[9] or None) if len(icfg) > 9 else None
    # what "something was clamped" looks like in the forward's one-word flag (0: the library
    # clears the word itself with a launch of its own and uses "non-zero")
    cfg.flag_token = icfg[10] if len(icfg) > 10 else 0
    (cfg.inp_res, cfg.out_res, cfg.out_bound, cfg.out_noise, cfg.ir_decay,
     cfg.ir_input_min_percentage) = fcfg
    cfg.seed, cfg.offset = seed, offset
    return cfg


LIB = torch.library.Library("aihwkit_hip", "DEF")

LIB.define("sliced_absmax(Tensor x, int[] in_sizes, bool tile_stats) -> (Tensor, Tensor, Tensor)")
LIB.define("sliced_std(Tensor x, int[] in_sizes) -> Tensor")
LIB.define("row_nonzero(Tensor x) -> Tensor")
LIB.define("sliced_std_kept(Tensor x, int[] in_sizes) -> Tensor")
LIB.define("sliced_quantile(Tensor x, int[] in_sizes, float q) -> Tensor")
LIB.define(
    "ir_moving_update(Tensor(a!) ir, Tensor(b!) idx, Tensor val, float alpha, bool val_in_dtype) -> ()"
)
LIB.define(
    "ir_init_update(Tensor(a!) ir, Tensor(b!) idx, Tensor std, float init_from_data, "
    "float alpha) -> ()"
)
LIB.define("running_absmax(Tensor x, int[] in_sizes, Tensor(a!) cache) -> ()")
LIB.define(
    "ir_fast_update(Tensor x, int[] in_sizes, Tensor(a!) ir, Tensor(b!) idx, Tensor(c!) x_min, "
    "Tensor(d!) x_max, float init_from_data, float momentum) -> ()"
)
LIB.define("clip_weights(Tensor(a!) w, float sigma, int kind) -> ()")
LIB.define("col_sum(Tensor x) -> Tensor")
LIB.define(
    "weight_prep(Tensor w, int[] in_sizes, int quant_type, int noise_type, float res, "
    "float std_dev, int seed, int offset, bool want_eff, bool skip_tile_stats=False, "
    "int seed_state=0) -> (Tensor, Tensor, Tensor, Tensor)"
)
LIB.define("quantize_weights(Tensor(a!) w, int[] in_sizes, int quant_type, float res) -> ()")
LIB.define(
    "weight_prep_clip(Tensor w, Tensor clip, int[] in_sizes, int quant_type, int noise_type, "
    "float res, float std_dev, int seed, int offset, int seed_state=0) -> (Tensor, Tensor, Tensor)"
)
LIB.define(
    "learned_clip_bwd(Tensor(a!) dw, Tensor w, Tensor clip, Tensor tile_min, int[] in_sizes, "
    "int quant_type, float res) -> Tensor"
)
LIB.define(
    "dac(Tensor x, Tensor? ir, int[] in_sizes, int[] icfg, float[] fcfg) -> (Tensor, Tensor)"
)
LIB.define(
    "linear_fwd(Tensor? x, Tensor? xq, Tensor w_eff, Tensor? bias, Tensor? ir, Tensor? wmax, "
    "Tensor? tile_max, int[] in_sizes, int[] icfg, float[] fcfg, bool want_keep) "
    "-> (Tensor, Tensor, Tensor)"
)
LIB.define(
    "linear_bwd_dx(Tensor g, Tensor? keep, Tensor? clamp_flag, Tensor w_eff, Tensor? x, "
    "Tensor? ir, int[] in_sizes, int[] icfg, float[] fcfg) -> (Tensor, Tensor)"
)
LIB.define(
    "linear_bwd_dw(Tensor g, Tensor? keep, Tensor? clamp_flag, Tensor? x, Tensor? xq, Tensor? ir, "
    "int[] in_sizes, int[] icfg, float[] fcfg, bool want_bias) -> (Tensor, Tensor)"
)
LIB.define("pad_tiles(Tensor x, int[] in_sizes, int stride) -> Tensor")
LIB.define("unpad_tiles(Tensor x, int[] in_sizes, int stride) -> Tensor")
LIB.define("im2col(Tensor x, int[] geom) -> Tensor")
LIB.define("col2im(Tensor dcols, int[] geom) -> Tensor")
LIB.define("transpose_batched(Tensor src) -> Tensor")


_NOISE_STATES = {}


def noise_state(device: torch.device, create: bool = True) -> Optional[Tensor]:
    """The device-resident noise state of ``device``: int64 ``[2]`` = (Philox key, call counter).

    Launches that are replayed from a HIP graph cannot carry their seed by value (every replay
    would draw the same noise): under stream capture the layers point their kernels at this
    state and record one :func:`seed_advance` per call. The key is drawn from torch's CPU
    generator when the state is created, so ``torch.manual_seed`` makes graphed runs reproducible.
    It has to exist before a capture starts (creating it copies from the host)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    state = _NOISE_STATES.get(index)
    if state is None and create:
        key = int(torch.randint(0, 2**62, (1,)).item())
        state = torch.tensor([key, 0], dtype=torch.int64, device=torch.device("cuda", index))
        _NOISE_STATES[index] = state
    return state


def seed_advance(state: Tensor, delta: int) -> None:
    """``state[1] += delta`` on the device (one small launch on the current stream)."""
    L.check(_lib().ahl_seed_advance(_ptr(state), int(delta), _stream()), "ahl_seed_advance")


def tile_stride(k_in: int, n_tiles: int, dtype: torch.dtype) -> int:
    """Column stride of the padded tile layout the fast kernels want for this split, or 0 when
    the dense layout already suits them (host arithmetic in the library)."""
    return int(_lib().ahl_tile_stride(k_in, n_tiles, dtype_id(dtype)))


def pad_tiles(x: Tensor, in_sizes: List[int], stride: int) -> Tensor:
    """Dense ``[rows, K]`` to the padded tile layout ``[rows, T * stride]``."""
    lib = _lib()
    x = _rows2d(x, "x")
    rows, k_in = x.shape
    n_tiles = len(in_sizes)
    out = torch.empty((rows, n_tiles * stride), dtype=x.dtype, device=x.device)
    L.check(lib.ahl_pad_tiles(_ptr(x), _ld(x), dtype_id(x.dtype), rows, k_in,
                              L.tile_ends_array(in_sizes), n_tiles, stride, _ptr(out),
                              n_tiles * stride, _stream()), "ahl_pad_tiles")
    return out


def unpad_tiles(x: Tensor, in_sizes: List[int], stride: int) -> Tensor:
    """Padded tile layout ``[rows, T * stride]`` back to dense ``[rows, K]``."""
    lib = _lib()
    x = _rows2d(x, "x")
    rows, k_in, n_tiles = x.size(0), sum(in_sizes), len(in_sizes)
    out = torch.empty((rows, k_in), dtype=x.dtype, device=x.device)
    L.check(lib.ahl_unpad_tiles(_ptr(x), _ld(x), dtype_id(x.dtype), rows, k_in,
                                L.tile_ends_array(in_sizes), n_tiles, stride, _ptr(out), k_in,
                                _stream()), "ahl_unpad_tiles")
    return out


def conv_geom(geom: List[int]) -> L.AhlConvGeom:
    """``[batch, channels, in(3), kernel(3), stride(3), padding(3), dilation(3)]`` as the ABI's
    geometry struct."""
    if len(geom) != 17:
        raise HipBackendError(f"a convolution geometry has 17 integers, got {len(geom)}")
    if _SHAPES_ONLY.depth:
        return None
    out = L.AhlConvGeom()
    out.batch, out.channels = int(geom[0]), int(geom[1])
    for i in range(3):
        out.in_size[i] = int(geom[2 + i])
        out.kernel[i] = int(geom[5 + i])
        out.stride[i] = int(geom[8 + i])
        out.padding[i] = int(geom[11 + i])
        out.dilation[i] = int(geom[14 + i])
    return out


def conv_out_size(geom: List[int]) -> List[int]:
    """Output extents (3) of a convolution geometry; host arithmetic in the library."""
    if _SHAPES_ONLY.depth:   # the same formula on what may be symbolic sizes
        return [(geom[2 + i] + 2 * geom[11 + i] - geom[14 + i] * (geom[5 + i] - 1) - 1) // geom[8 + i] + 1
                for i in range(3)]
    out = (L.c_int32 * 3)()
    L.check(_lib().ahl_conv_out_size(byref(conv_geom(geom)), out), "ahl_conv_out_size")
    return [int(v) for v in out]


def im2col(x: Tensor, geom: List[int]) -> Tensor:
    """Patches ``[B, L, C * kD * kH * kW]`` of ``x [B, C, D, H, W]``."""
    lib = _lib()
    x = x.contiguous()
    cgeom = conv_geom(geom)
    if x.numel() != geom[0] * geom[1] * geom[2] * geom[3] * geom[4]:
        raise HipBackendError(f"input of shape {tuple(x.shape)} does not match geometry {geom}")
    out_size = conv_out_size(geom)
    n_pos = out_size[0] * out_size[1] * out_size[2]
    k_in = geom[1] * geom[5] * geom[6] * geom[7]
    cols = torch.empty((geom[0], n_pos, k_in), dtype=x.dtype, device=x.device)
    L.check(lib.ahl_im2col(_ptr(x), _ref(cgeom), dtype_id(x.dtype), _ptr(cols), k_in, _stream()),
            "ahl_im2col")
    return cols


def col2im(dcols: Tensor, geom: List[int]) -> Tensor:
    """Adjoint of :func:`im2col`: ``[B, L, K]`` patch gradients to ``[B, C, D, H, W]``."""
    lib = _lib()
    dcols = dcols.contiguous()
    cgeom = conv_geom(geom)
    out_size = conv_out_size(geom)
    k_in = geom[1] * geom[5] * geom[6] * geom[7]
    if dcols.numel() != geom[0] * out_size[0] * out_size[1] * out_size[2] * k_in:
        raise HipBackendError(f"patches of shape {tuple(dcols.shape)} do not match geometry {geom}")
    dx = torch.empty((geom[0], geom[1], geom[2], geom[3], geom[4]), dtype=dcols.dtype,
                     device=dcols.device)
    L.check(lib.ahl_col2im(_ptr(dcols), k_in, _ref(cgeom), dtype_id(dcols.dtype), _ptr(dx),
                           _stream()), "ahl_col2im")
    return dx


def transpose_batched(src: Tensor) -> Tensor:
    """``dst[b, c, r] = src[b, r, c]`` as a new contiguous tensor."""
    lib = _lib()
    if src.dim() != 3:
        raise HipBackendError(f"transpose_batched takes a 3-D tensor, got {tuple(src.shape)}")
    src = src.contiguous()
    batch, rows, cols = src.shape
    dst = torch.empty((batch, cols, rows), dtype=src.dtype, device=src.device)
    if src.numel() > 0:
        L.check(lib.ahl_transpose_batched(_ptr(src), cols, dtype_id(src.dtype), batch, rows, cols,
                                          _ptr(dst), rows, _stream()), "ahl_transpose_batched")
    return dst


def sliced_absmax(x: Tensor, in_sizes: List[int], tile_stats: bool) -> Tuple[Tensor, Tensor, Tensor]:
    """``out[t, r] = max |x[r, tile t]|`` (+ per-tile max/min over rows)."""
    lib = _lib()
    x = _rows2d(x, "x")
    n_tiles, rows = len(in_sizes), x.size(0)
    out = torch.empty((n_tiles, rows), dtype=x.dtype, device=x.device)
    n_stats = n_tiles if tile_stats else 0
    tile_max = torch.empty((n_stats,), dtype=torch.float32, device=x.device)
    tile_min = torch.empty((n_stats,), dtype=torch.float32, device=x.device)
    L.check(
        lib.ahl_sliced_absmax(
            _ptr(x), dtype_id(x.dtype), rows, x.size(1), _ld(x), L.tile_ends_array(in_sizes), n_tiles,
            _ptr(out), _ptr(tile_max) if tile_stats else None,
            _ptr(tile_min) if tile_stats else None, _stream(),
        ),
        "ahl_sliced_absmax",
    )
    return out, tile_max, tile_min


def sliced_std(x: Tensor, in_sizes: List[int]) -> Tensor:
    """Unbiased std of every K-tile over all rows, float32 ``[T]``."""
    lib = _lib()
    x = _rows2d(x, "x")
    n_tiles = len(in_sizes)
    out = torch.empty((n_tiles,), dtype=torch.float32, device=x.device)
    ws = torch.empty((lib.ahl_sliced_std_ws_bytes(x.size(0), n_tiles),), dtype=torch.uint8,
                     device=x.device)
    L.check(
        lib.ahl_sliced_std(
            _ptr(x), dtype_id(x.dtype), x.size(0), x.size(1), _ld(x), L.tile_ends_array(in_sizes),
            n_tiles, _ptr(out), _ptr(ws), _stream(),
        ),
        "ahl_sliced_std",
    )
    return out


def row_nonzero(x: Tensor) -> Tensor:
    """uint8 ``[rows]``: 1 for every row of ``x`` that is not all zero."""
    lib = _lib()
    x = _rows2d(x, "x")
    kept = torch.empty((x.size(0),), dtype=torch.uint8, device=x.device)
    count = torch.empty((1,), dtype=torch.int32, device=x.device)
    L.check(
        lib.ahl_row_nonzero(_ptr(x), dtype_id(x.dtype), x.size(0), x.size(1), _ld(x), _ptr(kept),
                            _ptr(count), _stream()),
        "ahl_row_nonzero",
    )
    return kept


def sliced_std_kept(x: Tensor, in_sizes: List[int]) -> Tensor:
    """Unbiased std of every K-tile over the rows that are not all zero, float32 ``[T]``."""
    lib = _lib()
    x = _rows2d(x, "x")
    n_tiles = len(in_sizes)
    out = torch.empty((n_tiles,), dtype=torch.float32, device=x.device)
    ws = torch.empty((lib.ahl_sliced_std_kept_ws_bytes(x.size(0), n_tiles),), dtype=torch.uint8,
                     device=x.device)
    L.check(
        lib.ahl_sliced_std_kept(
            _ptr(x), dtype_id(x.dtype), x.size(0), x.size(1), _ld(x), L.tile_ends_array(in_sizes),
            n_tiles, _ptr(out), _ptr(ws), _stream(),
        ),
        "ahl_sliced_std_kept",
    )
    return out


def sliced_quantile(x: Tensor, in_sizes: List[int], q: float) -> Tensor:
    """``torch.quantile(x[kept rows, tile].float().flatten(), q)`` of every K-tile, float32
    ``[T]``; kept rows are those that are not all zero."""
    lib = _lib()
    x = _rows2d(x, "x")
    n_tiles = len(in_sizes)
    out = torch.empty((n_tiles,), dtype=torch.float32, device=x.device)
    ws = torch.empty((lib.ahl_sliced_quantile_ws_bytes(x.size(0), n_tiles),), dtype=torch.uint8,
                     device=x.device)
    L.check(
        lib.ahl_sliced_quantile(
            _ptr(x), dtype_id(x.dtype), x.size(0), x.size(1), _ld(x), L.tile_ends_array(in_sizes),
            n_tiles, float(q), _ptr(out), _ptr(ws), _stream(),
        ),
        "ahl_sliced_quantile",
    )
    return out


def ir_moving_update(ir: Tensor, idx: Tensor, val: Tensor, alpha: float, val_in_dtype: bool) -> None:
    """In-place moving-average step of the calibrated ranges; ``idx`` is int32 ``[T]``."""
    lib = _lib()
    if not (ir.is_contiguous() and idx.is_contiguous() and idx.dtype == torch.int32
            and val.dtype == torch.float32 and val.is_contiguous()):
        raise HipBackendError("ir_moving_update: contiguous ir, int32 idx and float32 val expected")
    L.check(
        lib.ahl_ir_moving_update(_ptr(ir), _ptr(idx), _ptr(val), dtype_id(ir.dtype), ir.numel(),
                                 float(alpha), int(val_in_dtype), _stream()),
        "ahl_ir_moving_update",
    )


def ir_init_update(ir: Tensor, idx: Tensor, std: Tensor, init_from_data: float, alpha: float) -> None:
    """In-place input-range initialisation step from the per-tile std."""
    lib = _lib()
    if not (ir.is_contiguous() and idx.is_contiguous() and ir.dtype == idx.dtype):
        raise HipBackendError("input_range and input_range_update_idx must be contiguous, same dtype")
    L.check(
        lib.ahl_ir_init_update(
            _ptr(ir), _ptr(idx), _ptr(std), dtype_id(ir.dtype), ir.numel(), init_from_data, alpha,
            _stream(),
        ),
        "ahl_ir_init_update",
    )


def running_absmax(x: Tensor, in_sizes: List[int], cache: Tensor) -> None:
    """``cache[t] = max(cache[t], max |x[:, tile t]|)``; cache is float32 ``[T]`` on the device."""
    lib = _lib()
    if cache.dtype != torch.float32 or not cache.is_contiguous() or cache.numel() != len(in_sizes):
        raise HipBackendError("cache must be a contiguous float32 tensor with one entry per tile")
    # a calibration pass calls this once per layer and batch, and the launch is short: the usual
    # case (a contiguous 2-D batch) skips the general stride handling
    if x.dim() == 2 and x.is_contiguous():
        rows, cols = x.shape
        ld = cols
    else:
        x = _rows2d(x, "x")
        rows, cols, ld = x.size(0), x.size(1), _ld(x)
    L.check(
        lib.ahl_running_absmax(
            _ptr(x), dtype_id(x.dtype), rows, cols, ld, L.tile_ends_array(in_sizes),
            len(in_sizes), _ptr(cache), _stream(),
        ),
        "ahl_running_absmax",
    )


def ir_fast_update(x: Tensor, in_sizes: List[int], ir: Tensor, idx: Tensor, x_min: Tensor,
                   x_max: Tensor, init_from_data: float, momentum: float) -> None:
    """In-place fast_mode update of the running min / max, the step counter and the range."""
    lib = _lib()
    x = _rows2d(x, "x")
    for buf in (ir, idx, x_min, x_max):
        if not (buf.is_contiguous() and buf.dtype == x.dtype and buf.numel() == len(in_sizes)):
            raise HipBackendError("input_range, its counter, x_min and x_max must be contiguous "
                                  "[n_tiles] tensors of the input dtype")
    ws = torch.empty((lib.ahl_ir_fast_update_ws_bytes(x.size(0), len(in_sizes)),), dtype=torch.uint8,
                     device=x.device)
    L.check(
        lib.ahl_ir_fast_update(
            _ptr(x), dtype_id(x.dtype), x.size(0), x.size(1), _ld(x), L.tile_ends_array(in_sizes),
            len(in_sizes), _ptr(ir), _ptr(idx), _ptr(x_min), _ptr(x_max), init_from_data, momentum,
            _ptr(ws), _stream(),
        ),
        "ahl_ir_fast_update",
    )


def clip_weights(w: Tensor, sigma: float, kind: int) -> None:
    """In-place clamp of ``w`` at ``sigma`` standard deviations (per matrix or per row)."""
    lib = _lib()
    if w.dim() != 2 or w.stride(1) != 1:
        raise HipBackendError("weight must be a row-major 2-D tensor")
    ws = torch.empty((lib.ahl_clip_weights_ws_bytes(w.size(0)),), dtype=torch.uint8, device=w.device)
    L.check(
        lib.ahl_clip_weights(
            _ptr(w), dtype_id(w.dtype), w.size(0), w.size(1), _ld(w), sigma, kind, _ptr(ws), _stream()
        ),
        "ahl_clip_weights",
    )


def col_sum(x: Tensor) -> Tensor:
    """Column sums of a 2-D tensor in its dtype (float accumulation)."""
    lib = _lib()
    x = _rows2d(x, "x")
    out = torch.empty((x.size(1),), dtype=x.dtype, device=x.device)
    ws = torch.empty((lib.ahl_col_sum_ws_bytes(x.size(1)),), dtype=torch.uint8, device=x.device)
    L.check(
        lib.ahl_col_sum(
            _ptr(x), dtype_id(x.dtype), x.size(0), x.size(1), _ld(x), _ptr(out), _ptr(ws), _stream()
        ),
        "ahl_col_sum",
    )
    return out


def _modifier_cfg(dtype, quant_type, noise_type, res, std_dev, seed, offset,
                  seed_state: int = 0) -> L.AhlModifierCfg:
    cfg = L.AhlModifierCfg()
    cfg.dtype = dtype_id(dtype)
    cfg.quant_type, cfg.noise_type = quant_type, noise_type
    # The reference derives the number of states as max(res, 1 / res) in Python (double) and only
    # then enters tensor arithmetic; the library would do the same in float, where 1 / (1 / 30) is
    # 29.999998. The number of states itself is passed (a value >= 1 is taken as it is).
    cfg.res = max(res, 1.0 / res) if res > 0 else res
    cfg.std_dev = std_dev
    cfg.seed, cfg.offset = seed, offset
    cfg.seed_state = seed_state or None
    return cfg


def weight_prep(
    w: Tensor, in_sizes: List[int], quant_type: int, noise_type: int, res: float, std_dev: float,
    seed: int, offset: int, want_eff: bool, skip_tile_stats: bool = False, seed_state: int = 0,
) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """wmax ``[T, N]``, tile max/min ``[T]`` and, if wanted, the modified copy ``[N, K]``.
    ``skip_tile_stats``: the caller does not use tile max/min (they may come back unwritten)."""
    lib = _lib()
    if w.dim() != 2 or w.stride(1) != 1:
        raise HipBackendError("weight must be a row-major 2-D tensor")
    n_out, n_in = w.shape
    n_tiles = len(in_sizes)
    dev = w.device
    wmax = torch.empty((n_tiles, n_out), dtype=w.dtype, device=dev)
    tile_max = torch.empty((n_tiles,), dtype=torch.float32, device=dev)
    tile_min = torch.empty((n_tiles,), dtype=torch.float32, device=dev)
    w_eff = torch.empty((n_out, n_in) if want_eff else (0,), dtype=w.dtype, device=dev)
    cfg = _modifier_cfg(w.dtype, quant_type, noise_type, res, std_dev, seed, offset, seed_state)
    cfg.skip_tile_stats = int(skip_tile_stats)
    L.check(
        lib.ahl_weight_prep(
            _ptr(w), n_out, n_in, _ld(w), L.tile_ends_array(in_sizes), n_tiles, byref(cfg), _ptr(wmax),
            _ptr(tile_max), _ptr(tile_min), _ptr(w_eff) if want_eff else None, n_in, _stream(),
        ),
        "ahl_weight_prep",
    )
    return wmax, tile_max, tile_min, w_eff


def weight_prep_clip(
    w: Tensor, clip: Tensor, in_sizes: List[int], quant_type: int, noise_type: int, res: float,
    std_dev: float, seed: int, offset: int, seed_state: int = 0,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Weights under a learnable per-channel clip ``clip [T, N]`` (which also takes the place of
    the per-tile abs-max): tile max/min of the clip and the clipped (+ quantised, + noisy) copy."""
    lib = _lib()
    if w.dim() != 2 or w.stride(1) != 1:
        raise HipBackendError("weight must be a row-major 2-D tensor")
    n_out, n_in = w.shape
    n_tiles = len(in_sizes)
    if clip.shape != (n_tiles, n_out) or not clip.is_contiguous() or clip.dtype != w.dtype:
        raise HipBackendError("learnable_weight_clip must be a contiguous [n_tiles, out] tensor")
    tile_max = torch.empty((n_tiles,), dtype=torch.float32, device=w.device)
    tile_min = torch.empty((n_tiles,), dtype=torch.float32, device=w.device)
    w_eff = torch.empty((n_out, n_in), dtype=w.dtype, device=w.device)
    cfg = _modifier_cfg(w.dtype, quant_type, noise_type, res, std_dev, seed, offset, seed_state)
    cfg.wmax_given = 1
    L.check(
        lib.ahl_weight_prep(
            _ptr(w), n_out, n_in, _ld(w), L.tile_ends_array(in_sizes), n_tiles, byref(cfg), _ptr(clip),
            _ptr(tile_max), _ptr(tile_min), _ptr(w_eff), n_in, _stream(),
        ),
        "ahl_weight_prep",
    )
    return tile_max, tile_min, w_eff


def learned_clip_bwd(dw: Tensor, w: Tensor, clip: Tensor, tile_min: Tensor, in_sizes: List[int],
                     quant_type: int, res: float) -> Tensor:
    """LSQ backward of the learnable clip: ``dw`` (gradient w.r.t. the clipped weights) becomes
    the gradient w.r.t. the weights in place; returns the gradient of the clip ``[T, N]``."""
    lib = _lib()
    if dw.stride(1) != 1 or w.stride(1) != 1:
        raise HipBackendError("weight and its gradient must be row-major")
    n_out, n_in = w.shape
    dclip = torch.empty_like(clip)
    cfg = _modifier_cfg(w.dtype, quant_type, L.AHL_NOISE_NONE, res, 0.0, 0, 0)
    L.check(
        lib.ahl_learned_clip_bwd(
            _ptr(dw), _ld(dw), _ptr(w), _ld(w), _ptr(clip), _ptr(tile_min), _ptr(dclip), n_out, n_in,
            L.tile_ends_array(in_sizes), len(in_sizes), byref(cfg), _stream(),
        ),
        "ahl_learned_clip_bwd",
    )
    return dclip


def quantize_weights(w: Tensor, in_sizes: List[int], quant_type: int, res: float) -> None:
    """In-place per-tile weight quantisation with scales from each slice's own abs-max."""
    lib = _lib()
    if w.dim() != 2 or w.stride(1) != 1:
        raise HipBackendError("weight must be a row-major 2-D tensor")
    n_tiles = len(in_sizes)
    ws_wmax = torch.empty((n_tiles, w.size(0)), dtype=w.dtype, device=w.device)
    ws_tile = torch.empty((2 * n_tiles,), dtype=torch.float32, device=w.device)
    cfg = _modifier_cfg(w.dtype, quant_type, L.AHL_NOISE_NONE, res, 0.0, 0, 0)
    L.check(
        lib.ahl_quantize_weights(
            _ptr(w), w.size(0), w.size(1), _ld(w), L.tile_ends_array(in_sizes), n_tiles, byref(cfg),
            _ptr(ws_wmax), _ptr(ws_tile), _stream(),
        ),
        "ahl_quantize_weights",
    )


def dac(x: Tensor, ir: Optional[Tensor], in_sizes: List[int], icfg: List[int],
        fcfg: List[float]) -> Tuple[Tensor, Tensor]:
    """Clamp + DAC pre-pass: returns ``xq [M, K]`` and, in dynamic mode, the ranges ``[T, M]``."""
    lib = _lib()
    x = _rows2d(x, "x")
    m_rows, k_in = x.shape
    n_tiles = len(in_sizes)
    cfg = _linear_cfg(x.dtype, icfg, fcfg)
    # padded tile layout: n_tiles * stride columns per row
    q_cols = n_tiles * cfg.tile_stride if cfg.tile_stride > 0 else k_in
    xq = torch.empty((m_rows, q_cols), dtype=x.dtype, device=x.device)
    dynamic = cfg.ir_mode == L.AHL_IR_DYNAMIC
    ir_dyn = torch.empty((n_tiles, m_rows) if dynamic else (0,), dtype=x.dtype, device=x.device)
    L.check(
        lib.ahl_dac(
            _ptr(x), _ld(x), _ptr(xq), q_cols, _ptr(ir), _ptr(ir_dyn) if dynamic else None, m_rows,
            k_in, L.tile_ends_array(in_sizes), n_tiles, byref(cfg), _stream(),
        ),
        "ahl_dac",
    )
    return xq, ir_dyn


@lru_cache(maxsize=4096)
def _fwd_ws_bytes(m_rows: int, k_in: int, n_out: int, n_tiles: int, dtype: int) -> int:
    """The library's answer per shape (host arithmetic there; asked once per shape here)."""
    return int(_lib().ahl_linear_fwd_ws_bytes(m_rows, k_in, n_out, n_tiles, dtype))


# Hand the forward a workspace for calls of few rows (one K-tile per block, summed in tile order
# afterwards). The result is the same bit for bit either way; the switch exists for comparisons.
SPLIT_FEW_ROW_FORWARD = True


def linear_fwd(
    x: Optional[Tensor], xq: Optional[Tensor], w_eff: Tensor, bias: Optional[Tensor],
    ir: Optional[Tensor], wmax: Optional[Tensor], tile_max: Optional[Tensor], in_sizes: List[int],
    icfg: List[int], fcfg: List[float], want_keep: bool,
) -> Tuple[Tensor, Tensor, Tensor]:
    """The analog forward; returns ``y [M, N]``, the clamp mask (empty if not wanted) and the
    one-word "anything clamped" flag."""
    lib = _lib()
    ref = x if x is not None else xq
    if x is not None:
        x = _rows2d(x, "x")
    if xq is not None:
        xq = _rows2d(xq, "xq")
    m_rows, k_in = ref.size(0), sum(in_sizes)
    n_out = w_eff.size(0)
    n_tiles = len(in_sizes)
    cfg = _linear_cfg(ref.dtype, icfg, fcfg)
    y = torch.empty((m_rows, n_out), dtype=ref.dtype, device=ref.device)
    # clamp mask: one bit per (tile, row, column), 32 columns of one row per word
    # rows padded to a multiple of 64 (the kernels never write or use the padding rows)
    keep = torch.empty((n_tiles, (n_out + 31) // 32, (m_rows + 63) // 64 * 64) if want_keep else (0,),
                       dtype=torch.int32, device=ref.device)
    if want_keep and m_rows % 64 != 0:
        keep[:, :, m_rows:].zero_()   # the padding rows: defined contents for whoever compares masks
    flag = torch.empty((1,) if want_keep else (0,), dtype=torch.int32, device=ref.device)
    ws_bytes = 0
    if xq is not None and SPLIT_FEW_ROW_FORWARD and not _SHAPES_ONLY.depth:
        ws_bytes = _fwd_ws_bytes(m_rows, k_in, n_out, n_tiles, cfg.dtype)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=ref.device) if ws_bytes else None
    L.check(
        lib.ahl_linear_fwd(
            _ptr(x), _ld(x) if x is not None else 0, _ptr(xq), _ld(xq) if xq is not None else 0,
            _ptr(w_eff), _ld(w_eff), _ptr(bias), _ptr(y), n_out, _ptr(keep) if want_keep else None,
            _ptr(flag) if want_keep else None, _ptr(ir), _ptr(wmax), _ptr(tile_max), m_rows, k_in,
            n_out, L.tile_ends_array(in_sizes), n_tiles, byref(cfg), _ptr(ws), _stream(),
        ),
        "ahl_linear_fwd",
    )
    return y, keep, flag


def linear_bwd_dx(
    g: Tensor, keep: Optional[Tensor], clamp_flag: Optional[Tensor], w_eff: Tensor,
    x: Optional[Tensor], ir: Optional[Tensor], in_sizes: List[int], icfg: List[int],
    fcfg: List[float],
) -> Tuple[Tensor, Tensor]:
    """Input gradient ``[M, K]`` and input-range gradient ``[T]`` (empty unless static range)."""
    lib = _lib()
    g = _rows2d(g, "g")
    m_rows, n_out = g.shape
    k_in = sum(in_sizes)
    n_tiles = len(in_sizes)
    cfg = _linear_cfg(g.dtype, icfg, fcfg)
    if cfg.tile_stride > 0:
        g = _vector_aligned(g)
    static = cfg.ir_mode == L.AHL_IR_STATIC
    dx = torch.empty((m_rows, k_in), dtype=g.dtype, device=g.device)
    ir_grad = torch.empty((n_tiles,) if static else (0,), dtype=g.dtype, device=g.device)
    ws = torch.empty((lib.ahl_linear_bwd_dx_ws_bytes(m_rows, k_in, n_out, n_tiles, cfg.dtype,
                                                     cfg.tile_stride),),
                     dtype=torch.uint8, device=g.device)
    if x is not None:
        x = _rows2d(x, "x")
        if cfg.tile_stride > 0 and (not _aligned16(x) or _ld(x) != k_in):
            x = x.clone(memory_format=torch.contiguous_format)  # same row stride and alignment as dx
    L.check(
        lib.ahl_linear_bwd_dx(
            _ptr(g), _ld(g), _ptr(keep), _ptr(clamp_flag), _ptr(w_eff), _ld(w_eff), _ptr(x),
            _ld(x) if x is not None else 0, _ptr(ir), _ptr(dx), k_in,
            _ptr(ir_grad) if static else None, m_rows, k_in, n_out, L.tile_ends_array(in_sizes),
            n_tiles, byref(cfg), _ptr(ws), _stream(),
        ),
        "ahl_linear_bwd_dx",
    )
    return dx, ir_grad


def linear_bwd_dw(
    g: Tensor, keep: Optional[Tensor], clamp_flag: Optional[Tensor], x: Optional[Tensor],
    xq: Optional[Tensor], ir: Optional[Tensor], in_sizes: List[int], icfg: List[int],
    fcfg: List[float], want_bias: bool,
) -> Tuple[Tensor, Tensor]:
    """Weight gradient ``[N, K]`` from the raw input ``x`` or the saved quantised input ``xq``,
    and (if wanted, else empty) the bias gradient ``[N]``, the column sums of ``g``."""
    lib = _lib()
    g = _rows2d(g, "g")
    ref = xq if xq is not None else x
    if x is not None:
        x = _rows2d(x, "x")
    if xq is not None:
        xq = _rows2d(xq, "xq")
    m_rows, n_out = g.shape
    k_in = sum(in_sizes)
    n_tiles = len(in_sizes)
    cfg = _linear_cfg(g.dtype, icfg, fcfg)
    if cfg.tile_stride > 0:
        g = _vector_aligned(g)
    dw = torch.empty((n_out, k_in), dtype=g.dtype, device=g.device)
    dbias = torch.empty((n_out,) if want_bias else (0,), dtype=g.dtype, device=g.device)
    ws_bytes = lib.ahl_linear_bwd_dw_ws_bytes(m_rows, k_in, n_out, n_tiles, cfg.dtype,
                                              0 if keep is None else 1, cfg.tile_stride)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=g.device)
    L.check(
        lib.ahl_linear_bwd_dw(
            _ptr(g), _ld(g), _ptr(keep), _ptr(clamp_flag), _ptr(x), _ld(x) if x is not None else 0,
            _ptr(xq), _ld(xq) if xq is not None else 0, _ptr(ir), _ptr(dw), k_in,
            _ptr(dbias) if want_bias else None, m_rows, k_in, n_out, L.tile_ends_array(in_sizes),
            n_tiles, byref(cfg), _ptr(ws), _stream(),
        ),
        "ahl_linear_bwd_dw",
    )
    return dw, dbias


# ---------------------------------------------------------------------------------------------
# Gate arithmetic of the recurrent cells (called from the cells' autograd functions directly; no
# dispatcher entry: they are internal to those functions)
def gates_supported(igates: Tensor, hgates: Optional[Tensor], state: Tensor, n_gates: int) -> bool:
    """Whether the fused gate kernels can take these operands: everything on one GPU in one of
    float32 / bfloat16, ``state [rows, hidden]`` with the hidden size in whole 16-byte vectors,
    the projections ``[rows, n_gates * hidden]``. (The kernels read raw pointers: a projection
    in another dtype or shape than the state would be read out of bounds; such calls take the
    torch formula, which type-promotes.)"""
    if not state.is_cuda or state.dtype not in _DTYPES or state.dim() != 2 or state.size(0) == 0:
        return False
    rows, hidden = state.shape
    if hidden % (16 // state.element_size()) != 0:
        return False
    for gates in (igates, hgates):
        if gates is None:
            continue
        if (gates.device != state.device or gates.dtype != state.dtype
                or tuple(gates.shape) != (rows, n_gates * hidden)):
            return False
    return True


def dense(tensor: Optional[Tensor]) -> Optional[Tensor]:
    """``tensor`` as a dense, 16-byte aligned matrix (itself if it already is one)."""
    if tensor is None:
        return None
    if not tensor.is_contiguous() or not _aligned16(tensor):
        tensor = tensor.clone(memory_format=torch.contiguous_format)
    return tensor


def lstm_gates_fwd(igates: Tensor, hgates: Optional[Tensor], c_x: Tensor,
                   want_act: bool) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
    """``(h_y, c_y, activated gates or None)`` of an LSTM step."""
    lib = _lib()
    igates, hgates, c_x = dense(igates), dense(hgates), dense(c_x)
    rows, hidden = c_x.shape
    h_y, c_y = torch.empty_like(c_x), torch.empty_like(c_x)
    act = torch.empty_like(igates) if want_act else None
    L.check(lib.ahl_lstm_gates_fwd(_ptr(igates), _ptr(hgates), _ptr(c_x), dtype_id(c_x.dtype), rows,
                                   hidden, _ptr(h_y), _ptr(c_y), _ptr(act), _stream()),
            "ahl_lstm_gates_fwd")
    return h_y, c_y, act


def lstm_gates_bwd(dh_y: Tensor, dc_y: Optional[Tensor], act: Tensor, c_x: Tensor,
                   c_y: Tensor) -> Tuple[Tensor, Tensor]:
    """``(dgates [rows, 4H], dc_x)``."""
    lib = _lib()
    dh_y, dc_y = dense(dh_y), dense(dc_y)
    rows, hidden = c_x.shape
    dgates, dc_x = torch.empty_like(act), torch.empty_like(c_x)
    L.check(lib.ahl_lstm_gates_bwd(_ptr(dh_y), _ptr(dc_y), _ptr(act), _ptr(c_x), _ptr(c_y),
                                   dtype_id(c_x.dtype), rows, hidden, _ptr(dgates), _ptr(dc_x),
                                   _stream()),
            "ahl_lstm_gates_bwd")
    return dgates, dc_x


def gru_gates_fwd(igates: Tensor, hgates: Tensor, h_x: Tensor,
                  want_act: bool) -> Tuple[Tensor, Optional[Tensor]]:
    """``(h_y, (reset, update, new) or None)`` of a GRU step."""
    lib = _lib()
    igates, hgates, h_x = dense(igates), dense(hgates), dense(h_x)
    rows, hidden = h_x.shape
    h_y = torch.empty_like(h_x)
    act = torch.empty_like(igates) if want_act else None
    L.check(lib.ahl_gru_gates_fwd(_ptr(igates), _ptr(hgates), _ptr(h_x), dtype_id(h_x.dtype), rows,
                                  hidden, _ptr(h_y), _ptr(act), _stream()),
            "ahl_gru_gates_fwd")
    return h_y, act


def gru_gates_bwd(dh_y: Tensor, act: Tensor, hgates: Tensor,
                  h_x: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """``(digates, dhgates [rows, 3H], dh_x)``."""
    lib = _lib()
    dh_y = dense(dh_y)
    rows, hidden = h_x.shape
    digates, dhgates, dh_x = torch.empty_like(act), torch.empty_like(act), torch.empty_like(h_x)
    L.check(lib.ahl_gru_gates_bwd(_ptr(dh_y), _ptr(act), _ptr(hgates), _ptr(h_x),
                                  dtype_id(h_x.dtype), rows, hidden, _ptr(digates), _ptr(dhgates),
                                  _ptr(dh_x), _stream()),
            "ahl_gru_gates_bwd")
    return digates, dhgates, dh_x


for _name, _fn in [
    ("sliced_absmax", sliced_absmax), ("sliced_std", sliced_std),
    ("row_nonzero", row_nonzero), ("sliced_std_kept", sliced_std_kept), ("sliced_quantile", sliced_quantile),
    ("ir_moving_update", ir_moving_update), ("ir_init_update", ir_init_update),
    ("running_absmax", running_absmax), ("ir_fast_update", ir_fast_update),
    ("clip_weights", clip_weights), ("col_sum", col_sum),
    ("weight_prep", weight_prep), ("quantize_weights", quantize_weights),
    ("weight_prep_clip", weight_prep_clip), ("learned_clip_bwd", learned_clip_bwd),
    ("pad_tiles", pad_tiles), ("unpad_tiles", unpad_tiles),
    ("im2col", im2col), ("col2im", col2im), ("transpose_batched", transpose_batched),
    ("dac", dac), ("linear_fwd", linear_fwd), ("linear_bwd_dx", linear_bwd_dx), ("linear_bwd_dw", linear_bwd_dw),
]:
    LIB.impl(_name, _fn, "CUDA")
    torch.library.register_fake(f"aihwkit_hip::{_name}", _shapes_only(_fn), lib=LIB)

OPS = torch.ops.aihwkit_hip

# what the autograd functions that call the library themselves (hip_conv.py) share with the ops here
ptr, linear_cfg, current_stream = _ptr, _linear_cfg, _stream


def os_environ_no_rounding() -> bool:
    """The reference's test switch ``_AIHWKIT_NO_ROUNDING``."""
    return bool(os.environ.get("_AIHWKIT_NO_ROUNDING", False))


def direct(tensor: Tensor):
    """Where code that is never traced (an autograd node's own body, a calibration hook) takes its
    operator calls from: this module's functions themselves for a tensor on the current device --
    the dispatcher adds nothing there but time, about 10 us per call -- and the registered ops,
    whose dispatch switches the device, for a tensor elsewhere."""
    if tensor.device.index == torch.cuda.current_device():
        return sys.modules[__name__]
    return OPS
