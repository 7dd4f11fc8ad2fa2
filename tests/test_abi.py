"""The C-ABI library loads and exports exactly what include/analog_hip.h declares (no GPU)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "analog_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ahl_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    names = declared_symbols()
    for must in ("ahl_linear_fwd", "ahl_linear_bwd_dx", "ahl_linear_bwd_dw", "ahl_sliced_absmax",
                 "ahl_sliced_std", "ahl_clip_weights", "ahl_weight_prep", "ahl_quantize_weights",
                 "ahl_running_absmax", "ahl_ir_init_update"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    if not os.path.exists(L.lib_path()):
        pytest.fail(f"{L.lib_path()} is missing: run python aihwkit-lightning_amd/build.py")
    lib = L.load()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(L.SIGNATURES) == declared_symbols(), "ctypes table and header disagree"
    assert lib.ahl_abi_version() == L.ABI_VERSION


def test_header_compiles_as_c():
    src = '#include "analog_hip.h"\nint main(void){AhlLinearCfg c; c.dtype = AHL_BF16; return c.dtype - 1;}\n'
    proc = subprocess.run(
        ["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", os.path.dirname(HEADER), "-x",
         "c", "-"], input=src, text=True, capture_output=True)
    assert proc.returncode == 0, proc.stderr


def test_struct_layout_matches_ctypes():
    import ctypes
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    src = ('#include <stdio.h>\n#include <stddef.h>\n#include "analog_hip.h"\n'
           'int main(void){printf("%zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(AhlLinearCfg), '
           'offsetof(AhlLinearCfg, seed), offsetof(AhlLinearCfg, ir_decay), sizeof(AhlModifierCfg), '
           'offsetof(AhlModifierCfg, seed), sizeof(AhlConvGeom), offsetof(AhlConvGeom, kernel), '
           'offsetof(AhlConvGeom, dilation)); return 0;}\n')
    exe = "/tmp/ahl_layout_probe"
    proc = subprocess.run(["gcc", "-I", os.path.dirname(HEADER), "-x", "c", "-", "-o", exe],
                          input=src, text=True, capture_output=True)
    assert proc.returncode == 0, proc.stderr
    got = [int(v) for v in subprocess.run([exe], capture_output=True, text=True).stdout.split()]
    want = [ctypes.sizeof(L.AhlLinearCfg), L.AhlLinearCfg.seed.offset, L.AhlLinearCfg.ir_decay.offset,
            ctypes.sizeof(L.AhlModifierCfg), L.AhlModifierCfg.seed.offset,
            ctypes.sizeof(L.AhlConvGeom), L.AhlConvGeom.kernel.offset, L.AhlConvGeom.dilation.offset]
    assert got == want


def test_host_side_errors_without_gpu():
    import torch
    from aihwkit_lightning.exceptions import ConfigError, HipBackendError
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig, WeightClipType

    with pytest.raises(ValueError):
        AnalogLinear(4, 4)
    cfg = TorchInferenceRPUConfig()
    layer = AnalogLinear(8, 4, rpu_config=cfg)
    with pytest.raises(HipBackendError):
        layer(torch.randn(2, 8))
    cfg2 = TorchInferenceRPUConfig()
    cfg2.clip.type = WeightClipType.LAYER_GAUSSIAN
    cfg2.clip.sigma = 2.0
    layer2 = AnalogLinear(8, 4, rpu_config=cfg2)
    with pytest.raises(HipBackendError):
        layer2.clip_weights()
    assert issubclass(HipBackendError, Exception) and issubclass(ConfigError, Exception)
