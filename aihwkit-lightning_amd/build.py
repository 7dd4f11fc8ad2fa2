"""Build ``libanalog_hip.so`` for gfx950 with hipcc, in-tree.

    python aihwkit-lightning_amd/build.py [--force]

Sources: ``csrc/*.hip`` -> objects in ``csrc/build/`` -> ``aihwkit_lightning/_lib/libanalog_hip.so``.
hipcc cross-compiles without a GPU. The flags matter for numerics: no fp contraction (every
rounding step of the bf16-faithful arithmetic is explicit) and no compiler-generated packed-fp32
instructions.
"""
import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(HERE, "aihwkit_lightning", "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libanalog_hip.so")
SOURCES = ["ahl_reduce.hip", "ahl_weights.hip", "ahl_gemm.hip", "ahl_fast.hip", "ahl_fwd_pipe.hip", "ahl_fast_bwd.hip",
           "ahl_conv.hip", "ahl_conv_direct.hip", "ahl_layout.hip", "ahl_calib.hip", "ahl_rnn.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unused-value",
] + os.environ.get("AHL_EXTRA_FLAGS", "").split()


def _newest_dep() -> float:
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h"))]
    deps.append(os.path.join(HERE, "..", "include", "analog_hip.h"))
    return max(os.path.getmtime(p) for p in deps)


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stderr}")
    return obj


def build(force: bool = True, verbose: bool = True) -> str:
    """Compile and link; returns the library path. ``force=False`` skips an up-to-date library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    if not force and os.path.exists(LIB_PATH) and os.path.getmtime(LIB_PATH) >= _newest_dep():
        return LIB_PATH
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("--if-stale", action="store_true", help="skip when the library is newer")
    ns = parser.parse_args()
    try:
        build(force=not ns.if_stale)
    except RuntimeError as exc:
        print(exc, file=sys.stderr)
        sys.exit(1)
