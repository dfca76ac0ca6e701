"""Build libjigsaw_hip.so (gfx950) from the HIP sources under ``csrc/``.

Usage: ``python -m jigsaw_amd.build [--jobs N] [--force]``. hipcc cross-compiles
for gfx950 without a GPU present. Objects go to ``csrc/build/``, the library to
``lib/libjigsaw_hip.so`` (both git-ignored; the library travels with the tree).
"""

from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
OBJ = CSRC / "build"
LIB = ROOT / "lib" / "libjigsaw_hip.so"
ARCH = "gfx950"

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # Packed-fp32 VALU forms are kept out of the generated code on purpose.
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


# Kernels whose vector instructions read or scale their matrix accumulators (softmax on the scores, the
# running rescale, epilogues) keep the accumulators in ordinary vector registers: left to its default the
# compiler puts them in the accumulation registers and moves them over and back with v_accvgpr_read /
# v_accvgpr_write around every such use (64 moves per loop iteration in the wide attention forward).
PER_FILE_FLAGS = {
    name: ["-mllvm", "-amdgpu-mfma-vgpr-form"]
    for name in ("attn_wide.hip", "attn_swin.hip", "attn_window.hip", "attn_f32_mfma.hip", "proj_mfma.hip")
}


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm under /opt/rocm")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _newer(a: Path, deps: list[Path]) -> bool:
    if not a.exists():
        return False
    t = a.stat().st_mtime
    return all(d.stat().st_mtime <= t for d in deps)


def _compile(src: Path, force: bool, extra: list[str]) -> Path:
    obj = OBJ / (src.stem + ".o")
    deps = [src, *CSRC.glob("*.h"), ROOT.parent / "include" / "jigsaw_hip.h"]
    if not force and _newer(obj, deps):
        return obj
    cmd = [hipcc(), *HIPCC_FLAGS, *PER_FILE_FLAGS.get(src.name, []), *extra, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; harmless.
    err = "\n".join(
        ln for ln in proc.stderr.splitlines() if "packed-fp32-ops" not in ln
    )
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(jobs: int = 8, force: bool = False, extra: list[str] | None = None) -> Path:
    """Compile every ``csrc/*.hip`` and link ``lib/libjigsaw_hip.so``."""
    extra = list(extra or [])
    OBJ.mkdir(parents=True, exist_ok=True)
    LIB.parent.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    with cf.ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs = list(pool.map(lambda s: _compile(s, force, extra), srcs))
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB)]
    cmd += [str(o) for o in objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--save-temps", action="store_true", help="keep ISA under csrc/build/")
    ns = ap.parse_args()
    extra = ["-save-temps=obj"] if ns.save_temps else []
    print(build(ns.jobs, ns.force, extra))


if __name__ == "__main__":
    main()
