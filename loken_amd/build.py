"""Builds ``libloken_gfx950.so`` in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libloken_gfx950.so"
# measurement kernels: a library of their own that only the benchmark loads
PROBES_SRC = HERE / "probes_csrc" / "probes.hip"
PROBES_LIB = HERE / "libloken_probes.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fno-fast-math",
    # packed-FP32 instructions stay off: the compiler forms them from plain float code otherwise
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]
# MFMA results are consumed by VALU fix-ups right away: keep them in VGPRs instead of the
# accumulator file, which would cost one v_accvgpr_read per value.
_VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
PER_FILE_FLAGS = {"mmq.hip": _VGPR_FORM, "mmq_q4k_f16.hip": _VGPR_FORM, "mmq_q4k_wide.hip": _VGPR_FORM}


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _fresh(src: Path, obj: Path) -> bool:
    """True when `obj` is newer than `src` and every header it may include."""
    if not obj.exists():
        return False
    deps = [src, *CSRC.glob("*.h"), *(HERE.parent / "include").glob("*.h*"), Path(__file__)]
    return obj.stat().st_mtime > max(d.stat().st_mtime for d in deps)


def _compile(src: Path, incremental: bool = False) -> Path:
    obj = CSRC / (src.stem + ".o")
    if incremental and _fresh(src, obj):
        return obj
    cmd = [HIPCC, *FLAGS, *PER_FILE_FLAGS.get(src.name, []), "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{r.stderr[-6000:]}")
    return obj


def build(jobs: int = 8, verbose: bool = False, incremental: bool = False) -> Path:
    """Compiles every source (always, unless `incremental`: then only those older than their object)."""
    srcs = sources()
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(srcs)))) as pool:
        objs = list(pool.map(lambda s: _compile(s, incremental), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-6000:]}")
    probes_obj = PROBES_SRC.with_suffix(".o")
    if not (incremental and _fresh(PROBES_SRC, probes_obj)):
        r = subprocess.run([HIPCC, *FLAGS, "-c", str(PROBES_SRC), "-o", str(probes_obj)], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {PROBES_SRC.name}:\n{r.stderr[-6000:]}")
    # lk_launch_status and the knob reader live in the product's objects: the probes link the one they use
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(PROBES_LIB), str(probes_obj),
                        str(CSRC / "device.o")], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-6000:]}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources and {PROBES_LIB.name}")
    return LIB


if __name__ == "__main__":
    build(verbose=True, incremental="--incremental" in sys.argv)
    sys.exit(0)
