"""Builds libcgptx.so (HIP kernels + C-ABI, gfx950) in-tree with hipcc.

`python -m cgpt_amd.build` compiles every translation unit under
cgpt_amd/csrc into cgpt_amd/lib/libcgptx.so. hipcc cross-compiles for gfx950
without a GPU, so this runs in a CPU-only container.
"""
from __future__ import annotations

import concurrent.futures
import os
import pathlib
import shutil
import subprocess
import sys

ROOT = pathlib.Path(__file__).resolve().parent.parent
CSRC = ROOT / "cgpt_amd" / "csrc"
LIB_DIR = ROOT / "cgpt_amd" / "lib"
OBJ_DIR = ROOT / "build" / "obj"
LIB_PATH = LIB_DIR / "libcgptx.so"

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

DEVICE_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # Keep the compiler from forming packed-fp32 VALU ops.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


# Per-file additions. attention.hip: MFMA results in vector registers (the softmax arithmetic reads them in
# place). The option belongs to the compiler's backend, not to its documented interface: it is probed once and
# left out, with a warning, when this hipcc does not know it (the kernels are correct either way, the
# accumulators are then copied between the two register files).
FILE_FLAGS = {"attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}
_probed_flags: dict[tuple[str, ...], bool] = {}


def _compiler_accepts(flags: list[str]) -> bool:
    key = tuple(flags)
    if key not in _probed_flags:
        proc = subprocess.run([HIPCC, "--offload-arch=gfx950", "-x", "hip", "-c", "/dev/null", "-o", "/dev/null", *flags],
                              capture_output=True, text=True)
        _probed_flags[key] = proc.returncode == 0
        if proc.returncode != 0:
            print(f"cgpt_amd.build: {HIPCC} rejects {' '.join(flags)}; building without it", file=sys.stderr)
    return _probed_flags[key]


def file_flags(name: str) -> list[str]:
    flags = FILE_FLAGS.get(name, [])
    return flags if not flags or _compiler_accepts(flags) else []


def sources() -> list[pathlib.Path]:
    return sorted(CSRC.glob("*.hip")) + sorted(CSRC.glob("*.cpp"))


def _compile(src: pathlib.Path, force: bool) -> pathlib.Path:
    obj = OBJ_DIR / (src.name + ".o")
    deps = [src] + list(CSRC.glob("*.hpp")) + list((ROOT / "include").glob("*.h"))
    if not force and obj.exists() and all(obj.stat().st_mtime >= d.stat().st_mtime for d in deps):
        return obj
    cmd = [HIPCC, *DEVICE_FLAGS, *file_flags(src.name), "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build(force: bool = True, jobs: int | None = None) -> pathlib.Path:
    """Compiles all sources (always, when force) and links the shared library."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(LIB_PATH),
           *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


INTERFACE_TEST_SOURCES = [ROOT / "tests" / "cpp" / name
                          for name in ("ops_interface_test.cpp", "block_backward_test.cpp", "data_upload_test.cpp")]
INTERFACE_TEST_BINARY = ROOT / "tests" / "cpp" / "ops_interface_test.bin"


def build_interface_test() -> pathlib.Path:
    """Compiles the C++ programs that drive include/core, include/ops/**, include/optim/** against the library
    (tests/cpp/*.cpp -> *.bin). Host code only (the headers are inline wrappers over the C-ABI); linked with an
    rpath relative to the binary so that they run from any checkout location."""
    for source in INTERFACE_TEST_SOURCES:
        cmd = [HIPCC, "-std=c++20", "-O1", f"-I{ROOT / 'include'}", str(source), "-o", str(source.with_suffix(".bin")),
               f"-L{LIB_DIR}", "-lcgptx", "-Wl,-rpath,$ORIGIN/../../cgpt_amd/lib"]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"interface test build failed ({source.name}):\n{proc.stderr}")
    return INTERFACE_TEST_BINARY


if __name__ == "__main__":
    path = build(force="--incremental" not in sys.argv)
    print(path)
    print(build_interface_test())
