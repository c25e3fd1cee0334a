"""The C++ operator interface (include/core, include/ops, include/optim) over the C-ABI.

CPU part: every header of the interface is self-contained C++20 and the set declares the functions
the reference's callers use, in the reference's argument order. GPU part: the compiled test program
replays the reference tests' known answers through that interface (tests/cpp/ops_interface_test.cpp).
"""
import pathlib
import re
import shutil
import subprocess

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
INCLUDE = ROOT / "include"
HEADERS = sorted(p.relative_to(INCLUDE).as_posix() for p in INCLUDE.rglob("*.h") if p.parent != INCLUDE)

# name -> leading parameter names, as declared by the reference (include/ops/**, include/optim/adamw.h)
REFERENCE_SIGNATURES = {
    "rmsnorm_backward": ["grad_input", "grad_weight", "grad_output", "input", "weight", "epsilon", "stream"],
    "rope_backward": ["grad_query", "grad_key", "grad_rotated_query", "grad_rotated_key", "cos_cache", "sin_cache",
                      "stream", "rope_options"],
    "linear_backward": ["grad_input", "grad_weight", "grad_bias", "grad_output", "input", "weight"],
    "embedding_backward": ["grad_weight", "grad_output", "device_token_ids", "token_count", "stream", "options"],
    "cross_entropy_forward_backward": ["loss", "gradient", "logits", "device_targets", "target_count", "stream",
                                       "gradient_scale"],
    "cut_cross_entropy_forward_backward": ["loss", "input_gradient", "classifier_gradient", "input", "classifier",
                                           "device_targets", "target_count", "stream"],
    "flash_gqa_attention_backward_with_lse": ["grad_query", "grad_key", "grad_value", "grad_output", "output",
                                              "logsumexp", "query", "key", "value", "stream", "options",
                                              "accumulate_grads"],
    "flash_gqa_attention_backward": ["grad_query", "grad_key", "grad_value", "grad_output", "query", "key", "value",
                                     "stream", "options", "accumulate_grads"],
    "adamw_step": ["parameter", "gradient", "state", "options", "stream"],
    "adamw_step_many_async": ["entries", "options", "workspace", "stream"],
}


@pytest.mark.parametrize("header", HEADERS)
def test_header_is_self_contained(header, tmp_path):
    compiler = shutil.which("g++")
    if compiler is None or not pathlib.Path("/opt/rocm/include/hip/hip_runtime_api.h").exists():
        pytest.skip("needs g++ and the HIP runtime headers")
    source = tmp_path / "unit.cpp"
    source.write_text(f'#include "{header}"\nint main() {{ return 0; }}\n')
    proc = subprocess.run([compiler, "-std=c++20", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", f"-I{INCLUDE}",
                           "-I/opt/rocm/include", str(source)], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]


def test_signatures_follow_the_reference_order():
    text = "\n".join((INCLUDE / h).read_text() for h in HEADERS)
    for name, want in REFERENCE_SIGNATURES.items():
        match = re.search(r"inline\s+(?:void|bool)\s+" + name + r"\s*\(([^)]*)\)", text)
        assert match, f"{name} is not declared"
        params = [re.sub(r"\s*=.*", "", p).strip().split()[-1].lstrip("&*") for p in match.group(1).split(",")]
        params = [p for p in params if p not in ("GemmContext&",)]
        named = [p for p in params if re.fullmatch(r"[a-z_]+", p)]
        assert named[: len(want)] == want[: len(named)] or named == want, (name, named, want)


@pytest.mark.gpu
def test_interface_program_replays_reference_known_answers():
    binary = ROOT / "tests" / "cpp" / "ops_interface_test.bin"
    assert binary.exists(), "build it with `python -m cgpt_amd.build` (there is no fallback)"
    proc = subprocess.run([str(binary)], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 failure(s)" in proc.stdout


@pytest.mark.gpu
def test_token_batches_upload_through_the_data_header():
    """tests/cpp/data_upload_test.cpp: data::Batch / data::DeviceBatch / data::upload_batch
    (include/data/dataset_loader.h) over the library's upload entry points: alternating page-locked batches arrive
    bit for bit, device buffers keep their address, shape mismatches throw, copies are deep, moves carry the
    pending upload."""
    binary = ROOT / "tests" / "cpp" / "data_upload_test.bin"
    assert binary.exists(), "build it with `python -m cgpt_amd.build` (there is no fallback)"
    proc = subprocess.run([str(binary)], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 failure(s)" in proc.stdout


@pytest.mark.gpu
def test_callers_of_the_headers_reproduce_the_library_step():
    """tests/cpp/block_backward_test.cpp: the wrappers accept the reference's argument lists (compile-time), and
    the library's own table of operator calls (the step as the reference's call sequence, CGPTX_FUSE=0), made
    through include/ops/** eagerly and from a HipGraph capture, gives the library step's gradients bit for bit."""
    binary = ROOT / "tests" / "cpp" / "block_backward_test.bin"
    assert binary.exists(), "build it with `python -m cgpt_amd.build` (there is no fallback)"
    proc = subprocess.run([str(binary)], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 failure(s)" in proc.stdout
