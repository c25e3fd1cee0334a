"""cgptx_rmsnorm_backward_static — the entry point that allocates nothing (its working memory is a block inside
the library's device image) — against cgptx_rmsnorm_backward, through the C-ABI, bit for bit: the two share
their kernels and launch shapes, so any difference is a fault in how the built-in block is addressed. Two calls
in a row, the second with a smaller input (the block keeps the first call's contents), then a shape whose
partial sums exceed the block, which must be refused before anything is launched."""
import ctypes

import pytest
import torch

from cgpt_amd import capi
from tests.util import bits, randn

pytestmark = pytest.mark.gpu


def _call(name, dx, dw, dy, x, w, eps, stream):
    code = {torch.float16: capi.F16, torch.bfloat16: capi.BF16, torch.float32: capi.F32}[x.dtype]
    capi.call(name, ctypes.c_void_p(dx.data_ptr()), ctypes.c_void_p(dw.data_ptr()), ctypes.c_void_p(dy.data_ptr()),
              ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(w.data_ptr()), x.shape[0], x.shape[1], eps, code,
              ctypes.c_void_p(stream.cuda_stream))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_static_entry_point_matches_the_allocating_one_on_two_calls_in_a_row(device, dtype):
    stream = torch.cuda.Stream(device=device)
    # [rows, hidden]: the training shape's row count, then smaller inputs (row kernel and generic kernels)
    for call, (rows, hidden) in enumerate([(32768, 1024), (4096, 128), (777, 200), (5, 1024)]):
        x, dy = randn((rows, hidden), dtype, 10 + call).to(device), randn((rows, hidden), dtype, 20 + call).to(device)
        w = (1 + 0.1 * randn((hidden,), torch.float32, 30 + call)).to(dtype).to(device)
        want_dx, want_dw = torch.full_like(x, 3.0), torch.full_like(w, 3.0)
        got_dx, got_dw = torch.full_like(x, 5.0), torch.full_like(w, 5.0)
        torch.cuda.synchronize()
        _call("cgptx_rmsnorm_backward", want_dx, want_dw, dy, x, w, 1e-5, stream)
        _call("cgptx_rmsnorm_backward_static", got_dx, got_dw, dy, x, w, 1e-5, stream)
        stream.synchronize()
        assert (bits(got_dx) == bits(want_dx)).all(), f"dx differs on call {call} [{rows}, {hidden}]"
        assert (bits(got_dw) == bits(want_dw)).all(), f"dgamma differs on call {call} [{rows}, {hidden}]"


def test_static_entry_point_refuses_what_does_not_fit(device):
    stream = torch.cuda.Stream(device=device)
    rows, hidden = 4_300_000, 9   # off the row kernel's shapes: one fp32 statistic per row, 17.2 MB > 16 MiB
    x = torch.zeros(rows, hidden, dtype=torch.bfloat16, device=device)
    w = torch.ones(hidden, dtype=torch.bfloat16, device=device)
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    with pytest.raises(ValueError, match="working memory"):
        _call("cgptx_rmsnorm_backward_static", dx, dw, x, x, w, 1e-5, stream)
    with pytest.raises(ValueError):   # the shared validation still runs first
        _call("cgptx_rmsnorm_backward_static", dx, dw, x, x, w, 0.0, stream)


def test_static_entry_point_leaves_device_memory_as_it_is(device):
    """An eager call of the static entry point on a stream that has no scratch arena changes neither the free
    device memory nor the library's arenas (the allocating entry point, called the same way, takes its arena)."""
    stream = torch.cuda.Stream(device=device)
    rows, hidden = 8192, 1024
    x, dy = randn((rows, hidden), torch.bfloat16, 1).to(device), randn((rows, hidden), torch.bfloat16, 2).to(device)
    w = torch.ones(hidden, dtype=torch.bfloat16, device=device)
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    _call("cgptx_rmsnorm_backward_static", dx, dw, dy, x, w, 1e-5, stream)  # the device address is looked up here
    stream.synchronize()
    torch.cuda.synchronize()
    capi.call("cgptx_release_scratch")
    free_before, _ = torch.cuda.mem_get_info(device)
    _call("cgptx_rmsnorm_backward_static", dx, dw, dy, x, w, 1e-5, stream)
    stream.synchronize()
    free_after, _ = torch.cuda.mem_get_info(device)
    assert free_after == free_before, "the static entry point changed the amount of free device memory"
    _call("cgptx_rmsnorm_backward", dx, dw, dy, x, w, 1e-5, stream)
    stream.synchronize()
    free_with_arena, _ = torch.cuda.mem_get_info(device)
    assert free_with_arena < free_before, "the allocating entry point was expected to take its arena here"
    capi.call("cgptx_release_scratch")


_CAPTURE_FIRST = r"""
import ctypes, sys
import torch
sys.path.insert(0, sys.argv[1])
from cgpt_amd import capi
from tests.util import bits, randn

device = torch.device("cuda:0")
stream = torch.cuda.Stream(device=device)
rows, hidden = 4096, 1024
x, dy = randn((rows, hidden), torch.bfloat16, 1).to(device), randn((rows, hidden), torch.bfloat16, 2).to(device)
w = (1 + 0.1 * randn((hidden,), torch.float32, 3)).to(torch.bfloat16).to(device)
got_dx, got_dw = torch.full_like(x, 5.0), torch.full_like(w, 5.0)
args = lambda dx, dw: (ctypes.c_void_p(dx.data_ptr()), ctypes.c_void_p(dw.data_ptr()), ctypes.c_void_p(dy.data_ptr()),
                       ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(w.data_ptr()), rows, hidden, 1e-5, capi.BF16)
torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
# The library's very first call in this process happens while the stream is being captured: no eager call has
# sized an arena, and an arena cannot grow under capture, so any use of it would fail here.
with torch.cuda.graph(graph, stream=stream, capture_error_mode="thread_local"):
    capi.call("cgptx_rmsnorm_backward_static", *args(got_dx, got_dw), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
results = []
for replay in range(3):
    got_dx.fill_(7.0)
    got_dw.fill_(7.0)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    results.append((bits(got_dx).copy(), bits(got_dw).copy()))
want_dx, want_dw = torch.full_like(x, 3.0), torch.full_like(w, 3.0)
capi.call("cgptx_rmsnorm_backward", *args(want_dx, want_dw), ctypes.c_void_p(stream.cuda_stream))
stream.synchronize()
for replay, (dx_bits, dw_bits) in enumerate(results):
    assert (dx_bits == bits(want_dx)).all(), f"dx differs on replay {replay}"
    assert (dw_bits == bits(want_dw)).all(), f"dgamma differs on replay {replay}"
print("captured-first ok")
"""


def test_static_entry_point_as_the_first_call_of_a_process_under_capture(device):
    """In a fresh process: the static entry point is called for the first time while its stream is being captured
    (nothing ran eagerly before, so no arena exists and none may be created), the graph is replayed three times with
    the outputs overwritten and the device synchronised in between, and every replay equals the eager allocating
    entry point bit for bit."""
    import pathlib
    import subprocess
    import sys

    root = pathlib.Path(__file__).resolve().parent.parent
    proc = subprocess.run([sys.executable, "-c", _CAPTURE_FIRST, str(root)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and "captured-first ok" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-4000:]
