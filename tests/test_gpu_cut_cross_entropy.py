"""GPU parity tests of cut cross-entropy against the float64 statement (loss, dX, dC) and against the
dense path it must be equivalent to: cross_entropy(X·Cᵀ) followed by linear_backward."""
import math

import numpy as np
import pytest
import torch

from cgpt_amd import ops
from oracle import oracle64
from tests.util import DTYPES, DTYPE_IDS, STOL, TOL, assert_close, assert_scaled_close, randint, randn, to_np

pytestmark = pytest.mark.gpu


def run(device, x, c, targets, scale=1.0, accumulate=False, base=None):
    loss = torch.zeros(1, device=device)
    dx = torch.full_like(x, 3.0, device=device)
    dc = torch.full_like(c, 3.0, device=device) if base is None else base.to(device).clone()
    ops.cut_cross_entropy_forward_backward(loss, dx, dc, x.to(device), c.to(device), targets.to(device), x.shape[0],
                                           None, scale, accumulate)
    return loss.item(), dx, dc


def test_reference_test_case(device):
    """tests/cut_cross_entropy_test.cu:19-31 (F32, 2x2 input, 3 classes). Row 1 of dX and row 2 of dC are
    compared with the reference's formula rather than its constants, which disagree with its own kernels
    (see tests/test_oracle_pins.py::test_cut_cross_entropy_known_answer)."""
    x = torch.tensor([[1, 2], [3, 4.0]])
    c = torch.tensor([[1, 0], [0, 1], [1, 1.0]])
    targets = torch.tensor([2, 0], dtype=torch.int32)
    loss, dx, dc = run(device, x, c, targets)
    e = math.exp
    assert abs(loss - (math.log(e(1) + e(2) + e(3)) - 3 + math.log(e(3) + e(4) + e(7)) - 3) / 2) <= 2e-5
    assert np.abs(to_np(dx)[0] - [-0.1223642, -0.0450153]).max() <= 2e-5
    assert np.abs(to_np(dc)[:2].reshape(-1) - [-1.4295, -1.876, 0.193, 0.339]).max() <= 2e-3
    l64, dx64, dc64 = oracle64.cut_cross_entropy(x.numpy(), c.numpy(), targets.numpy())
    assert_close(dx, dx64, 1e-5, "dX")
    assert_close(dc, dc64, 1e-5, "dC")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows,hidden,vocab", [(5, 7, 11), (64, 64, 128), (300, 128, 1000), (1024, 256, 4096)])
def test_parity_with_float64(device, rows, hidden, vocab, dtype):
    x, c = randn((rows, hidden), dtype, 1), randn((vocab, hidden), dtype, 2, 0.05)
    targets = randint(vocab, (rows,), 3)
    l64, dx64, dc64 = oracle64.cut_cross_entropy(to_np(x), to_np(c), targets.numpy(), 1024.0)
    loss, dx, dc = run(device, x, c, targets, 1024.0)
    assert abs(loss - l64) <= (1e-4 if dtype == torch.float32 else 5e-3) * max(1.0, l64)
    assert_scaled_close(dx, dx64, STOL[dtype], "dX")
    assert_scaled_close(dc, dc64, STOL[dtype], "dC")
    base = randn((vocab, hidden), dtype, 4)
    _, _, dc2 = run(device, x, c, targets, 1024.0, True, base)
    want = dc64 + to_np(base)
    assert_scaled_close(dc2, want, STOL[dtype], "dC accumulate")


@pytest.mark.parametrize("logits_bytes", [None, 128 << 20], ids=["one-chunk", "three-chunks"])
def test_equivalent_to_dense_cross_entropy_plus_linear_backward(device, monkeypatch, logits_bytes):
    """bf16, [6000, 256] x [32000, 256], as one chunk of logits (the classifier gradient straight out of its
    contraction) and as several row chunks (CGPTX_CUT_CE_LOGITS_BYTES = 128 MiB: 3 chunks of 2048 rows, the
    classifier gradient accumulated in fp32 across them)."""
    if logits_bytes is not None:
        monkeypatch.setenv("CGPTX_CUT_CE_LOGITS_BYTES", str(logits_bytes))
    dtype = torch.bfloat16
    rows, hidden, vocab = 6000, 256, 32000
    x, c = randn((rows, hidden), dtype, 5).to(device), randn((vocab, hidden), dtype, 6, 0.05).to(device)
    targets = randint(vocab, (rows,), 7).to(device)
    loss, dx, dc = run(device, x, c, targets, 1024.0)
    logits = torch.empty(rows, vocab, dtype=dtype, device=device)
    ops.linear_forward(logits, x, c)
    dense_loss = torch.zeros(1, device=device)
    grad = torch.empty_like(logits)
    ops.cross_entropy_forward_backward(dense_loss, grad, logits, targets, rows, None, 1024.0)
    dx2, dc2 = torch.empty_like(x), torch.empty_like(c)
    ops.linear_backward(dx2, dc2, None, grad, x, c)
    assert abs(loss - dense_loss.item()) <= 1e-5 * dense_loss.item()
    assert_scaled_close(dx, dx2, STOL[dtype], "dX vs dense path")
    assert_scaled_close(dc, dc2, STOL[dtype], "dC vs dense path")
    again = run(device, x, c, targets, 1024.0)
    assert again[0] == loss and torch.equal(again[1], dx) and torch.equal(again[2], dc)


@pytest.mark.parametrize("rows", [1024, 1025, 1281, 2049], ids=["at-the-bound", "one-row-over", "ragged-second-chunk", "three-chunks"])
def test_row_counts_on_both_sides_of_the_chunk_bound(device, monkeypatch, rows):
    """CGPTX_CUT_CE_LOGITS_BYTES = 64 MiB at V = 32000 in bf16 allows 1024 rows per chunk: 1024 rows are one chunk
    (the classifier gradient straight out of its contraction), 1025 rows two chunks of 768 and 257 rows, 2049 three.
    Loss, dX and dC against float64 on every side of the bound; both gradient paths round the same fp32 sums once."""
    monkeypatch.setenv("CGPTX_CUT_CE_LOGITS_BYTES", str(64 << 20))
    dtype = torch.bfloat16
    hidden, vocab = 64, 32000
    x, c = randn((rows, hidden), dtype, 40 + rows), randn((vocab, hidden), dtype, 41, 0.05)
    targets = randint(vocab, (rows,), 42)
    loss, dx, dc = run(device, x.to(device), c.to(device), targets.to(device), 64.0)
    z = to_np(x) @ to_np(c).T
    lse = np.log(np.exp(z - z.max(axis=1, keepdims=True)).sum(axis=1)) + z.max(axis=1)
    want_loss = float((lse - z[np.arange(rows), targets.numpy()]).mean())
    prob = np.exp(z - lse[:, None])
    prob[np.arange(rows), targets.numpy()] -= 1.0
    prob *= 64.0 / rows
    assert abs(loss - want_loss) <= 1e-4 * want_loss
    assert_scaled_close(dx, prob @ to_np(c), STOL[dtype], f"dX, {rows} rows")
    assert_scaled_close(dc, prob.T @ to_np(x), STOL[dtype], f"dC, {rows} rows")


@pytest.mark.parametrize("logits_bytes", [None, 2 << 30], ids=["two-chunks-by-default", "one-chunk"])
@pytest.mark.parametrize("hidden", [1024, 768], ids=["preset-1024", "secondary-768"])
def test_training_shape_against_the_dense_path_and_float64_rows(device, monkeypatch, hidden, logits_bytes):
    """[32768, hidden] x [32000, hidden] bf16, loss scale 1024, with the default bound on the logits scratch (two
    chunks of 16384 rows) and as one chunk: loss, dX and dC against the dense path (logits contraction,
    cross-entropy operator, linear_backward), the dX rows of 256 rows against float64 (a row's gradient
    does not depend on the other rows), and two runs are bit-identical."""
    if logits_bytes is not None:
        monkeypatch.setenv("CGPTX_CUT_CE_LOGITS_BYTES", str(logits_bytes))
    dtype = torch.bfloat16
    rows, vocab = 32768, 32000
    x, c = randn((rows, hidden), dtype, 31), randn((vocab, hidden), dtype, 32, 0.02)
    targets = randint(vocab, (rows,), 33)
    dx_, dc_, dt = x.to(device), c.to(device), targets.to(device)
    loss, dx, dc = run(device, dx_, dc_, dt, 1024.0)
    logits = torch.empty(rows, vocab, dtype=dtype, device=device)
    ops.linear_forward(logits, dx_, dc_)
    dense_loss, grad = torch.zeros(1, device=device), torch.empty_like(logits)
    ops.cross_entropy_forward_backward(dense_loss, grad, logits, dt, rows, None, 1024.0)
    dx2, dc2 = torch.empty_like(dx_), torch.empty_like(dc_)
    ops.linear_backward(dx2, dc2, None, grad, dx_, dc_)
    del logits, grad
    assert abs(loss - dense_loss.item()) <= 1e-5 * dense_loss.item()
    assert_scaled_close(dx, dx2, STOL[dtype], "dX vs dense path")
    assert_scaled_close(dc, dc2, STOL[dtype], "dC vs dense path")
    # float64 on a slice: the per-row loss terms and the dX rows do not depend on the other rows
    pick = np.arange(0, rows, rows // 256)
    z = to_np(x)[pick].astype(np.float64) @ to_np(c).astype(np.float64).T
    lse = np.log(np.exp(z - z.max(axis=1, keepdims=True)).sum(axis=1)) + z.max(axis=1)
    prob = np.exp(z - lse[:, None])
    prob[np.arange(len(pick)), targets.numpy()[pick]] -= 1.0
    dx64 = prob @ to_np(c).astype(np.float64) * (1024.0 / rows)
    assert_scaled_close(dx.cpu()[pick], dx64, STOL[dtype], "dX rows vs float64")
    again = run(device, dx_, dc_, dt, 1024.0)
    assert again[0] == loss and torch.equal(again[1], dx) and torch.equal(again[2], dc)


def test_argument_errors(device):
    x, c = torch.zeros(4, 8, device=device), torch.zeros(5, 8, device=device)
    t = torch.zeros(4, dtype=torch.int32, device=device)
    loss = torch.zeros(1, device=device)
    with pytest.raises(ValueError):
        ops.cut_cross_entropy_forward_backward(loss, x.clone(), c.clone(), x, torch.zeros(5, 7, device=device), t, 4)
    with pytest.raises(ValueError):
        ops.cut_cross_entropy_forward_backward(loss, x.clone(), c.clone(), x, c, t, 3)
    with pytest.raises(ValueError):
        ops.cut_cross_entropy_forward_backward(loss.half(), x.clone(), c.clone(), x, c, t, 4)
