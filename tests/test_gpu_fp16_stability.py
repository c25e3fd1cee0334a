"""fp16 storage with large magnitudes: the inputs of tests/fp16_numerical_stability_test.cu (values cycling through
+scale, -scale, 1e-3 at the same tiny shapes), through the C-ABI. The reference only asks for finite results; here
every result is also compared with the float64 formulas. Tolerance: max |a-b| / max(1, |b|) <= 2e-2 (fp16)."""
import math

import numpy as np
import pytest
import torch

from cgpt_amd import ops
from oracle import oracle64
from tests.util import TOL, assert_close, to_np

pytestmark = pytest.mark.gpu

F16 = torch.float16
BOUND = TOL[F16]


def cycle(shape, scale=64.0):
    """fp16_numerical_stability_test.cu:36-41: +scale, -scale, 1e-3, repeating over the flattened tensor."""
    idx = np.arange(int(np.prod(shape))) % 3
    values = np.where(idx == 0, scale, np.where(idx == 1, -scale, 1.0e-3))
    return torch.tensor(values, dtype=torch.float32).reshape(shape).to(F16)


def finite_and_close(actual, expected, what):
    assert torch.isfinite(actual.float()).all(), f"{what}: non-finite values"
    assert_close(actual, expected, BOUND, what)


def test_rmsnorm_and_swiglu_with_large_values(device):
    """fp16_numerical_stability_test.cu:43-66."""
    x, w, dy = cycle((2, 8)), cycle((8,), 1.0), cycle((2, 8), 2.0)
    y = torch.empty_like(x, device=device)
    ops.rmsnorm_forward(y, x.to(device), w.to(device), 1e-5)
    finite_and_close(y, oracle64.rmsnorm_forward(to_np(x), to_np(w), 1e-5), "rmsnorm forward")
    dx, dw = torch.empty_like(x, device=device), torch.empty_like(w, device=device)
    ops.rmsnorm_backward(dx, dw, dy.to(device), x.to(device), w.to(device), 1e-5)
    dx64, dw64 = oracle64.rmsnorm_backward(to_np(dy), to_np(x), to_np(w), 1e-5)
    finite_and_close(dx, dx64, "rmsnorm backward dx")
    finite_and_close(dw, dw64, "rmsnorm backward dgamma")

    gate, up, dy = cycle((2, 8)), cycle((2, 8)), cycle((2, 8), 1.0)
    act = torch.empty_like(gate, device=device)
    ops.swiglu_forward(act, gate.to(device), up.to(device))
    finite_and_close(act, oracle64.swiglu_forward(to_np(gate), to_np(up)), "swiglu forward")
    dg, du = torch.empty_like(gate, device=device), torch.empty_like(gate, device=device)
    ops.swiglu_backward(dg, du, dy.to(device), gate.to(device), up.to(device))
    dg64, du64 = oracle64.swiglu_backward(to_np(dy), to_np(gate), to_np(up))
    finite_and_close(dg, dg64, "swiglu backward dgate")
    finite_and_close(du, du64, "swiglu backward dup")


def test_cross_entropy_with_large_logits(device):
    """fp16_numerical_stability_test.cu:68-80 (its softmax operator is not part of the backward path)."""
    logits = cycle((2, 8), 64.0)
    targets = torch.tensor([0, 3], dtype=torch.int32)
    loss = torch.zeros(1, dtype=torch.float32, device=device)
    grad = torch.empty_like(logits, device=device)
    ops.cross_entropy_forward_backward(loss, grad, logits.to(device), targets.to(device), 2)
    loss64, grad64 = oracle64.cross_entropy(to_np(logits), targets.numpy())
    assert math.isfinite(loss.item()) and abs(loss.item() - loss64) <= 1e-4 * max(1.0, abs(loss64))
    finite_and_close(grad, grad64, "cross-entropy gradient")


def test_linear_with_large_values(device):
    """fp16_numerical_stability_test.cu:82-94: products of 32 * 32 summed over 4 terms stay inside fp16."""
    x, w, b, dy = cycle((2, 4), 32.0), cycle((4, 4), 32.0), cycle((4,), 1.0), cycle((2, 4), 1.0)
    y = torch.empty((2, 4), dtype=F16, device=device)
    ops.linear_forward(y, x.to(device), w.to(device), bias=b.to(device))
    finite_and_close(y, oracle64.linear_forward(to_np(x), to_np(w), to_np(b)), "linear forward")
    dx = torch.empty((2, 4), dtype=F16, device=device)
    dw = torch.empty((4, 4), dtype=F16, device=device)
    db = torch.empty((4,), dtype=F16, device=device)
    ops.linear_backward(dx, dw, db, dy.to(device), x.to(device), w.to(device))
    dx64, dw64, db64 = oracle64.linear_backward(to_np(dy), to_np(x), to_np(w))
    finite_and_close(dx, dx64, "linear backward dx")
    finite_and_close(dw, dw64, "linear backward dw")
    finite_and_close(db, db64, "linear backward db")


def test_attention_with_large_scores(device):
    """fp16_numerical_stability_test.cu:96-111: 2 queries against 3 keys, 2:1 heads of 32, not causal; scores reach
    16 * 16 * 32 / sqrt(32) = 1448, far outside what exp() holds without the row maximum."""
    q, k, v = cycle((1, 2, 2, 32), 16.0), cycle((1, 3, 1, 32), 16.0), cycle((1, 3, 1, 32), 16.0)
    do = cycle((1, 2, 2, 32), 1.0)
    options = ops.FlashAttentionOptions(2, 1, 32, 1.0 / math.sqrt(32.0), False, 0, 2, 128, True)
    out = torch.empty_like(q, device=device)
    ops.flash_gqa_attention_forward(out, q.to(device), k.to(device), v.to(device), options=options)
    out64, _ = oracle64.attention_forward(to_np(q), to_np(k), to_np(v), 2, 1, 32, options.attention_scale, False)
    finite_and_close(out, out64, "attention forward")
    dq, dk, dv = (torch.empty_like(t, device=device) for t in (q, k, v))
    ops.flash_gqa_attention_backward(dq, dk, dv, do.to(device), q.to(device), k.to(device), v.to(device),
                                     options=options)
    dq64, dk64, dv64 = oracle64.attention_backward(to_np(do), to_np(q), to_np(k), to_np(v), 2, 1, 32,
                                                   options.attention_scale, False)
    finite_and_close(dq, dq64, "attention backward dq")
    finite_and_close(dk, dk64, "attention backward dk")
    finite_and_close(dv, dv64, "attention backward dv")


def test_rope_and_embedding_with_large_values(device):
    """fp16_numerical_stability_test.cu:113-143."""
    q, k = cycle((1, 2, 1, 8)), cycle((1, 2, 1, 8))
    dq_rot, dk_rot = cycle((1, 2, 1, 8), 1.0), cycle((1, 2, 1, 8), 1.0)
    cos = torch.full((2, 4), 0.7071, dtype=torch.float32).to(F16)
    sin = torch.full((2, 4), 0.7071, dtype=torch.float32).to(F16)
    q_dev, k_dev = q.to(device), k.to(device)
    ops.rope_forward(q_dev, k_dev, cos.to(device), sin.to(device))
    finite_and_close(q_dev, oracle64.rope_forward(to_np(q), to_np(cos), to_np(sin)), "rope forward q")
    finite_and_close(k_dev, oracle64.rope_forward(to_np(k), to_np(cos), to_np(sin)), "rope forward k")
    dq, dk = torch.empty_like(q, device=device), torch.empty_like(k, device=device)
    ops.rope_backward(dq, dk, dq_rot.to(device), dk_rot.to(device), cos.to(device), sin.to(device))
    finite_and_close(dq, oracle64.rope_backward(to_np(dq_rot), to_np(cos), to_np(sin)), "rope backward q")
    finite_and_close(dk, oracle64.rope_backward(to_np(dk_rot), to_np(cos), to_np(sin)), "rope backward k")

    weight, dy = cycle((4, 8)), cycle((3, 8), 1.0)
    ids = torch.tensor([0, 1, 3], dtype=torch.int32)
    out = torch.empty((3, 8), dtype=F16, device=device)
    ops.embedding_forward(out, ids.to(device), 3, weight.to(device))
    assert torch.equal(out.cpu(), weight[ids.long()])
    dweight = torch.full((4, 8), 7.0, dtype=F16, device=device)
    ops.embedding_backward(dweight, dy.to(device), ids.to(device), 3)
    expected = oracle64.embedding_backward(to_np(dy), ids.numpy(), 4)
    assert torch.equal(dweight.cpu().double(), torch.from_numpy(expected)), "embedding backward"
