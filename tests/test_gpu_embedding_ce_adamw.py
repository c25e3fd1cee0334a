"""GPU parity tests: embedding gather/scatter (bit-exact), dense cross-entropy, AdamW."""
import math

import numpy as np
import pytest
import torch

from cgpt_amd import ops
from oracle import cpu_ops, oracle64
from tests.util import DTYPES, DTYPE_IDS, TOL, assert_close, randint, randn, to_np

pytestmark = pytest.mark.gpu


def dev(t, device):
    return t.to(device).contiguous()


# ---------------------------------------------------------------------- Embedding
@pytest.mark.parametrize("dtype,tol", [(torch.float16, 1e-2), (torch.bfloat16, 5e-2), (torch.float32, 1e-6)])
def test_embedding_backward_repeated_tokens_known_answer(device, dtype, tol):
    """tests/embedding_test.cu:183-203."""
    dy = torch.tensor([1, 2, 3, 4, 0.5, 1.5, -1, 2, 7, 8, 9, 10.0]).reshape(3, 4).to(dtype)
    ids = torch.tensor([1, 1, 2], dtype=torch.int32)
    gw = torch.full((3, 4), 5.0, dtype=dtype, device=device)
    ops.embedding_backward(gw, dev(dy, device), dev(ids, device), 3)
    assert np.abs(to_np(gw).reshape(-1) - [0, 0, 0, 0, 1.5, 3.5, 2, 6, 7, 8, 9, 10]).max() <= tol


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("tokens,vocab,hidden,accumulate", [
    (64, 7, 16, False), (64, 7, 16, True), (1000, 50, 24, True), (4096, 1000, 128, False), (300, 5, 7, True),
    (1, 3, 8, False), (4097, 900, 40, True), (6000, 50, 24, False),
])
def test_embedding_backward_bit_exact(device, tokens, vocab, hidden, accumulate, dtype):
    """Heavy id collisions, out-of-range ids, odd widths: which rows receive which tokens is integer work
    and the per-add rounding follows the CPU operator, so the whole table is compared bit for bit."""
    ids = randint(vocab + 2, (tokens,), 3)  # ids vocab and vocab+1 are out of range and must be skipped
    dy = randn((tokens, hidden), dtype, 4)
    gw = randn((vocab, hidden), dtype, 5)
    dgw = dev(gw, device).clone()
    cpu_ops.embedding_backward(gw, dy, ids, True, accumulate)
    ops.embedding_backward(dgw, dev(dy, device), dev(ids, device), tokens, None,
                           ops.EmbeddingBackwardOptions(accumulate_weight=accumulate))
    assert torch.equal(dgw.cpu(), gw)


def test_embedding_backward_all_tokens_same_id(device):
    dtype = torch.bfloat16
    ids = torch.full((5000,), 3, dtype=torch.int32)
    dy = randn((5000, 64), dtype, 6)
    gw = torch.zeros(8, 64, dtype=dtype)
    dgw = torch.ones(8, 64, dtype=dtype, device=device)
    cpu_ops.embedding_backward(gw, dy, ids)
    ops.embedding_backward(dgw, dev(dy, device), dev(ids, device), 5000)
    assert torch.equal(dgw.cpu(), gw)


def test_embedding_backward_training_shape_bit_exact_and_deterministic(device):
    """32768 tokens into a [32000, 1024] bf16 table that already holds the lm_head gradient (tied weights)."""
    dtype = torch.bfloat16
    ids = randint(32000, (32768,), 7)
    dy = randn((32768, 1024), dtype, 8)
    base = randn((32000, 1024), dtype, 9)
    want = base.clone()
    cpu_ops.embedding_backward(want, dy, ids, True, True)
    d_ids, d_dy = dev(ids, device), dev(dy, device)
    results = []
    for _ in range(2):
        got = dev(base, device).clone()
        ops.embedding_backward(got, d_dy, d_ids, 32768, None, ops.EmbeddingBackwardOptions(accumulate_weight=True))
        results.append(got.cpu())
    assert torch.equal(results[0], results[1])
    assert torch.equal(results[0], want)
    # integer side: exactly the rows named by the ids changed
    changed = (results[0] != base).any(dim=1).nonzero().flatten().tolist()
    assert set(changed) <= set(ids.tolist())


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_embedding_forward_bit_exact(device, dtype):
    for vocab, hidden, tokens in ((11, 24, 40), (100, 1024, 256), (7, 5, 9)):
        w = randn((vocab, hidden), dtype, 10)
        ids = randint(vocab + 1, (tokens,), 11)
        out = torch.empty(tokens, hidden, dtype=dtype)
        cpu_ops.embedding_forward(out, ids, w)
        dout = torch.full((tokens, hidden), 9.0, dtype=dtype, device=device)
        ops.embedding_forward(dout, dev(ids, device), tokens, dev(w, device))
        assert torch.equal(dout.cpu(), out)


def test_embedding_argument_errors(device):
    gw = torch.zeros(3, 4, device=device)
    dy = torch.zeros(2, 4, device=device)
    ids = torch.zeros(2, dtype=torch.int32, device=device)
    with pytest.raises(ValueError):
        ops.embedding_backward(gw, dy, ids, 3)
    with pytest.raises(ValueError):
        ops.embedding_backward(gw, dy.half(), ids, 2)
    with pytest.raises(ValueError):
        ops.embedding_backward(gw, dy, ids, 0)


# ------------------------------------------------------------------ Cross entropy
def test_cross_entropy_known_answers(device):
    """tests/cross_entropy_test.cu:33-56."""
    logits = torch.tensor([1, 2, 3, 1, 1, 1.0]).reshape(2, 3).to(device)
    targets = torch.tensor([2, 0], dtype=torch.int32, device=device)
    loss, grad = torch.zeros(1, device=device), torch.zeros(2, 3, device=device)
    ops.cross_entropy_forward_backward(loss, grad, logits, targets, 2)
    want = (math.log(math.exp(1) + math.exp(2) + math.exp(3)) - 3 + math.log(3)) / 2
    assert abs(loss.item() - want) <= 1e-5
    assert np.abs(to_np(grad).reshape(-1) -
                  [0.0450153, 0.1223642, -0.1673795, -0.3333333, 0.1666667, 0.1666667]).max() <= 1e-5
    only = torch.zeros(1, device=device)
    ops.cross_entropy_forward(only, logits, targets, 2)
    assert abs(only.item() - want) <= 1e-5
    loss, grad = torch.zeros(1, device=device), torch.zeros(1, 2, device=device)
    ops.cross_entropy_forward_backward(loss, grad, torch.zeros(1, 2, device=device),
                                       torch.tensor([0], dtype=torch.int32, device=device), 1, None, 1024.0)
    assert abs(loss.item() - math.log(2)) <= 1e-6
    assert grad.reshape(-1).tolist() == [-512.0, 512.0]
    with pytest.raises(ValueError):  # target count does not match the rows (tests/cross_entropy_test.cu:58-63)
        ops.cross_entropy_forward_backward(loss, torch.zeros(2, 3, device=device), torch.zeros(2, 3, device=device),
                                           targets, 1)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows,vocab", [(5, 11), (64, 1000), (7, 32000), (3, 50257), (16, 8), (2, 50264), (2, 65544)])
def test_cross_entropy_parity(device, rows, vocab, dtype):
    # Row lengths for each kernel: unaligned rows stream (11, 50257); aligned rows of up to 8192 vectors stay
    # in registers, in 2, 8 or 16 vectors per thread (8 .. 50264); longer ones stream again (65544).
    logits = randn((rows, vocab), dtype, 12, 3.0)
    targets = randint(vocab, (rows,), 13)
    targets[0] = vocab + 5  # out of range: no loss, gradient stays the softmax
    loss, grad = torch.empty(1), torch.empty_like(logits)
    cpu_ops.cross_entropy_forward_backward(loss, grad, logits, targets, 1024.0)
    dloss, dgrad = torch.zeros(1, device=device), torch.empty_like(logits, device=device)
    ops.cross_entropy_forward_backward(dloss, dgrad, dev(logits, device), dev(targets, device), rows, None, 1024.0)
    l64, g64 = oracle64.cross_entropy(to_np(logits), targets.numpy(), 1024.0)
    assert abs(dloss.item() - l64) <= 1e-4 * max(1.0, abs(l64))
    assert abs(dloss.item() - loss.item()) <= 1e-4 * max(1.0, abs(l64))
    assert_close(dgrad, grad, TOL[dtype], "grad vs float32 checker")
    assert_close(dgrad, g64, TOL[dtype], "grad vs float64")
    only = torch.zeros(1, device=device)
    ops.cross_entropy_forward(only, dev(logits, device), dev(targets, device), rows)
    assert abs(only.item() - l64) <= 1e-4 * max(1.0, abs(l64))


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_cross_entropy_rows_that_start_off_a_16_byte_boundary(device, dtype):
    """A vocabulary that is not a multiple of the vector width: every row starts at another offset from a 16-byte
    boundary. In place (gradient = logits), and with a gradient whose rows have a different offset than the logits'."""
    rows, vocab = 9, 50257
    logits = randn((rows, vocab), dtype, 21, 3.0)
    targets = randint(vocab, (rows,), 22)
    l64, g64 = oracle64.cross_entropy(to_np(logits), targets.numpy(), 8.0)
    d_targets = dev(targets, device)
    in_place, loss = dev(logits, device).clone(), torch.zeros(1, device=device)
    ops.cross_entropy_forward_backward(loss, in_place, in_place, d_targets, rows, None, 8.0)
    assert abs(loss.item() - l64) <= 1e-4 * max(1.0, abs(l64))
    assert_close(in_place, g64, TOL[dtype], "in place")
    storage = torch.empty(rows * vocab + 1, dtype=dtype, device=device)
    shifted = storage[1:].view(rows, vocab)  # one element off the logits' alignment
    ops.cross_entropy_forward_backward(loss, shifted, dev(logits, device), d_targets, rows, None, 8.0)
    assert_close(shifted, g64, TOL[dtype], "gradient rows at another offset")


def test_cross_entropy_training_shape_rows_sum_to_zero(device):
    """[8192, 32000] bf16 (a quarter of the training rows; 524 MB): every gradient row sums to ~0, the target
    entry is the only negative one, the loss equals the float64 value on a row sample, twice identical."""
    dtype = torch.bfloat16
    rows, vocab = 8192, 32000
    logits = randn((rows, vocab), dtype, 14, 2.0)
    targets = randint(vocab, (rows,), 15)
    dl, dt = dev(logits, device), dev(targets, device)
    runs = []
    for _ in range(2):
        loss, grad = torch.zeros(1, device=device), torch.empty_like(dl)
        ops.cross_entropy_forward_backward(loss, grad, dl, dt, rows, None, 1024.0)
        runs.append((loss.item(), grad))
    assert runs[0][0] == runs[1][0] and torch.equal(runs[0][1], runs[1][1])
    grad = runs[0][1].float()
    assert grad.sum(dim=1).abs().max().item() <= 2e-2 * 1024.0 / rows * 40
    negatives = (grad < 0).sum(dim=1)
    assert torch.all(negatives == 1)
    assert torch.equal((grad < 0).float().argmax(dim=1).int().cpu(), targets)
    sample = slice(0, 64)
    l64, g64 = oracle64.cross_entropy(to_np(logits[sample]), targets[sample].numpy(), 1024.0 * 64 / rows)
    assert_close(runs[0][1][sample], g64, TOL[dtype], "grad rows vs float64")
    full = torch.empty(1)
    cpu_ops.cross_entropy_forward(full, logits, targets)
    assert abs(runs[0][0] - full.item()) <= 1e-4 * full.item()


# -------------------------------------------------------------------------- AdamW
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.float16, 2e-3), (torch.bfloat16, 1e-2)])
def test_adamw_step_known_answers(device, dtype, tol):
    """tests/adamw_test.cu:21-57."""
    p = torch.tensor([1.0, -2.0]).to(dtype).to(device)
    g = torch.tensor([0.1, -0.2]).to(dtype).to(device)
    state = ops.AdamWState.for_parameter(p)
    options = ops.AdamWOptions(learning_rate=0.1, beta1=0.9, beta2=0.999, epsilon=1e-8, weight_decay=0.01)
    assert ops.adamw_step(p, g, state, options)
    assert np.abs(to_np(p) - [0.899, -1.898]).max() <= tol
    assert np.abs(to_np(state.first_moment) - [0.01, -0.02]).max() <= tol
    assert np.abs(to_np(state.second_moment) - [0.00001, 0.00004]).max() <= tol
    assert state.step == 1
    assert ops.adamw_step(p, g, state, options)
    assert np.abs(to_np(p) - [0.798101, -1.796102]).max() <= tol
    assert state.step == 2

    p = torch.tensor([1.0, -1.0]).to(dtype).to(device)
    g = torch.tensor([8.0, 0.0]).to(dtype).to(device)
    state = ops.AdamWState.for_parameter(p)
    options = ops.AdamWOptions(learning_rate=0.1, weight_decay=0.0, loss_scale=4.0, max_grad_norm=1.0)
    assert ops.adamw_step(p, g, state, options)
    assert np.abs(to_np(p) - [0.9, -1.0]).max() <= tol
    assert np.abs(to_np(state.master_parameter) - [0.9, -1.0]).max() <= 2e-6
    before = p.clone()
    g = torch.tensor([float("inf"), 0.0]).to(dtype).to(device)
    assert not ops.adamw_step(p, g, state, options)
    assert torch.equal(p, before) and state.step == 1


def test_adamw_validation(device):
    p = torch.zeros(1, device=device)
    state = ops.AdamWState.for_parameter(p)
    with pytest.raises(ValueError):
        ops.adamw_step(p, torch.zeros(2, device=device), state)
    with pytest.raises(ValueError):
        ops.adamw_step(p, torch.zeros(1, device=device), state, ops.AdamWOptions(beta2=1.0))


def test_adamw_batched_non_finite_gradient(device):
    """tests/adamw_test.cu:70-91."""
    p = torch.tensor([1.0, -1.0], device=device)
    g = torch.tensor([1.0, 0.0], device=device)
    state = ops.AdamWState.for_parameter(p)
    ws = ops.AdamWWorkspace()
    entry = [ops.AdamWBatchEntry(p, g, state)]
    ops.adamw_step_many_async(entry, ops.AdamWOptions(learning_rate=0.1, weight_decay=0.0), ws)
    assert ops.adamw_check(ws)
    assert np.abs(to_np(p) - [0.9, -1.0]).max() <= 1e-6 and state.step == 1
    g.copy_(torch.tensor([float("inf"), 0.0]))
    ops.adamw_step_many_async(entry, ops.AdamWOptions(), ws)
    assert not ops.adamw_check(ws)
    assert np.abs(to_np(p) - [0.9, -1.0]).max() <= 1e-6 and state.step == 1
    # the sticky flag was cleared by the check; a finite step goes through again
    g.copy_(torch.tensor([1.0, 0.0]))
    ops.adamw_step_many_async(entry, ops.AdamWOptions(learning_rate=0.1, weight_decay=0.0), ws)
    assert ops.adamw_check(ws) and state.step == 2
    with pytest.raises(ValueError):  # the workspace is bound to its first entry list
        ops.adamw_step_many_async(entry + entry, ops.AdamWOptions(), ws)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_adamw_many_parity_three_steps(device, dtype):
    """Ragged tensor sizes (1 .. 70001 elements, crossing the 4096-element chunking), global-norm clipping,
    loss scale 1024, three steps, against the float64 statement of src/optim/adamw.cu:148-187."""
    sizes = [1, 7, 4096, 4097, 70001, 513, 8192]
    params = [randn((n,), dtype, 100 + i, 0.5) for i, n in enumerate(sizes)]
    d_params = [dev(p, device).clone() for p in params]
    states = [ops.AdamWState.for_parameter(p) for p in d_params]
    d_grads = [torch.empty_like(p) for p in d_params]
    entries = [ops.AdamWBatchEntry(p, g, s) for p, g, s in zip(d_params, d_grads, states)]
    ws = ops.AdamWWorkspace()
    options = ops.AdamWOptions(learning_rate=3e-4, beta1=0.9, beta2=0.95, epsilon=1e-8, weight_decay=0.1,
                               loss_scale=1024.0, max_grad_norm=1.0)
    masters = [to_np(p) for p in params]
    ms = [np.zeros(n) for n in sizes]
    vs = [np.zeros(n) for n in sizes]
    step = 0
    for it in range(3):
        grads = [randn((n,), dtype, 200 + 10 * it + i, 1024.0 * 0.01) for i, n in enumerate(sizes)]
        for dg, g in zip(d_grads, grads):
            dg.copy_(g)
        ops.adamw_step_many_async(entries, options, ws)
        ok, masters, ms, vs, step = oracle64.adamw(None, [to_np(g) for g in grads], masters, ms, vs, step, 3e-4, 0.9,
                                                   0.95, 1e-8, 0.1, 1024.0, 1.0)
        assert ok
    assert ops.adamw_check(ws) and states[0].step == 3 == step
    for p, s, m64, mm, vv in zip(d_params, states, masters, ms, vs):
        assert_close(s.master_parameter, m64, 1e-5, "master")
        assert_close(s.first_moment, mm, 1e-5, "m")
        assert np.abs(to_np(s.second_moment) - vv).max() <= 1e-5 * max(1e-12, np.abs(vv).max()) + 1e-12
        assert_close(p, m64, TOL[dtype], "param")
        assert torch.equal(p, s.master_parameter.to(dtype))


def test_adamw_matches_cpu_restatement_single_tensor(device):
    n = 10007
    p, g = randn((n,), torch.float32, 300), randn((n,), torch.float32, 301, 5.0)
    dp, dg = dev(p, device).clone(), dev(g, device)
    state = ops.AdamWState.for_parameter(dp)
    master, m, v = p.clone(), torch.zeros(n), torch.zeros(n)
    options = ops.AdamWOptions(learning_rate=1e-2, beta2=0.95, weight_decay=0.1, loss_scale=2.0, max_grad_norm=1.0)
    for step in (1, 2):
        assert cpu_ops.adamw(p, g, master, m, v, step, 1e-2, 0.9, 0.95, 1e-8, 0.1, 2.0, 1.0)
        assert ops.adamw_step(dp, dg, state, options)
    assert_close(dp, p, 1e-6, "param")
    assert_close(state.first_moment, m, 1e-6, "m")
    assert_close(state.second_moment, v, 1e-6, "v")
