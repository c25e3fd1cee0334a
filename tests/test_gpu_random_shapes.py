"""Seeded random-shape sweep of every operator on the path against the float64 formulas (the float32 CPU checker for
the rotary embedding, bit for bit for the embedding scatter): shapes the fixed lists of the other test files do not name — odd widths,
ragged row counts, every dtype, group sizes, offsets, accumulate flags. The shapes stay small enough for the float64
formulas to finish in a fraction of a second each; the seeds are fixed, so a failure names a reproducible case."""
import numpy as np
import pytest
import torch

from cgpt_amd import ops
from oracle import cpu_ops, oracle64
from tests.util import DTYPES, STOL, TOL, assert_close, assert_scaled_close, randint, randn, to_np

pytestmark = pytest.mark.gpu

SEEDS = list(range(40))


def dev(t, device):
    return t.to(device).contiguous()


def pick(rng, values):
    return values[int(rng.integers(0, len(values)))]


def case_dtype(rng):
    return DTYPES[int(rng.integers(0, len(DTYPES)))]


@pytest.mark.parametrize("seed", SEEDS)
def test_rmsnorm_backward_random_shapes(device, seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = case_dtype(rng)
    rows = int(rng.integers(1, 3000))
    hidden = pick(rng, [int(rng.integers(1, 300)), 64, 128, 8 * int(rng.integers(1, 200)), 768, 1024, 4096])
    print(f"rmsnorm rows={rows} hidden={hidden} {dtype}", flush=True)
    x, dy = randn((rows, hidden), dtype, seed), randn((rows, hidden), dtype, seed + 1)
    w = (1.0 + 0.2 * randn((hidden,), torch.float32, seed + 2)).to(dtype)
    dx64, dw64 = oracle64.rmsnorm_backward(to_np(dy), to_np(x), to_np(w), 1e-5)
    dx, dw = torch.full_like(x, 3.0, device=device), torch.full_like(w, 3.0, device=device)
    ops.rmsnorm_backward(dx, dw, dev(dy, device), dev(x, device), dev(w, device), 1e-5)
    assert_close(dx, dx64, TOL[dtype], "dx")
    assert_scaled_close(dw, dw64, STOL[dtype], "dgamma")
    y = torch.empty_like(x, device=device)
    ops.rmsnorm_forward(y, dev(x, device), dev(w, device), 1e-5)
    assert_close(y, oracle64.rmsnorm_forward(to_np(x), to_np(w), 1e-5), TOL[dtype], "y")


@pytest.mark.parametrize("seed", SEEDS)
def test_rope_and_swiglu_random_shapes(device, seed):
    rng = np.random.default_rng(2000 + seed)
    dtype = case_dtype(rng)
    b, s = int(rng.integers(1, 4)), int(rng.integers(1, 40))
    hkv = int(rng.integers(1, 5))
    hq = hkv * int(rng.integers(1, 5))
    d = 2 * int(rng.integers(1, 65))
    rotary = pick(rng, [0, 2 * int(rng.integers(1, d // 2 + 1))])
    off = int(rng.integers(0, 9))
    print(f"rope b={b} s={s} {hq}:{hkv} d={d} rotary={rotary} off={off} {dtype}", flush=True)
    r = rotary or d
    pos = torch.arange(off + s + 1, dtype=torch.float32)[:, None]
    theta = pos / torch.pow(torch.tensor(10000.0), 2.0 * torch.arange(r // 2, dtype=torch.float32)[None, :] / r)
    cos, sin = torch.cos(theta).to(dtype).contiguous(), torch.sin(theta).to(dtype).contiguous()
    q, k = randn((b, s, hq, d), dtype, seed), randn((b, s, hkv, d), dtype, seed + 1)
    gq, gk = torch.empty_like(q), torch.empty_like(k)
    cpu_ops.rope_backward(gq, gk, q, k, cos, sin, rotary, off)
    dq, dk = torch.full_like(q, 3.0, device=device), torch.full_like(k, 3.0, device=device)
    ops.rope_backward(dq, dk, dev(q, device), dev(k, device), dev(cos, device), dev(sin, device), None,
                      ops.RopeOptions(rotary, off))
    assert_close(dq, gq, TOL[dtype], "rope dq")
    assert_close(dk, gk, TOL[dtype], "rope dk")

    rows, inter = int(rng.integers(1, 700)), int(rng.integers(1, 500))
    print(f"swiglu rows={rows} inter={inter}", flush=True)
    gate, up, dy = randn((rows, inter), dtype, seed + 2, 2.0), randn((rows, inter), dtype, seed + 3), randn((rows, inter), dtype, seed + 4)
    dg64, du64 = oracle64.swiglu_backward(to_np(dy), to_np(gate), to_np(up))
    dg, du = torch.empty_like(gate, device=device), torch.empty_like(up, device=device)
    ops.swiglu_backward(dg, du, dev(dy, device), dev(gate, device), dev(up, device))
    assert_close(dg, dg64, TOL[dtype], "dgate")
    assert_close(du, du64, TOL[dtype], "dup")
    packed = torch.cat([gate, up], dim=1).contiguous()
    dpacked = torch.empty_like(packed, device=device)
    ops.swiglu_backward_packed(dpacked, dev(dy, device), dev(packed, device))
    assert_close(dpacked[:, :inter], dg64, TOL[dtype], "packed dgate")
    assert_close(dpacked[:, inter:], du64, TOL[dtype], "packed dup")


@pytest.mark.parametrize("seed", SEEDS)
def test_linear_backward_random_shapes(device, seed):
    rng = np.random.default_rng(3000 + seed)
    dtype = case_dtype(rng)
    aligned = bool(rng.integers(0, 2))  # multiples of 32 take the matrix-core kernels in 16-bit storage
    rows, fin, fout = (int(rng.integers(1, 40)) * 32 if aligned else int(rng.integers(1, 900)) for _ in range(3))
    accumulate = bool(rng.integers(0, 2))
    print(f"linear rows={rows} in={fin} out={fout} accumulate={accumulate} {dtype}", flush=True)
    x, w, dy = randn((rows, fin), dtype, seed), randn((fout, fin), dtype, seed + 1, 0.1), randn((rows, fout), dtype, seed + 2)
    dx64, dw64, db64 = oracle64.linear_backward(to_np(dy), to_np(x), to_np(w))
    base_x, base_w, base_b = randn((rows, fin), dtype, seed + 3), randn((fout, fin), dtype, seed + 4), randn((fout,), dtype, seed + 5)
    gi, gw, gb = dev(base_x, device).clone(), dev(base_w, device).clone(), dev(base_b, device).clone()
    options = ops.LinearBackwardOptions(accumulate_input=accumulate, accumulate_weight=accumulate, accumulate_bias=accumulate)
    ops.linear_backward(gi, gw, gb, dev(dy, device), dev(x, device), dev(w, device), None, None, options)
    if accumulate:
        dx64, dw64, db64 = dx64 + to_np(base_x), dw64 + to_np(base_w), db64 + to_np(base_b)
    assert_scaled_close(gi, dx64, STOL[dtype], "dX")
    assert_scaled_close(gw, dw64, STOL[dtype], "dW")
    assert_scaled_close(gb, db64, STOL[dtype], "db")
    y = torch.empty(rows, fout, dtype=dtype, device=device)
    ops.linear_forward(y, dev(x, device), dev(w, device))
    assert_scaled_close(y, oracle64.linear_forward(to_np(x), to_np(w)), STOL[dtype], "Y")


@pytest.mark.parametrize("seed", SEEDS[:24])
def test_stacked_weight_gradients_random_shapes(device, seed):
    """Weight gradients of several layers in one call: tile-aligned shapes take the stacked launch (any number of
    K slices and rounds), the others one weight gradient per layer; layers may be slices of larger blocks."""
    rng = np.random.default_rng(8000 + seed)
    dtype = case_dtype(rng)
    aligned = bool(rng.integers(0, 4))
    count = int(rng.integers(1, 7))
    if aligned:
        rows, fin, fout = int(rng.integers(1, 60)) * 32, int(rng.integers(1, 40)) * 8, int(rng.integers(1, 5)) * 256
    else:
        rows, fin, fout = (int(rng.integers(1, 500)) for _ in range(3))
    extra_rows = int(rng.integers(0, 3)) * 8  # rows of the block a layer is a slice of, beyond the layer's own
    print(f"stacked dW count={count} rows={rows} in={fin} out={fout} extra_rows={extra_rows} {dtype}", flush=True)
    dy_block = randn((count, rows + extra_rows, fout), dtype, seed).to(device)
    x_block = randn((count, rows + extra_rows, fin), dtype, seed + 1).to(device)
    dy, x = dy_block[:, :rows], x_block[:, :rows]
    gw = torch.full((count, fout, fin), 5.0, dtype=dtype, device=device)
    ops.linear_backward_weights_stacked(gw, dy, x)
    for j in range(count):
        assert_scaled_close(gw[j], to_np(dy[j]).T @ to_np(x[j]), STOL[dtype], f"dW of layer {j}")


@pytest.mark.parametrize("seed", SEEDS)
def test_attention_random_shapes(device, seed):
    rng = np.random.default_rng(4000 + seed)
    dtype = case_dtype(rng)
    hkv = int(rng.integers(1, 4))
    hq = hkv * int(rng.integers(1, 5))
    d = pick(rng, [8 * int(rng.integers(1, 17)), 64, 128, int(rng.integers(1, 129))])
    b, qs = int(rng.integers(1, 3)), int(rng.integers(1, 200))
    causal = bool(rng.integers(0, 4))
    off = int(rng.integers(0, 40)) if causal else 0
    ks = qs + off + (int(rng.integers(0, 30)) if causal else int(rng.integers(0, 150)))
    scale = pick(rng, [0.0, 0.0, 0.3])
    with_lse, accumulate = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    print(f"attention b={b} qs={qs} ks={ks} {hq}:{hkv} d={d} causal={causal} off={off} scale={scale} lse={with_lse} "
          f"accumulate={accumulate} {dtype}", flush=True)
    q, k, v = randn((b, qs, hq, d), dtype, seed), randn((b, ks, hkv, d), dtype, seed + 1), randn((b, ks, hkv, d), dtype, seed + 2)
    do = randn((b, qs, hq, d), dtype, seed + 3)
    opt = ops.FlashAttentionOptions(hq, hkv, d, scale, causal, off)
    o64, lse64 = oracle64.attention_forward(to_np(q), to_np(k), to_np(v), hq, hkv, d, scale, causal, off)
    want = oracle64.attention_backward(to_np(do), to_np(q), to_np(k), to_np(v), hq, hkv, d, scale, causal, off)
    out, lse = torch.empty_like(q, device=device), torch.empty(b, qs, hq, device=device)
    dq_, dk_, dv_, ddo = dev(q, device), dev(k, device), dev(v, device), dev(do, device)
    ops.flash_gqa_attention_forward_with_lse(out, lse, dq_, dk_, dv_, None, opt)
    assert_close(out, o64, TOL[dtype], "O")
    assert_close(lse, lse64, 1e-3 if dtype != torch.float32 else 1e-4, "LSE")
    base = [randn(t.shape, dtype, seed + 4 + i) for i, t in enumerate((q, k, v))]
    grads = [dev(t, device).clone() for t in base]
    if with_lse:
        ops.flash_gqa_attention_backward_with_lse(*grads, ddo, out, lse, dq_, dk_, dv_, None, opt, accumulate)
    else:
        ops.flash_gqa_attention_backward(*grads, ddo, dq_, dk_, dv_, None, opt, accumulate)
    for g, w, bs, name in zip(grads, want, base, ("dQ", "dK", "dV")):
        assert_scaled_close(g, w + to_np(bs) if accumulate else w, STOL[dtype], name)


@pytest.mark.parametrize("seed", SEEDS)
def test_embedding_and_cross_entropy_random_shapes(device, seed):
    rng = np.random.default_rng(5000 + seed)
    dtype = case_dtype(rng)
    tokens = pick(rng, [int(rng.integers(1, 300)), int(rng.integers(3000, 6000))])  # both sides of the sort-free limit
    vocab, hidden = int(rng.integers(1, 400)), int(rng.integers(1, 200))
    accumulate = bool(rng.integers(0, 2))
    print(f"embedding tokens={tokens} vocab={vocab} hidden={hidden} accumulate={accumulate} {dtype}", flush=True)
    ids = randint(vocab + 2, (tokens,), seed)  # two ids out of range
    dy, gw = randn((tokens, hidden), dtype, seed + 1), randn((vocab, hidden), dtype, seed + 2)
    dgw = dev(gw, device).clone()
    cpu_ops.embedding_backward(gw, dy, ids, True, accumulate)
    ops.embedding_backward(dgw, dev(dy, device), dev(ids, device), tokens, None,
                           ops.EmbeddingBackwardOptions(accumulate_weight=accumulate))
    assert torch.equal(dgw.cpu(), gw)

    rows = int(rng.integers(1, 40))
    width = pick(rng, [int(rng.integers(2, 3000)), 8 * int(rng.integers(1, 2000)), 32000, 50257])
    scale = pick(rng, [1.0, 1024.0])
    print(f"cross entropy rows={rows} vocab={width} scale={scale}", flush=True)
    logits = randn((rows, width), dtype, seed + 3, 3.0)
    targets = randint(width + 1, (rows,), seed + 4)  # an occasional target out of range
    l64, g64 = oracle64.cross_entropy(to_np(logits), targets.numpy(), scale)
    loss, grad = torch.zeros(1, device=device), torch.empty_like(logits, device=device)
    ops.cross_entropy_forward_backward(loss, grad, dev(logits, device), dev(targets, device), rows, None, scale)
    assert abs(loss.item() - l64) <= 1e-4 * max(1.0, abs(l64))
    assert_close(grad, g64, TOL[dtype], "gradient")

    crows, chidden, cvocab = int(rng.integers(1, 300)), int(rng.integers(1, 200)), int(rng.integers(2, 600))
    print(f"cut cross entropy rows={crows} hidden={chidden} vocab={cvocab}", flush=True)
    x, c = randn((crows, chidden), dtype, seed + 5), randn((cvocab, chidden), dtype, seed + 6, 0.05)
    ctargets = randint(cvocab, (crows,), seed + 7)
    cl64, dx64, dc64 = oracle64.cut_cross_entropy(to_np(x), to_np(c), ctargets.numpy(), scale)
    closs, dx, dc = torch.zeros(1, device=device), torch.empty_like(x, device=device), torch.empty_like(c, device=device)
    ops.cut_cross_entropy_forward_backward(closs, dx, dc, dev(x, device), dev(c, device), dev(ctargets, device), crows, None, scale)
    assert abs(closs.item() - cl64) <= (1e-4 if dtype == torch.float32 else 5e-3) * max(1.0, cl64)
    assert_scaled_close(dx, dx64, STOL[dtype], "dX")
    assert_scaled_close(dc, dc64, STOL[dtype], "dC")


@pytest.mark.parametrize("seed", SEEDS[:16])
def test_adamw_many_random_tensor_lists(device, seed):
    """Random lists of 1 to 12 tensors of 1 to 40000 elements each (mixed storage dtypes within a list), random
    hyper-parameters, clipping on or off, three steps of which one may carry a non-finite gradient (skipped as a
    whole: no tensor changes, the step counter stays), against the float64 update of src/optim/adamw.cu:148-187."""
    rng = np.random.default_rng(6000 + seed)
    count = int(rng.integers(1, 13))
    sizes = [int(rng.integers(1, 40000)) if rng.integers(0, 4) else int(rng.integers(1, 9)) for _ in range(count)]
    dtypes = [DTYPES[int(rng.integers(0, 3))] for _ in range(count)]
    lr, wd = float(10 ** rng.uniform(-4, -2)), float(rng.uniform(0, 0.2))
    beta1, beta2 = float(rng.uniform(0.8, 0.95)), float(rng.uniform(0.9, 0.999))
    loss_scale = float(pick(rng, [1.0, 64.0, 1024.0]))
    max_norm = float(pick(rng, [float("inf"), 1.0, 0.05]))
    bad_step = int(rng.integers(0, 6))  # 0..2: that step's gradients hold an Inf or NaN somewhere
    print(f"adamw sizes={sizes} lr={lr:.2e} wd={wd:.3f} betas=({beta1:.3f},{beta2:.4f}) scale={loss_scale} "
          f"max_norm={max_norm} bad_step={bad_step}", flush=True)
    params = [randn((n,), t, seed * 100 + i, 0.5) for i, (n, t) in enumerate(zip(sizes, dtypes))]
    d_params = [dev(p, device).clone() for p in params]
    states = [ops.AdamWState.for_parameter(p) for p in d_params]
    d_grads = [torch.empty_like(p) for p in d_params]
    entries = [ops.AdamWBatchEntry(p, g, s) for p, g, s in zip(d_params, d_grads, states)]
    ws = ops.AdamWWorkspace()
    options = ops.AdamWOptions(learning_rate=lr, beta1=beta1, beta2=beta2, epsilon=1e-8, weight_decay=wd,
                               loss_scale=loss_scale, max_grad_norm=max_norm)
    masters = [to_np(p) for p in params]
    ms, vs, step = [np.zeros(n) for n in sizes], [np.zeros(n) for n in sizes], 0
    for it in range(3):
        grads = [randn((n,), t, seed * 1000 + 10 * it + i, loss_scale * 0.02) for i, (n, t) in enumerate(zip(sizes, dtypes))]
        if it == bad_step:
            victim = int(rng.integers(0, count))
            grads[victim][int(rng.integers(0, sizes[victim]))] = float("inf") if rng.integers(0, 2) else float("nan")
        for dg, g in zip(d_grads, grads):
            dg.copy_(g)
        ops.adamw_step_many_async(entries, options, ws)
        ok, masters, ms, vs, step = oracle64.adamw(None, [to_np(g) for g in grads], masters, ms, vs, step, lr, beta1, beta2,
                                                   1e-8, wd, loss_scale, max_norm)
        assert ops.adamw_check(ws) == ok
        assert states[0].step == step
    for p, s, m64, mm, vv, t in zip(d_params, states, masters, ms, vs, dtypes):
        assert_close(s.master_parameter, m64, 1e-5, "master")
        assert_close(s.first_moment, mm, 1e-5, "m")
        assert np.abs(to_np(s.second_moment) - vv).max() <= 1e-5 * max(1e-12, np.abs(vv).max()) + 1e-12
        assert torch.equal(p, s.master_parameter.to(t))
