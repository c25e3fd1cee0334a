"""Pins both CPU checkers (oracle/cgpt_cpu_ops.c and oracle/oracle64.py) before
anything is compared with them.

Sources of truth used here, none of which is the checker's own formula:
  * literal known-answer vectors held by the reference's tests (cited per test);
  * central finite differences of the *forward* definition in float64, which
    catch a dropped term, a wrong sign or a transposed operand in a backward;
  * algebraic identities (inverse rotation undoes rotation, rows of dS sum to
    zero, accumulate = overwrite + previous, causal visibility counts).
"""
import math

import numpy as np
import pytest
import torch

from oracle import cpu_ops, oracle64
from tests.util import DTYPES, DTYPE_IDS, assert_close, randn, to_np

F32 = torch.float32


def t(values, shape, dtype=F32):
    return torch.tensor(values, dtype=torch.float32).reshape(shape).to(dtype).contiguous()


def fd_grad(f, x, eps=1e-6):
    """Central finite differences of scalar f at float64 array x."""
    g = np.zeros_like(x)
    flat, gflat = x.reshape(-1), g.reshape(-1)
    for i in range(flat.size):
        old = flat[i]
        flat[i] = old + eps
        hi = f(x)
        flat[i] = old - eps
        lo = f(x)
        flat[i] = old
        gflat[i] = (hi - lo) / (2 * eps)
    return g


# ------------------------------------------------------------------------ RMSNorm
def test_rmsnorm_backward_matches_finite_differences_of_forward():
    rng = np.random.default_rng(1)
    x, w, dy = rng.normal(size=(3, 7)), rng.normal(size=7), rng.normal(size=(3, 7))
    eps = 1e-5

    def fwd(xv, wv):  # definition of the op: include/ops/rmsnorm.h
        return xv / np.sqrt((xv * xv).mean(axis=1, keepdims=True) + eps) * wv

    dx_fd = fd_grad(lambda xv: (fwd(xv, w) * dy).sum(), x.copy())
    dw_fd = fd_grad(lambda wv: (fwd(x, wv) * dy).sum(), w.copy())
    dx, dw = oracle64.rmsnorm_backward(dy, x, w, eps)
    np.testing.assert_allclose(dx, dx_fd, atol=1e-7)
    np.testing.assert_allclose(dw, dw_fd, atol=1e-7)
    np.testing.assert_allclose(oracle64.rmsnorm_forward(x, w, eps), fwd(x, w), atol=1e-12)
    # float32 restatement against the pinned float64 one
    gi, gw = torch.empty(3, 7), torch.empty(7)
    cpu_ops.rmsnorm_backward(gi, gw, t(dy, (3, 7)), t(x, (3, 7)), t(w, (7,)), eps)
    assert_close(gi, dx, 1e-5, "dx")
    assert_close(gw, dw, 1e-5, "dw")


@pytest.mark.parametrize("rows,hidden,dtype,tol", [(3, 7, torch.float32, 2e-4), (2, 4096, torch.float16, 5e-3),
                                                   (129, 513, torch.bfloat16, 2.5e-1)])
def test_rmsnorm_backward_reference_test_cases(rows, hidden, dtype, tol):
    """Inputs and tolerances of tests/rmsnorm_test.cu:268-322, 412-415."""
    idx = np.arange(rows * hidden)
    x = 0.125 * ((idx % 13) - 6).astype(np.float64)
    dy = 0.25 * ((idx % 9) - 4).astype(np.float64)
    w = 0.5 + 0.125 * np.arange(hidden)
    xt, dyt, wt = t(x, (rows, hidden), dtype), t(dy, (rows, hidden), dtype), t(w, (hidden,), dtype)
    dx, dw = oracle64.rmsnorm_backward(to_np(dyt), to_np(xt), to_np(wt), 1e-5)
    gi, gw = torch.empty_like(xt), torch.empty_like(wt)
    cpu_ops.rmsnorm_backward(gi, gw, dyt, xt, wt, 1e-5)
    # the reference test scales its tolerance by max(1, |expected|) (tests/rmsnorm_test.cu:80-85)
    assert_close(gi, dx, tol, "dx")
    assert_close(gw, dw, tol, "dw")


# --------------------------------------------------------------------------- RoPE
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.float16, 3e-3), (torch.bfloat16, 2e-2)])
def test_rope_backward_known_answer(dtype, tol):
    """tests/rope_test.cu:99-127: cos/sin in {0,1}, rotary_dim 2 of head_dim 4."""
    q = t([1, 2, 30, 40, 3, 4, 50, 60, 5, 6, 70, 80, 7, 8, 90, 100], (1, 2, 2, 4), dtype)
    k = t([1, -2, 30, 40, 5, -6, 70, 80], (1, 2, 1, 4), dtype)
    cos, sin = t([1, 0], (2, 1), dtype), t([0, 1], (2, 1), dtype)
    want_q = [1, 2, 30, 40, 3, 4, 50, 60, 6, -5, 70, 80, 8, -7, 90, 100]
    want_k = [1, -2, 30, 40, -6, -5, 70, 80]
    gq, gk = torch.empty_like(q), torch.empty_like(k)
    cpu_ops.rope_backward(gq, gk, q, k, cos, sin, rotary_dim=2)
    assert np.abs(to_np(gq).reshape(-1) - want_q).max() <= tol
    assert np.abs(to_np(gk).reshape(-1) - want_k).max() <= tol
    assert np.abs(oracle64.rope_backward(to_np(q), to_np(cos), to_np(sin), 2).reshape(-1) - want_q).max() <= tol
    assert np.abs(oracle64.rope_backward(to_np(k), to_np(cos), to_np(sin), 2).reshape(-1) - want_k).max() <= tol


def test_rope_backward_inverts_forward_and_uses_position_offset():
    rng = np.random.default_rng(2)
    x = rng.normal(size=(2, 5, 3, 8))
    theta = rng.uniform(0, 6.28, size=(9, 3))
    cos, sin = np.cos(theta), np.sin(theta)
    y = oracle64.rope_forward(x, cos, sin, rotary_dim=6, position_offset=4)
    np.testing.assert_allclose(oracle64.rope_backward(y, cos, sin, rotary_dim=6, position_offset=4), x, atol=1e-12)
    # offset really selects rows 4.. of the cache
    y0 = oracle64.rope_forward(x, cos[4:], sin[4:], rotary_dim=6, position_offset=0)
    np.testing.assert_allclose(y, y0, atol=0)
    # float32 restatement: forward then backward returns the input
    q, k = t(x, x.shape), t(x[:, :, :1], (2, 5, 1, 8))
    c32, s32 = t(cos, cos.shape), t(sin, sin.shape)
    q2, k2 = q.clone(), k.clone()
    cpu_ops.rope_forward(q2, k2, c32, s32, rotary_dim=6, position_offset=4)
    assert_close(q2, y, 1e-5, "rope forward")
    gq, gk = torch.empty_like(q), torch.empty_like(k)
    cpu_ops.rope_backward(gq, gk, q2, k2, c32, s32, rotary_dim=6, position_offset=4)
    assert_close(gq, x, 1e-5, "rope roundtrip q")
    assert_close(gk, x[:, :, :1], 1e-5, "rope roundtrip k")


# ------------------------------------------------------------------------- SwiGLU
def test_swiglu_backward_matches_finite_differences_of_forward():
    rng = np.random.default_rng(3)
    g, u, dy = rng.normal(size=17) * 3, rng.normal(size=17), rng.normal(size=17)

    def fwd(gv, uv):  # include/ops/swiglu.h: silu(gate) * up
        return gv / (1 + np.exp(-gv)) * uv

    dg_fd = fd_grad(lambda gv: (fwd(gv, u) * dy).sum(), g.copy())
    du_fd = fd_grad(lambda uv: (fwd(g, uv) * dy).sum(), u.copy())
    dg, du = oracle64.swiglu_backward(dy, g, u)
    np.testing.assert_allclose(dg, dg_fd, atol=1e-7)
    np.testing.assert_allclose(du, du_fd, atol=1e-7)
    gg, gu = torch.empty(17), torch.empty(17)
    cpu_ops.swiglu_backward(gg, gu, t(dy, (17,)), t(g, (17,)), t(u, (17,)))
    assert_close(gg, dg, 1e-5, "dgate")
    assert_close(gu, du, 1e-5, "dup")
    # accumulate = overwrite + previous; packed layout = separate layout
    prev_g, prev_u = gg.clone(), gu.clone()
    cpu_ops.swiglu_backward(gg, gu, t(dy, (17,)), t(g, (17,)), t(u, (17,)), True, True)
    assert_close(gg, 2 * to_np(prev_g), 1e-6, "accumulate gate")
    assert_close(gu, 2 * to_np(prev_u), 1e-6, "accumulate up")
    packed = torch.cat([t(g, (1, 17)), t(u, (1, 17))], dim=1).contiguous()
    out = torch.empty(1, 34)
    cpu_ops.swiglu_backward_packed(out, t(dy, (1, 17)), packed)
    assert_close(out[0, :17], to_np(prev_g), 1e-6, "packed gate")
    assert_close(out[0, 17:], to_np(prev_u), 1e-6, "packed up")


# ------------------------------------------------------------------------- Linear
def test_linear_backward_known_answer_and_accumulation():
    """tests/linear_backward_test.cu:20-45."""
    x, w, dy = t([1, 2, 3, 4, 5, 6], (2, 3)), t([1, 0, 2, -1, 3, 1], (2, 3)), t([2, -1, 3, 4], (2, 2))
    gi, gw, gb = torch.empty(2, 3), torch.empty(2, 3), torch.empty(2)
    cpu_ops.linear_backward(gi, gw, gb, dy, x, w)
    assert gi.reshape(-1).tolist() == [3, -3, 3, -1, 12, 10]
    assert gw.reshape(-1).tolist() == [14, 19, 24, 15, 18, 21]
    assert gb.tolist() == [5, 3]
    cpu_ops.linear_backward(gi, gw, gb, dy, x, w, True, True, True)
    assert gi.reshape(-1).tolist() == [6, -6, 6, -2, 24, 20]
    assert gw.reshape(-1).tolist() == [28, 38, 48, 30, 36, 42]
    assert gb.tolist() == [10, 6]
    dx, dw, db = oracle64.linear_backward(to_np(dy), to_np(x), to_np(w))
    assert dx.reshape(-1).tolist() == [3, -3, 3, -1, 12, 10]
    assert dw.reshape(-1).tolist() == [14, 19, 24, 15, 18, 21]
    assert db.tolist() == [5, 3]


def test_linear_backward_batched_f16_known_answer():
    """tests/linear_backward_test.cu:47-58."""
    f16 = torch.float16
    x, w = t([1, 2, 3, 4, 5, 6, 7, 8], (2, 2, 2), f16), t([1, 2, 3, 4, 5, 6], (3, 2), f16)
    dy = t(list(range(1, 13)), (2, 2, 3), f16)
    gi, gw, gb = torch.empty_like(x), torch.empty_like(w), torch.empty(3, dtype=f16)
    cpu_ops.linear_backward(gi, gw, gb, dy, x, w)
    assert np.abs(to_np(gi).reshape(-1) - [22, 28, 49, 64, 76, 100, 103, 136]).max() <= 0.1
    assert np.abs(to_np(gw).reshape(-1) - [118, 140, 134, 160, 150, 180]).max() <= 0.2
    assert np.abs(to_np(gb) - [22, 26, 30]).max() <= 0.1


def test_linear_forward_is_x_times_w_transposed_plus_bias():
    x, w, b = randn((5, 19), F32, 1), randn((11, 19), F32, 2), randn((11,), F32, 3)
    y = torch.empty(5, 11)
    cpu_ops.linear_forward(y, x, w, b)
    assert_close(y, to_np(x) @ to_np(w).T + to_np(b), 1e-5, "linear forward")
    assert_close(y, oracle64.linear_forward(to_np(x), to_np(w), to_np(b)), 1e-5, "linear forward 64")


# ---------------------------------------------------------------------- Embedding
@pytest.mark.parametrize("dtype,tol", [(torch.float16, 1e-2), (torch.bfloat16, 5e-2)])
def test_embedding_backward_repeated_tokens_known_answer(dtype, tol):
    """tests/embedding_test.cu:183-203."""
    dy = t([1, 2, 3, 4, 0.5, 1.5, -1, 2, 7, 8, 9, 10], (3, 4), dtype)
    ids = torch.tensor([1, 1, 2], dtype=torch.int32)
    want = [0, 0, 0, 0, 1.5, 3.5, 2, 6, 7, 8, 9, 10]
    gw = torch.full((3, 4), 99.0).to(dtype)
    cpu_ops.embedding_backward(gw, dy, ids)
    assert np.abs(to_np(gw).reshape(-1) - want).max() <= tol
    assert np.abs(oracle64.embedding_backward(to_np(dy), ids.numpy(), 3).reshape(-1) - want).max() <= tol
    # accumulate keeps what was there; out-of-range ids are skipped
    gw2 = torch.ones(3, 4).to(dtype)
    cpu_ops.embedding_backward(gw2, dy, torch.tensor([1, 7, 2], dtype=torch.int32), accumulate_weight=True)
    want2 = np.ones((3, 4))
    want2[1] += [1, 2, 3, 4]
    want2[2] += [7, 8, 9, 10]
    assert np.abs(to_np(gw2) - want2).max() <= tol


# ------------------------------------------------------------------ Cross entropy
def test_cross_entropy_known_answers():
    """tests/cross_entropy_test.cu:33-56."""
    logits = t([1, 2, 3, 1, 1, 1], (2, 3))
    targets = torch.tensor([2, 0], dtype=torch.int32)
    want_loss = (math.log(math.exp(1) + math.exp(2) + math.exp(3)) - 3 + math.log(3)) / 2
    want_grad = [0.0450153, 0.1223642, -0.1673795, -0.3333333, 0.1666667, 0.1666667]
    loss, grad = torch.empty(1), torch.empty(2, 3)
    cpu_ops.cross_entropy_forward_backward(loss, grad, logits, targets)
    assert abs(loss.item() - want_loss) <= 1e-5
    assert np.abs(to_np(grad).reshape(-1) - want_grad).max() <= 1e-5
    l64, g64 = oracle64.cross_entropy(to_np(logits), targets.numpy())
    assert abs(l64 - want_loss) <= 1e-7 and np.abs(g64.reshape(-1) - want_grad).max() <= 1e-6
    only = torch.empty(1)
    cpu_ops.cross_entropy_forward(only, logits, targets)
    assert abs(only.item() - want_loss) <= 1e-5
    # gradient scale 1024 on two equal logits gives -512 / +512, loss unchanged
    loss, grad = torch.empty(1), torch.empty(1, 2)
    cpu_ops.cross_entropy_forward_backward(loss, grad, t([0, 0], (1, 2)), torch.tensor([0], dtype=torch.int32), 1024.0)
    assert abs(loss.item() - math.log(2)) <= 1e-6 and grad.reshape(-1).tolist() == [-512.0, 512.0]
    l64, g64 = oracle64.cross_entropy(np.zeros((1, 2)), np.array([0]), 1024.0)
    assert abs(l64 - math.log(2)) <= 1e-12 and g64.reshape(-1).tolist() == [-512.0, 512.0]


def test_cross_entropy_out_of_range_target_row():
    """Rows with target >= vocab add no loss but keep the softmax gradient (src/ops/cross_entropy.cu:209-232)."""
    logits = t([1, 2, 3, 1, 1, 1], (2, 3))
    targets = torch.tensor([2, 9], dtype=torch.int32)
    loss, grad = torch.empty(1), torch.empty(2, 3)
    cpu_ops.cross_entropy_forward_backward(loss, grad, logits, targets)
    assert abs(loss.item() - (math.log(math.exp(1) + math.exp(2) + math.exp(3)) - 3) / 2) <= 1e-5
    assert np.abs(to_np(grad)[1] - [1 / 6, 1 / 6, 1 / 6]).max() <= 1e-6
    l64, g64 = oracle64.cross_entropy(to_np(logits), targets.numpy())
    assert abs(l64 - loss.item()) <= 1e-5 and np.abs(g64 - to_np(grad)).max() <= 1e-6


def test_cut_cross_entropy_known_answer():
    """tests/cut_cross_entropy_test.cu:19-31."""
    x, c = np.array([[1, 2], [3, 4.0]]), np.array([[1, 0], [0, 1], [1, 1.0]])
    loss, dx, dc = oracle64.cut_cross_entropy(x, c, np.array([2, 0]))
    e = math.exp
    want_loss = (math.log(e(1) + e(2) + e(3)) - 3 + math.log(e(3) + e(4) + e(7)) - 3) / 2
    assert abs(loss - want_loss) <= 1e-9
    # Row 0 of dX and rows 0-1 of dC match the reference's constants within its tolerances (2e-5, 2e-3).
    assert np.abs(dx[0] - [-0.1223642, -0.0450153]).max() <= 2e-5
    assert np.abs(dc[:2].reshape(-1) - [-1.4295, -1.876, 0.193, 0.339]).max() <= 2e-3
    # Row 2 of dC in the reference test (1.7365, 2.537) equals Σ_r p_r2·x_r / rows WITHOUT the one-hot term of
    # row 0 (target 2), which the reference's kernel does subtract (src/ops/cut_cross_entropy.cu:137-146):
    # the constant and the kernel differ by x_0 / rows = (0.5, 1.0). The formula is followed, not the constant.
    assert np.abs(dc[2] + x[0] / 2 - [1.7365, 2.537]).max() <= 2e-3
    # Row 1 of dX: the constants in the reference test (-0.0234640, 0.4915309) are 1.6e-4 away from what the
    # reference's own kernels compute, (softmax(z)·C - C[target]) / rows with z = (3, 4, 7)
    # (src/ops/cut_cross_entropy.cu:118-135), so they are checked at 2e-4 and the value is pinned by
    # finite differences of the loss instead.
    assert np.abs(dx[1] - [-0.0234640, 0.4915309]).max() <= 2e-4
    tg = np.array([2, 0])
    np.testing.assert_allclose(dx, fd_grad(lambda a: oracle64.cut_cross_entropy(a, c, tg)[0], x.copy()), atol=1e-8)
    np.testing.assert_allclose(dc, fd_grad(lambda a: oracle64.cut_cross_entropy(x, a, tg)[0], c.copy()), atol=1e-8)


# ---------------------------------------------------------------------- Attention
def _values(count, phase):
    """Input pattern of tests/flash_attention_test.cu:176-183."""
    i = np.arange(count, dtype=np.float64)
    return 0.45 * np.sin(phase + i * 0.31) + 0.1 * np.cos(i * 0.17)


ATTENTION_CASES = [  # tests/flash_attention_test.cu:365-388
    dict(b=2, qs=3, ks=5, hq=4, hkv=2, d=32, off=2, scale=0.23),
    dict(b=1, qs=3, ks=35, hq=4, hkv=1, d=64, off=32, scale=0.11),
    dict(b=1, qs=3, ks=35, hq=4, hkv=1, d=128, off=32, scale=0.11),
]


def attention_case_inputs(c):
    q = _values(c["b"] * c["qs"] * c["hq"] * c["d"], 0.2).reshape(c["b"], c["qs"], c["hq"], c["d"])
    k = _values(c["b"] * c["ks"] * c["hkv"] * c["d"], 0.7).reshape(c["b"], c["ks"], c["hkv"], c["d"])
    v = _values(k.size, 1.4).reshape(k.shape)
    do = _values(q.size, 2.1).reshape(q.shape)
    return q, k, v, do


def test_attention_forward_definition_and_lse():
    c = ATTENTION_CASES[0]
    q, k, v, _ = attention_case_inputs(c)
    out, lse = oracle64.attention_forward(q, k, v, c["hq"], c["hkv"], c["d"], c["scale"], True, c["off"])
    # brute force from the definition, element by element
    g = c["hq"] // c["hkv"]
    for b in range(c["b"]):
        for i in range(c["qs"]):
            for h in range(c["hq"]):
                visible = c["off"] + i + 1
                s = np.array([c["scale"] * q[b, i, h] @ k[b, j, h // g] for j in range(visible)])
                p = np.exp(s - s.max())
                p /= p.sum()
                np.testing.assert_allclose(out[b, i, h], p @ v[b, :visible, h // g], atol=1e-12)
                np.testing.assert_allclose(lse[b, i, h], np.log(np.exp(s).sum()), atol=1e-12)
    o32, l32 = torch.empty(q.shape), torch.empty(q.shape[:3])
    cpu_ops.attention_forward(o32, l32, t(q, q.shape), t(k, k.shape), t(v, v.shape), c["hq"], c["hkv"], c["d"],
                              c["scale"], True, c["off"])
    assert_close(o32, out, 1e-5, "attention forward")
    assert_close(l32, lse, 1e-5, "lse")


@pytest.mark.parametrize("case", range(2))
def test_attention_backward_matches_finite_differences_of_forward(case):
    c = dict(ATTENTION_CASES[case])
    if case == 1:
        c.update(ks=9, off=6, d=8)  # keep the finite-difference loop small
    else:
        c.update(d=8)
    q, k, v, do = attention_case_inputs(c)

    def loss(qv, kv, vv):
        return (oracle64.attention_forward(qv, kv, vv, c["hq"], c["hkv"], c["d"], c["scale"], True, c["off"])[0]
                * do).sum()

    dq, dk, dv = oracle64.attention_backward(do, q, k, v, c["hq"], c["hkv"], c["d"], c["scale"], True, c["off"])
    np.testing.assert_allclose(dq, fd_grad(lambda a: loss(a, k, v), q.copy()), atol=2e-7)
    np.testing.assert_allclose(dk, fd_grad(lambda a: loss(q, a, v), k.copy()), atol=2e-7)
    np.testing.assert_allclose(dv, fd_grad(lambda a: loss(q, k, a), v.copy()), atol=2e-7)


@pytest.mark.parametrize("case", range(3))
def test_attention_backward_cpu_restatement_on_reference_cases(case):
    """Shapes, offsets, scales and the 3e-2 tolerance of tests/flash_attention_test.cu:310-388."""
    c = ATTENTION_CASES[case]
    q, k, v, do = attention_case_inputs(c)
    dq, dk, dv = oracle64.attention_backward(do, q, k, v, c["hq"], c["hkv"], c["d"], c["scale"], True, c["off"])
    for dtype, tol in ((torch.float32, 1e-5), (torch.float16, 3e-2)):
        qt, kt, vt, dot = (t(a, a.shape, dtype) for a in (q, k, v, do))
        gq, gk, gv = torch.empty_like(qt), torch.empty_like(kt), torch.empty_like(vt)
        cpu_ops.attention_backward(gq, gk, gv, dot, qt, kt, vt, c["hq"], c["hkv"], c["d"], c["scale"], True, c["off"])
        assert np.abs(to_np(gq) - dq).max() <= tol
        assert np.abs(to_np(gk) - dk).max() <= tol
        assert np.abs(to_np(gv) - dv).max() <= tol
    # keys beyond the causal horizon of the last query receive exactly zero gradient
    horizon = c["off"] + c["qs"]
    assert np.all(dk[:, horizon:] == 0) and np.all(dv[:, horizon:] == 0)


def test_attention_backward_accumulate_and_non_causal():
    c = dict(ATTENTION_CASES[0], d=16)
    q, k, v, do = attention_case_inputs(c)
    qt, kt, vt, dot = (t(a, a.shape) for a in (q, k, v, do))
    gq, gk, gv = torch.empty_like(qt), torch.empty_like(kt), torch.empty_like(vt)
    cpu_ops.attention_backward(gq, gk, gv, dot, qt, kt, vt, 4, 2, 16, 0.0, False, 0)
    dq, dk, dv = oracle64.attention_backward(do, q, k, v, 4, 2, 16, 0.0, False, 0)  # scale 0 -> 1/sqrt(d)
    assert_close(gq, dq, 1e-5, "dq non-causal")
    assert_close(gk, dk, 1e-5, "dk non-causal")
    first = (gq.clone(), gk.clone(), gv.clone())
    cpu_ops.attention_backward(gq, gk, gv, dot, qt, kt, vt, 4, 2, 16, 0.0, False, 0, accumulate_grads=True)
    for got, base in zip((gq, gk, gv), first):
        assert_close(got, 2 * to_np(base), 1e-5, "accumulate")


# -------------------------------------------------------------------------- AdamW
@pytest.mark.parametrize("parallel", [False, True])
def test_adamw_known_answers(parallel):
    """tests/adamw_test.cu:21-57."""
    p, g = t([1, -2], (2,)), t([0.1, -0.2], (2,))
    master, m, v = p.clone(), torch.zeros(2), torch.zeros(2)
    kw = dict(learning_rate=0.1, beta1=0.9, beta2=0.999, epsilon=1e-8, weight_decay=0.01, parallel=parallel)
    assert cpu_ops.adamw(p, g, master, m, v, 1, **kw)
    assert np.abs(to_np(p) - [0.899, -1.898]).max() <= 2e-6
    assert np.abs(to_np(m) - [0.01, -0.02]).max() <= 2e-6
    assert np.abs(to_np(v) - [0.00001, 0.00004]).max() <= 2e-6
    assert cpu_ops.adamw(p, g, master, m, v, 2, **kw)
    assert np.abs(to_np(p) - [0.798101, -1.796102]).max() <= 2e-6
    # loss scale 4, clip to norm 1, then an infinite gradient is rejected untouched
    p, g = t([1, -1], (2,)), t([8, 0], (2,))
    master, m, v = p.clone(), torch.zeros(2), torch.zeros(2)
    kw = dict(learning_rate=0.1, weight_decay=0.0, loss_scale=4.0, max_grad_norm=1.0, parallel=parallel)
    assert cpu_ops.adamw(p, g, master, m, v, 1, **kw)
    assert np.abs(to_np(p) - [0.9, -1.0]).max() <= 2e-6
    before = (p.clone(), master.clone(), m.clone(), v.clone())
    assert not cpu_ops.adamw(p, t([float("inf"), 0], (2,)), master, m, v, 2, **kw)
    for got, want in zip((p, master, m, v), before):
        assert torch.equal(got, want)


def test_adamw_float64_statement_known_answers():
    ok, p, m, v, step = oracle64.adamw([None], [np.array([0.1, -0.2])], [np.array([1.0, -2.0])], [np.zeros(2)],
                                       [np.zeros(2)], 0, 0.1, 0.9, 0.999, 1e-8, 0.01, 1.0, float("inf"))
    assert ok and step == 1
    np.testing.assert_allclose(p[0], [0.899, -1.898], atol=2e-6)
    ok, p, m, v, step = oracle64.adamw([None], [np.array([0.1, -0.2])], p, m, v, step, 0.1, 0.9, 0.999, 1e-8, 0.01,
                                       1.0, float("inf"))
    np.testing.assert_allclose(p[0], [0.798101, -1.796102], atol=2e-6)
    ok, p, m, v, step = oracle64.adamw([None], [np.array([8.0, 0.0])], [np.array([1.0, -1.0])], [np.zeros(2)],
                                       [np.zeros(2)], 0, 0.1, 0.9, 0.999, 1e-8, 0.0, 4.0, 1.0)
    np.testing.assert_allclose(p[0], [0.9, -1.0], atol=2e-6)
    ok, *_ = oracle64.adamw([None], [np.array([np.inf, 0.0])], p, m, v, step, 0.1, 0.9, 0.999, 1e-8, 0.0, 4.0, 1.0)
    assert not ok


def test_storage_rounding_helpers():
    """BF16 store is round-to-nearest-even, F16 goes through F16C (every reference CPU op, e.g.
    src/ops/cpu/backward/rmsnorm_backward_cpu.cpp:27-58)."""
    x = torch.tensor([1.0 + 2**-8, 1.0 + 3 * 2**-8, 65519.0, 1e-8], dtype=torch.float32)
    for dtype in (torch.bfloat16, torch.float16):
        out = torch.empty(4, dtype=dtype)
        cpu_ops.add(out, x.to(torch.float32).to(dtype).to(dtype), torch.zeros(4, dtype=dtype))
        assert torch.equal(out, x.to(dtype))
    out = torch.empty(4, dtype=torch.bfloat16)
    # float32 inputs rounded by the C store: tie to even (1+2^-8 -> 1.0, 1+3*2^-8 -> 1+2^-6)
    a = torch.tensor([1.0, 1.0, 0, 0], dtype=torch.bfloat16)
    b = torch.tensor([2**-8, 3 * 2**-8, 0, 0], dtype=torch.bfloat16)
    cpu_ops.add(out, a, b)
    assert out[0].item() == 1.0 and out[1].item() == 1.0 + 2**-6
