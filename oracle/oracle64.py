"""Float64 numpy statement of the formulas on the training hot path.

TEST INFRASTRUCTURE — only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this module. Inputs are numpy arrays (any float
dtype; they are widened to float64), outputs are float64 arrays. No storage
rounding happens here: callers round to the storage dtype when they need to.

Every function cites the reference formula it states (paths relative to the
reference checkout) and is pinned in tests/test_oracle_pins.py against the
known-answer vectors of the reference's tests plus independent checks
(finite differences, closed forms, brute force).
"""
from __future__ import annotations

import numpy as np


def _f64(a):
    return np.asarray(a, dtype=np.float64)


# -- RMSNorm: src/ops/cpu/backward/rmsnorm_backward_cpu.cpp:86-133 ------------------
def rmsnorm_forward(x, w, eps):
    x, w = _f64(x), _f64(w)
    inv = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    return x * inv * w


def rmsnorm_backward(dy, x, w, eps):
    dy, x, w = _f64(dy), _f64(x), _f64(w)
    hidden = x.shape[-1]
    inv = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    corr = (dy * w * x).sum(axis=-1, keepdims=True) * inv**3 / hidden
    dx = dy * w * inv - x * corr
    dw = (dy * x * inv).reshape(-1, hidden).sum(axis=0)
    return dx, dw


# -- RoPE: src/ops/cpu/backward/rope_backward_cpu.cpp:110-141, rope_cpu.cpp:110-120 ---
def _rope(x, cos, sin, rotary_dim, position_offset, inverse):
    x, cos, sin = _f64(x), _f64(cos), _f64(sin)
    b, s, h, d = x.shape
    r = rotary_dim or d
    pos = position_offset + np.arange(s)
    c = cos[pos][None, :, None, :]  # [1, s, 1, r/2]
    sn = sin[pos][None, :, None, :]
    out = x.copy()
    even, odd = x[..., 0:r:2], x[..., 1:r:2]
    if inverse:
        out[..., 0:r:2] = even * c + odd * sn
        out[..., 1:r:2] = -even * sn + odd * c
    else:
        out[..., 0:r:2] = even * c - odd * sn
        out[..., 1:r:2] = even * sn + odd * c
    return out


def rope_forward(x, cos, sin, rotary_dim=0, position_offset=0):
    return _rope(x, cos, sin, rotary_dim, position_offset, False)


def rope_backward(dy, cos, sin, rotary_dim=0, position_offset=0):
    return _rope(dy, cos, sin, rotary_dim, position_offset, True)


# -- SwiGLU: src/ops/cpu/backward/swiglu_backward_cpu.cpp:92-141 -----------------------
def swiglu_forward(gate, up):
    gate, up = _f64(gate), _f64(up)
    return gate / (1.0 + np.exp(-gate)) * up


def swiglu_backward(dy, gate, up):
    dy, gate, up = _f64(dy), _f64(gate), _f64(up)
    s = 1.0 / (1.0 + np.exp(-gate))
    return dy * up * s * (1.0 + gate * (1.0 - s)), dy * gate * s


# -- Linear: src/ops/cpu/backward/linear_backward_cpu.cpp:131-165 ---------------------
def linear_forward(x, w, b=None):
    y = _f64(x).reshape(-1, w.shape[1]) @ _f64(w).T
    if b is not None:
        y = y + _f64(b)
    return y


def linear_backward(dy, x, w):
    dy2 = _f64(dy).reshape(-1, w.shape[0])
    x2 = _f64(x).reshape(-1, w.shape[1])
    return dy2 @ _f64(w), dy2.T @ x2, dy2.sum(axis=0)


# -- Embedding: src/ops/cpu/backward/embedding_backward_cpu.cpp:89-114 ----------------
def embedding_backward(dy, ids, vocab, base=None):
    dy = _f64(dy)
    hidden = dy.shape[-1]
    dw = np.zeros((vocab, hidden)) if base is None else _f64(base).copy()
    for t, i in enumerate(np.asarray(ids).reshape(-1)):
        if i < vocab:
            dw[i] += dy.reshape(-1, hidden)[t]
    return dw


# -- Cross entropy: src/ops/cpu/backward/cross_entropy_backward_cpu.cpp:122-148 --------
def cross_entropy(logits, targets, gradient_scale=1.0):
    z = _f64(logits)
    n, vocab = z.shape
    targets = np.asarray(targets).reshape(-1).astype(np.int64)
    mx = z.max(axis=1, keepdims=True)
    e = np.exp(z - mx)
    den = e.sum(axis=1, keepdims=True)
    lse = np.log(den) + mx
    valid = targets < vocab
    safe = np.where(valid, targets, 0)
    loss = ((lse[:, 0] - z[np.arange(n), safe]) * valid).sum() / n
    grad = e / den
    grad[np.arange(n)[valid], targets[valid]] -= 1.0
    return loss, grad * (gradient_scale / n)


# -- Cut cross-entropy: src/ops/cut_cross_entropy.cu:97-160 (semantics only) -----------
def cut_cross_entropy(x, c, targets, gradient_scale=1.0):
    x, c = _f64(x), _f64(c)
    loss, dz = cross_entropy(x @ c.T, targets, gradient_scale)
    return loss, dz @ c, dz.T @ x


# -- Attention: src/ops/cpu/backward/attention_backward_cpu.cpp:206-280 ----------------
def _scores(q, k, h, kv, scale, causal, off):
    # q [QS, D], k [KS, D]
    s = (q @ k.T) * scale
    if causal:
        qs, ks = s.shape
        mask = np.arange(ks)[None, :] > (off + np.arange(qs))[:, None]
        s = np.where(mask, -np.inf, s)
    return s


def attention_forward(q, k, v, num_query_heads, num_kv_heads, head_dim, attention_scale=0.0, causal=True,
                      query_position_offset=0):
    q, k, v = _f64(q), _f64(k), _f64(v)
    b, qs = q.shape[:2]
    scale = attention_scale if attention_scale > 0 else 1.0 / np.sqrt(head_dim)
    group = num_query_heads // num_kv_heads
    out = np.zeros_like(q)
    lse = np.zeros((b, qs, num_query_heads))
    for bi in range(b):
        for h in range(num_query_heads):
            kv = h // group
            s = _scores(q[bi, :, h], k[bi, :, kv], h, kv, scale, causal, query_position_offset)
            mx = s.max(axis=1, keepdims=True)
            e = np.exp(s - mx)
            den = e.sum(axis=1, keepdims=True)
            out[bi, :, h] = (e / den) @ v[bi, :, kv]
            lse[bi, :, h] = (np.log(den) + mx)[:, 0]
    return out, lse


def attention_backward(do, q, k, v, num_query_heads, num_kv_heads, head_dim, attention_scale=0.0, causal=True,
                       query_position_offset=0):
    do, q, k, v = _f64(do), _f64(q), _f64(k), _f64(v)
    b = q.shape[0]
    scale = attention_scale if attention_scale > 0 else 1.0 / np.sqrt(head_dim)
    group = num_query_heads // num_kv_heads
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    for bi in range(b):
        for h in range(num_query_heads):
            kv = h // group
            s = _scores(q[bi, :, h], k[bi, :, kv], h, kv, scale, causal, query_position_offset)
            mx = s.max(axis=1, keepdims=True)
            e = np.exp(s - mx)
            p = e / e.sum(axis=1, keepdims=True)
            dp = do[bi, :, h] @ v[bi, :, kv].T
            delta = (p * dp).sum(axis=1, keepdims=True)
            ds = p * (dp - delta)
            dq[bi, :, h] = scale * ds @ k[bi, :, kv]
            dk[bi, :, kv] += scale * ds.T @ q[bi, :, h]
            dv[bi, :, kv] += p.T @ do[bi, :, h]
    return dq, dk, dv


# -- AdamW: src/optim/adamw.cu:148-187 (batched, global norm) and 193-225 -------------
def adamw(params, grads, masters, ms, vs, step, lr, beta1, beta2, eps, wd, loss_scale, max_grad_norm):
    """One global-norm update over lists of arrays. Returns (applied, new masters, ms, vs, step)."""
    grads = [_f64(g) / loss_scale for g in grads]
    if not all(np.isfinite(g).all() for g in grads):
        return False, [_f64(p) for p in masters], [_f64(m) for m in ms], [_f64(v) for v in vs], step
    norm = np.sqrt(sum((g * g).sum() for g in grads))
    clip = max_grad_norm / norm if norm > max_grad_norm else 1.0
    step += 1
    bc1, bc2 = 1.0 - beta1**step, 1.0 - beta2**step
    out_p, out_m, out_v = [], [], []
    for g, p, m, v in zip(grads, masters, ms, vs):
        g = g * clip
        m = beta1 * _f64(m) + (1 - beta1) * g
        v = beta2 * _f64(v) + (1 - beta2) * g * g
        p = _f64(p) * (1 - lr * wd) - lr * (m / bc1) / (np.sqrt(v / bc2) + eps)
        out_p.append(p)
        out_m.append(m)
        out_v.append(v)
    return True, out_p, out_m, out_v, step
