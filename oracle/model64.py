"""Float64 statement of the whole train step (forward, loss, backward) of the reference's
decoder, composed from oracle64's operator formulas in the reference's order.

TEST INFRASTRUCTURE — only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
may import this module.

Order of operations: forward src/core/transformer_model.cu:195-241 and
src/core/transformer_block.cu:405-611; backward src/core/transformer_model.cu:336-381 and
src/core/transformer_block.cu:644-748. `rnd` models the rounding of every operator output
to the storage dtype (identity for a pure float64 run). The composition itself is pinned
in tests/test_oracle_pins.py by central finite differences of the loss on a tiny model.
"""
from __future__ import annotations

import numpy as np

from oracle import oracle64 as o

LAYER_KEYS = ("attention_norm", "q", "k", "q_norm", "k_norm", "v", "o", "ffn_norm", "gate", "up", "down")


def rope_cache(sequence, rotary_dim, base=10000.0):
    """train/train.cpp:322-333, computed in float32 like there."""
    pos = np.arange(sequence, dtype=np.float32)[:, None]
    i = np.arange(rotary_dim // 2, dtype=np.float32)[None, :]
    theta = pos / np.power(np.float32(base), np.float32(2.0) * i / np.float32(rotary_dim))
    return np.cos(theta).astype(np.float32), np.sin(theta).astype(np.float32)


def forward_backward(params, tokens, targets, cfg, loss_scale=1.0, rnd=lambda a: a, cos=None, sin=None):
    """params: {"embedding": [V,H], "final_norm": [H], "layers": [{key: array}]} (float64 arrays).
    Returns (loss, grads with the same structure, saved dict)."""
    B, T = tokens.shape
    H, HQ, HKV, D = cfg["hidden"], cfg["hq"], cfg["hkv"], cfg["d"]
    eps, rotary = cfg["eps"], cfg.get("rotary", 0) or cfg["d"]
    N = B * T
    if cos is None:
        cos, sin = rope_cache(T, rotary, cfg.get("rope_base", 10000.0))
        cos, sin = rnd(cos.astype(np.float64)), rnd(sin.astype(np.float64))
    E = params["embedding"]
    V = E.shape[0]
    ids = tokens.reshape(-1)
    x = np.where((ids < V)[:, None], E[np.minimum(ids, V - 1)], 0.0)
    saved = []
    hidden = [x]
    for w in params["layers"]:
        s = {}
        s["norm_a"] = rnd(o.rmsnorm_forward(x, w["attention_norm"], eps))
        s["q_pre"] = rnd(o.linear_forward(s["norm_a"], w["q"]))
        s["k_pre"] = rnd(o.linear_forward(s["norm_a"], w["k"]))
        s["v"] = rnd(o.linear_forward(s["norm_a"], w["v"])).reshape(B, T, HKV, D)
        qn = rnd(o.rmsnorm_forward(s["q_pre"].reshape(N * HQ, D), w["q_norm"], eps)).reshape(B, T, HQ, D)
        kn = rnd(o.rmsnorm_forward(s["k_pre"].reshape(N * HKV, D), w["k_norm"], eps)).reshape(B, T, HKV, D)
        s["q"] = rnd(o.rope_forward(qn, cos, sin, rotary))
        s["k"] = rnd(o.rope_forward(kn, cos, sin, rotary))
        attn, _ = o.attention_forward(s["q"], s["k"], s["v"], HQ, HKV, D)
        s["attn_out"] = rnd(attn).reshape(N, HQ * D)
        attn_proj = rnd(o.linear_forward(s["attn_out"], w["o"]))
        s["norm_f"] = rnd(o.rmsnorm_forward(x, w["ffn_norm"], eps))
        s["gate"] = rnd(o.linear_forward(s["norm_f"], w["gate"]))
        s["up"] = rnd(o.linear_forward(s["norm_f"], w["up"]))
        s["act"] = rnd(o.swiglu_forward(s["gate"], s["up"]))
        ffn = rnd(o.linear_forward(s["act"], w["down"]))
        out = rnd(rnd(x + attn_proj) + ffn)
        s["x"] = x
        saved.append(s)
        x = out
        hidden.append(x)
    normalized = rnd(o.rmsnorm_forward(x, params["final_norm"], eps))
    logits = rnd(o.linear_forward(normalized, E))
    loss, dlogits = o.cross_entropy(logits, targets.reshape(-1), loss_scale)
    dlogits = rnd(dlogits)

    grads = {"layers": []}
    d_normalized, dE, _ = o.linear_backward(dlogits, normalized, E)
    d_normalized, dE = rnd(d_normalized), rnd(dE)
    cur, grads["final_norm"] = o.rmsnorm_backward(d_normalized, x, params["final_norm"], eps)
    cur, grads["final_norm"] = rnd(cur), rnd(grads["final_norm"])
    for w, s in zip(reversed(params["layers"]), reversed(saved)):
        g = {}
        xin = s["x"]
        d_act, g["down"], _ = o.linear_backward(cur, s["act"], w["down"])
        d_act, g["down"] = rnd(d_act), rnd(g["down"])
        d_gate, d_up = o.swiglu_backward(d_act, s["gate"], s["up"])
        d_gate, d_up = rnd(d_gate), rnd(d_up)
        d_in, g["gate"], _ = o.linear_backward(d_gate, s["norm_f"], w["gate"])
        d_in, g["gate"] = rnd(d_in), rnd(g["gate"])
        d_in2, g["up"], _ = o.linear_backward(d_up, s["norm_f"], w["up"])
        d_in, g["up"] = rnd(d_in + d_in2), rnd(g["up"])
        d_res, g["ffn_norm"] = o.rmsnorm_backward(d_in, xin, w["ffn_norm"], eps)
        d_res, g["ffn_norm"] = rnd(d_res), rnd(g["ffn_norm"])
        prev = rnd(cur + d_res)
        d_attn_out, g["o"], _ = o.linear_backward(cur, s["attn_out"], w["o"])
        d_attn_out, g["o"] = rnd(d_attn_out), rnd(g["o"])
        dq, dk, dv = o.attention_backward(d_attn_out.reshape(B, T, HQ, D), s["q"], s["k"], s["v"], HQ, HKV, D)
        dq, dk, dv = rnd(dq), rnd(dk), rnd(dv)
        dq_pre = rnd(o.rope_backward(dq, cos, sin, rotary))
        dk_pre = rnd(o.rope_backward(dk, cos, sin, rotary))
        dq2, g["q_norm"] = o.rmsnorm_backward(dq_pre.reshape(N * HQ, D), s["q_pre"].reshape(N * HQ, D), w["q_norm"], eps)
        dk2, g["k_norm"] = o.rmsnorm_backward(dk_pre.reshape(N * HKV, D), s["k_pre"].reshape(N * HKV, D), w["k_norm"],
                                              eps)
        dq2, dk2, g["q_norm"], g["k_norm"] = rnd(dq2), rnd(dk2), rnd(g["q_norm"]), rnd(g["k_norm"])
        d_in, g["q"], _ = o.linear_backward(dq2.reshape(N, HQ * D), s["norm_a"], w["q"])
        d_in, g["q"] = rnd(d_in), rnd(g["q"])
        d_in2, g["k"], _ = o.linear_backward(dk2.reshape(N, HKV * D), s["norm_a"], w["k"])
        d_in, g["k"] = rnd(d_in + d_in2), rnd(g["k"])
        d_in2, g["v"], _ = o.linear_backward(dv.reshape(N, HKV * D), s["norm_a"], w["v"])
        d_in, g["v"] = rnd(d_in + d_in2), rnd(g["v"])
        d_res, g["attention_norm"] = o.rmsnorm_backward(d_in, xin, w["attention_norm"], eps)
        d_res, g["attention_norm"] = rnd(d_res), rnd(g["attention_norm"])
        cur = rnd(prev + d_res)
        grads["layers"].insert(0, g)
    grads["embedding"] = o.embedding_backward(cur, ids, V, base=dE)
    return loss, grads, {"hidden": hidden, "normalized": normalized, "logits": logits}


def loss_only(params, tokens, targets, cfg):
    return forward_backward(params, tokens, targets, cfg)[0]
