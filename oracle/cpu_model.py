"""The reference's CPU path for one train step, composed from the float32 C checker.

TEST INFRASTRUCTURE — only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this module. Forward order follows src/core/generation_cpu.cpp:323-379 (the reference's
CPU forward) and src/core/transformer_block.cu:405-611; backward order follows
src/core/transformer_block.cu:644-748 and src/core/transformer_model.cu:336-381 with the
`*_backward_cpu` operators; the update is adamw_cpu (src/optim/adamw.cu:193-225). Everything is
float32, which is what the reference's CPU tensors hold in its configuration 1.
"""
from __future__ import annotations

import time

import torch

from oracle import cpu_ops as c


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    H, I, D = cfg["hidden"], cfg["inter"], cfg["d"]
    QW, KW = cfg["hq"] * D, cfg["hkv"] * D

    def mat(o, i, std=0.02):
        return (torch.randn(o, i, generator=g) * std).contiguous()

    residual = 0.02 / (2.0 * cfg["layers"]) ** 0.5
    layers = []
    for _ in range(cfg["layers"]):
        layers.append({"attention_norm": torch.ones(H), "q": mat(QW, H), "k": mat(KW, H), "q_norm": torch.ones(D),
                       "k_norm": torch.ones(D), "v": mat(KW, H), "o": mat(H, QW, residual), "ffn_norm": torch.ones(H),
                       "gate": mat(I, H), "up": mat(I, H), "down": mat(H, I, residual)})
    return {"embedding": mat(cfg["vocab"], H), "final_norm": torch.ones(H), "layers": layers}


def rope_cache(sequence, rotary_dim, base=10000.0):
    pos = torch.arange(sequence, dtype=torch.float32)[:, None]
    i = torch.arange(rotary_dim // 2, dtype=torch.float32)[None, :]
    theta = pos / torch.pow(torch.tensor(base), 2.0 * i / rotary_dim)
    return torch.cos(theta).contiguous(), torch.sin(theta).contiguous()


def forward(w, tokens, cfg):
    """The reference's CPU forward for whole sequences (src/core/generation_cpu.cpp:323-379: embedding, per layer
    {RMSNorm, q/k/v projections, per-head RMSNorm, RoPE, attention, o-projection, RMSNorm, gate/up, SwiGLU, down,
    two adds}, final norm, classifier). Returns (hidden states entering each layer + the last one, the tensors the
    backward pass needs, normalized, logits)."""
    B, T = tokens.shape
    N, H, I, D, HQ, HKV, V = B * T, cfg["hidden"], cfg["inter"], cfg["d"], cfg["hq"], cfg["hkv"], cfg["vocab"]
    QW, KW, eps = HQ * D, HKV * D, cfg["eps"]
    cos, sin = rope_cache(T, D)
    ids = tokens.reshape(-1).to(torch.int32).contiguous()
    E = w["embedding"]
    x = torch.empty(N, H)
    c.embedding_forward(x, ids, E)
    saved = []
    for lw in w["layers"]:
        s = {"x": x}
        s["norm_a"] = torch.empty(N, H)
        c.rmsnorm_forward(s["norm_a"], x, lw["attention_norm"], eps)
        s["q_pre"], s["k_pre"], s["v"] = torch.empty(N, QW), torch.empty(N, KW), torch.empty(N, KW)
        c.linear_forward(s["q_pre"], s["norm_a"], lw["q"])
        c.linear_forward(s["k_pre"], s["norm_a"], lw["k"])
        c.linear_forward(s["v"], s["norm_a"], lw["v"])
        q, k = torch.empty(N * HQ, D), torch.empty(N * HKV, D)
        c.rmsnorm_forward(q, s["q_pre"].view(N * HQ, D), lw["q_norm"], eps)
        c.rmsnorm_forward(k, s["k_pre"].view(N * HKV, D), lw["k_norm"], eps)
        s["q"], s["k"] = q.view(B, T, HQ, D), k.view(B, T, HKV, D)
        c.rope_forward(s["q"], s["k"], cos, sin)
        s["attn_out"], s["lse"] = torch.empty(B, T, HQ, D), torch.empty(B, T, HQ)
        c.attention_forward(s["attn_out"], s["lse"], s["q"], s["k"], s["v"].view(B, T, HKV, D), HQ, HKV, D)
        proj = torch.empty(N, H)
        c.linear_forward(proj, s["attn_out"].view(N, QW), lw["o"])
        s["norm_f"] = torch.empty(N, H)
        c.rmsnorm_forward(s["norm_f"], x, lw["ffn_norm"], eps)
        s["gate"], s["up"], s["act"] = torch.empty(N, I), torch.empty(N, I), torch.empty(N, I)
        c.linear_forward(s["gate"], s["norm_f"], lw["gate"])
        c.linear_forward(s["up"], s["norm_f"], lw["up"])
        c.swiglu_forward(s["act"], s["gate"], s["up"])
        ffn = torch.empty(N, H)
        c.linear_forward(ffn, s["act"], lw["down"])
        out = torch.empty(N, H)
        c.add(out, x, proj)
        c.add(out, out, ffn)
        saved.append(s)
        x = out
    normalized, logits = torch.empty(N, H), torch.empty(N, V)
    c.rmsnorm_forward(normalized, x, w["final_norm"], eps)
    c.linear_forward(logits, normalized, E)
    return [s["x"] for s in saved] + [x], saved, normalized, logits


def forward_loss(w, tokens, targets, cfg):
    """Forward + cross_entropy_forward_cpu (src/ops/cpu/cross_entropy_cpu.cpp): the reference's CPU-runnable
    configuration. Returns (loss, hidden states [layers + 1], float64 sum of the logits as a checksum)."""
    hidden, _, _, logits = forward(w, tokens, cfg)
    loss = torch.empty(1)
    c.cross_entropy_forward(loss, logits, targets.reshape(-1).to(torch.int32).contiguous())
    return loss.item(), hidden, float(logits.double().sum())


def timed_forward_loss(cfg, batch, sequence, seed=0):
    """Seconds, loss and logits checksum of one CPU forward + loss on a seeded random batch."""
    w = make_weights(cfg, seed)
    g = torch.Generator().manual_seed(seed + 1)
    tokens = torch.randint(0, cfg["vocab"], (batch, sequence), generator=g)
    targets = torch.randint(0, cfg["vocab"], (batch, sequence), generator=g)
    start = time.perf_counter()
    loss, _, checksum = forward_loss(w, tokens, targets, cfg)
    return time.perf_counter() - start, loss, checksum


def train_step(w, tokens, targets, cfg, loss_scale=1.0, optimizer=None, step=1):
    """One float32 CPU step. Returns (loss, grads). `optimizer` = dict of AdamW options to also update."""
    B, T = tokens.shape
    N, H, I, D, HQ, HKV, V = B * T, cfg["hidden"], cfg["inter"], cfg["d"], cfg["hq"], cfg["hkv"], cfg["vocab"]
    QW, KW, eps = HQ * D, HKV * D, cfg["eps"]
    cos, sin = rope_cache(T, D)
    ids = tokens.reshape(-1).to(torch.int32).contiguous()
    tg = targets.reshape(-1).to(torch.int32).contiguous()
    E = w["embedding"]
    hidden, saved, normalized, logits = forward(w, tokens, cfg)
    x = hidden[-1]
    loss, dlogits = torch.empty(1), torch.empty(N, V)
    c.cross_entropy_forward_backward(loss, dlogits, logits, tg, loss_scale)

    grads = {"layers": [None] * len(w["layers"])}
    bias = torch.empty(max(V, I, H))
    d_norm, grads["embedding"] = torch.empty(N, H), torch.empty(V, H)
    c.linear_backward(d_norm, grads["embedding"], bias[:V], dlogits, normalized, E)
    cur, grads["final_norm"] = torch.empty(N, H), torch.empty(H)
    c.rmsnorm_backward(cur, grads["final_norm"], d_norm, x, w["final_norm"], eps)
    for l in range(len(w["layers"]) - 1, -1, -1):
        lw, s, g = w["layers"][l], saved[l], {}
        d_act, g["down"] = torch.empty(N, I), torch.empty(H, I)
        c.linear_backward(d_act, g["down"], bias[:H], cur, s["act"], lw["down"])
        d_gate, d_up = torch.empty(N, I), torch.empty(N, I)
        c.swiglu_backward(d_gate, d_up, d_act, s["gate"], s["up"])
        d_in, g["gate"], g["up"] = torch.empty(N, H), torch.empty(I, H), torch.empty(I, H)
        c.linear_backward(d_in, g["gate"], bias[:I], d_gate, s["norm_f"], lw["gate"])
        c.linear_backward(d_in, g["up"], bias[:I], d_up, s["norm_f"], lw["up"], accumulate_input=True)
        d_res, g["ffn_norm"] = torch.empty(N, H), torch.empty(H)
        c.rmsnorm_backward(d_res, g["ffn_norm"], d_in, s["x"], lw["ffn_norm"], eps)
        prev = torch.empty(N, H)
        c.add(prev, cur, d_res)
        d_attn, g["o"] = torch.empty(N, QW), torch.empty(H, QW)
        c.linear_backward(d_attn, g["o"], bias[:H], cur, s["attn_out"].view(N, QW), lw["o"])
        dq, dk, dv = torch.empty(B, T, HQ, D), torch.empty(B, T, HKV, D), torch.empty(B, T, HKV, D)
        c.attention_backward(dq, dk, dv, d_attn.view(B, T, HQ, D), s["q"], s["k"], s["v"].view(B, T, HKV, D), HQ, HKV, D)
        dq_pre, dk_pre = torch.empty_like(dq), torch.empty_like(dk)
        c.rope_backward(dq_pre, dk_pre, dq, dk, cos, sin)
        g["q_norm"], g["k_norm"] = torch.empty(D), torch.empty(D)
        c.rmsnorm_backward(dq.view(N * HQ, D), g["q_norm"], dq_pre.view(N * HQ, D), s["q_pre"].view(N * HQ, D),
                           lw["q_norm"], eps)
        c.rmsnorm_backward(dk.view(N * HKV, D), g["k_norm"], dk_pre.view(N * HKV, D), s["k_pre"].view(N * HKV, D),
                           lw["k_norm"], eps)
        g["q"], g["k"], g["v"] = torch.empty(QW, H), torch.empty(KW, H), torch.empty(KW, H)
        c.linear_backward(d_in, g["q"], bias[:QW], dq.view(N, QW), s["norm_a"], lw["q"])
        c.linear_backward(d_in, g["k"], bias[:KW], dk.view(N, KW), s["norm_a"], lw["k"], accumulate_input=True)
        c.linear_backward(d_in, g["v"], bias[:KW], dv.view(N, KW), s["norm_a"], lw["v"], accumulate_input=True)
        g["attention_norm"] = torch.empty(H)
        c.rmsnorm_backward(d_res, g["attention_norm"], d_in, s["x"], lw["attention_norm"], eps)
        c.add(prev, prev, d_res)
        cur = prev
        grads["layers"][l] = g
    c.embedding_backward(grads["embedding"], cur, ids, True, True)

    if optimizer is not None:
        state = optimizer.setdefault("state", {})
        flat = [("embedding", w["embedding"], grads["embedding"]), ("final_norm", w["final_norm"], grads["final_norm"])]
        for l, (lw, g) in enumerate(zip(w["layers"], grads["layers"])):
            flat += [(f"{l}.{k}", lw[k], g[k]) for k in lw]
        # one global norm over all tensors: concatenate views (adamw_cpu works on one tensor)
        params = torch.cat([p.reshape(-1) for _, p, _ in flat])
        grad = torch.cat([g.reshape(-1) for _, _, g in flat])
        if "m" not in state:
            state["master"], state["m"], state["v"] = params.clone(), torch.zeros_like(params), torch.zeros_like(params)
        c.adamw(params, grad, state["master"], state["m"], state["v"], step, optimizer["learning_rate"],
                optimizer["beta1"], optimizer["beta2"], optimizer["epsilon"], optimizer["weight_decay"], loss_scale,
                optimizer["max_grad_norm"], parallel=True)
        offset = 0
        for _, p, _ in flat:
            p.copy_(params[offset:offset + p.numel()].view_as(p))
            offset += p.numel()
    return loss.item(), grads


def timed_train_step(cfg, batch, sequence, seed=0):
    """Seconds for one CPU train step (forward + loss + backward + AdamW) on a seeded random batch."""
    w = make_weights(cfg, seed)
    g = torch.Generator().manual_seed(seed + 1)
    tokens = torch.randint(0, cfg["vocab"], (batch, sequence), generator=g)
    targets = torch.randint(0, cfg["vocab"], (batch, sequence), generator=g)
    options = dict(learning_rate=3e-4, beta1=0.9, beta2=0.95, epsilon=1e-8, weight_decay=0.1, max_grad_norm=1.0)
    start = time.perf_counter()
    loss, _ = train_step(w, tokens, targets, cfg, 1024.0, options, 1)
    return time.perf_counter() - start, loss
