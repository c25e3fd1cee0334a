"""Writes tests/golden/hot_path_vectors.npz: seeded inputs (already rounded to bf16) and the float64
oracle's outputs for the operators of the hot path, at shapes small enough to commit (a few hundred
KiB). The fixture freezes the oracle: tests/test_golden.py checks that today's oracle still
reproduces it (CPU) and that the HIP kernels match it (GPU).

Run from the repository root:  python tests/golden/make_golden.py
"""
from __future__ import annotations

import pathlib
import sys

import numpy as np

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import oracle64  # noqa: E402

OUT = pathlib.Path(__file__).resolve().parent / "hot_path_vectors.npz"


def bf16(a):
    """Round float64/float32 values to bfloat16 (nearest even) and return them as float32."""
    f = np.asarray(a, dtype=np.float32)
    bits = f.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).reshape(f.shape)


def main() -> None:
    rng = np.random.default_rng(20240607)
    v = {}
    # attention: heads of 128 in groups of two, 70 tokens: one full and one ragged 64-row tile
    B, T, HQ, HKV, D = 1, 70, 4, 2, 128
    q, k, val = (bf16(rng.normal(size=s)) for s in ((B, T, HQ, D), (B, T, HKV, D), (B, T, HKV, D)))
    do = bf16(rng.normal(size=(B, T, HQ, D)))
    out, lse = oracle64.attention_forward(q, k, val, HQ, HKV, D)
    dq, dk, dv = oracle64.attention_backward(do, q, k, val, HQ, HKV, D)
    v.update(attn_q=q, attn_k=k, attn_v=val, attn_do=do, attn_out=out, attn_lse=lse, attn_dq=dq, attn_dk=dk, attn_dv=dv)
    # RMSNorm backward, hidden 1024 and head-norm width 128
    for tag, rows, hidden in (("h", 12, 1024), ("d", 70, 128)):
        x, dy = bf16(rng.normal(size=(rows, hidden))), bf16(rng.normal(size=(rows, hidden)))
        w = bf16(1 + 0.1 * rng.normal(size=hidden))
        dx, dw = oracle64.rmsnorm_backward(dy, x, w, 1e-5)
        v.update({f"rms_{tag}_x": x, f"rms_{tag}_dy": dy, f"rms_{tag}_w": w, f"rms_{tag}_dx": dx, f"rms_{tag}_dw": dw})
    # SwiGLU backward and RoPE backward
    g, u, dy = (bf16(rng.normal(size=(33, 256))) for _ in range(3))
    gg, gu = oracle64.swiglu_backward(dy, g, u)
    v.update(swiglu_g=g, swiglu_u=u, swiglu_dy=dy, swiglu_dg=gg, swiglu_du=gu)
    pos = np.arange(16)[:, None] / (10000.0 ** (np.arange(64)[None, :] * 2 / 128))
    cos, sin = bf16(np.cos(pos)), bf16(np.sin(pos))
    rq = bf16(rng.normal(size=(2, 16, 4, 128)))
    v.update(rope_dy=rq, rope_cos=cos, rope_sin=sin, rope_dx=oracle64.rope_backward(rq, cos, sin))
    # linear backward and cut cross-entropy (vocabulary 300, hidden 64)
    x, w, dy = bf16(rng.normal(size=(96, 64))), bf16(0.1 * rng.normal(size=(40, 64))), bf16(rng.normal(size=(96, 40)))
    dx, dw, db = oracle64.linear_backward(dy, x, w)
    v.update(lin_x=x, lin_w=w, lin_dy=dy, lin_dx=dx, lin_dw=dw, lin_db=db)
    x, c = bf16(rng.normal(size=(50, 64))), bf16(0.2 * rng.normal(size=(300, 64)))
    targets = rng.integers(0, 300, size=50).astype(np.uint32)
    loss, dx, dc = oracle64.cut_cross_entropy(x, c, targets, 64.0)
    v.update(cce_x=x, cce_c=c, cce_targets=targets, cce_loss=np.float64(loss), cce_dx=dx, cce_dc=dc)
    # embedding scatter with heavy collisions (integer work: exact)
    ids = rng.integers(0, 9, size=200).astype(np.uint32)
    dy = bf16(rng.normal(size=(200, 32)))
    v.update(emb_ids=ids, emb_dy=dy, emb_dw=oracle64.embedding_backward(dy, ids, 7))
    # inputs (exactly representable in bf16) are stored as their bf16 bit patterns, float64 results as float32
    inputs = {"attn_q", "attn_k", "attn_v", "attn_do", "rms_h_x", "rms_h_dy", "rms_h_w", "rms_d_x", "rms_d_dy", "rms_d_w",
              "swiglu_g", "swiglu_u", "swiglu_dy", "rope_dy", "rope_cos", "rope_sin", "lin_x", "lin_w", "lin_dy", "cce_x",
              "cce_c", "emb_dy"}
    packed = {}
    for name, a in v.items():
        a = np.asarray(a)
        if name in inputs:
            packed[name] = (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        elif a.dtype == np.float64 and a.ndim > 0:
            packed[name] = a.astype(np.float32)
        else:
            packed[name] = a
    np.savez_compressed(OUT, **packed)
    print(OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
