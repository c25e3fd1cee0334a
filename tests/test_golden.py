"""Committed golden vectors (tests/golden/hot_path_vectors.npz, written by tests/golden/make_golden.py).

CPU: the float64 oracle of today still reproduces the frozen outputs (guards the checker itself).
GPU: the HIP kernels, called through the operator interface, match the frozen outputs to the
16-bit parity bar; the embedding scatter exactly.
"""
import pathlib

import numpy as np
import pytest
import torch

from oracle import oracle64

GOLDEN = pathlib.Path(__file__).resolve().parent / "golden" / "hot_path_vectors.npz"


@pytest.fixture(scope="module")
def vec():
    data = np.load(GOLDEN, allow_pickle=False)
    out = {}
    for name in data.files:
        a = data[name]
        if a.dtype == np.uint16:  # bf16 bit patterns -> float32
            a = (a.astype(np.uint32) << 16).view(np.float32)
        out[name] = a
    return out


def close(got, want, tol, what):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, what
    err = np.abs(got - want).max() / max(1.0, np.abs(want).max())
    assert err <= tol, f"{what}: {err}"


def test_oracle_reproduces_the_frozen_vectors(vec):
    v = vec
    out, lse = oracle64.attention_forward(v["attn_q"], v["attn_k"], v["attn_v"], 4, 2, 128)
    dq, dk, dv = oracle64.attention_backward(v["attn_do"], v["attn_q"], v["attn_k"], v["attn_v"], 4, 2, 128)
    for got, name in ((out, "attn_out"), (lse, "attn_lse"), (dq, "attn_dq"), (dk, "attn_dk"), (dv, "attn_dv")):
        close(got, v[name], 1e-6, name)
    for tag in ("h", "d"):
        dx, dw = oracle64.rmsnorm_backward(v[f"rms_{tag}_dy"], v[f"rms_{tag}_x"], v[f"rms_{tag}_w"], 1e-5)
        close(dx, v[f"rms_{tag}_dx"], 1e-6, "rmsnorm dx")
        close(dw, v[f"rms_{tag}_dw"], 1e-6, "rmsnorm dgamma")
    gg, gu = oracle64.swiglu_backward(v["swiglu_dy"], v["swiglu_g"], v["swiglu_u"])
    close(gg, v["swiglu_dg"], 1e-6, "swiglu dgate")
    close(gu, v["swiglu_du"], 1e-6, "swiglu dup")
    close(oracle64.rope_backward(v["rope_dy"], v["rope_cos"], v["rope_sin"]), v["rope_dx"], 1e-6, "rope")
    dx, dw, db = oracle64.linear_backward(v["lin_dy"], v["lin_x"], v["lin_w"])
    close(dx, v["lin_dx"], 1e-6, "linear dx")
    close(dw, v["lin_dw"], 1e-6, "linear dw")
    close(db, v["lin_db"], 1e-6, "linear db")
    loss, dx, dc = oracle64.cut_cross_entropy(v["cce_x"], v["cce_c"], v["cce_targets"], 64.0)
    assert abs(loss - float(v["cce_loss"])) <= 1e-9
    close(dx, v["cce_dx"], 1e-6, "cut-CE dx")
    close(dc, v["cce_dc"], 1e-6, "cut-CE dc")
    close(oracle64.embedding_backward(v["emb_dy"], v["emb_ids"], 7), v["emb_dw"], 1e-6, "embedding")


@pytest.mark.gpu
def test_kernels_match_the_frozen_vectors(vec, device):
    from cgpt_amd import ops

    bf = torch.bfloat16
    v = vec

    def dev(name):
        return torch.from_numpy(np.ascontiguousarray(v[name])).to(bf).to(device)

    def empty(name, dtype=bf):
        return torch.empty(v[name].shape, dtype=dtype, device=device)

    tol = 2e-2
    options = ops.FlashAttentionOptions(4, 2, 128)
    q, k, val, do = dev("attn_q"), dev("attn_k"), dev("attn_v"), dev("attn_do")
    out, lse = empty("attn_out"), empty("attn_lse", torch.float32)
    ops.flash_gqa_attention_forward_with_lse(out, lse, q, k, val, None, options)
    dq, dk, dv = empty("attn_dq"), empty("attn_dk"), empty("attn_dv")
    ops.flash_gqa_attention_backward_with_lse(dq, dk, dv, do, out, lse, q, k, val, None, options)
    for got, name in ((out, "attn_out"), (lse, "attn_lse"), (dq, "attn_dq"), (dk, "attn_dk"), (dv, "attn_dv")):
        close(got.float().cpu().numpy(), v[name], tol, name)
    for tag in ("h", "d"):
        dx, dw = empty(f"rms_{tag}_dx"), empty(f"rms_{tag}_dw")
        ops.rmsnorm_backward(dx, dw, dev(f"rms_{tag}_dy"), dev(f"rms_{tag}_x"), dev(f"rms_{tag}_w"), 1e-5)
        close(dx.float().cpu().numpy(), v[f"rms_{tag}_dx"], tol, "rmsnorm dx")
        close(dw.float().cpu().numpy(), v[f"rms_{tag}_dw"], tol, "rmsnorm dgamma")
    gg, gu = empty("swiglu_dg"), empty("swiglu_du")
    ops.swiglu_backward(gg, gu, dev("swiglu_dy"), dev("swiglu_g"), dev("swiglu_u"))
    close(gg.float().cpu().numpy(), v["swiglu_dg"], tol, "swiglu dgate")
    close(gu.float().cpu().numpy(), v["swiglu_du"], tol, "swiglu dup")
    dy = dev("rope_dy")
    gq, gk = torch.empty_like(dy), torch.empty_like(dy[:, :, :1].contiguous())
    ops.rope_backward(gq, gk, dy, dy[:, :, :1].contiguous(), dev("rope_cos"), dev("rope_sin"))
    close(gq.float().cpu().numpy(), v["rope_dx"], tol, "rope")
    dx, dw, db = empty("lin_dx"), empty("lin_dw"), empty("lin_db")
    ops.linear_backward(dx, dw, db, dev("lin_dy"), dev("lin_x"), dev("lin_w"))
    close(dx.float().cpu().numpy(), v["lin_dx"], tol, "linear dx")
    close(dw.float().cpu().numpy(), v["lin_dw"], tol, "linear dw")
    close(db.float().cpu().numpy(), v["lin_db"], tol, "linear db")
    targets = torch.from_numpy(v["cce_targets"].astype(np.int32)).to(device)
    loss = torch.zeros(1, device=device)
    dx, dc = empty("cce_dx"), empty("cce_dc")
    ops.cut_cross_entropy_forward_backward(loss, dx, dc, dev("cce_x"), dev("cce_c"), targets, 50, None, 64.0)
    assert abs(loss.item() - float(v["cce_loss"])) <= 2e-2 * float(v["cce_loss"])
    close(dx.float().cpu().numpy(), v["cce_dx"], tol, "cut-CE dx")
    close(dc.float().cpu().numpy(), v["cce_dc"], tol, "cut-CE dc")
    ids = torch.from_numpy(v["emb_ids"].astype(np.int32)).to(device)
    gw = torch.empty((7, 32), dtype=torch.float32, device=device)
    ops.embedding_backward(gw, dev("emb_dy").float(), ids, 200)
    close(gw.cpu().numpy(), v["emb_dw"], 1e-5, "embedding (fp32 table, ids 7 and 8 out of range)")
