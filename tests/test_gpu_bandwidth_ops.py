"""GPU parity tests of the bandwidth-bound kernels (RMSNorm, RoPE, SwiGLU, residual add) against
the float32 CPU checker, through the C-ABI. Tolerance: max |a-b| / max(1, |b|) <= 1e-4 (fp32),
2e-2 (fp16 / bf16)."""
import numpy as np
import pytest
import torch

from cgpt_amd import ops
from oracle import cpu_ops, oracle64
from tests.util import DTYPES, DTYPE_IDS, TOL, assert_close, randn, to_np

pytestmark = pytest.mark.gpu


def dev(t, device):
    return t.to(device).contiguous()


# ------------------------------------------------------------------------ RMSNorm
RMS_SHAPES = [(3, 7), (2, 4096), (129, 513), (64, 128), (257, 128), (33, 768), (40, 1024), (5, 2048), (7, 64),
              (9, 256), (4, 5000)]


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows,hidden", RMS_SHAPES)
def test_rmsnorm_backward_parity(device, rows, hidden, dtype):
    x, dy = randn((rows, hidden), dtype, 1), randn((rows, hidden), dtype, 2)
    w = (1.0 + 0.1 * randn((hidden,), torch.float32, 3)).to(dtype)
    gi, gw = torch.empty_like(x), torch.empty_like(w)
    cpu_ops.rmsnorm_backward(gi, gw, dy, x, w, 1e-5)
    dgi, dgw = torch.full_like(x, 7.0, device=device), torch.full_like(w, 7.0, device=device)
    ops.rmsnorm_backward(dgi, dgw, dev(dy, device), dev(x, device), dev(w, device), 1e-5)
    torch.cuda.synchronize()
    assert_close(dgi, gi, TOL[dtype], "dx")
    # dgamma sums `rows` terms; the checker rounds once at the end like the kernel
    dw64 = oracle64.rmsnorm_backward(to_np(dy), to_np(x), to_np(w), 1e-5)[1]
    assert_close(dgw, dw64, TOL[dtype], "dgamma vs float64")
    assert_close(dgw, gw, TOL[dtype], "dgamma vs float32 checker")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.float16, 5e-3), (torch.bfloat16, 2.5e-1)])
def test_rmsnorm_backward_reference_test_inputs(device, dtype, tol):
    """Inputs of tests/rmsnorm_test.cu:268-322 at its three shapes, checked against the float64 formulas."""
    for rows, hidden in ((3, 7), (2, 4096), (129, 513)):
        idx = np.arange(rows * hidden)
        x = torch.tensor(0.125 * ((idx % 13) - 6), dtype=torch.float32).reshape(rows, hidden).to(dtype)
        dy = torch.tensor(0.25 * ((idx % 9) - 4), dtype=torch.float32).reshape(rows, hidden).to(dtype)
        w = torch.tensor(0.5 + 0.125 * np.arange(hidden), dtype=torch.float32).to(dtype)
        dx64, dw64 = oracle64.rmsnorm_backward(to_np(dy), to_np(x), to_np(w), 1e-5)
        gi, gw = torch.empty_like(x, device=device), torch.empty_like(w, device=device)
        ops.rmsnorm_backward(gi, gw, dev(dy, device), dev(x, device), dev(w, device), 1e-5)
        assert_close(gi, dx64, tol, "dx")
        assert_close(gw, dw64, tol, "dgamma")


def test_rmsnorm_backward_is_deterministic_and_full_size(device):
    """[32768, 1024] bf16 (the training shape), the QK-norm shapes [262144, 128] (q: the 8 heads of every token, the pass
    a step runs once per layer) and [65536, 128] (k), and the 768-wide shapes ([32768, 768]; [131072, 64] for its 4
    kv-heads of 64): run twice, bit-identical, and equal to the CPU checker."""
    for rows, hidden in ((32768, 1024), (262144, 128), (65536, 128), (32768, 768), (131072, 64)):
        dtype = torch.bfloat16
        x, dy = randn((rows, hidden), dtype, 11), randn((rows, hidden), dtype, 12)
        w = (1.0 + 0.1 * randn((hidden,), torch.float32, 13)).to(dtype)
        gi, gw = torch.empty_like(x), torch.empty_like(w)
        cpu_ops.rmsnorm_backward(gi, gw, dy, x, w, 1e-5)
        dx_, dy_, dw_ = dev(x, device), dev(dy, device), dev(w, device)
        out = []
        for _ in range(2):
            dgi, dgw = torch.empty_like(dx_), torch.empty_like(dw_)
            ops.rmsnorm_backward(dgi, dgw, dy_, dx_, dw_, 1e-5)
            out.append((dgi.cpu(), dgw.cpu()))
        assert torch.equal(out[0][0], out[1][0]) and torch.equal(out[0][1], out[1][1])
        assert_close(out[0][0], gi, TOL[dtype], "dx")
        dw64 = oracle64.rmsnorm_backward(to_np(dy), to_np(x), to_np(w), 1e-5)[1]
        # a sum of 32768+ terms of size ~1: compare relative to the column scale
        assert np.abs(to_np(out[0][1]) - dw64).max() <= TOL[dtype] * max(1.0, np.abs(dw64).max())


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows,hidden", [(3, 7), (64, 128), (33, 768), (40, 1024), (4, 5000)])
def test_rmsnorm_forward_parity(device, rows, hidden, dtype):
    x = randn((rows, hidden), dtype, 4)
    w = (1.0 + 0.1 * randn((hidden,), torch.float32, 5)).to(dtype)
    y = torch.empty_like(x)
    cpu_ops.rmsnorm_forward(y, x, w, 1e-5)
    dy_ = torch.empty_like(x, device=device)
    ops.rmsnorm_forward(dy_, dev(x, device), dev(w, device), 1e-5)
    assert_close(dy_, y, TOL[dtype], "y")


def test_rmsnorm_argument_errors(device):
    x = torch.zeros(2, 4, device=device)
    w = torch.zeros(4, device=device)
    with pytest.raises(ValueError):
        ops.rmsnorm_backward(x.clone(), w.clone(), x, x, torch.zeros(3, device=device), 1e-5)
    with pytest.raises(ValueError):
        ops.rmsnorm_backward(x.clone(), w.clone(), x, x, w, 0.0)
    with pytest.raises(ValueError):
        ops.rmsnorm_backward(x.clone(), w.clone(), x, x.cpu(), w, 1e-5)
    with pytest.raises(ValueError):
        ops.rmsnorm_backward(x.clone(), w.clone(), x, x.half(), w, 1e-5)


# --------------------------------------------------------------------------- RoPE
def rope_cache(positions, rotary_dim, dtype):
    pos = torch.arange(positions, dtype=torch.float32)[:, None]
    i = torch.arange(rotary_dim // 2, dtype=torch.float32)[None, :]
    theta = pos / torch.pow(torch.tensor(10000.0), 2.0 * i / rotary_dim)  # train/train.cpp:322-333
    return torch.cos(theta).to(dtype).contiguous(), torch.sin(theta).to(dtype).contiguous()


ROPE_CASES = [  # batch, seq, hq, hkv, d, rotary, offset
    (1, 2, 2, 1, 4, 2, 0), (2, 5, 3, 1, 8, 6, 4), (2, 16, 8, 2, 128, 0, 0), (1, 7, 12, 4, 64, 0, 3),
    (2, 9, 4, 2, 64, 32, 0), (1, 3, 2, 2, 24, 16, 1),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("case", ROPE_CASES)
def test_rope_backward_parity(device, case, dtype):
    b, s, hq, hkv, d, rotary, off = case
    r = rotary or d
    cos, sin = rope_cache(off + s + 2, r, dtype)
    q, k = randn((b, s, hq, d), dtype, 6), randn((b, s, hkv, d), dtype, 7)
    gq, gk = torch.empty_like(q), torch.empty_like(k)
    cpu_ops.rope_backward(gq, gk, q, k, cos, sin, rotary, off)
    dq, dk = torch.full_like(q, 3.0, device=device), torch.full_like(k, 3.0, device=device)
    ops.rope_backward(dq, dk, dev(q, device), dev(k, device), dev(cos, device), dev(sin, device), None,
                      ops.RopeOptions(rotary, off))
    assert_close(dq, gq, TOL[dtype], "dq")
    assert_close(dk, gk, TOL[dtype], "dk")
    # forward in place, then backward, returns the input up to two roundings
    fq, fk = dev(q, device).clone(), dev(k, device).clone()
    ops.rope_forward(fq, fk, dev(cos, device), dev(sin, device), None, ops.RopeOptions(rotary, off))
    cq, ck = q.clone(), k.clone()
    cpu_ops.rope_forward(cq, ck, cos, sin, rotary, off)
    assert_close(fq, cq, TOL[dtype], "rope forward q")
    assert_close(fk, ck, TOL[dtype], "rope forward k")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.float16, 3e-3), (torch.bfloat16, 2e-2)])
def test_rope_backward_known_answer(device, dtype, tol):
    """tests/rope_test.cu:99-127."""
    q = torch.tensor([1, 2, 30, 40, 3, 4, 50, 60, 5, 6, 70, 80, 7, 8, 90, 100.0]).reshape(1, 2, 2, 4).to(dtype)
    k = torch.tensor([1, -2, 30, 40, 5, -6, 70, 80.0]).reshape(1, 2, 1, 4).to(dtype)
    cos, sin = torch.tensor([[1.0], [0.0]]).to(dtype), torch.tensor([[0.0], [1.0]]).to(dtype)
    gq, gk = torch.empty_like(q, device=device), torch.empty_like(k, device=device)
    ops.rope_backward(gq, gk, dev(q, device), dev(k, device), dev(cos, device), dev(sin, device), None,
                      ops.RopeOptions(rotary_dim=2))
    assert np.abs(to_np(gq).reshape(-1) - [1, 2, 30, 40, 3, 4, 50, 60, 6, -5, 70, 80, 8, -7, 90, 100]).max() <= tol
    assert np.abs(to_np(gk).reshape(-1) - [1, -2, 30, 40, -6, -5, 70, 80]).max() <= tol


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (12, 4, 64)], ids=["preset-8:2x128", "secondary-12:4x64"])
def test_rope_backward_full_size_bit_exact_vs_checker(device, hq, hkv, d):
    """q[32,1024,8,128] + k[32,1024,2,128] and q[32,1024,12,64] + k[32,1024,4,64], bf16: same fp32 arithmetic and one
    rounding as the CPU checker, so the result is compared bit for bit."""
    dtype = torch.bfloat16
    cos, sin = rope_cache(1024, d, dtype)
    q, k = randn((32, 1024, hq, d), dtype, 21), randn((32, 1024, hkv, d), dtype, 22)
    gq, gk = torch.empty_like(q), torch.empty_like(k)
    cpu_ops.rope_backward(gq, gk, q, k, cos, sin)
    dq, dk = torch.empty_like(q, device=device), torch.empty_like(k, device=device)
    ops.rope_backward(dq, dk, dev(q, device), dev(k, device), dev(cos, device), dev(sin, device))
    assert torch.equal(dq.cpu(), gq) and torch.equal(dk.cpu(), gk)


def test_rope_argument_errors(device):
    q = torch.zeros(1, 2, 2, 4, device=device)
    k = torch.zeros(1, 2, 1, 4, device=device)
    c = torch.zeros(2, 2, device=device)
    with pytest.raises(ValueError):  # cache shorter than offset + sequence
        ops.rope_backward(q.clone(), k.clone(), q, k, c, c, None, ops.RopeOptions(0, 1))
    with pytest.raises(ValueError):  # rotary_dim does not match the cache width
        ops.rope_backward(q.clone(), k.clone(), q, k, c, c, None, ops.RopeOptions(2, 0))
    with pytest.raises(ValueError):
        ops.rope_backward(q.clone(), k.clone(), q, torch.zeros(1, 3, 1, 4, device=device), c, c)


# ------------------------------------------------------------------------- SwiGLU
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("shape", [(17,), (3, 24), (64, 2048), (5, 7, 9)])
@pytest.mark.parametrize("acc", [(False, False), (True, False), (True, True)])
def test_swiglu_backward_parity(device, shape, dtype, acc):
    g, u, dy = randn(shape, dtype, 8, 2.0), randn(shape, dtype, 9), randn(shape, dtype, 10)
    gg, gu = randn(shape, dtype, 11), randn(shape, dtype, 12)
    dgg, dgu = dev(gg, device).clone(), dev(gu, device).clone()
    cpu_ops.swiglu_backward(gg, gu, dy, g, u, *acc)
    ops.swiglu_backward(dgg, dgu, dev(dy, device), dev(g, device), dev(u, device), None,
                        ops.SwiGLUBackwardOptions(*acc))
    assert_close(dgg, gg, TOL[dtype], "dgate")
    assert_close(dgu, gu, TOL[dtype], "dup")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows,hidden", [(3, 5), (16, 256)])
@pytest.mark.parametrize("acc", [False, True])
def test_swiglu_backward_packed_parity(device, rows, hidden, dtype, acc):
    gu, dy = randn((rows, 2 * hidden), dtype, 13, 2.0), randn((rows, hidden), dtype, 14)
    out = randn((rows, 2 * hidden), dtype, 15)
    dout = dev(out, device).clone()
    cpu_ops.swiglu_backward_packed(out, dy, gu, acc)
    ops.swiglu_backward_packed(dout, dev(dy, device), dev(gu, device), None,
                               ops.SwiGLUBackwardOptions(accumulate_gate_up=acc))
    assert_close(dout, out, TOL[dtype], "packed")


def test_swiglu_backward_full_size(device):
    """[32768, 2048] bf16 against the CPU checker, plus extreme gate values stay finite."""
    dtype = torch.bfloat16
    shape = (32768, 2048)
    g, u, dy = randn(shape, dtype, 31, 2.0), randn(shape, dtype, 32), randn(shape, dtype, 33)
    g[0, :8] = torch.tensor([-60000.0, 60000.0, -88.0, 88.0, 0.0, -0.0, 1e-30, -1e-30]).to(dtype)
    gg, gu = torch.empty_like(g), torch.empty_like(g)
    cpu_ops.swiglu_backward(gg, gu, dy, g, u)
    dgg, dgu = torch.empty_like(g, device=device), torch.empty_like(g, device=device)
    ops.swiglu_backward(dgg, dgu, dev(dy, device), dev(g, device), dev(u, device))
    assert_close(dgg, gg, TOL[dtype], "dgate")
    assert_close(dgu, gu, TOL[dtype], "dup")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_swiglu_forward_and_add_parity(device, dtype):
    g, u = randn((33, 100), dtype, 16, 2.0), randn((33, 100), dtype, 17)
    out = torch.empty_like(g)
    cpu_ops.swiglu_forward(out, g, u)
    dout = torch.empty_like(g, device=device)
    ops.swiglu_forward(dout, dev(g, device), dev(u, device))
    assert_close(dout, out, TOL[dtype], "swiglu forward")
    cpu_ops.add(out, g, u)
    ops.add_tensors(dout, dev(g, device), dev(u, device))
    assert torch.equal(dout.cpu(), out)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows,hidden", [(7, 24), (64, 2048), (5, 13)])
def test_swiglu_forward_packed_parity(device, rows, hidden, dtype):
    """Concatenated [gate | up] input (include/ops/swiglu.h:33-37): same values as the two-tensor form."""
    gu = randn((rows, 2 * hidden), dtype, 41)
    out = torch.empty((rows, hidden), dtype=dtype)
    cpu_ops.swiglu_forward(out, gu[:, :hidden].contiguous(), gu[:, hidden:].contiguous())
    dout = torch.empty((rows, hidden), dtype=dtype, device=device)
    ops.swiglu_forward(dout, dev(gu, device))
    assert_close(dout, out, TOL[dtype], "packed swiglu forward")
    with pytest.raises(ValueError):
        ops.swiglu_forward(dout, dev(gu, device)[:, : 2 * hidden - 1].contiguous())


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_tensors_without_elements_are_accepted_and_nothing_is_written(device, dtype):
    """The reference returns early for RoPE and SwiGLU tensors with no elements (src/ops/rope.cu:606-608,
    src/ops/backward/rope_backward.cu:326-328, src/ops/swiglu.cu:530-532 and 581-583,
    src/ops/backward/swiglu_backward.cu:772-774 and 839-841): zero rows, a zero batch or a zero sequence are not
    errors. A guard tensor next to the calls keeps its contents."""
    guard = torch.full((64,), 3.0, dtype=dtype, device=device)
    empty = torch.zeros(0, 16, dtype=dtype, device=device)
    ops.swiglu_backward(empty.clone(), empty.clone(), empty, empty, empty)
    ops.swiglu_forward(empty.clone(), empty, empty)
    packed = torch.zeros(0, 32, dtype=dtype, device=device)
    ops.swiglu_backward_packed(packed.clone(), empty, packed)
    ops.swiglu_forward(empty.clone(), packed)
    cos = torch.zeros(4, 4, dtype=dtype, device=device)
    for shape_q, shape_k in (((0, 4, 2, 8), (0, 4, 1, 8)), ((2, 0, 2, 8), (2, 0, 1, 8))):
        q, k = torch.zeros(shape_q, dtype=dtype, device=device), torch.zeros(shape_k, dtype=dtype, device=device)
        ops.rope_backward(q.clone(), k.clone(), q, k, cos, cos)
        ops.rope_forward(q, k, cos, cos)
    torch.cuda.synchronize()
    assert torch.equal(guard, torch.full_like(guard, 3.0))


def test_swiglu_argument_errors(device):
    a = torch.zeros(4, 4, device=device)
    with pytest.raises(ValueError):
        ops.swiglu_backward(a.clone(), a.clone(), a, a, torch.zeros(4, 5, device=device))
    with pytest.raises(ValueError):
        ops.swiglu_backward(a.clone(), a.clone(), a, a, a.half())
