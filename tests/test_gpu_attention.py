"""GPU parity tests of causal GQA flash attention (forward with LSE, backward with and without
saved LSE) against the float64 formulas and the float32 CPU checker, through the C-ABI.
Tolerance: max |a-b| / max(1, |b|) <= 2e-2 for fp16 / bf16 storage (the reference's own
test uses 3e-2 absolute, tests/flash_attention_test.cu:342-344)."""
import numpy as np
import pytest
import torch

from cgpt_amd import ops
from oracle import cpu_ops, oracle64
from tests.util import STOL, TOL, assert_close, assert_scaled_close, randn, to_np

pytestmark = pytest.mark.gpu

HALF = [torch.float16, torch.bfloat16]
HALF_IDS = ["f16", "bf16"]


def dev(t, device):
    return t.to(device).contiguous()


def options(c):
    return ops.FlashAttentionOptions(num_query_heads=c["hq"], num_kv_heads=c["hkv"], head_dim=c["d"],
                                     attention_scale=c.get("scale", 0.0), causal=c.get("causal", True),
                                     query_position_offset=c.get("off", 0))


def oracle_args(c):
    return (c["hq"], c["hkv"], c["d"], c.get("scale", 0.0), c.get("causal", True), c.get("off", 0))


def run_forward(device, q, k, v, c):
    out = torch.full_like(q, 7.0, device=device)
    lse = torch.full(q.shape[:3], 7.0, dtype=torch.float32, device=device)
    ops.flash_gqa_attention_forward_with_lse(out, lse, dev(q, device), dev(k, device), dev(v, device), None,
                                             options(c))
    return out, lse


def run_backward(device, do, q, k, v, c, with_lse=True, accumulate=False, base=None):
    dq, dk, dv = (torch.full_like(t, 3.0, device=device) for t in (q, k, v))
    if base is not None:
        dq, dk, dv = (dev(t, device).clone() for t in base)
    dq_, dk_, dv_, ddo = dev(q, device), dev(k, device), dev(v, device), dev(do, device)
    if with_lse:
        out, lse = run_forward(device, q, k, v, c)
        ops.flash_gqa_attention_backward_with_lse(dq, dk, dv, ddo, out, lse, dq_, dk_, dv_, None, options(c),
                                                  accumulate)
    else:
        ops.flash_gqa_attention_backward(dq, dk, dv, ddo, dq_, dk_, dv_, None, options(c), accumulate)
    return dq, dk, dv


def _values(count, phase):
    """Input pattern of tests/flash_attention_test.cu:176-183."""
    i = np.arange(count, dtype=np.float64)
    return 0.45 * np.sin(phase + i * 0.31) + 0.1 * np.cos(i * 0.17)


REFERENCE_CASES = [  # tests/flash_attention_test.cu:365-388
    dict(b=2, qs=3, ks=5, hq=4, hkv=2, d=32, off=2, scale=0.23),
    dict(b=1, qs=3, ks=35, hq=4, hkv=1, d=64, off=32, scale=0.11),
    dict(b=1, qs=3, ks=35, hq=4, hkv=1, d=128, off=32, scale=0.11),
]


@pytest.mark.parametrize("case", range(3))
@pytest.mark.parametrize("with_lse", [False, True])
def test_backward_reference_test_cases(device, case, with_lse):
    c = REFERENCE_CASES[case]
    f16 = torch.float16
    q = torch.tensor(_values(c["b"] * c["qs"] * c["hq"] * c["d"], 0.2)).reshape(c["b"], c["qs"], c["hq"], c["d"])
    k = torch.tensor(_values(c["b"] * c["ks"] * c["hkv"] * c["d"], 0.7)).reshape(c["b"], c["ks"], c["hkv"], c["d"])
    v = torch.tensor(_values(k.numel(), 1.4)).reshape(k.shape)
    do = torch.tensor(_values(q.numel(), 2.1)).reshape(q.shape)
    want = oracle64.attention_backward(do.numpy(), q.numpy(), k.numpy(), v.numpy(), *oracle_args(c))
    got = run_backward(device, do.to(f16), q.to(f16), k.to(f16), v.to(f16), c, with_lse)
    for g, w, name in zip(got, want, ("dQ", "dK", "dV")):
        assert np.abs(to_np(g) - w).max() <= 3e-2, name


CASES = [
    dict(b=2, qs=64, ks=64, hq=8, hkv=2, d=128),                       # training layout, one tile
    dict(b=1, qs=200, ks=200, hq=8, hkv=2, d=128),                     # several tiles, ragged end
    dict(b=2, qs=150, ks=150, hq=12, hkv=4, d=64),                     # secondary shape: group of 3, d 64
    dict(b=1, qs=70, ks=100, hq=4, hkv=2, d=32, off=30, scale=0.2),    # offset, explicit scale, d 32
    dict(b=1, qs=129, ks=257, hq=2, hkv=1, d=64, causal=False),        # non-causal, qs != ks
    dict(b=1, qs=33, ks=33, hq=3, hkv=3, d=24),                        # head_dim below the tile width
    dict(b=3, qs=1, ks=1, hq=2, hkv=1, d=128),                         # a single token
    dict(b=1, qs=130, ks=130, hq=4, hkv=1, d=128, scale=0.05),
    dict(b=1, qs=300, ks=300, hq=4, hkv=2, d=96),                      # padded columns on the 65..128 path, 3 key blocks
    dict(b=1, qs=100, ks=260, hq=2, hkv=1, d=128, causal=False),       # non-causal on the 65..128 path, qs != ks
    dict(b=1, qs=90, ks=150, hq=4, hkv=2, d=72, off=60, scale=0.3),    # offset on the 65..128 path
    dict(b=2, qs=520, ks=520, hq=2, hkv=2, d=128),                     # 5 key blocks: pairs (0,4), (1,3) and 2 alone
]


def make_inputs(c, dtype, seed):
    q = randn((c["b"], c["qs"], c["hq"], c["d"]), dtype, seed)
    k = randn((c["b"], c["ks"], c["hkv"], c["d"]), dtype, seed + 1)
    v = randn((c["b"], c["ks"], c["hkv"], c["d"]), dtype, seed + 2)
    do = randn((c["b"], c["qs"], c["hq"], c["d"]), dtype, seed + 3)
    return q, k, v, do


@pytest.fixture(params=["lds-direct", "register-staged"])
def kernel_family(request, monkeypatch):
    """Both kernel families take every case: the LDS-direct kernels are the default, the register-staged
    ones serve inputs beyond 32-bit offsets and CGPTX_ATTENTION_WIDE=0 (read per call)."""
    if request.param == "register-staged":
        monkeypatch.setenv("CGPTX_ATTENTION_WIDE", "0")
    else:
        monkeypatch.delenv("CGPTX_ATTENTION_WIDE", raising=False)
    return request.param


@pytest.mark.parametrize("dtype", HALF, ids=HALF_IDS)
@pytest.mark.parametrize("case", range(len(CASES)))
def test_forward_parity(device, case, dtype, kernel_family):
    c = CASES[case]
    q, k, v, _ = make_inputs(c, dtype, 10 * case)
    out, lse = run_forward(device, q, k, v, c)
    want_out, want_lse = oracle64.attention_forward(to_np(q), to_np(k), to_np(v), *oracle_args(c))
    assert_close(out, want_out, TOL[dtype], "O")
    assert_close(lse, want_lse, 1e-3, "LSE")
    # no-LSE entry point writes the same output
    out2 = torch.empty_like(out)
    ops.flash_gqa_attention_forward(out2, dev(q, device), dev(k, device), dev(v, device), None, options(c))
    assert torch.equal(out, out2)


@pytest.mark.parametrize("dtype", HALF, ids=HALF_IDS)
@pytest.mark.parametrize("case", range(len(CASES)))
@pytest.mark.parametrize("with_lse", [True, False])
def test_backward_parity(device, case, dtype, with_lse, kernel_family):
    c = CASES[case]
    q, k, v, do = make_inputs(c, dtype, 10 * case)
    want = oracle64.attention_backward(to_np(do), to_np(q), to_np(k), to_np(v), *oracle_args(c))
    got = run_backward(device, do, q, k, v, c, with_lse)
    for g, w, name in zip(got, want, ("dQ", "dK", "dV")):
        # dK/dV sum over up to qs*group terms of rounded products: the bound follows the result's scale
        assert_scaled_close(g, w, STOL[dtype], f"{name} case {case}")


def test_backward_matches_float32_cpu_checker(device):
    """Small shape where the cubic-cost CPU operator finishes quickly; both sides take the same fp16 inputs."""
    c = dict(b=1, qs=40, ks=48, hq=4, hkv=2, d=32, off=8, scale=0.3)
    dtype = torch.float16
    q, k, v, do = make_inputs(c, dtype, 77)
    gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    cpu_ops.attention_backward(gq, gk, gv, do, q, k, v, 4, 2, 32, 0.3, True, 8)
    got = run_backward(device, do, q, k, v, c)
    for g, w, name in zip(got, (gq, gk, gv), ("dQ", "dK", "dV")):
        assert_scaled_close(g, w, STOL[dtype], name)
    out, lse = run_forward(device, q, k, v, c)
    co, cl = torch.empty_like(q), torch.empty(q.shape[:3])
    cpu_ops.attention_forward(co, cl, q, k, v, 4, 2, 32, 0.3, True, 8)
    assert_close(out, co, TOL[dtype], "O")
    assert_close(lse, cl, 1e-3, "LSE")


@pytest.mark.parametrize("with_lse", [True, False])
def test_backward_accumulate_adds_to_existing_gradients(device, with_lse):
    c = CASES[1]
    dtype = torch.bfloat16
    q, k, v, do = make_inputs(c, dtype, 5)
    base = (randn(q.shape, dtype, 91), randn(k.shape, dtype, 92), randn(v.shape, dtype, 93))
    plain = run_backward(device, do, q, k, v, c, with_lse)
    acc = run_backward(device, do, q, k, v, c, with_lse, accumulate=True, base=base)
    for a, p_, b_, name in zip(acc, plain, base, ("dQ", "dK", "dV")):
        want = to_np(p_) + to_np(b_)
        assert_scaled_close(a, want, STOL[dtype], name)


def test_causal_horizon_and_value_gradient_identity(device):
    """Keys beyond offset+qs get exactly zero gradient; since every row of P sums to one,
    Σ_keys dV = Σ_{heads of the group} Σ_queries dO (independent of Q and K)."""
    c = dict(b=2, qs=100, ks=160, hq=8, hkv=2, d=128, off=20)
    dtype = torch.bfloat16
    q, k, v, do = make_inputs(c, dtype, 31)
    dq, dk, dv = run_backward(device, do, q, k, v, c)
    assert torch.all(dk[:, 120:] == 0) and torch.all(dv[:, 120:] == 0)
    lhs = to_np(dv).sum(axis=1)                                        # [b, hkv, d]
    rhs = to_np(do).reshape(2, 100, 2, 4, 128).sum(axis=(1, 3))        # [b, hkv, d]
    assert np.abs(lhs - rhs).max() <= 2e-2 * np.abs(rhs).max()


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (12, 4, 64)], ids=["preset-8:2x128", "secondary-12:4x64"])
def test_training_shape_against_float64_and_determinism(device, hq, hkv, d):
    """B=32, T=1024, bf16, the preset's 8:2 heads of 128 and the 12:4 heads of 64 of the 768-wide shape: two runs are
    bit-identical, the Σ dV identity holds for every batch, and two batches are compared element-wise with the float64
    formulas."""
    c = dict(b=32, qs=1024, ks=1024, hq=hq, hkv=hkv, d=d)
    dtype = torch.bfloat16
    q, k, v, do = make_inputs(c, dtype, 1234)
    first = run_backward(device, do, q, k, v, c)
    second = run_backward(device, do, q, k, v, c)
    for a, b_ in zip(first, second):
        assert torch.equal(a, b_)
    dq, dk, dv = (t.cpu() for t in first)
    lhs = to_np(dv).sum(axis=1)
    rhs = to_np(do).reshape(32, 1024, hkv, hq // hkv, d).sum(axis=(1, 3))
    assert np.abs(lhs - rhs).max() <= 2e-2 * np.abs(rhs).max()
    for bi in (0, 31):
        sl = slice(bi, bi + 1)
        want = oracle64.attention_backward(to_np(do[sl]), to_np(q[sl]), to_np(k[sl]), to_np(v[sl]), hq, hkv, d)
        for g, w, name in zip((dq[sl], dk[sl], dv[sl]), want, ("dQ", "dK", "dV")):
            assert_scaled_close(g, w, STOL[dtype], f"{name} batch {bi}")
        out, lse = run_forward(device, q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), dict(c, b=1))
        wo, wl = oracle64.attention_forward(to_np(q[sl]), to_np(k[sl]), to_np(v[sl]), hq, hkv, d)
        assert_close(out, wo, TOL[dtype], "O")
        assert_close(lse, wl, 1e-3, "LSE")


def test_long_context_variant(device):
    """B=1 slice of the B=8, T=4096 configuration against float64."""
    c = dict(b=1, qs=4096, ks=4096, hq=8, hkv=2, d=128)
    dtype = torch.bfloat16
    q, k, v, do = make_inputs(c, dtype, 99)
    got = run_backward(device, do, q, k, v, c)
    want = oracle64.attention_backward(to_np(do), to_np(q), to_np(k), to_np(v), 8, 2, 128)
    for g, w, name in zip(got, want, ("dQ", "dK", "dV")):
        assert_scaled_close(g, w, STOL[dtype], name)


SCALAR_CASES = [  # served by the scalar family: fp32 storage, head_dim not a multiple of 8, unaligned tensors
    (torch.float32, dict(b=2, qs=40, ks=40, hq=8, hkv=2, d=128)),
    (torch.float32, dict(b=1, qs=33, ks=70, hq=6, hkv=2, d=64, off=37, scale=0.2)),
    (torch.float32, dict(b=1, qs=50, ks=90, hq=2, hkv=1, d=20, causal=False)),
    (torch.float32, dict(b=3, qs=1, ks=1, hq=2, hkv=1, d=128)),
    (torch.float16, dict(b=1, qs=48, ks=48, hq=4, hkv=2, d=36)),
    (torch.bfloat16, dict(b=2, qs=30, ks=45, hq=3, hkv=1, d=100, off=15)),
    (torch.bfloat16, dict(b=1, qs=20, ks=20, hq=2, hkv=2, d=7)),
    (torch.float32, dict(b=1, qs=3, ks=35, hq=4, hkv=1, d=128, off=32, scale=0.11)),  # flash_attention_test.cu:382-388 in fp32
]


@pytest.mark.parametrize("case", range(len(SCALAR_CASES)))
@pytest.mark.parametrize("with_lse", [True, False])
def test_scalar_family_parity(device, case, with_lse):
    """What the reference serves with its warp-per-row kernels (src/ops/backward/attention_backward.cu:352-504,
    2044-2068): fp32 storage and any head_dim up to 128. fp32 storage: max |a-b| / max(1, |b|) <= 1e-4 against
    the float64 formulas; 16-bit storage: 2e-2 of the result's scale."""
    dtype, c = SCALAR_CASES[case]
    q, k, v, do = make_inputs(c, dtype, 100 + case)
    out, lse = run_forward(device, q, k, v, c)
    want_out, want_lse = oracle64.attention_forward(to_np(q), to_np(k), to_np(v), *oracle_args(c))
    assert_close(out, want_out, TOL[dtype], "O")
    assert_close(lse, want_lse, 1e-4 if dtype == torch.float32 else 1e-3, "LSE")
    want = oracle64.attention_backward(to_np(do), to_np(q), to_np(k), to_np(v), *oracle_args(c))
    got = run_backward(device, do, q, k, v, c, with_lse)
    for g, w, name in zip(got, want, ("dQ", "dK", "dV")):
        if dtype == torch.float32:
            assert_close(g, w, TOL[dtype], f"{name} scalar case {case}")
        else:
            assert_scaled_close(g, w, STOL[dtype], f"{name} scalar case {case}")
    base = (randn(q.shape, dtype, 91), randn(k.shape, dtype, 92), randn(v.shape, dtype, 93))
    acc = run_backward(device, do, q, k, v, c, with_lse, accumulate=True, base=base)
    for a, w, b_, name in zip(acc, want, base, ("dQ", "dK", "dV")):
        assert_scaled_close(a, w + to_np(b_), STOL[dtype], f"{name} accumulate")
    again = run_backward(device, do, q, k, v, c, with_lse)
    for a, b_ in zip(got, again):
        assert torch.equal(a, b_)   # no atomics: results do not depend on scheduling


def test_unaligned_tensors_take_the_scalar_family(device):
    """Views that start 2 bytes into an allocation are not 16-byte aligned: same results as the aligned call
    to storage precision (the two families round differently)."""
    c = dict(b=1, qs=64, ks=64, hq=4, hkv=2, d=64)
    dtype = torch.float16
    q, k, v, do = make_inputs(c, dtype, 3)

    def shifted(t):
        flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=device)
        view = flat[1:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 != 0
        return view

    out, lse = torch.empty_like(q, device=device), torch.empty(q.shape[:3], device=device)
    ops.flash_gqa_attention_forward_with_lse(out, lse, shifted(q), shifted(k), shifted(v), None, options(c))
    dq, dk, dv = torch.empty_like(out), torch.empty_like(k, device=device), torch.empty_like(v, device=device)
    ops.flash_gqa_attention_backward_with_lse(dq, dk, dv, shifted(do), out, lse, shifted(q), shifted(k), shifted(v), None,
                                              options(c))
    want = oracle64.attention_backward(to_np(do), to_np(q), to_np(k), to_np(v), *oracle_args(c))
    for g, w, name in zip((dq, dk, dv), want, ("dQ", "dK", "dV")):
        assert_scaled_close(g, w, STOL[dtype], name)


def test_argument_errors(device):
    q = torch.zeros(1, 4, 4, 32, dtype=torch.float16, device=device)
    k = torch.zeros(1, 4, 2, 32, dtype=torch.float16, device=device)
    lse = torch.zeros(1, 4, 4, device=device)
    good = ops.FlashAttentionOptions(4, 2, 32)
    with pytest.raises(ValueError):  # heads not divisible
        ops.flash_gqa_attention_backward(q.clone(), k.clone(), k.clone(), q, q, k, k, None,
                                         ops.FlashAttentionOptions(4, 3, 32))
    with pytest.raises(ValueError):  # causal range exceeds keys
        ops.flash_gqa_attention_backward(q.clone(), k.clone(), k.clone(), q, q, k, k, None,
                                         ops.FlashAttentionOptions(4, 2, 32, query_position_offset=1))
    with pytest.raises(ValueError):  # LSE must be F32 [b, qs, hq]
        ops.flash_gqa_attention_backward_with_lse(q.clone(), k.clone(), k.clone(), q, q, lse.half(), q, k, k, None,
                                                  good)
    with pytest.raises(ValueError):  # gradient shape mismatch
        ops.flash_gqa_attention_backward(q.clone(), q.clone(), k.clone(), q, q, k, k, None, good)
    wide_q = torch.zeros(1, 4, 2, 136, device=device)  # src/ops/backward/attention_backward.cu:1886-1887
    with pytest.raises(ValueError):
        ops.flash_gqa_attention_backward(wide_q.clone(), wide_q.clone(), wide_q.clone(), wide_q, wide_q, wide_q, wide_q, None,
                                         ops.FlashAttentionOptions(2, 2, 136))
