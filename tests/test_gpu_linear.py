"""GPU parity tests of linear_forward / linear_backward (MFMA contraction kernels and the plain
fallback) against the CPU checker and float64 matmuls, through the C-ABI."""
import numpy as np
import pytest
import torch

from cgpt_amd import ops
from oracle import cpu_ops, oracle64
from tests.util import DTYPES, DTYPE_IDS, TOL, assert_close, randn, to_np

pytestmark = pytest.mark.gpu


def dev(t, device):
    return t.to(device).contiguous()


def test_linear_backward_known_answer_and_accumulation(device):
    """tests/linear_backward_test.cu:20-45 (F32, 2x3)."""
    x = torch.tensor([1, 2, 3, 4, 5, 6.0]).reshape(2, 3).to(device)
    w = torch.tensor([1, 0, 2, -1, 3, 1.0]).reshape(2, 3).to(device)
    dy = torch.tensor([2, -1, 3, 4.0]).reshape(2, 2).to(device)
    gi, gw, gb = torch.zeros(2, 3, device=device), torch.zeros(2, 3, device=device), torch.zeros(2, device=device)
    ops.linear_backward(gi, gw, gb, dy, x, w)
    assert gi.reshape(-1).tolist() == [3, -3, 3, -1, 12, 10]
    assert gw.reshape(-1).tolist() == [14, 19, 24, 15, 18, 21]
    assert gb.tolist() == [5, 3]
    options = ops.LinearBackwardOptions(accumulate_input=True, accumulate_weight=True, accumulate_bias=True)
    ops.linear_backward(gi, gw, gb, dy, x, w, None, None, options)
    assert gi.reshape(-1).tolist() == [6, -6, 6, -2, 24, 20]
    assert gw.reshape(-1).tolist() == [28, 38, 48, 30, 36, 42]
    assert gb.tolist() == [10, 6]


def test_linear_backward_batched_f16_known_answer(device):
    """tests/linear_backward_test.cu:47-58."""
    f16 = torch.float16
    x = torch.tensor([1, 2, 3, 4, 5, 6, 7, 8.0]).reshape(2, 2, 2).to(f16).to(device)
    w = torch.tensor([1, 2, 3, 4, 5, 6.0]).reshape(3, 2).to(f16).to(device)
    dy = torch.arange(1, 13, dtype=torch.float32).reshape(2, 2, 3).to(f16).to(device)
    gi, gw, gb = torch.empty_like(x), torch.empty_like(w), torch.empty(3, dtype=f16, device=device)
    ops.linear_backward(gi, gw, gb, dy, x, w)
    assert np.abs(to_np(gi).reshape(-1) - [22, 28, 49, 64, 76, 100, 103, 136]).max() <= 0.1
    assert np.abs(to_np(gw).reshape(-1) - [118, 140, 134, 160, 150, 180]).max() <= 0.2
    assert np.abs(to_np(gb) - [22, 26, 30]).max() <= 0.1


def check_against_float64(got, want64, dtype, what, terms):
    """A dot product of `terms` rounded inputs: compare relative to the result's scale."""
    scale = max(1.0, float(np.abs(want64).max()))
    err = np.abs(to_np(got) - want64).max()
    assert np.isfinite(to_np(got)).all()
    assert err <= TOL[dtype] * scale, f"{what}: abs err {err:.3e} vs scale {scale:.3e}"


SHAPES = [  # rows, in, out
    (5, 7, 3), (33, 20, 17), (64, 64, 64), (128, 128, 256), (256, 192, 128), (136, 64, 72), (200, 256, 264),
    (384, 1024, 256), (1024, 320, 1024),
    # every reduction length (in for Y, out for dX, rows for dW) is an odd multiple of 32
    (288, 96, 160), (1056, 160, 352),
    # a single K tile; partial tiles in both directions with more work items than persistent blocks
    (64, 32, 64), (1000, 96, 520), (4104, 64, 2056),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows,fin,fout", SHAPES)
def test_linear_forward_backward_parity(device, rows, fin, fout, dtype):
    x, w = randn((rows, fin), dtype, 1), randn((fout, fin), dtype, 2, 0.1)
    dy, b = randn((rows, fout), dtype, 3), randn((fout,), dtype, 4)
    dx_, dw_, ddy_, db_ = dev(x, device), dev(w, device), dev(dy, device), dev(b, device)

    y = torch.empty(rows, fout, dtype=dtype, device=device)
    ops.linear_forward(y, dx_, dw_, None, None, db_)
    check_against_float64(y, oracle64.linear_forward(to_np(x), to_np(w), to_np(b)), dtype, "y", fin)

    gi = torch.full((rows, fin), 5.0, dtype=dtype, device=device)
    gw = torch.full((fout, fin), 5.0, dtype=dtype, device=device)
    gb = torch.full((fout,), 5.0, dtype=dtype, device=device)
    ops.linear_backward(gi, gw, gb, ddy_, dx_, dw_)
    dx64, dw64, db64 = oracle64.linear_backward(to_np(dy), to_np(x), to_np(w))
    check_against_float64(gi, dx64, dtype, "dX", fout)
    check_against_float64(gw, dw64, dtype, "dW", rows)
    check_against_float64(gb, db64, dtype, "db", rows)

    if rows * fin * fout <= 256 * 192 * 128:  # the scalar CPU checker is O(rows*in*out)
        ci, cw, cb = torch.empty_like(x), torch.empty_like(w), torch.empty_like(b)
        cpu_ops.linear_backward(ci, cw, cb, dy, x, w)
        check_against_float64(gi, to_np(ci), dtype, "dX vs checker", fout)
        check_against_float64(gw, to_np(cw), dtype, "dW vs checker", rows)
        check_against_float64(gb, to_np(cb), dtype, "db vs checker", rows)

    # accumulate adds the same product onto what is there
    before = (gi.clone(), gw.clone(), gb.clone())
    options = ops.LinearBackwardOptions(accumulate_input=True, accumulate_weight=True, accumulate_bias=True)
    ops.linear_backward(gi, gw, gb, ddy_, dx_, dw_, None, None, options)
    check_against_float64(gi, to_np(before[0]) + dx64, dtype, "dX accumulate", fout)
    check_against_float64(gw, to_np(before[1]) + dw64, dtype, "dW accumulate", rows)
    check_against_float64(gb, to_np(before[2]) + db64, dtype, "db accumulate", rows)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_linear_backward_integer_valued_inputs_are_exact(device, dtype):
    """Small integers make every product and partial sum exactly representable: the MFMA path (incl. split-K
    for dW) must return the exact integers whatever the summation order."""
    rows, fin, fout = 2048, 256, 128
    g = torch.Generator().manual_seed(5)
    x = torch.randint(-2, 3, (rows, fin), generator=g).to(dtype)
    w = torch.randint(-2, 3, (fout, fin), generator=g).to(dtype)
    dy = torch.randint(-1, 2, (rows, fout), generator=g).to(dtype)
    dx64, dw64, db64 = oracle64.linear_backward(to_np(dy), to_np(x), to_np(w))
    gi = torch.empty(rows, fin, dtype=dtype, device=device)
    gw = torch.empty(fout, fin, dtype=dtype, device=device)
    ops.linear_backward(gi, gw, None, dev(dy, device), dev(x, device), dev(w, device))
    assert np.array_equal(to_np(gi), to_np(torch.tensor(dx64).to(dtype)))
    assert np.array_equal(to_np(gw), to_np(torch.tensor(dw64).to(dtype)))
    y = torch.empty(rows, fout, dtype=dtype, device=device)
    ops.linear_forward(y, dev(x, device), dev(w, device))
    assert np.array_equal(to_np(y), to_np(torch.tensor(to_np(x) @ to_np(w).T).to(dtype)))


def test_linear_backward_layer_shapes_of_the_104m_model(device):
    """One layer's projection shapes at 4096 of the 32768 training rows (k/v 256x1024, q/o 1024x1024,
    gate/up 2048x1024, down 1024x2048), bf16, against float64 matmuls, run twice bit-identically."""
    dtype = torch.bfloat16
    rows = 4096
    for fout, fin in ((256, 1024), (1024, 1024), (2048, 1024), (1024, 2048)):
        x, w, dy = randn((rows, fin), dtype, 6), randn((fout, fin), dtype, 7, 0.02), randn((rows, fout), dtype, 8)
        dx64, dw64, _ = oracle64.linear_backward(to_np(dy), to_np(x), to_np(w))
        outs = []
        for _ in range(2):
            gi = torch.empty(rows, fin, dtype=dtype, device=device)
            gw = torch.empty(fout, fin, dtype=dtype, device=device)
            ops.linear_backward(gi, gw, None, dev(dy, device), dev(x, device), dev(w, device))
            outs.append((gi.cpu(), gw.cpu()))
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
        check_against_float64(outs[0][0], dx64, dtype, f"dX {fout}x{fin}", fout)
        check_against_float64(outs[0][1], dw64, dtype, f"dW {fout}x{fin}", rows)


@pytest.mark.parametrize("fout,fin", [(256, 1024), (1024, 1024), (4096, 1024), (1024, 2048), (32000, 1024)],
                         ids=["kv-256x1024", "q-o-1024x1024", "gate_up-4096x1024", "down-1024x2048", "lm_head-32000x1024"])
def test_linear_backward_at_the_32768_training_rows_sampled_against_float64(device, fout, fin):
    """linear_backward at the real row count of a B=32, T=1024 step (the weight gradient's split-K depth is the 32768
    rows; the classifier shape is the one the cut cross-entropy contracts), bf16. Checked against float64 dot products
    on samples that touch every output tile: 256 rows of dX (two per 256-row tile, all columns), 64 rows and 64 columns
    of dW (all of the other index, i.e. sums over all 32768 rows), with the tolerance of the 16-bit parity bar relative
    to each result's scale. Inputs are made on the device; only the sampled slices travel to the host."""
    dtype = torch.bfloat16
    rows = 32768
    gen = torch.Generator(device=device).manual_seed(fout + fin)
    x = torch.randn(rows, fin, device=device, generator=gen).to(dtype)
    w = (torch.randn(fout, fin, device=device, generator=gen) * 0.02).to(dtype)
    dy = torch.randn(rows, fout, device=device, generator=gen).to(dtype)
    gi = torch.empty(rows, fin, dtype=dtype, device=device)
    gw = torch.empty(fout, fin, dtype=dtype, device=device)
    ops.linear_backward(gi, gw, None, dy, x, w)
    torch.cuda.synchronize()
    rng = np.random.default_rng(fout * 7 + fin)
    # dX rows: two per 256-row tile.
    picked = np.sort(np.concatenate([tile * 256 + rng.choice(256, 2, replace=False) for tile in range(rows // 256)]))
    index = torch.as_tensor(picked, device=device)
    want = to_np(dy[index]) @ to_np(w)
    check_against_float64(gi[index], want, dtype, f"dX rows {fout}x{fin}", fout)
    # dW rows (outputs o) and columns (inputs i), each a sum over all rows: accumulated over row chunks on the host.
    some_out = np.sort(rng.choice(fout, 64, replace=False))
    some_in = np.sort(rng.choice(fin, 64, replace=False))
    out_index, in_index = torch.as_tensor(some_out, device=device), torch.as_tensor(some_in, device=device)
    want_rows = np.zeros((64, fin))
    want_cols = np.zeros((fout, 64))
    for r0 in range(0, rows, 2048):
        dy_chunk, x_chunk = dy[r0:r0 + 2048], x[r0:r0 + 2048]
        want_rows += to_np(dy_chunk[:, out_index]).T @ to_np(x_chunk)
        want_cols += to_np(dy_chunk).T @ to_np(x_chunk[:, in_index])
    check_against_float64(gw[out_index], want_rows, dtype, f"dW rows {fout}x{fin}", rows)
    check_against_float64(gw[:, in_index], want_cols, dtype, f"dW columns {fout}x{fin}", rows)
    # dX columns over all rows for the layer shapes (the classifier's dY is too large to widen on the host).
    if fout <= 4096:
        want_dx_cols = np.concatenate([to_np(dy[r0:r0 + 4096]) @ to_np(w[:, in_index]) for r0 in range(0, rows, 4096)])
        check_against_float64(gi[:, in_index], want_dx_cols, dtype, f"dX columns {fout}x{fin}", fout)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
@pytest.mark.parametrize("count,rows,fout,fin", [
    (8, 2048, 256, 512),    # 16 tiles: the launch splits the row sum
    (3, 1056, 512, 264),    # ragged columns, three slices' worth of K tiles
    (5, 4096, 768, 1024),   # 60 tiles
    (40, 1024, 2048, 256),  # 320 tiles: more than one round of the persistent blocks
    (2, 520, 96, 200),      # out_features not a multiple of 256: separate weight gradients
    (1, 2048, 256, 512),    # a stack of one
], ids=["8x256x512", "3x512x264", "5x768x1024", "40x2048x256", "fallback", "single"])
def test_linear_backward_weights_stacked_matches_float64_and_integers(device, count, rows, fout, fin, dtype):
    """The weight gradients of several layers in one launch against float64 products (the bound of the single
    weight gradient), and exact on small integers whatever the number of slices the launch picks."""
    g = torch.Generator().manual_seed(11)
    dy = (torch.randn((count, rows, fout), generator=g) * 1.0).to(dtype)
    x = (torch.randn((count, rows, fin), generator=g) * 1.0).to(dtype)
    gw = torch.full((count, fout, fin), 7.0, dtype=dtype, device=device)
    ops.linear_backward_weights_stacked(gw, dev(dy, device), dev(x, device))
    for j in range(count):
        want = to_np(dy[j]).T @ to_np(x[j])
        check_against_float64(gw[j].cpu(), want, dtype, f"dW of layer {j}", rows)
    # twice, bit-identical
    again = torch.empty_like(gw)
    ops.linear_backward_weights_stacked(again, dev(dy, device), dev(x, device))
    assert torch.equal(gw, again)
    if dtype != torch.float32:
        dy = torch.randint(-1, 2, (count, rows, fout), generator=g).to(dtype)
        x = torch.randint(-2, 3, (count, rows, fin), generator=g).to(dtype)
        ops.linear_backward_weights_stacked(gw, dev(dy, device), dev(x, device))
        for j in range(count):
            want = torch.tensor(to_np(dy[j]).T @ to_np(x[j])).to(dtype)
            assert np.array_equal(to_np(gw[j]), to_np(want)), f"layer {j}"


def test_linear_backward_weights_stacked_with_strided_layers_and_errors(device):
    """Layers taken out of larger blocks (strides beyond rows x features), and the argument checks."""
    dtype = torch.bfloat16
    count, rows, fout, fin = 4, 1024, 256, 256
    g = torch.Generator().manual_seed(12)
    dy_block = torch.randn((count, rows + 64, fout), generator=g).to(dtype).to(device)
    x_block = torch.randn((count, rows + 32, fin), generator=g).to(dtype).to(device)
    dy, x = dy_block[:, :rows], x_block[:, :rows]
    gw = torch.empty((count, fout, fin), dtype=dtype, device=device)
    ops.linear_backward_weights_stacked(gw, dy, x)
    for j in range(count):
        check_against_float64(gw[j].cpu(), to_np(dy[j]).T @ to_np(x[j]), dtype, f"dW of layer {j}", rows)
    with pytest.raises(ValueError):
        ops.linear_backward_weights_stacked(gw, dy[:3], x)
    with pytest.raises(ValueError):
        ops.linear_backward_weights_stacked(gw, dy, x[:, :, :128])
    with pytest.raises(ValueError):
        ops.linear_backward_weights_stacked(gw.cpu(), dy, x)


def test_linear_argument_errors(device):
    x, w, dy = torch.zeros(4, 8, device=device), torch.zeros(3, 8, device=device), torch.zeros(4, 3, device=device)
    gi, gw, gb = torch.zeros_like(x), torch.zeros_like(w), torch.zeros(3, device=device)
    with pytest.raises(ValueError):
        ops.linear_backward(gi, gw, gb, torch.zeros(4, 4, device=device), x, w)
    with pytest.raises(ValueError):
        ops.linear_backward(gi, gw, gb, dy, x.half(), w)
    with pytest.raises(ValueError):
        ops.linear_backward(gi, torch.zeros(3, 7, device=device), gb, dy, x, w)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("rows,fin,hidden", [(4096, 256, 1664), (4104, 64, 1664), (2056, 96, 3328), (64, 32, 64), (520, 96, 200)],
                         ids=["fused", "fused-ragged-rows", "fused-wide", "small", "unaligned-columns"])
def test_linear_swiglu_forward_equals_the_two_operators(device, rows, fin, hidden, dtype):
    """Gate/up projection with the SwiGLU product from its epilogue (one contraction over interleaved
    gate and up columns when the shape fills the chip) against linear_forward into the concatenated
    layout followed by swiglu_forward: the same bits, and the float64 product within the 16-bit tolerance."""
    g = torch.Generator().manual_seed(rows + hidden)
    x = torch.randn(rows, fin, generator=g).to(dtype).to(device)
    w = (torch.randn(2 * hidden, fin, generator=g) * 0.3).to(dtype).to(device)
    want_gate_up = torch.empty(rows, 2 * hidden, dtype=dtype, device=device)
    want_act = torch.empty(rows, hidden, dtype=dtype, device=device)
    ops.linear_forward(want_gate_up, x, w)
    ops.swiglu_forward(want_act, want_gate_up)
    got_gate_up = torch.full_like(want_gate_up, float("nan"))
    got_act = torch.full_like(want_act, float("nan"))
    ops.linear_swiglu_forward(got_gate_up, got_act, x, w)
    torch.cuda.synchronize()
    assert torch.equal(got_gate_up, want_gate_up)
    assert torch.equal(got_act, want_act)
    exact = x.double().cpu() @ w.double().cpu().t()
    gate, up = exact[:, :hidden], exact[:, hidden:]
    reference = gate / (1 + torch.exp(-gate)) * up
    err = (got_act.double().cpu() - reference).abs().max() / reference.abs().max()
    assert err <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("rows,out,hidden", [(4096, 256, 3328), (4104, 64, 3328), (4096, 96, 3336), (64, 32, 64), (520, 96, 200)],
                         ids=["fused", "fused-ragged-rows", "fused-ragged-columns", "small", "unaligned-columns"])
def test_linear_swiglu_backward_equals_the_two_operators(device, rows, out, hidden, dtype):
    """Input gradient of the down projection with the SwiGLU gradient from its epilogue (when the shape
    fills the chip) against linear_backward followed by the packed swiglu_backward: the same bits, rows and
    columns past the matrix untouched, and the float64 gradient within the 16-bit tolerance."""
    g = torch.Generator().manual_seed(rows + hidden + 1)
    dy = torch.randn(rows, out, generator=g).to(dtype).to(device)
    w = (torch.randn(out, hidden, generator=g) * 0.3).to(dtype).to(device)
    gate_up = torch.randn(rows, 2 * hidden, generator=g).to(dtype).to(device)
    act = torch.empty(rows, hidden, dtype=dtype, device=device)  # the projection's input: unused by its input gradient
    d_act = torch.empty(rows, hidden, dtype=dtype, device=device)
    want = torch.empty(rows, 2 * hidden, dtype=dtype, device=device)
    ops.linear_backward(d_act, None, None, dy, act, w)
    ops.swiglu_backward_packed(want, d_act, gate_up)
    guarded = torch.full((rows + 8, 2 * hidden), 7.0, dtype=dtype, device=device)  # rows after the output
    got = guarded[:rows]
    work = torch.empty_like(d_act)
    ops.linear_swiglu_backward(got, work, dy, w, gate_up)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert bool((guarded[rows:] == 7.0).all())
    exact = dy.double().cpu() @ w.double().cpu()
    gate, up = gate_up.double().cpu()[:, :hidden], gate_up.double().cpu()[:, hidden:]
    sig = 1 / (1 + torch.exp(-gate))
    reference = torch.cat([exact * up * sig * (1 + gate * (1 - sig)), exact * gate * sig], dim=1)
    err = (got.double().cpu() - reference).abs().max() / reference.abs().max()
    assert err <= 2e-2


def test_linear_swiglu_backward_argument_errors(device):
    bf = torch.bfloat16
    dy = torch.zeros(8, 16, dtype=bf, device=device)
    w = torch.zeros(16, 32, dtype=bf, device=device)
    gate_up = torch.zeros(8, 64, dtype=bf, device=device)
    grad = torch.zeros(8, 64, dtype=bf, device=device)
    work = torch.zeros(8, 32, dtype=bf, device=device)
    ops.linear_swiglu_backward(grad, work, dy, w, gate_up)  # valid
    with pytest.raises(ValueError):
        ops.linear_swiglu_backward(grad, torch.zeros(8, 16, dtype=bf, device=device), dy, w, gate_up)
    with pytest.raises(ValueError):
        ops.linear_swiglu_backward(grad, work, dy, torch.zeros(15, 32, dtype=bf, device=device), gate_up)
    with pytest.raises(ValueError):
        ops.linear_swiglu_backward(grad.float(), work, dy, w, gate_up)
    from cgpt_amd import capi
    with pytest.raises(ValueError):  # the C entry point rejects null tensors itself
        capi.call("cgptx_linear_swiglu_backward", grad.data_ptr(), None, dy.data_ptr(), w.data_ptr(), gate_up.data_ptr(),
                  8, 32, 16, 1, None)


def test_linear_swiglu_forward_argument_errors(device):
    x = torch.zeros(8, 32, dtype=torch.bfloat16, device=device)
    w = torch.zeros(64, 32, dtype=torch.bfloat16, device=device)
    gate_up = torch.zeros(8, 64, dtype=torch.bfloat16, device=device)
    act = torch.zeros(8, 32, dtype=torch.bfloat16, device=device)
    ops.linear_swiglu_forward(gate_up, act, x, w)  # valid
    with pytest.raises(ValueError):
        ops.linear_swiglu_forward(gate_up, torch.zeros(8, 16, dtype=torch.bfloat16, device=device), x, w)
    with pytest.raises(ValueError):
        ops.linear_swiglu_forward(gate_up, act, x, torch.zeros(63, 32, dtype=torch.bfloat16, device=device))
    with pytest.raises(ValueError):
        ops.linear_swiglu_forward(gate_up, act.float(), x, w)
    from cgpt_amd import capi
    with pytest.raises(ValueError):  # the C entry point rejects null tensors itself
        capi.call("cgptx_linear_swiglu_forward", None, act.data_ptr(), x.data_ptr(), w.data_ptr(), 8, 32, 32, 1, None)
