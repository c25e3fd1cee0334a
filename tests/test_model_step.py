"""The composed train step: the float64 composition is pinned by finite differences (CPU), then
the GPU step (eager and hipGraph replay, dense and cut loss) is compared with it."""
import numpy as np
import pytest
import torch

from oracle import model64
from tests.util import to_np

TINY = dict(vocab=50, layers=2, hidden=32, inter=48, hq=4, hkv=2, d=8, eps=1e-5)


def random_params(cfg, rng, scale=0.3):
    H, I, QW, KW = cfg["hidden"], cfg["inter"], cfg["hq"] * cfg["d"], cfg["hkv"] * cfg["d"]
    layers = []
    for _ in range(cfg["layers"]):
        layers.append({
            "attention_norm": 1 + 0.1 * rng.normal(size=H), "q": scale * rng.normal(size=(QW, H)),
            "k": scale * rng.normal(size=(KW, H)), "q_norm": 1 + 0.1 * rng.normal(size=cfg["d"]),
            "k_norm": 1 + 0.1 * rng.normal(size=cfg["d"]), "v": scale * rng.normal(size=(KW, H)),
            "o": scale * rng.normal(size=(H, QW)), "ffn_norm": 1 + 0.1 * rng.normal(size=H),
            "gate": scale * rng.normal(size=(I, H)), "up": scale * rng.normal(size=(I, H)),
            "down": scale * rng.normal(size=(H, I)),
        })
    return {"embedding": scale * rng.normal(size=(cfg["vocab"], H)), "final_norm": 1 + 0.1 * rng.normal(size=H),
            "layers": layers}


def test_float64_composition_matches_finite_differences():
    """Pins oracle/model64.py: its analytic gradients equal central differences of its own loss,
    for a sample of entries of every parameter tensor (incl. the tied embedding, which receives
    both the classifier and the lookup gradient)."""
    cfg = dict(TINY, layers=2)
    rng = np.random.default_rng(0)
    params = random_params(cfg, rng)
    tokens = rng.integers(0, cfg["vocab"], size=(2, 5))
    targets = rng.integers(0, cfg["vocab"], size=(2, 5))
    tokens[0, 1] = tokens[0, 3]  # a repeated id
    loss, grads, _ = model64.forward_backward(params, tokens, targets, cfg)
    assert np.isfinite(loss)

    def check(array, grad, name):
        flat = array.reshape(-1)
        for idx in rng.choice(flat.size, size=min(6, flat.size), replace=False):
            old = flat[idx]
            flat[idx] = old + 1e-6
            hi = model64.loss_only(params, tokens, targets, cfg)
            flat[idx] = old - 1e-6
            lo = model64.loss_only(params, tokens, targets, cfg)
            flat[idx] = old
            fd = (hi - lo) / 2e-6
            assert abs(fd - grad.reshape(-1)[idx]) <= 1e-6 + 1e-5 * abs(fd), (name, idx, fd, grad.reshape(-1)[idx])

    check(params["embedding"], grads["embedding"], "embedding")
    check(params["final_norm"], grads["final_norm"], "final_norm")
    for l, (w, g) in enumerate(zip(params["layers"], grads["layers"])):
        for key in model64.LAYER_KEYS:
            check(w[key], g[key], f"layer{l}.{key}")
    # the embedding row of a token that is used twice and is also a target gets all three contributions
    used = tokens[0, 1]
    assert np.abs(grads["embedding"][used]).max() > 0


# --------------------------------------------------------------------------------- GPU
def torch_round(dtype):
    def rnd(a):
        return torch.from_numpy(np.asarray(a, dtype=np.float64)).to(torch.float32).to(dtype).to(torch.float64).numpy()
    return rnd


def build(device, dtype, batch, seq, cfg, seed=3):
    from cgpt_amd.model import Model, ModelConfig

    config = ModelConfig(vocabulary_size=cfg["vocab"], num_layers=cfg["layers"], hidden_size=cfg["hidden"],
                         intermediate_size=cfg["inter"], num_query_heads=cfg["hq"], num_kv_heads=cfg["hkv"],
                         head_dim=cfg["d"], rotary_dim=cfg["d"], rms_epsilon=cfg["eps"], dtype=dtype)
    return Model(config, batch, seq, seed=seed, device=device)


def params_from_model(model, cfg):
    """Reads the library's (rounded) weights back as the float64 parameter structure."""
    H, I, QW, KW, D = cfg["hidden"], cfg["inter"], cfg["hq"] * cfg["d"], cfg["hkv"] * cfg["d"], cfg["d"]
    shapes = {"attention_norm": (H,), "q": (QW, H), "k": (KW, H), "q_norm": (D,), "k_norm": (D,), "v": (KW, H),
              "o": (H, QW), "ffn_norm": (H,), "gate": (I, H), "up": (I, H), "down": (H, I)}
    names = {"input_layernorm.weight": "attention_norm", "self_attn.q_proj.weight": "q",
             "self_attn.k_proj.weight": "k", "self_attn.q_norm.weight": "q_norm", "self_attn.k_norm.weight": "k_norm",
             "self_attn.v_proj.weight": "v", "self_attn.o_proj.weight": "o",
             "post_attention_layernorm.weight": "ffn_norm", "mlp.gate_proj.weight": "gate",
             "mlp.up_proj.weight": "up", "mlp.down_proj.weight": "down"}
    params = {"layers": [dict() for _ in range(cfg["layers"])]}
    grads = {"layers": [dict() for _ in range(cfg["layers"])]}
    for name, p, g in model.parameters():
        if name == "model.embed_tokens.weight":
            params["embedding"], grads["embedding"] = to_np(p).reshape(cfg["vocab"], H), g
        elif name == "model.norm.weight":
            params["final_norm"], grads["final_norm"] = to_np(p), g
        else:
            _, _, layer, rest = name.split(".", 3)
            key = names[rest]
            params["layers"][int(layer)][key] = to_np(p).reshape(shapes[key])
            grads["layers"][int(layer)][key] = g
    return params, grads


def compare_gradients(got, want, tol, loss_scale):
    worst = [0.0, ""]

    def one(g, w, name):
        w = np.asarray(w).reshape(-1)
        scale = max(np.abs(w).max(), 1e-3 * loss_scale)
        got_flat = to_np(g).reshape(-1)
        err = np.abs(got_flat - w).max() / scale
        assert np.isfinite(got_flat).all(), name
        if err > worst[0]:
            worst[:] = [err, name]
        assert err <= tol, f"{name}: error {err:.3e} of the tensor's scale"
    one(got["embedding"], want["embedding"], "embedding")
    one(got["final_norm"], want["final_norm"], "final_norm")
    for l, (g, w) in enumerate(zip(got["layers"], want["layers"])):
        for key in model64.LAYER_KEYS:
            one(g[key], w[key], f"layer{l}.{key}")
    print(f"[parity] composed step: worst gradient error {worst[0]:.3e} of its tensor's scale ({worst[1]}; bound {tol:.1e})")


MODEL_CFG = dict(vocab=96, layers=2, hidden=64, inter=128, hq=2, hkv=1, d=32, eps=1e-5)


# Heads of 128 with 256-wide q and k/v projections, 64 rows: the shape class in which the step runs the
# q/k/v projections as one contraction over segmented operands and attention on its head_dim-128 kernels.
WIDE_CFG = dict(vocab=96, layers=1, hidden=256, inter=128, hq=2, hkv=2, d=128, eps=1e-5)


# Three layers with tile-aligned projections (256-wide q, k, v, hidden and [gate | up]) and 64 rows: the shape class in
# which the projections' weight gradients of all layers run as four launches at the end of the backward pass.
STACKED_CFG = dict(vocab=96, layers=3, hidden=256, inter=128, hq=2, hkv=2, d=128, eps=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("loss_mode", [0, 1], ids=["dense", "cut"])
@pytest.mark.parametrize("shape", [(MODEL_CFG, 2, 24), (WIDE_CFG, 2, 32), (STACKED_CFG, 2, 32)],
                         ids=["heads32", "heads128-fused-qkv", "stacked-weight-gradients"])
def test_gpu_step_matches_float64_composition(device, dtype, loss_mode, shape):
    """Hidden 64, 2:1 heads of 32, T=24, B=2, two layers (and the wide-head variant above): every parameter
    gradient of the GPU step against the float64 composition that rounds each operator output to the storage
    dtype where the GPU stores it.
    Tolerance: 3e-2 of each tensor's largest gradient entry (the operators' own bar is 2e-2, and a gradient here has
    passed through several of them; the observed worst is printed)."""
    cfg, batch, seq = shape
    loss_scale = 64.0
    model = build(device, dtype, batch, seq, cfg)
    rng = np.random.default_rng(5)
    tokens = rng.integers(0, cfg["vocab"], size=(batch, seq))
    targets = rng.integers(0, cfg["vocab"], size=(batch, seq))
    tokens[1, 2] = tokens[1, 7]
    model.set_tokens(tokens, targets)
    model.forward_backward(loss_scale, loss_mode, use_graph=False)
    loss, _, _ = model.status()
    params, grads = params_from_model(model, cfg)
    want_loss, want, saved = model64.forward_backward(params, tokens, targets, cfg, loss_scale, torch_round(dtype))
    assert abs(loss - want_loss) <= 2e-2 * want_loss
    for l in range(cfg["layers"] + 1):
        hidden = to_np(model.activation(f"hidden.{l}")).reshape(batch * seq, cfg["hidden"])
        assert np.abs(hidden - saved["hidden"][l]).max() <= 4e-2 * max(1.0, np.abs(saved["hidden"][l]).max())
    compare_gradients(grads, want, 3e-2, loss_scale)
    model.close()


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(16))
def test_gpu_step_matches_float64_composition_on_random_configurations(device, seed):
    """Seeded random small models — 1 to 3 layers, 1 to 4 kv-heads with groups of 1 to 4, heads of 16 to 128, odd
    feed-forward widths, every storage dtype, both loss paths, eager and recorded — against the float64 composition:
    the shape classes in which the step falls back from its fused launches to the separate operators are exactly
    the ones fixed shape lists tend to miss."""
    rng = np.random.default_rng(700 + seed)
    dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
    hkv = int(rng.integers(1, 5))
    hq = hkv * int(rng.integers(1, 5))
    d = [16, 32, 64, 128][int(rng.integers(0, 4))]
    if hq * d > 1024:
        d = 32
    cfg = dict(vocab=int(rng.integers(40, 300)), layers=int(rng.integers(1, 4)), hidden=hq * d,
               inter=int(rng.integers(1, 40)) * 8 if rng.integers(0, 2) else int(rng.integers(8, 300)), hq=hq, hkv=hkv, d=d,
               eps=1e-5)
    batch, seq = int(rng.integers(1, 4)), int(rng.integers(2, 70))
    loss_mode, use_graph = int(rng.integers(0, 2)), bool(rng.integers(0, 2))
    loss_scale = 64.0
    print(f"model {cfg} batch={batch} seq={seq} loss_mode={loss_mode} graph={use_graph} {dtype}", flush=True)
    model = build(device, dtype, batch, seq, cfg, seed=seed)
    tokens = rng.integers(0, cfg["vocab"], size=(batch, seq))
    targets = rng.integers(0, cfg["vocab"], size=(batch, seq))
    model.set_tokens(tokens, targets)
    stream = torch.cuda.Stream(device=device)
    for _ in range(2 if use_graph else 1):  # the second call replays the recorded step
        model.forward_backward(loss_scale, loss_mode, use_graph=use_graph, stream=stream)
    loss, _, _ = model.status(stream)
    params, grads = params_from_model(model, cfg)
    want_loss, want, saved = model64.forward_backward(params, tokens, targets, cfg, loss_scale, torch_round(dtype))
    sixteen = dtype != torch.float32
    assert abs(loss - want_loss) <= (2e-2 if sixteen else 1e-4) * want_loss
    for l in range(cfg["layers"] + 1):
        hidden = to_np(model.activation(f"hidden.{l}")).reshape(batch * seq, cfg["hidden"])
        assert np.abs(hidden - saved["hidden"][l]).max() <= (4e-2 if sixteen else 1e-4) * max(1.0, np.abs(saved["hidden"][l]).max())
    compare_gradients(grads, want, 3e-2 if sixteen else 1e-3, loss_scale)
    model.close()


@pytest.mark.gpu
def test_graph_replay_equals_eager_and_losses_agree_between_modes(device):
    cfg = MODEL_CFG
    dtype = torch.bfloat16
    batch, seq = 2, 40
    rng = np.random.default_rng(6)
    tokens = rng.integers(0, cfg["vocab"], size=(batch, seq))
    targets = rng.integers(0, cfg["vocab"], size=(batch, seq))
    stream = torch.cuda.Stream(device=device)
    results = {}
    for mode in (0, 1):
        model = build(device, dtype, batch, seq, cfg)
        model.set_tokens(tokens, targets)
        model.forward_backward(1024.0, mode, use_graph=False, stream=stream)
        loss_eager = model.status(stream)[0]
        eager = [g.clone() for _, _, g in model.parameters()]
        model.forward_backward(1024.0, mode, use_graph=True, stream=stream)   # eager run + capture
        for replay in range(3):
            for _, _, g in model.parameters():
                g.zero_()
            torch.cuda.synchronize()
            model.forward_backward(1024.0, mode, use_graph=True, stream=stream)  # replay
            loss_graph = model.status(stream)[0]
            assert loss_graph == loss_eager
            for (name, _, g), e in zip(model.parameters(), eager):
                assert torch.equal(g, e), f"{name} differs on replay {replay}"
        results[mode] = (loss_eager, eager)
        model.close()
    assert abs(results[0][0] - results[1][0]) <= 1e-3 * results[0][0]
    for a, b in zip(results[0][1], results[1][1]):
        scale = max(float(a.float().abs().max()), 1e-3)
        assert float((a.float() - b.float()).abs().max()) <= 3e-2 * scale


@pytest.mark.gpu
def test_train_steps_reduce_the_loss_and_count_steps(device):
    cfg = MODEL_CFG
    from cgpt_amd.ops import AdamWOptions

    model = build(device, torch.bfloat16, 4, 32, cfg)
    rng = np.random.default_rng(7)
    tokens = rng.integers(0, cfg["vocab"], size=(4, 32))
    model.set_tokens(tokens, np.roll(tokens, -1, axis=1))
    options = AdamWOptions(learning_rate=1e-2, beta1=0.9, beta2=0.95, weight_decay=0.1, loss_scale=1024.0,
                           max_grad_norm=1.0)
    stream = torch.cuda.Stream(device=device)
    losses = []
    for _ in range(30):
        model.train_step(options, loss_mode=1, use_graph=True, stream=stream)
        losses.append(model.status(stream))
    assert all(finite for _, finite, _ in losses)
    assert losses[-1][2] == 30
    assert losses[-1][0] < 0.5 * losses[0][0]
    assert abs(losses[0][0] - np.log(cfg["vocab"])) < 0.5   # random init: loss starts near ln(vocab)
    model.close()


@pytest.mark.gpu
def test_recorded_train_step_follows_a_changing_learning_rate_and_skips_like_the_eager_one(device):
    """With use_graph the AdamW update is part of the recorded step and reads its options on the device. Two models
    from one seed take the same eight steps, one eagerly and one from the recording, with a learning rate, weight
    decay and clipping norm that change every step and one step whose gradients are made non-finite (both must skip
    it and count it): parameters, master copies and moments agree bit for bit after every step."""
    cfg = MODEL_CFG
    from cgpt_amd.ops import AdamWOptions

    batch, seq = 2, 24
    rng = np.random.default_rng(17)
    tokens = rng.integers(0, cfg["vocab"], size=(batch, seq))
    targets = rng.integers(0, cfg["vocab"], size=(batch, seq))
    stream = torch.cuda.Stream(device=device)
    models = [build(device, torch.bfloat16, batch, seq, cfg, seed=3) for _ in range(2)]
    for model in models:
        model.set_tokens(tokens, targets)
    saved = None
    for step in range(8):
        options = AdamWOptions(learning_rate=1e-2 / (1 + step), beta1=0.9, beta2=0.95, weight_decay=0.1 * (step % 3),
                               loss_scale=256.0, max_grad_norm=[1.0, float("inf"), 0.5][step % 3])
        if step == 4:  # a weight that overflows the forward pass: every gradient becomes non-finite
            saved = [models[i].parameters()[1][1].clone() for i in range(2)]
            for model in models:
                model.parameters()[1][1].fill_(float("inf"))
            torch.cuda.synchronize()
        for use_graph, model in zip((False, True), models):
            model.train_step(options, loss_mode=1, use_graph=use_graph, stream=stream)
        states = [model.status(stream) for model in models]
        assert states[0][1:] == states[1][1:], f"step {step}: {states}"
        assert states[0][1] == (step != 4), f"step {step}: finite flag {states[0][1]}"
        if step == 4:
            for i, model in enumerate(models):
                model.parameters()[1][1].copy_(saved[i])
            torch.cuda.synchronize()
        for index, ((name, p0, _), (_, p1, _)) in enumerate(zip(models[0].parameters(), models[1].parameters())):
            assert torch.equal(p0, p1), f"step {step}: {name} differs between the eager and the recorded step"
            for a, b in zip(models[0].optimizer_state(index), models[1].optimizer_state(index)):
                assert torch.equal(a, b), f"step {step}: optimizer state of {name} differs"
    assert models[0].status(stream)[2] == 7  # eight calls, one skipped
    for model in models:
        model.close()


@pytest.mark.gpu
def test_model_argument_errors(device):
    from cgpt_amd.model import Model, ModelConfig

    with pytest.raises(ValueError):
        Model(ModelConfig(num_query_heads=8, num_kv_heads=3), 1, 8, device=device)
    with pytest.raises(ValueError):
        Model(ModelConfig(hidden_size=1000), 1, 8, device=device)
    model = build(device, torch.bfloat16, 1, 8, MODEL_CFG)
    with pytest.raises(ValueError):
        model.forward_backward(0.0, 1)
    with pytest.raises(ValueError):
        model.forward_backward(1.0, 1, use_graph=True, stream=0)   # capture needs a real stream
    model.close()


def test_cpu_float32_step_matches_float64_composition():
    """oracle/cpu_model.py (the CPU baseline that bench.py times) against oracle/model64.py on a tiny model."""
    from oracle import cpu_model

    cfg = dict(TINY)
    w = cpu_model.make_weights(cfg, seed=1)
    for lw in w["layers"]:
        for key in lw:
            if lw[key].dim() == 2:
                lw[key].mul_(10.0)   # make the gradients large enough to compare
    w["embedding"].mul_(10.0)
    g = torch.Generator().manual_seed(2)
    tokens = torch.randint(0, cfg["vocab"], (2, 6), generator=g)
    targets = torch.randint(0, cfg["vocab"], (2, 6), generator=g)
    params = {"embedding": to_np(w["embedding"]), "final_norm": to_np(w["final_norm"]),
              "layers": [{k: to_np(v) for k, v in lw.items()} for lw in w["layers"]]}
    loss, grads = cpu_model.train_step(w, tokens, targets, cfg, 8.0)
    want_loss, want, _ = model64.forward_backward(params, tokens.numpy(), targets.numpy(), cfg, 8.0)
    assert abs(loss - want_loss) <= 1e-5 * want_loss
    compare_gradients(grads, want, 1e-4, 8.0)


@pytest.mark.gpu
@pytest.mark.parametrize("head_dim,rotary_dim,kv_heads,seq,dtype", [
    (64, 32, 2, 48, torch.bfloat16),     # the general row kernel, part of the head rotated
    (128, 128, 2, 48, torch.bfloat16),   # the kernel for head_dim 128; a group of four k rows spans two tokens
    (128, 128, 1, 333, torch.float16),   # the same with one kv head (four tokens per group), several trips per wavefront
    (128, 128, 4, 47, torch.bfloat16),   # 2 * 47 * 4 = 376 k rows and as many q rows per head group
], ids=["d64-r32", "d128-kv2", "d128-kv1-f16", "d128-kv4"])
def test_fused_qk_norm_rope_is_bit_identical_to_the_separate_operators(device, monkeypatch, head_dim, rotary_dim,
                                                                      kv_heads, seq, dtype):
    """Per-head RMSNorm + rotary embedding run as one pass (forward and backward) when head_dim is
    served by the row kernels; the pass keeps the separate operators' intermediate roundings, so a whole
    step gives the same bits either way. CGPTX_FUSE_QK=0 selects the separate operators."""
    from cgpt_amd.model import LOSS_DENSE, Model, ModelConfig
    config = ModelConfig(vocabulary_size=128, num_layers=2, hidden_size=4 * head_dim, intermediate_size=256,
                         num_query_heads=4, num_kv_heads=kv_heads, head_dim=head_dim, rotary_dim=rotary_dim, dtype=dtype)
    rng = np.random.default_rng(3)
    inputs = rng.integers(0, 128, size=2 * seq).astype(np.uint32)
    targets = rng.integers(0, 128, size=2 * seq).astype(np.uint32)
    results = []
    for fuse in ("1", "0"):
        monkeypatch.setenv("CGPTX_FUSE_QK", fuse)
        model = Model(config, 2, seq, seed=4, device=device)
        model.set_tokens(inputs, targets)
        model.forward_backward(loss_scale=4.0, loss_mode=LOSS_DENSE)
        loss = model.status()[0]
        results.append((loss, [g.clone() for _, _, g in model.parameters()], model.activation("hidden.2").clone()))
    assert results[0][0] == results[1][0]
    assert torch.equal(results[0][2], results[1][2])
    for a, b in zip(results[0][1], results[1][1]):
        assert torch.equal(a, b)


@pytest.mark.gpu
def test_norm_weight_gradients_reduced_at_the_end_of_the_backward_pass_are_bit_identical(device, monkeypatch):
    """The norm-backward passes of a step leave the reduction of their weight-gradient partial sums to one pair of
    launches at the end of the backward pass (same additions, same order); CGPTX_FUSE_DGAMMA=0 reduces after each
    pass. Eager passes (the first sizes the memory for the partial sums and still reduces at once, the later ones
    defer) and graph replays all give the same bits, with the block norms fused and separate."""
    from cgpt_amd.model import LOSS_CUT, Model, ModelConfig
    config = ModelConfig(vocabulary_size=512, num_layers=3, hidden_size=1024, intermediate_size=512, num_query_heads=8,
                         num_kv_heads=2, head_dim=128, rotary_dim=128, dtype=torch.bfloat16)
    batch, seq = 4, 512
    rng = np.random.default_rng(5)
    inputs = rng.integers(0, 512, size=batch * seq).astype(np.uint32)
    targets = rng.integers(0, 512, size=batch * seq).astype(np.uint32)
    stream = torch.cuda.Stream(device=device)

    def gradients(model):
        stream.synchronize()
        return [g.clone() for _, _, g in model.parameters()]

    for norms in ("1", "0"):
        monkeypatch.setenv("CGPTX_FUSE_NORMS", norms)
        monkeypatch.setenv("CGPTX_FUSE_DGAMMA", "0")
        model = Model(config, batch, seq, seed=6, device=device)
        model.set_tokens(inputs, targets)
        model.forward_backward(8.0, LOSS_CUT, use_graph=False, stream=stream)
        want = gradients(model)
        model.close()
        monkeypatch.setenv("CGPTX_FUSE_DGAMMA", "1")
        model = Model(config, batch, seq, seed=6, device=device)
        model.set_tokens(inputs, targets)
        for use_graph in (False, False, True, True, True, False):
            for _, _, g in model.parameters():
                g.zero_()
            torch.cuda.synchronize()
            model.forward_backward(8.0, LOSS_CUT, use_graph=use_graph, stream=stream)
            for (name, _, _), a, b in zip(model.parameters(), gradients(model), want):
                assert torch.equal(a, b), f"{name} (block norms fused: {norms}, graph: {use_graph})"
        model.close()


@pytest.mark.gpu
def test_swiglu_in_the_projection_epilogues_is_bit_identical_to_the_separate_operators(device, monkeypatch):
    """The SwiGLU product rides in the gate/up projection's epilogue and its gradient in the epilogue of the
    down projection's input gradient when the shapes fill the chip (here 4096 rows x 3328 feed-forward
    columns); both work from the rounded 16-bit values the separate operators would exchange, so a whole
    step gives the same bits either way. CGPTX_FUSE_SWIGLU=0 selects the separate operators."""
    from cgpt_amd.model import LOSS_DENSE, Model, ModelConfig
    config = ModelConfig(vocabulary_size=128, num_layers=2, hidden_size=256, intermediate_size=3328, num_query_heads=4,
                         num_kv_heads=2, head_dim=64, rotary_dim=64, dtype=torch.bfloat16)
    rng = np.random.default_rng(5)
    inputs = rng.integers(0, 128, size=4 * 1024).astype(np.uint32)
    targets = rng.integers(0, 128, size=4 * 1024).astype(np.uint32)
    results = []
    for fuse in ("1", "0"):
        monkeypatch.setenv("CGPTX_FUSE_SWIGLU", fuse)
        model = Model(config, 4, 1024, seed=6, device=device)
        model.set_tokens(inputs, targets)
        model.forward_backward(loss_scale=4.0, loss_mode=LOSS_DENSE)
        loss = model.status()[0]
        results.append((loss, [g.clone() for _, _, g in model.parameters()], model.activation("hidden.2").clone()))
    assert np.isfinite(results[0][0]) and results[0][0] == results[1][0]
    assert torch.equal(results[0][2], results[1][2])
    for a, b in zip(results[0][1], results[1][1]):
        assert torch.equal(a, b)


@pytest.mark.gpu
def test_block_norms_in_one_pass_match_the_separate_operators(device, monkeypatch):
    """The attention and feed-forward norms of a block read the same input and run as one pass: forward
    bit-identical; backward adds the two branch gradients before the one rounding instead of rounding
    after each, so gradients agree to storage precision, not bit for bit. CGPTX_FUSE_NORMS=0 selects
    the separate operators."""
    from cgpt_amd.model import LOSS_DENSE, Model, ModelConfig
    config = ModelConfig(vocabulary_size=128, num_layers=2, hidden_size=256, intermediate_size=256, num_query_heads=4,
                         num_kv_heads=2, head_dim=64, rotary_dim=64, dtype=torch.bfloat16)
    rng = np.random.default_rng(5)
    inputs = rng.integers(0, 128, size=2 * 40).astype(np.uint32)
    targets = rng.integers(0, 128, size=2 * 40).astype(np.uint32)
    results = []
    for fuse in ("1", "0"):
        monkeypatch.setenv("CGPTX_FUSE_NORMS", fuse)
        model = Model(config, 2, 40, seed=6, device=device)
        model.set_tokens(inputs, targets)
        model.forward_backward(loss_scale=4.0, loss_mode=LOSS_DENSE)
        loss = model.status()[0]
        results.append((loss, {n: g.float().cpu() for n, _, g in model.parameters()}, model.activation("hidden.2").clone()))
    assert results[0][0] == results[1][0]
    assert torch.equal(results[0][2], results[1][2])
    for name, fused in results[0][1].items():
        separate = results[1][1][name]
        scale = separate.abs().max().item() + 1e-12
        assert (fused - separate).abs().max().item() <= 2e-2 * scale, name


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_weight_gradients_of_all_layers_in_one_launch_agree_with_the_launches_per_layer(device, monkeypatch, dtype):
    """Tile-aligned models leave the projections' weight gradients to the end of the backward pass and compute
    them for all layers at once (CGPTX_STACK_DW=0 keeps one launch per layer and projection). Nothing else
    changes: loss, activations and every other gradient are bit-identical; the projections' weight gradients are
    the same sums over the rows taken in a different number of slices, equal to storage precision; eager and
    recorded passes of the stacked step give the same bits."""
    from cgpt_amd.model import LOSS_CUT, Model, ModelConfig
    config = ModelConfig(vocabulary_size=256, num_layers=4, hidden_size=512, intermediate_size=256, num_query_heads=4,
                         num_kv_heads=2, head_dim=128, rotary_dim=128, dtype=dtype)
    batch, seq = 2, 96
    rng = np.random.default_rng(9)
    inputs = rng.integers(0, 256, size=batch * seq).astype(np.uint32)
    targets = rng.integers(0, 256, size=batch * seq).astype(np.uint32)
    results = {}
    stream = torch.cuda.Stream(device=device)
    for stack in ("1", "0"):
        monkeypatch.setenv("CGPTX_STACK_DW", stack)
        model = Model(config, batch, seq, seed=8, device=device)
        model.set_tokens(inputs, targets)
        model.forward_backward(16.0, LOSS_CUT, use_graph=False, stream=stream)
        stream.synchronize()
        eager = {n: g.clone() for n, _, g in model.parameters()}
        for use_graph in (True, True):
            for _, _, g in model.parameters():
                g.zero_()
            torch.cuda.synchronize()
            model.forward_backward(16.0, LOSS_CUT, use_graph=use_graph, stream=stream)
            stream.synchronize()
            for n, _, g in model.parameters():
                assert torch.equal(g, eager[n]), f"{n}: recorded pass differs from the eager one (stack={stack})"
        results[stack] = (model.status(stream)[0], eager, model.activation(f"hidden.{config.num_layers}").clone())
        model.close()
    assert results["1"][0] == results["0"][0]
    assert torch.equal(results["1"][2], results["0"][2])
    projections = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")
    seen = 0
    for name, stacked in results["1"][1].items():
        separate = results["0"][1][name]
        if any(part in name for part in projections):
            seen += 1
            scale = separate.float().abs().max().item() + 1e-12
            assert (stacked.float() - separate.float()).abs().max().item() <= 1e-2 * scale, name
        else:
            assert torch.equal(stacked, separate), name
    assert seen == 7 * config.num_layers


HEADLINE = dict(vocabulary_size=32000, num_layers=8, hidden_size=1024, intermediate_size=2048, num_query_heads=8,
                num_kv_heads=2, head_dim=128, rotary_dim=128)
HEADLINE_CFG = dict(vocab=32000, layers=8, hidden=1024, inter=2048, hq=8, hkv=2, d=128, eps=1e-5)


# The 12-layer, 768-wide decoder with 12:4 heads of 64 that is named beside the preset as the 104m shape.
SECONDARY = dict(vocabulary_size=32000, num_layers=12, hidden_size=768, intermediate_size=2048, num_query_heads=12,
                 num_kv_heads=4, head_dim=64, rotary_dim=64)


@pytest.mark.gpu
@pytest.mark.parametrize("dims,batch,seq", [(HEADLINE, 32, 1024), (HEADLINE, 8, 4096), (SECONDARY, 32, 1024)],
                         ids=["b32-t1024", "long-context-b8-t4096", "12x768-b32-t1024"])
def test_headline_configuration_scales_exactly_replays_exactly_and_starts_at_the_closed_form_loss(device, dims, batch, seq):
    """The 104m preset at the benchmark's sizes (B=32, T=1024 and the long-context variant B=8, T=4096, bf16) and the
    12 x 768 shape at B=32, T=1024, where no CPU composition finishes in test time: properties that hold at any size.
    The backward pass is linear in the loss scale, and a factor of two is exact in binary floating point, so every
    gradient at scale 2048 is exactly twice the one at 1024; a hipGraph replay repeats the eager pass bit for bit; the
    two loss paths agree; a random-init model starts at the closed-form loss of Gaussian logits."""
    from cgpt_amd.model import LOSS_CUT, LOSS_DENSE, Model, ModelConfig

    config = ModelConfig(dtype=torch.bfloat16, **dims)
    model = Model(config, batch, seq, seed=0, device=device)
    assert model.num_parameters == (104_090_624 if dims is HEADLINE else 100_094_208)
    rng = np.random.default_rng(0)
    model.set_tokens(rng.integers(0, 32000, size=(batch, seq)), rng.integers(0, 32000, size=(batch, seq)))
    stream = torch.cuda.Stream(device=device)

    model.forward_backward(1024.0, LOSS_CUT, use_graph=False, stream=stream)
    loss, _, _ = model.status(stream)
    # Rows leave the final norm with unit RMS and the tied classifier is N(0, 0.02^2): logits are close to
    # N(0, H * 0.02^2) and independent of the target, so E[loss] = ln V + variance / 2.
    assert abs(loss - (np.log(32000.0) + 0.5 * dims["hidden_size"] * 0.02 ** 2)) < 0.02
    base = [g.clone() for _, _, g in model.parameters()]
    for (name, _, _), g in zip(model.parameters(), base):
        assert bool(torch.isfinite(g.float()).all()), name
        assert float(g.float().abs().max()) > 0.0, name

    model.forward_backward(2048.0, LOSS_CUT, use_graph=False, stream=stream)
    assert model.status(stream)[0] == loss
    for (name, _, g), b in zip(model.parameters(), base):
        assert torch.equal(g.float(), 2.0 * b.float()), f"{name}: not exactly twice the gradient at half the scale"

    model.forward_backward(1024.0, LOSS_CUT, use_graph=True, stream=stream)  # eager pass + capture
    for replay in range(2):
        for _, _, g in model.parameters():
            g.zero_()
        torch.cuda.synchronize()
        model.forward_backward(1024.0, LOSS_CUT, use_graph=True, stream=stream)
        assert model.status(stream)[0] == loss
        for (name, _, g), b in zip(model.parameters(), base):
            assert torch.equal(g, b), f"{name} differs on replay {replay}"

    model.forward_backward(1024.0, LOSS_DENSE, use_graph=False, stream=stream)
    assert abs(model.status(stream)[0] - loss) <= 1e-4 * loss
    for (name, _, g), b in zip(model.parameters(), base):
        scale = max(float(b.float().abs().max()), 1e-6)
        assert float((g.float() - b.float()).abs().max()) <= 3e-2 * scale, name
    model.close()


@pytest.mark.gpu
def test_adamw_over_all_104m_parameters_matches_the_float64_update(device):
    """Two full train steps of the 104m preset at B=32, T=1024 (hipGraph step + adamw_step_many_async over the 90
    tensors / 104,090,624 parameters: src/optim/adamw.cu:276-346). After each step the master copies, both
    moments and the 16-bit parameters of every tensor are compared with the float64 update
    (oracle64.adamw: unscale by the loss scale, one global norm over all tensors, clip to 1, bias correction)
    applied to the gradients the step left on the device."""
    from cgpt_amd.model import LOSS_CUT, Model, ModelConfig
    from cgpt_amd.ops import AdamWOptions
    from oracle import oracle64

    batch, seq = 32, 1024
    model = Model(ModelConfig(dtype=torch.bfloat16, **HEADLINE), batch, seq, seed=0, device=device)
    rng = np.random.default_rng(1)
    model.set_tokens(rng.integers(0, 32000, size=(batch, seq)), rng.integers(0, 32000, size=(batch, seq)))
    stream = torch.cuda.Stream(device=device)
    opt = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, wd=0.1, loss_scale=1024.0, max_grad_norm=1.0)
    options = AdamWOptions(learning_rate=opt["lr"], beta1=opt["beta1"], beta2=opt["beta2"], epsilon=opt["eps"],
                           weight_decay=opt["wd"], loss_scale=opt["loss_scale"], max_grad_norm=opt["max_grad_norm"])
    tensors = model.parameters()
    assert len(tensors) == 90 and sum(p.numel() for _, p, _ in tensors) == 104_090_624
    state = [tuple(to_np(t) for t in model.optimizer_state(i)) for i in range(len(tensors))]
    for (name, p, _), (master, m, v) in zip(tensors, state):   # masters start as the 16-bit parameters, moments at 0
        assert np.array_equal(master, to_np(p)), name
        assert not m.any() and not v.any(), name
    step = 0
    eps32 = float(np.finfo(np.float32).eps)
    for _ in range(2):
        model.train_step(options, LOSS_CUT, use_graph=True, stream=stream)
        loss, finite, steps = model.status(stream)
        grads = [to_np(g) for _, _, g in tensors]
        norm = np.sqrt(sum(((g / opt["loss_scale"]) ** 2).sum() for g in grads))
        applied, masters, ms, vs, step = oracle64.adamw(
            None, grads, [s[0] for s in state], [s[1] for s in state], [s[2] for s in state], step, opt["lr"],
            opt["beta1"], opt["beta2"], opt["eps"], opt["wd"], opt["loss_scale"], opt["max_grad_norm"])
        assert applied and finite and steps == step, (loss, finite, steps)
        print(f"[parity] AdamW step {step}: loss {loss:.4f}, unscaled gradient norm {norm:.4f} "
              f"({'clipped' if norm > opt['max_grad_norm'] else 'not clipped'})")
        worst = dict(master=0.0, m=0.0, v=0.0)
        for i, (name, p, _) in enumerate(tensors):
            got_master, got_m, got_v = (to_np(t) for t in model.optimizer_state(i))
            # master: the update is lr-sized on parameters up to 1 (norm weights): a thousandth of lr plus the
            # fp32 representation of the value itself
            bound = 1e-3 * opt["lr"] + 2 * eps32 * np.abs(masters[i])
            err = np.abs(got_master - masters[i])
            assert (err <= bound).all(), f"{name}: master differs by {err.max():.3e}"
            worst["master"] = max(worst["master"], float(err.max()))
            for key, got, want in (("m", got_m, ms[i]), ("v", got_v, vs[i])):
                scale = max(float(np.abs(want).max()), 1e-30)
                rel = float(np.abs(got - want).max()) / scale
                assert rel <= 2e-5, f"{name}: {key} differs by {rel:.3e} of its largest entry"
                worst[key] = max(worst[key], rel)
            # the 16-bit parameter is the master copy rounded to nearest even
            assert torch.equal(p, model.optimizer_state(i)[0].to(torch.bfloat16)), name
            state[i] = (got_master, got_m, got_v)   # the next step starts from what the device holds
        print(f"[parity] AdamW step {step}: worst master error {worst['master']:.3e} (lr {opt['lr']:.0e}), "
              f"worst m {worst['m']:.3e}, v {worst['v']:.3e} of the tensor's largest entry")
    model.close()


def cpu_weights_from_model(model, cfg):
    """The library's weights as the float32 tensors oracle/cpu_model.py takes."""
    params, _ = params_from_model(model, cfg)
    as_f32 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).float().contiguous()
    return {"embedding": as_f32(params["embedding"]), "final_norm": as_f32(params["final_norm"]),
            "layers": [{k: as_f32(v) for k, v in lw.items()} for lw in params["layers"]]}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 4e-2), (torch.float32, 1e-4)], ids=["bf16", "f32"])
def test_cpu_plumbing_configuration_forward_and_loss_against_the_cpu_port(device, dtype, tol):
    """The reference's CPU-runnable configuration: 104m dims, B=1, T=256, forward + cross-entropy loss in the
    order of src/core/generation_cpu.cpp:323-379 + cross_entropy_forward_cpu (oracle/cpu_model.forward_loss, the
    float32 port; about 40 s on one core, since linear_forward_cpu is serial for more than one row). The GPU
    forward runs on the same weights (the CPU side reads the library's rounded weights back): the hidden state
    entering every layer and leaving the last one, and the loss, must agree. bf16 rounds every operator output
    (2e-2 each, several operators deep: 4e-2 of the state's scale); fp32 storage accumulates in a different
    order only (1e-4 of the scale; 2e-6 observed)."""
    from cgpt_amd.model import LOSS_DENSE, Model, ModelConfig
    from oracle import cpu_model

    cfg, batch, seq = HEADLINE_CFG, 1, 256
    model = Model(ModelConfig(dtype=dtype, **HEADLINE), batch, seq, seed=0, device=device)
    g = torch.Generator().manual_seed(1)
    tokens = torch.randint(0, cfg["vocab"], (batch, seq), generator=g)
    targets = torch.randint(0, cfg["vocab"], (batch, seq), generator=g)
    model.set_tokens(tokens.numpy(), targets.numpy())
    model.forward_backward(1.0, LOSS_DENSE, use_graph=False)
    loss, _, _ = model.status()
    want_loss, want_hidden, want_checksum = cpu_model.forward_loss(cpu_weights_from_model(model, cfg), tokens, targets, cfg)
    print(f"[parity] configuration 1 ({dtype}): GPU loss {loss:.6f}, CPU port {want_loss:.6f}, logits checksum {want_checksum:.4f}")
    assert abs(loss - want_loss) <= (5e-3 if dtype == torch.bfloat16 else 1e-4) * want_loss
    for l, want in enumerate(want_hidden):
        got = to_np(model.activation(f"hidden.{l}")).reshape(batch * seq, cfg["hidden"])
        scale = max(1.0, float(want.abs().max()))
        err = float(np.abs(got - to_np(want)).max()) / scale
        print(f"[parity] hidden.{l}: {err:.3e} of scale {scale:.3g}")
        assert err <= tol, f"hidden state {l}: {err:.3e}"
    # the checksum follows from logits that agree element by element: N*V terms with errors below tol each
    logits = to_np(model.activation("logits"))
    assert abs(logits.sum() - want_checksum) <= tol * np.abs(logits).sum()
    model.close()


@pytest.mark.gpu
def test_graph_is_recorded_again_after_the_scratch_arena_moves(device):
    """A recorded step holds addresses inside the stream's scratch arena. Releasing the arena
    (cgptx_release_scratch), or an operator on the same stream that needs a larger one, frees that block: the
    next graph step must notice, run eagerly and record again, and give the same bits as before."""
    from cgpt_amd import capi, ops

    cfg, dtype, batch, seq = MODEL_CFG, torch.bfloat16, 2, 40
    rng = np.random.default_rng(8)
    model = build(device, dtype, batch, seq, cfg)
    model.set_tokens(rng.integers(0, cfg["vocab"], size=(batch, seq)), rng.integers(0, cfg["vocab"], size=(batch, seq)))
    stream = torch.cuda.Stream(device=device)

    def step():
        for _, _, g in model.parameters():
            g.zero_()
        torch.cuda.synchronize()
        model.forward_backward(64.0, 1, use_graph=True, stream=stream)
        return model.status(stream)[0], [g.clone() for _, _, g in model.parameters()]

    step()                      # eager + capture
    want = step()               # replay
    capi.call("cgptx_release_scratch")
    # fill the freed block with other data so that a stale replay could not pass by accident
    junk = [torch.full((1 << 20,), 1e30, device=device) for _ in range(8)]
    after_release = step()
    with torch.cuda.stream(stream):   # a larger request on the same stream reallocates the arena
        big_rows = 1 << 16
        x = torch.randn(big_rows, 1024, device=device).to(dtype)
        dx, dw = torch.empty_like(x), torch.empty(1024, dtype=dtype, device=device)
        ops.rmsnorm_backward(dx, dw, x, x, torch.ones(1024, dtype=dtype, device=device), 1e-5, stream=stream)
    torch.cuda.synchronize()
    after_growth = step()
    replay = step()
    del junk
    for name, (loss, grads) in (("release", after_release), ("growth", after_growth), ("replay", replay)):
        assert loss == want[0], name
        for a, b in zip(grads, want[1]):
            assert torch.equal(a, b), name
    model.close()


@pytest.mark.gpu
def test_step_as_the_reference_call_sequence_agrees_with_the_fused_step(device, monkeypatch):
    """CGPTX_FUSE=0 runs the step as the reference's own call sequence (one public operator per call: separate
    q / k / v and gate / up projections with accumulating input gradients, separate SwiGLU, RoPE and residual
    additions). The default step fuses across those boundaries and rounds less often: the two agree to storage
    precision, the loss almost exactly."""
    from cgpt_amd.model import LOSS_CUT, Model, ModelConfig
    config = ModelConfig(vocabulary_size=512, num_layers=2, hidden_size=256, intermediate_size=512, num_query_heads=2,
                         num_kv_heads=2, head_dim=128, rotary_dim=128, dtype=torch.bfloat16)
    rng = np.random.default_rng(9)
    inputs, targets = rng.integers(0, 512, size=(2, 64)), rng.integers(0, 512, size=(2, 64))
    results = []
    for fuse in ("1", "0"):
        monkeypatch.setenv("CGPTX_FUSE", fuse)
        model = Model(config, 2, 64, seed=6, device=device)
        model.set_tokens(inputs, targets)
        model.forward_backward(loss_scale=64.0, loss_mode=LOSS_CUT)
        results.append((model.status()[0], {n: g.float().cpu() for n, _, g in model.parameters()},
                        model.activation("hidden.2").float().cpu()))
        model.close()
    assert abs(results[0][0] - results[1][0]) <= 1e-3 * results[1][0]
    assert (results[0][2] - results[1][2]).abs().max().item() <= 4e-2 * max(1.0, results[1][2].abs().max().item())
    for name, fused in results[0][1].items():
        separate = results[1][1][name]
        scale = separate.abs().max().item() + 1e-12
        assert (fused - separate).abs().max().item() <= 3e-2 * scale, name
