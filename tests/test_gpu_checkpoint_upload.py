"""The callers' data formats either side of the train step: safetensors checkpoints with the
reference exporter's names (src/core/huggingface_export.cpp:135-158, 345-380, 400-430) and the
double-buffered page-locked token upload (src/data/dataset_loader.cpp:120-166, train/train.cpp:463-465,
570-574). The files are read back with the independent `safetensors` package, and files written by
that package are loaded by the library."""
import json
import struct

import numpy as np
import pytest
import torch

from cgpt_amd.model import LOSS_CUT, LOSS_DENSE, AdamWOptions, Model, ModelConfig, TokenUpload

pytestmark = pytest.mark.gpu

CFG = dict(vocabulary_size=96, num_layers=2, hidden_size=64, intermediate_size=96, num_query_heads=4, num_kv_heads=2,
           head_dim=16, rotary_dim=16)
BATCH, SEQ = 2, 16


def make(device, seed, dtype=torch.bfloat16):
    return Model(ModelConfig(dtype=dtype, **CFG), BATCH, SEQ, seed=seed, device=device)


def tokens(seed):
    rng = np.random.default_rng(seed)
    return (rng.integers(0, CFG["vocabulary_size"], size=BATCH * SEQ).astype(np.uint32),
            rng.integers(0, CFG["vocabulary_size"], size=BATCH * SEQ).astype(np.uint32))


def reference_names(layers):
    """Tensor list of export_huggingface_model, in its order."""
    names = ["model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"]
    for l in range(layers):
        p = f"model.layers.{l}."
        names += [p + s for s in ("input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight",
                                  "self_attn.q_norm.weight", "self_attn.k_norm.weight", "self_attn.v_proj.weight",
                                  "self_attn.o_proj.weight", "post_attention_layernorm.weight", "mlp.gate_proj.weight",
                                  "mlp.up_proj.weight", "mlp.down_proj.weight")]
    return names


def read_header(path):
    raw = path.read_bytes()
    (size,) = struct.unpack("<Q", raw[:8])
    return size, json.loads(raw[8:8 + size].decode()), raw[8 + size:]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
def test_checkpoint_has_the_reference_layout_and_the_models_values(device, tmp_path, dtype):
    from safetensors.torch import load_file
    model = make(device, 3, dtype)
    model.save_checkpoint(tmp_path, max_position_embeddings=512)
    config = json.loads((tmp_path / "config.json").read_text())
    assert list(config) == ["architectures", "model_type", "torch_dtype", "vocab_size", "hidden_size", "intermediate_size",
                            "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "head_dim",
                            "max_position_embeddings", "rms_norm_eps", "rope_theta", "use_parallel_residual",
                            "tie_word_embeddings"]
    assert config["architectures"] == ["CGPTForCausalLM"] and config["model_type"] == "cgpt"
    assert (config["vocab_size"], config["hidden_size"], config["intermediate_size"], config["num_hidden_layers"]) == (96, 64, 96, 2)
    assert (config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]) == (4, 2, 16)
    assert config["max_position_embeddings"] == 512 and config["rope_theta"] == 10000.0
    assert abs(config["rms_norm_eps"] - 1e-5) < 1e-12 and config["use_parallel_residual"] and config["tie_word_embeddings"]

    size, header, data = read_header(tmp_path / "model.safetensors")
    assert size % 8 == 0
    assert list(header) == reference_names(2)  # names and order
    tag = {torch.bfloat16: "BF16", torch.float16: "F16", torch.float32: "F32"}[dtype]
    end = 0
    for name, entry in header.items():
        assert entry["dtype"] == tag and entry["data_offsets"][0] == end  # contiguous, in order
        end = entry["data_offsets"][1]
    assert end == len(data)
    H, I, QW, KW = 64, 96, 64, 32
    assert header["model.embed_tokens.weight"]["shape"] == [96, H] and header["lm_head.weight"]["shape"] == [96, H]
    assert header["model.layers.1.self_attn.q_proj.weight"]["shape"] == [QW, H]
    assert header["model.layers.1.self_attn.k_proj.weight"]["shape"] == [KW, H]
    assert header["model.layers.0.self_attn.o_proj.weight"]["shape"] == [H, QW]
    assert header["model.layers.0.mlp.up_proj.weight"]["shape"] == [I, H]
    assert header["model.layers.0.mlp.down_proj.weight"]["shape"] == [H, I]
    assert header["model.layers.0.self_attn.q_norm.weight"]["shape"] == [16]

    loaded = load_file(str(tmp_path / "model.safetensors"))  # the independent reader
    for name, value, _ in model.parameters():
        assert torch.equal(loaded[name].reshape(-1), value.cpu()), name
    assert torch.equal(loaded["lm_head.weight"], loaded["model.embed_tokens.weight"])  # tied


def test_checkpoint_round_trip_and_a_file_written_by_the_safetensors_package(device, tmp_path):
    from safetensors.torch import load_file, save_file
    a, b, c = make(device, 0), make(device, 1), make(device, 2)
    assert not torch.equal(a.parameters()[0][1], b.parameters()[0][1])
    a.save_checkpoint(tmp_path)
    b.load_checkpoint(tmp_path)
    for (name, pa, _), (_, pb, _) in zip(a.parameters(), b.parameters()):
        assert torch.equal(pa, pb), name
    # masters restart from the loaded values
    for i, (_, value, _) in enumerate(b.parameters()):
        assert torch.equal(b.optimizer_state(i)[0], value.float())
    # the package writes keys sorted and adds a __metadata__ object: still loads
    other = tmp_path / "other"
    other.mkdir()
    save_file(load_file(str(tmp_path / "model.safetensors")), str(other / "model.safetensors"), metadata={"format": "pt"})
    c.load_checkpoint(other)
    inputs, targets = tokens(5)
    losses = []
    for m in (a, b, c):
        m.set_tokens(inputs, targets)
        m.forward_backward(loss_mode=LOSS_DENSE)
        losses.append(m.status()[0])
    assert losses[0] == losses[1] == losses[2]


def test_checkpoint_errors_name_the_tensor(device, tmp_path):
    from safetensors.torch import load_file, save_file
    model = make(device, 0)
    with pytest.raises(RuntimeError, match="cannot open"):
        model.load_checkpoint(tmp_path)
    model.save_checkpoint(tmp_path)
    tensors = load_file(str(tmp_path / "model.safetensors"))
    missing = dict(tensors)
    del missing["model.layers.1.mlp.up_proj.weight"]
    (tmp_path / "m").mkdir()
    save_file(missing, str(tmp_path / "m" / "model.safetensors"))
    with pytest.raises(RuntimeError, match="missing tensor model.layers.1.mlp.up_proj.weight"):
        model.load_checkpoint(tmp_path / "m")
    wrong = dict(tensors)
    wrong["model.norm.weight"] = torch.ones(65, dtype=torch.bfloat16)
    (tmp_path / "w").mkdir()
    save_file(wrong, str(tmp_path / "w" / "model.safetensors"))
    with pytest.raises(RuntimeError, match="shape mismatch for tensor model.norm.weight"):
        model.load_checkpoint(tmp_path / "w")
    wrong = dict(tensors)
    wrong["model.norm.weight"] = torch.ones(64, dtype=torch.float32)
    (tmp_path / "d").mkdir()
    save_file(wrong, str(tmp_path / "d" / "model.safetensors"))
    with pytest.raises(RuntimeError, match="dtype mismatch for tensor model.norm.weight"):
        model.load_checkpoint(tmp_path / "d")
    (tmp_path / "t").mkdir()
    (tmp_path / "t" / "model.safetensors").write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(RuntimeError, match="invalid header"):
        model.load_checkpoint(tmp_path / "t")


def test_training_resumes_bit_identically_from_weights_plus_optimizer_state(device, tmp_path):
    options = AdamWOptions(learning_rate=1e-2, weight_decay=0.1, max_grad_norm=1.0, loss_scale=8.0)
    a = make(device, 0)
    batches = [tokens(s) for s in range(4)]
    for inputs, targets in batches[:2]:
        a.set_tokens(inputs, targets)
        a.train_step(options, loss_mode=LOSS_CUT, use_graph=False)
    _, finite, step = a.status()
    assert finite and step == 2
    a.save_checkpoint(tmp_path)
    a.save_optimizer(tmp_path / "optimizer.safetensors", step)
    _, header, _ = read_header(tmp_path / "optimizer.safetensors")
    assert header["step"] == {"dtype": "U64", "shape": [1], "data_offsets": [0, 8]}
    assert header["model.norm.weight.exp_avg_sq"]["dtype"] == "F32"

    b = make(device, 7)
    b.load_checkpoint(tmp_path)
    assert b.load_optimizer(tmp_path / "optimizer.safetensors") == 2
    for inputs, targets in batches[2:]:
        for m in (a, b):
            m.set_tokens(inputs, targets)
            m.train_step(options, loss_mode=LOSS_CUT, use_graph=False)
    la, fa, sa = a.status()
    lb, fb, sb = b.status()
    assert (la, fa, sa) == (lb, fb, sb) and sa == 4
    for i, ((name, pa, _), (_, pb, _)) in enumerate(zip(a.parameters(), b.parameters())):
        assert torch.equal(pa, pb), name
        for x, y in zip(a.optimizer_state(i), b.optimizer_state(i)):
            assert torch.equal(x, y), name


def test_double_buffered_upload_feeds_eager_and_captured_steps(device):
    stream = torch.cuda.Stream(device=device)
    direct, fed = make(device, 0), make(device, 0)
    upload = TokenUpload(BATCH, SEQ)
    slots = []
    for step in range(5):
        inputs, targets = tokens(10 + step)
        direct.set_tokens(inputs, targets)
        direct.forward_backward(loss_mode=LOSS_CUT, use_graph=False)
        expected = direct.status()[0]
        host_inputs, host_targets = upload.acquire()
        slots.append(host_inputs.ctypes.data)
        host_inputs[:] = inputs
        host_targets[:] = targets
        with torch.cuda.stream(stream):
            fed.upload_tokens(upload, stream=stream)
            fed.forward_backward(loss_mode=LOSS_CUT, use_graph=step >= 1, stream=stream)  # captured from step 1 on
        # the next slot can be filled while this step runs: it is the other buffer
        assert fed.status(stream=stream)[0] == expected, step
    assert slots[0] != slots[1] and slots[0] == slots[2] == slots[4] and slots[1] == slots[3]
    assert torch.equal(fed.activation("loss").cpu(), direct.activation("loss").cpu())


def test_upload_into_plain_device_buffers_and_argument_errors(device):
    upload = TokenUpload(3, 5)
    dst_inputs = torch.zeros(15, dtype=torch.int32, device=device)
    dst_targets = torch.zeros(15, dtype=torch.int32, device=device)
    with pytest.raises(ValueError):
        upload.submit(dst_inputs, dst_targets)  # nothing acquired yet
    for round_ in range(3):
        a, b = upload.acquire()
        a[:] = np.arange(15) + 100 * round_
        b[:] = np.arange(15)[::-1] + 100 * round_
        upload.submit(dst_inputs, dst_targets)
        torch.cuda.synchronize()
        assert dst_inputs.cpu().tolist() == (np.arange(15) + 100 * round_).tolist()
        assert dst_targets.cpu().tolist() == (np.arange(15)[::-1] + 100 * round_).tolist()
    model = make(device, 0)
    upload.acquire()
    with pytest.raises(ValueError, match="do not match"):
        model.upload_tokens(upload)  # 15 tokens for a 32-token step
    empty = TokenUpload(0, 7)
    a, b = empty.acquire()
    assert a.size == 0
    empty.submit(dst_inputs, dst_targets)
