"""Python handle on the C-ABI train step (include/cgptx_train.h).

Mirrors what train/train.cpp keeps per run: model storage, workspaces, optimizer state and the
captured step. torch is used only to expose the library's device buffers as tensors for tests.
"""
from __future__ import annotations

import ctypes
import dataclasses

import numpy as np
import torch

from . import capi
from .ops import AdamWOptions, _stream

LOSS_DENSE, LOSS_CUT = 0, 1

_TORCH = {capi.F16: torch.float16, capi.BF16: torch.bfloat16, capi.F32: torch.float32}
_CODE = {v: k for k, v in _TORCH.items()}


@dataclasses.dataclass
class ModelConfig:
    """TransformerModelOptions of the reference; defaults are its `104m` preset (train/train.cpp:146-148)."""
    vocabulary_size: int = 32000
    num_layers: int = 8
    hidden_size: int = 1024
    intermediate_size: int = 2048
    num_query_heads: int = 8
    num_kv_heads: int = 2
    head_dim: int = 128
    rotary_dim: int = 128
    rms_epsilon: float = 1.0e-5
    rope_base: float = 10000.0
    dtype: torch.dtype = torch.bfloat16

    def to_c(self) -> capi.ModelConfig:
        return capi.ModelConfig(self.vocabulary_size, self.num_layers, self.hidden_size, self.intermediate_size,
                                self.num_query_heads, self.num_kv_heads, self.head_dim, self.rotary_dim,
                                self.rms_epsilon, self.rope_base, _CODE[self.dtype])


def _as_tensor(pointer: int, count: int, dtype: torch.dtype, device) -> torch.Tensor:
    """Wraps library-owned device memory (no copy, no ownership)."""
    class _Holder:
        pass
    holder = _Holder()
    itemsize = torch.empty((), dtype=dtype).element_size()
    holder.__cuda_array_interface__ = {
        "shape": (count,), "typestr": {2: "<u2", 4: "<u4"}[itemsize], "data": (pointer, False), "version": 3,
    }
    raw = torch.as_tensor(holder, device=device)
    return raw.view(dtype)


class Model:
    def __init__(self, config: ModelConfig, batch: int, sequence: int, seed: int = 0, device="cuda:0"):
        self.config, self.batch, self.sequence = config, batch, sequence
        self.device = torch.device(device)
        handle = ctypes.c_void_p()
        c_config = config.to_c()
        capi.call("cgptx_model_create", ctypes.byref(handle), ctypes.byref(c_config), batch, sequence, seed)
        self._handle = handle

    def close(self):
        if getattr(self, "_handle", None):
            capi.lib().cgptx_model_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def num_parameters(self) -> int:
        return capi.lib().cgptx_model_num_parameters(self._handle)

    def set_tokens(self, inputs, targets) -> None:
        a = np.ascontiguousarray(np.asarray(inputs, dtype=np.uint32).reshape(-1))
        b = np.ascontiguousarray(np.asarray(targets, dtype=np.uint32).reshape(-1))
        assert a.size == self.batch * self.sequence == b.size
        capi.call("cgptx_model_set_tokens", self._handle, a.ctypes.data_as(ctypes.c_void_p),
                  b.ctypes.data_as(ctypes.c_void_p))

    def upload_tokens(self, upload: "TokenUpload", stream=None) -> None:
        """Enqueues the asynchronous copy of the upload's acquired slot into the model's token buffers."""
        capi.call("cgptx_model_upload_tokens", self._handle, upload._handle, _stream(stream))

    def save_checkpoint(self, directory, max_position_embeddings=None) -> None:
        """config.json + model.safetensors with the reference exporter's names (directory must exist)."""
        capi.call("cgptx_model_save_checkpoint", self._handle, str(directory).encode(),
                  self.sequence if max_position_embeddings is None else max_position_embeddings)

    def load_checkpoint(self, directory) -> None:
        capi.call("cgptx_model_load_checkpoint", self._handle, str(directory).encode())

    def save_optimizer(self, path, step: int) -> None:
        capi.call("cgptx_model_save_optimizer", self._handle, str(path).encode(), step)

    def load_optimizer(self, path) -> int:
        step = ctypes.c_uint64(0)
        capi.call("cgptx_model_load_optimizer", self._handle, str(path).encode(), ctypes.byref(step))
        return step.value

    def optimizer_state(self, index: int):
        """(master, first moment, second moment) of parameter `index` as flat fp32 views."""
        count = self.parameters()[index][1].numel()
        m, a, b = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
        capi.call("cgptx_model_optimizer_state", self._handle, index, ctypes.byref(m), ctypes.byref(a), ctypes.byref(b))
        return tuple(_as_tensor(x.value, count, torch.float32, self.device) for x in (m, a, b))

    def forward_backward(self, loss_scale=1.0, loss_mode=LOSS_CUT, use_graph=False, stream=None) -> None:
        capi.call("cgptx_model_forward_backward", self._handle, loss_scale, loss_mode, int(use_graph),
                  _stream(stream))

    def optimizer_step(self, options: AdamWOptions, stream=None) -> None:
        c = options.to_c()
        capi.call("cgptx_model_optimizer_step", self._handle, ctypes.byref(c), _stream(stream))

    def train_step(self, options: AdamWOptions, loss_mode=LOSS_CUT, use_graph=True, stream=None) -> None:
        c = options.to_c()
        capi.call("cgptx_model_train_step", self._handle, ctypes.byref(c), loss_mode, int(use_graph),
                  _stream(stream))

    def status(self, stream=None):
        """Synchronises; returns (loss, all_finite, optimizer_step)."""
        loss, finite, step = ctypes.c_float(0), ctypes.c_int(1), ctypes.c_uint64(0)
        capi.call("cgptx_model_status", self._handle, ctypes.byref(loss), ctypes.byref(finite), ctypes.byref(step),
                  _stream(stream))
        return loss.value, bool(finite.value), step.value

    def parameters(self):
        """[(name, parameter tensor, gradient tensor)] as flat views of the library's buffers."""
        out = []
        for i in range(capi.lib().cgptx_model_parameter_count(self._handle)):
            name, p, g, n = ctypes.c_char_p(), ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_size_t()
            capi.call("cgptx_model_parameter", self._handle, i, ctypes.byref(name), ctypes.byref(p), ctypes.byref(g),
                      ctypes.byref(n))
            out.append((name.value.decode(), _as_tensor(p.value, n.value, self.config.dtype, self.device),
                        _as_tensor(g.value, n.value, self.config.dtype, self.device)))
        return out

    def activation(self, name: str) -> torch.Tensor:
        p, n = ctypes.c_void_p(), ctypes.c_size_t()
        capi.call("cgptx_model_activation", self._handle, name.encode(), ctypes.byref(p), ctypes.byref(n))
        dtype = torch.float32 if name == "loss" else self.config.dtype
        return _as_tensor(p.value, n.value, dtype, self.device)

    def profile(self, loss_scale=1.0, loss_mode=LOSS_CUT, stream=None):
        """One eager pass with events around every operator call: {operator kind: milliseconds}."""
        capi.call("cgptx_model_profile", self._handle, loss_scale, loss_mode, _stream(stream))
        out = {}
        for i in range(capi.lib().cgptx_model_profile_count(self._handle)):
            label, ms = ctypes.c_char_p(), ctypes.c_float()
            capi.call("cgptx_model_profile_entry", self._handle, i, ctypes.byref(label), ctypes.byref(ms))
            out[label.value.decode()] = ms.value
        return out


class TokenUpload:
    """Two page-locked host slots for [batch, sequence] input and target ids and their asynchronous
    upload (the reference's pair of data::Batch with data::upload_batch, train/train.cpp:463-465,
    570-574). `acquire()` returns numpy views of the slot to fill next (waiting until its previous
    upload has finished); `Model.upload_tokens` or `submit` enqueues the copies and switches slots."""

    def __init__(self, batch: int, sequence: int):
        self.batch, self.sequence = batch, sequence
        handle = ctypes.c_void_p()
        capi.call("cgptx_token_upload_create", ctypes.byref(handle), batch, sequence)
        self._handle = handle

    def close(self):
        if getattr(self, "_handle", None):
            capi.call("cgptx_token_upload_destroy", self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def acquire(self):
        a, b = ctypes.c_void_p(), ctypes.c_void_p()
        capi.call("cgptx_token_upload_acquire", self._handle, ctypes.byref(a), ctypes.byref(b))
        n = self.batch * self.sequence
        as_array = lambda p: np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_uint32)), shape=(n,))
        return as_array(a), as_array(b)

    def submit(self, device_inputs: torch.Tensor, device_targets: torch.Tensor, stream=None) -> None:
        capi.call("cgptx_token_upload_submit", self._handle, ctypes.c_void_p(device_inputs.data_ptr()),
                  ctypes.c_void_p(device_targets.data_ptr()), _stream(stream))
