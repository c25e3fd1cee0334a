"""Host-side mirror of the reference operator interface over the C-ABI.

Function names, argument order (outputs first, then inputs, then stream and
options) and error behaviour follow the free functions of the reference's
include/ops/** and include/optim/**; tensors are torch device tensors used
only as owners of HBM. Argument errors raise ValueError / OverflowError where
the reference throws std::invalid_argument / std::overflow_error, before
anything is launched. Every call goes through libcgptx.so; there is no other
implementation behind these functions.
"""
from __future__ import annotations

import ctypes
import dataclasses
import math
from typing import Optional, Sequence

import torch

from . import capi

_DTYPE = {torch.float16: capi.F16, torch.bfloat16: capi.BF16, torch.float32: capi.F32}


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}") from None


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream(stream) -> ctypes.c_void_p:
    if stream is None:
        stream = torch.cuda.current_stream()
    if isinstance(stream, torch.cuda.Stream):
        return ctypes.c_void_p(stream.cuda_stream)
    return ctypes.c_void_p(int(stream))


def _require_device(name: str, *tensors: torch.Tensor) -> None:
    for t in tensors:
        if t.device.type != "cuda":
            raise ValueError(f"{name}: all tensors must be device tensors")
        if not t.is_contiguous():
            raise ValueError(f"{name}: tensors must be contiguous")


def _same_dtype(name: str, *tensors: torch.Tensor) -> None:
    for t in tensors:
        if t.dtype != tensors[0].dtype or t.dtype not in _DTYPE:
            raise ValueError(f"{name}: all tensors must have the same floating dtype")


def _ids(name: str, ids: torch.Tensor, count: int) -> None:
    if ids is None or ids.device.type != "cuda" or ids.dtype not in (torch.int32, torch.uint32) or ids.numel() < count:
        raise ValueError(f"{name}: token ids must be a device uint32 buffer with at least token_count entries")


# ---------------------------------------------------------------------------- options
@dataclasses.dataclass
class RopeOptions:  # include/ops/rope.h:6-11
    rotary_dim: int = 0
    position_offset: int = 0


@dataclasses.dataclass
class FlashAttentionOptions:  # include/ops/attention.h:8-32
    num_query_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    attention_scale: float = 0.0
    causal: bool = True
    query_position_offset: int = 0
    key_tile_size: int = 16
    block_size: int = 128
    use_tensor_cores: bool = True


@dataclasses.dataclass
class SwiGLUBackwardOptions:  # include/ops/backward/swiglu_backward.h:6-13
    accumulate_gate: bool = False
    accumulate_up: bool = False
    accumulate_gate_up: bool = False


@dataclasses.dataclass
class LinearBackwardOptions:  # include/ops/backward/linear_backward.h:10-22
    compute_type: str = "F32"
    workspace_bytes: int = 32 * 1024 * 1024
    accumulate_input: bool = False
    accumulate_weight: bool = False
    accumulate_bias: bool = False


@dataclasses.dataclass
class EmbeddingBackwardOptions:  # include/ops/backward/embedding_backward.h:6-14
    block_size: int = 0
    bounds_check: bool = True
    accumulate_weight: bool = False


@dataclasses.dataclass
class AdamWOptions:  # include/optim/adamw.h:12-27
    learning_rate: float = 1.0e-3
    beta1: float = 0.9
    beta2: float = 0.999
    epsilon: float = 1.0e-8
    weight_decay: float = 1.0e-2
    loss_scale: float = 1.0
    max_grad_norm: float = float("inf")

    def to_c(self) -> capi.AdamWOptions:
        return capi.AdamWOptions(self.learning_rate, self.beta1, self.beta2, self.epsilon, self.weight_decay,
                                 self.loss_scale, self.max_grad_norm)


# --------------------------------------------------------------------------- backward
def rmsnorm_backward(grad_input, grad_weight, grad_output, input, weight, epsilon, stream=None):
    """include/ops/backward/rmsnorm_backward.h:21-29."""
    name = "rmsnorm_backward"
    if not (math.isfinite(epsilon) and epsilon > 0):
        raise ValueError(f"{name}: epsilon must be finite and positive")
    _require_device(name, grad_input, grad_weight, grad_output, input, weight)
    _same_dtype(name, input, grad_input, grad_weight, grad_output, weight)
    if input.dim() != 2 or grad_output.shape != input.shape or grad_input.shape != input.shape:
        raise ValueError(f"{name}: input, grad_output and grad_input must have shape [rows, hidden]")
    if weight.dim() != 1 or grad_weight.dim() != 1 or weight.shape[0] != input.shape[1] or \
            grad_weight.shape[0] != input.shape[1]:
        raise ValueError(f"{name}: weight and grad_weight must have shape [hidden]")
    capi.call("cgptx_rmsnorm_backward", _ptr(grad_input), _ptr(grad_weight), _ptr(grad_output), _ptr(input),
              _ptr(weight), input.shape[0], input.shape[1], epsilon, _code(input), _stream(stream))


def _rope_check(name, q, k, cos_cache, sin_cache, options):
    for t in (q, k):
        if t.dim() != 4:
            raise ValueError(f"{name}: tensors must have shape [batch, sequence, heads, head_dim]")
    if q.shape[0] != k.shape[0] or q.shape[1] != k.shape[1] or q.shape[3] != k.shape[3]:
        raise ValueError(f"{name}: incompatible Q/K shapes")
    if cos_cache.dim() != 2 or sin_cache.shape != cos_cache.shape:
        raise ValueError(f"{name}: caches must have identical [max_sequence, rotary_dim / 2] shapes")
    rotary = options.rotary_dim or q.shape[3]
    if cos_cache.shape[1] * 2 != rotary:
        raise ValueError(f"{name}: cache does not cover the requested rotary positions")


def rope_backward(grad_query, grad_key, grad_rotated_query, grad_rotated_key, cos_cache, sin_cache, stream=None,
                  rope_options: RopeOptions = RopeOptions()):
    """include/ops/backward/rope_backward.h:22-31."""
    name = "rope_backward"
    _require_device(name, grad_query, grad_key, grad_rotated_query, grad_rotated_key, cos_cache, sin_cache)
    _same_dtype(name, grad_query, grad_key, grad_rotated_query, grad_rotated_key, cos_cache, sin_cache)
    if grad_query.shape != grad_rotated_query.shape or grad_key.shape != grad_rotated_key.shape:
        raise ValueError(f"{name}: incompatible Q/K gradient shapes")
    _rope_check(name, grad_query, grad_key, cos_cache, sin_cache, rope_options)
    b, s, hq, d = grad_query.shape
    capi.call("cgptx_rope_backward", _ptr(grad_query), _ptr(grad_key), _ptr(grad_rotated_query),
              _ptr(grad_rotated_key), _ptr(cos_cache), _ptr(sin_cache), b, s, hq, grad_key.shape[2], d,
              rope_options.rotary_dim, rope_options.position_offset, cos_cache.shape[0], _code(grad_query),
              _stream(stream))


def swiglu_backward(grad_gate, grad_up, grad_output, gate, up, stream=None,
                    options: SwiGLUBackwardOptions = SwiGLUBackwardOptions()):
    """include/ops/backward/swiglu_backward.h:30-38."""
    name = "swiglu_backward"
    _require_device(name, grad_gate, grad_up, grad_output, gate, up)
    _same_dtype(name, grad_output, grad_gate, grad_up, gate, up)
    for t in (grad_gate, grad_up, gate, up):
        if t.shape != grad_output.shape:
            raise ValueError(f"{name}: all tensors must have the same shape")
    capi.call("cgptx_swiglu_backward", _ptr(grad_gate), _ptr(grad_up), _ptr(grad_output), _ptr(gate), _ptr(up),
              grad_output.numel(), int(options.accumulate_gate), int(options.accumulate_up), _code(gate),
              _stream(stream))


def swiglu_backward_packed(grad_gate_up, grad_output, gate_up, stream=None,
                           options: SwiGLUBackwardOptions = SwiGLUBackwardOptions()):
    """Packed [.., 2*hidden] = [gate | up] overload (src/ops/backward/swiglu_backward.cu:830-883)."""
    name = "swiglu_backward"
    _require_device(name, grad_gate_up, grad_output, gate_up)
    _same_dtype(name, grad_output, grad_gate_up, gate_up)
    hidden = grad_output.shape[-1]
    if gate_up.dim() < 1 or gate_up.shape[-1] != 2 * hidden or gate_up.numel() != 2 * grad_output.numel() or \
            grad_gate_up.shape != gate_up.shape:
        raise ValueError(f"{name}: invalid fused tensors")
    if grad_output.numel() == 0:
        return  # nothing to do (src/ops/backward/swiglu_backward.cu:839-841)
    capi.call("cgptx_swiglu_backward_packed", _ptr(grad_gate_up), _ptr(grad_output), _ptr(gate_up),
              grad_output.numel() // hidden, hidden, int(options.accumulate_gate_up), _code(gate_up), _stream(stream))


def linear_backward(grad_input, grad_weight, grad_bias, grad_output, input, weight, gemm_context=None, stream=None,
                    options: LinearBackwardOptions = LinearBackwardOptions()):
    """include/ops/backward/linear_backward.h:36-46 (gemm_context stands where the cuBLASLt context is)."""
    name = "linear_backward"
    present = [t for t in (grad_input, grad_weight, grad_bias) if t is not None]
    _require_device(name, grad_output, input, weight, *present)
    _same_dtype(name, input, grad_output, weight, *present)
    if input.dim() < 1 or weight.dim() != 2 or grad_output.dim() != input.dim() or \
            input.shape[-1] != weight.shape[1] or grad_output.shape[-1] != weight.shape[0] or \
            tuple(grad_output.shape[:-1]) != tuple(input.shape[:-1]):
        raise ValueError(f"{name}: incompatible tensors")
    if grad_input is not None and grad_input.shape != input.shape:
        raise ValueError(f"{name}: grad_input must match input")
    if grad_weight is not None and grad_weight.shape != weight.shape:
        raise ValueError(f"{name}: grad_weight must match weight")
    if grad_bias is not None and (grad_bias.dim() != 1 or grad_bias.shape[0] != weight.shape[0]):
        raise ValueError(f"{name}: grad_bias must have shape [out_features]")
    out_features, in_features = weight.shape
    capi.call("cgptx_linear_backward", _ptr(grad_input), _ptr(grad_weight), _ptr(grad_bias), _ptr(grad_output),
              _ptr(input), _ptr(weight), input.numel() // in_features, in_features, out_features,
              int(options.accumulate_input), int(options.accumulate_weight), int(options.accumulate_bias),
              _code(input), _stream(stream))


def embedding_backward(grad_weight, grad_output, device_token_ids, token_count, stream=None,
                       options: EmbeddingBackwardOptions = EmbeddingBackwardOptions()):
    """include/ops/backward/embedding_backward.h:35-42."""
    name = "embedding_backward"
    _require_device(name, grad_weight, grad_output)
    _same_dtype(name, grad_weight, grad_output)
    if token_count == 0:
        raise ValueError(f"{name}: token_count must be positive")
    _ids(name, device_token_ids, token_count)
    if grad_weight.dim() != 2 or grad_output.dim() < 1 or grad_output.shape[-1] != grad_weight.shape[1] or \
            grad_output.numel() != token_count * grad_weight.shape[1]:
        raise ValueError(f"{name}: incompatible tensors or token count")
    capi.call("cgptx_embedding_backward", _ptr(grad_weight), _ptr(grad_output), _ptr(device_token_ids), token_count,
              grad_weight.shape[0], grad_weight.shape[1], int(options.bounds_check), int(options.accumulate_weight),
              _code(grad_weight), _stream(stream))


def _ce_check(name, loss, logits, targets, target_count):
    if target_count == 0 or logits.dim() != 2 or logits.shape[0] != target_count or logits.shape[1] == 0:
        raise ValueError(f"{name}: logits must be [target_count, vocabulary] with a positive target count")
    if loss.dtype != torch.float32 or loss.numel() != 1 or loss.device.type != "cuda":
        raise ValueError(f"{name}: loss must be a device F32 tensor with shape [1]")
    _ids(name, targets, target_count)


def cross_entropy_forward_backward(loss, gradient, logits, device_targets, target_count, stream=None,
                                   gradient_scale: float = 1.0):
    """include/ops/cross_entropy.h:25-32."""
    name = "cross_entropy_forward_backward"
    _require_device(name, gradient, logits)
    _same_dtype(name, logits, gradient)
    _ce_check(name, loss, logits, device_targets, target_count)
    if gradient.shape != logits.shape or not (math.isfinite(gradient_scale) and gradient_scale > 0):
        raise ValueError(f"{name}: invalid gradient tensor or scale")
    capi.call("cgptx_cross_entropy_forward_backward", _ptr(loss), _ptr(gradient), _ptr(logits),
              _ptr(device_targets), logits.shape[0], logits.shape[1], gradient_scale, _code(logits), _stream(stream))


def cross_entropy_forward(loss, logits, device_targets, target_count, stream=None):
    """include/ops/cross_entropy.h:37-42."""
    name = "cross_entropy_forward"
    _require_device(name, logits)
    _same_dtype(name, logits)
    _ce_check(name, loss, logits, device_targets, target_count)
    capi.call("cgptx_cross_entropy_forward", _ptr(loss), _ptr(logits), _ptr(device_targets), logits.shape[0],
              logits.shape[1], _code(logits), _stream(stream))


def cut_cross_entropy_forward_backward(loss, input_gradient, classifier_gradient, input, classifier, device_targets,
                                       target_count, stream=None, gradient_scale: float = 1.0,
                                       accumulate_classifier: bool = False):
    """include/ops/cut_cross_entropy.h:25-33; gradient_scale and accumulate_classifier are extensions."""
    name = "cut_cross_entropy_forward_backward"
    _require_device(name, input_gradient, classifier_gradient, input, classifier)
    _same_dtype(name, input, input_gradient, classifier_gradient, classifier)
    if input.dim() != 2 or classifier.dim() != 2 or input.shape[1] != classifier.shape[1] or \
            input.shape[0] != target_count or target_count == 0 or input_gradient.shape != input.shape or \
            classifier_gradient.shape != classifier.shape:
        raise ValueError(f"{name}: incompatible tensors")
    if loss.dtype != torch.float32 or loss.numel() != 1 or loss.device.type != "cuda":
        raise ValueError(f"{name}: loss must be a device F32 tensor with shape [1]")
    _ids(name, device_targets, target_count)
    capi.call("cgptx_cut_cross_entropy_forward_backward", _ptr(loss), _ptr(input_gradient),
              _ptr(classifier_gradient), _ptr(input), _ptr(classifier), _ptr(device_targets), input.shape[0],
              input.shape[1], classifier.shape[0], gradient_scale, int(accumulate_classifier), _code(input),
              _stream(stream))


def _attention_check(name, q, k, v, options: FlashAttentionOptions, others=()):
    _same_dtype(name, q, k, v, *others)
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape or not options.num_query_heads or \
            not options.num_kv_heads or not options.head_dim or options.num_query_heads % options.num_kv_heads or \
            q.shape[0] != k.shape[0] or q.shape[2] != options.num_query_heads or \
            k.shape[2] != options.num_kv_heads or q.shape[3] != options.head_dim or \
            k.shape[3] != options.head_dim or not math.isfinite(options.attention_scale):
        raise ValueError(f"{name}: invalid tensors or options")
    if options.causal and (options.query_position_offset > k.shape[1] or
                           q.shape[1] > k.shape[1] - options.query_position_offset):
        raise ValueError(f"{name}: causal range exceeds the key sequence")


def flash_gqa_attention_backward_with_lse(grad_query, grad_key, grad_value, grad_output, output, logsumexp, query,
                                          key, value, stream=None,
                                          options: FlashAttentionOptions = FlashAttentionOptions(),
                                          accumulate_grads: bool = False):
    """include/ops/backward/attention_backward.h:57-70."""
    name = "flash_gqa_attention_backward_with_lse"
    _require_device(name, grad_query, grad_key, grad_value, grad_output, output, logsumexp, query, key, value)
    _attention_check(name, query, key, value, options, (grad_query, grad_key, grad_value, grad_output, output))
    if grad_output.shape != query.shape or grad_query.shape != query.shape or grad_key.shape != key.shape or \
            grad_value.shape != key.shape or output.shape != query.shape:
        raise ValueError(f"{name}: gradient shapes must match their tensors")
    if logsumexp.dtype != torch.float32 or tuple(logsumexp.shape) != tuple(query.shape[:3]):
        raise ValueError(f"{name}: invalid output or logsumexp")
    capi.call("cgptx_flash_gqa_attention_backward_with_lse", _ptr(grad_query), _ptr(grad_key), _ptr(grad_value),
              _ptr(grad_output), _ptr(output), _ptr(logsumexp), _ptr(query), _ptr(key), _ptr(value), query.shape[0],
              query.shape[1], key.shape[1], options.num_query_heads, options.num_kv_heads, options.head_dim,
              options.attention_scale, int(options.causal), options.query_position_offset, int(accumulate_grads),
              _code(query), _stream(stream))


def flash_gqa_attention_backward(grad_query, grad_key, grad_value, grad_output, query, key, value, stream=None,
                                 options: FlashAttentionOptions = FlashAttentionOptions(),
                                 accumulate_grads: bool = False):
    """include/ops/backward/attention_backward.h:24-35."""
    name = "flash_gqa_attention_backward"
    _require_device(name, grad_query, grad_key, grad_value, grad_output, query, key, value)
    _attention_check(name, query, key, value, options, (grad_query, grad_key, grad_value, grad_output))
    if grad_output.shape != query.shape or grad_query.shape != query.shape or grad_key.shape != key.shape or \
            grad_value.shape != key.shape:
        raise ValueError(f"{name}: gradient shapes must match their tensors")
    capi.call("cgptx_flash_gqa_attention_backward", _ptr(grad_query), _ptr(grad_key), _ptr(grad_value),
              _ptr(grad_output), _ptr(query), _ptr(key), _ptr(value), query.shape[0], query.shape[1], key.shape[1],
              options.num_query_heads, options.num_kv_heads, options.head_dim, options.attention_scale,
              int(options.causal), options.query_position_offset, int(accumulate_grads), _code(query),
              _stream(stream))


# ------------------------------------------------------------------------------ AdamW
class AdamWState:
    """AdamWState (include/optim/adamw.h:33-46): F32 master copy and moments."""

    def __init__(self, master_parameter, first_moment, second_moment, step=0):
        self.master_parameter = master_parameter
        self.first_moment = first_moment
        self.second_moment = second_moment
        self.step = step

    @staticmethod
    def for_parameter(parameter: torch.Tensor, stream=None) -> "AdamWState":
        if parameter.dtype not in _DTYPE:
            raise ValueError("AdamWState: parameter must have a floating dtype")
        return AdamWState(parameter.detach().to(torch.float32).clone(), torch.zeros_like(parameter, dtype=torch.float32),
                          torch.zeros_like(parameter, dtype=torch.float32), 0)


@dataclasses.dataclass
class AdamWBatchEntry:  # include/optim/adamw.h:49-57
    parameter: torch.Tensor
    gradient: torch.Tensor
    state: AdamWState


def _validate_adamw_options(o: AdamWOptions, name: str) -> None:
    ok = (math.isfinite(o.learning_rate) and o.learning_rate >= 0 and 0 <= o.beta1 < 1 and 0 <= o.beta2 < 1 and
          math.isfinite(o.epsilon) and o.epsilon > 0 and math.isfinite(o.weight_decay) and o.weight_decay >= 0 and
          math.isfinite(o.loss_scale) and o.loss_scale > 0 and not math.isnan(o.max_grad_norm) and
          o.max_grad_norm > 0)
    if not ok:
        raise ValueError(f"{name}: invalid optimizer options")


def _validate_adamw_tensors(parameter, gradient, state: AdamWState, name: str) -> None:
    if parameter.dtype not in _DTYPE or gradient.dtype != parameter.dtype or gradient.shape != parameter.shape or \
            gradient.device != parameter.device:
        raise ValueError(f"{name}: parameter and gradient must share dtype, shape and device")
    for t in (state.master_parameter, state.first_moment, state.second_moment):
        if t.dtype != torch.float32 or t.shape != parameter.shape or t.device != parameter.device:
            raise ValueError(f"{name}: master parameter and moment buffers must be F32 and match the parameter")


class AdamWWorkspace:
    """AdamWWorkspace (include/optim/adamw.h:60-84): device scalars bound to one stable entry list."""

    def __init__(self):
        handle = ctypes.c_void_p()
        capi.call("cgptx_adamw_workspace_create", ctypes.byref(handle))
        self._handle = handle
        self._states = None
        self._c_entries = None

    def __del__(self):
        try:
            if getattr(self, "_handle", None):
                capi.lib().cgptx_adamw_workspace_destroy(self._handle)
                self._handle = None
        except Exception:
            pass


def adamw_step_many_async(entries: Sequence[AdamWBatchEntry], options: AdamWOptions, workspace: AdamWWorkspace,
                          stream=None) -> None:
    """include/optim/adamw.h:103-107."""
    name = "adamw_step_many_async"
    _validate_adamw_options(options, name)
    if len(entries) == 0:
        raise ValueError(f"{name}: empty parameter list")
    if workspace._states is None:
        initial_step = entries[0].state.step if entries[0].state is not None else 0
        for e in entries:
            if e.state is None or e.state.step != initial_step:
                raise ValueError(f"{name}: states must share one initial step")
    else:
        initial_step = 0
        if len(workspace._states) != len(entries):
            raise ValueError(f"{name}: workspace entries changed")
        for e, s in zip(entries, workspace._states):
            if e.state is not s:
                raise ValueError(f"{name}: workspace states changed")
    array = (capi.AdamWEntry * len(entries))()
    for i, e in enumerate(entries):
        if e.parameter is None or e.gradient is None or e.state is None:
            raise ValueError(f"{name}: null entry")
        _validate_adamw_tensors(e.parameter, e.gradient, e.state, name)
        if e.parameter.device.type != "cuda":
            raise ValueError(f"{name}: device tensors required")
        array[i] = capi.AdamWEntry(e.parameter.data_ptr(), e.gradient.data_ptr(), e.state.master_parameter.data_ptr(),
                                   e.state.first_moment.data_ptr(), e.state.second_moment.data_ptr(),
                                   e.parameter.numel(), _code(e.parameter))
    c_options = options.to_c()
    capi.call("cgptx_adamw_step_many_async", workspace._handle, array, len(entries), ctypes.byref(c_options),
              initial_step, _stream(stream))
    if workspace._states is None:
        workspace._states = [e.state for e in entries]


def adamw_check(workspace: AdamWWorkspace, stream=None) -> bool:
    """include/optim/adamw.h:114-115."""
    finite = ctypes.c_int(1)
    step = ctypes.c_uint64(0)
    capi.call("cgptx_adamw_check", workspace._handle, ctypes.byref(finite), ctypes.byref(step), _stream(stream))
    for s in workspace._states or ():
        s.step = step.value
    return bool(finite.value)


def adamw_step(parameter, gradient, state: AdamWState, options: AdamWOptions = AdamWOptions(), stream=None) -> bool:
    """include/optim/adamw.h:131-136 (device tensors only; the CPU branch of the reference is the checker's job)."""
    name = "adamw_step"
    _validate_adamw_options(options, name)
    _validate_adamw_tensors(parameter, gradient, state, name)
    if parameter.device.type != "cuda":
        raise ValueError(f"{name}: device tensors required")
    if state.step == 2**64 - 1:
        raise OverflowError(f"{name}: step counter overflow")
    updated = ctypes.c_int(0)
    c_options = options.to_c()
    capi.call("cgptx_adamw_step", _ptr(parameter), _ptr(gradient), _ptr(state.master_parameter),
              _ptr(state.first_moment), _ptr(state.second_moment), parameter.numel(), _code(parameter),
              ctypes.byref(c_options), state.step + 1, ctypes.byref(updated), _stream(stream))
    if updated.value:
        state.step += 1
    return bool(updated.value)


# ---------------------------------------------------------------------------- forward
def rmsnorm_forward(output, input, weight, epsilon, stream=None):
    """include/ops/rmsnorm.h."""
    name = "rmsnorm_forward"
    if not (math.isfinite(epsilon) and epsilon > 0):
        raise ValueError(f"{name}: epsilon must be finite and positive")
    _require_device(name, output, input, weight)
    _same_dtype(name, input, output, weight)
    if input.dim() != 2 or output.shape != input.shape or weight.dim() != 1 or weight.shape[0] != input.shape[1]:
        raise ValueError(f"{name}: incompatible shapes")
    capi.call("cgptx_rmsnorm_forward", _ptr(output), _ptr(input), _ptr(weight), input.shape[0], input.shape[1],
              epsilon, _code(input), _stream(stream))


def rope_forward(query, key, cos_cache, sin_cache, stream=None, rope_options: RopeOptions = RopeOptions()):
    """include/ops/rope.h:32-39 (in place)."""
    name = "rope_forward"
    _require_device(name, query, key, cos_cache, sin_cache)
    _same_dtype(name, query, key, cos_cache, sin_cache)
    _rope_check(name, query, key, cos_cache, sin_cache, rope_options)
    b, s, hq, d = query.shape
    capi.call("cgptx_rope_forward", _ptr(query), _ptr(key), _ptr(cos_cache), _ptr(sin_cache), b, s, hq, key.shape[2],
              d, rope_options.rotary_dim, rope_options.position_offset, cos_cache.shape[0], _code(query),
              _stream(stream))


def swiglu_forward(output, gate, up=None, stream=None):
    """include/ops/swiglu.h: (output, gate, up) or, with up omitted, (output, gate_up) with the
    projections concatenated along the last dimension."""
    name = "swiglu_forward"
    if up is None:
        gate_up = gate
        _require_device(name, output, gate_up)
        _same_dtype(name, gate_up, output)
        if gate_up.dim() == 0 or gate_up.shape[-1] % 2 != 0:
            raise ValueError(f"{name}: the last gate_up dimension must be even")
        hidden = gate_up.shape[-1] // 2
        if output.dim() != gate_up.dim() or tuple(output.shape[:-1]) != tuple(gate_up.shape[:-1]) or \
                output.shape[-1] != hidden:
            raise ValueError(f"{name}: output shape must match gate_up except for its last dimension")
        if output.numel() == 0:
            return  # nothing to do (src/ops/swiglu.cu:581-583)
        capi.call("cgptx_swiglu_forward_packed", _ptr(output), _ptr(gate_up), output.numel() // hidden, hidden,
                  _code(gate_up), _stream(stream))
        return
    _require_device(name, output, gate, up)
    _same_dtype(name, gate, output, up)
    if output.shape != gate.shape or up.shape != gate.shape:
        raise ValueError(f"{name}: all tensors must have the same shape")
    capi.call("cgptx_swiglu_forward", _ptr(output), _ptr(gate), _ptr(up), gate.numel(), _code(gate), _stream(stream))


def linear_forward(output, input, weight, gemm_context=None, stream=None, bias=None):
    """include/ops/linear.h."""
    name = "linear_forward"
    present = [bias] if bias is not None else []
    _require_device(name, output, input, weight, *present)
    _same_dtype(name, input, output, weight, *present)
    if weight.dim() != 2 or input.shape[-1] != weight.shape[1] or output.shape[-1] != weight.shape[0] or \
            tuple(output.shape[:-1]) != tuple(input.shape[:-1]):
        raise ValueError(f"{name}: incompatible tensors")
    out_features, in_features = weight.shape
    capi.call("cgptx_linear_forward", _ptr(output), _ptr(input), _ptr(weight), _ptr(bias),
              input.numel() // in_features, in_features, out_features, _code(input), _stream(stream))


def linear_swiglu_forward(gate_up, activated, input, weight, gemm_context=None, stream=None):
    """The feed-forward's gate and up projections and SwiGLU in one call (src/core/transformer_block.cu:586-590
    with the concatenated layouts of include/ops/swiglu.h:33-37): weight = [gate_proj; up_proj] ([2*hidden, in]),
    gate_up = [..., 2*hidden] = [gate | up], activated = [..., hidden] = silu(gate) * up."""
    name = "linear_swiglu_forward"
    _require_device(name, gate_up, activated, input, weight)
    _same_dtype(name, input, gate_up, activated, weight)
    if weight.dim() != 2 or weight.shape[0] % 2 != 0 or input.shape[-1] != weight.shape[1] or \
            gate_up.shape[-1] != weight.shape[0] or activated.shape[-1] * 2 != weight.shape[0] or \
            tuple(gate_up.shape[:-1]) != tuple(input.shape[:-1]) or tuple(activated.shape[:-1]) != tuple(input.shape[:-1]):
        raise ValueError(f"{name}: incompatible tensors")
    out_features, in_features = weight.shape
    capi.call("cgptx_linear_swiglu_forward", _ptr(gate_up), _ptr(activated), _ptr(input), _ptr(weight),
              input.numel() // in_features, in_features, out_features // 2, _code(input), _stream(stream))


def linear_swiglu_backward(grad_gate_up, grad_activated, grad_output, weight, gate_up, gemm_context=None, stream=None):
    """The input gradient of the down projection and the SwiGLU gradient in one call (src/core/transformer_block.cu:663-666
    with the concatenated layouts of src/ops/backward/swiglu_backward.cu:830-883): weight = down_proj ([out, hidden]),
    gate_up = the forward's [..., 2*hidden] = [gate | up], grad_gate_up = [..., 2*hidden] = [dgate | dup];
    grad_activated ([..., hidden]) is working memory (written only when the two operators run one after the other)."""
    name = "linear_swiglu_backward"
    _require_device(name, grad_gate_up, grad_activated, grad_output, weight, gate_up)
    _same_dtype(name, grad_output, grad_gate_up, grad_activated, weight, gate_up)
    if weight.dim() != 2 or grad_output.shape[-1] != weight.shape[0] or grad_activated.shape[-1] != weight.shape[1] or \
            gate_up.shape[-1] != 2 * weight.shape[1] or tuple(grad_gate_up.shape) != tuple(gate_up.shape) or \
            tuple(gate_up.shape[:-1]) != tuple(grad_output.shape[:-1]) or \
            tuple(grad_activated.shape[:-1]) != tuple(grad_output.shape[:-1]):
        raise ValueError(f"{name}: incompatible tensors")
    out_features, hidden = weight.shape
    capi.call("cgptx_linear_swiglu_backward", _ptr(grad_gate_up), _ptr(grad_activated), _ptr(grad_output), _ptr(weight),
              _ptr(gate_up), grad_output.numel() // out_features, hidden, out_features, _code(grad_output), _stream(stream))


def linear_backward_weights_stacked(grad_weight, grad_output, input, stream=None):
    """The weight gradients of several layers of one shape in one launch: grad_output [count, rows, out], input
    [count, rows, in], grad_weight [count, out, in] — `count` calls of linear_backward
    (include/ops/backward/linear_backward.h:36-46) for the weight gradient only."""
    name = "linear_backward_weights_stacked"
    _require_device(name, grad_weight)
    if grad_output.device.type != "cuda" or input.device.type != "cuda":  # layers may be slices of larger blocks
        raise ValueError(f"{name}: all tensors must be device tensors")
    _same_dtype(name, grad_weight, grad_output, input)
    if grad_weight.dim() != 3 or grad_output.dim() != 3 or input.dim() != 3 or \
            grad_output.shape[0] != grad_weight.shape[0] or input.shape[0] != grad_weight.shape[0] or \
            grad_output.shape[1] != input.shape[1] or grad_output.shape[2] != grad_weight.shape[1] or \
            input.shape[2] != grad_weight.shape[2] or not grad_weight.is_contiguous() or \
            grad_output.stride()[1:] != (grad_output.shape[2], 1) or input.stride()[1:] != (input.shape[2], 1):
        raise ValueError(f"{name}: incompatible tensors")
    count, out_features, in_features = grad_weight.shape
    capi.call("cgptx_linear_backward_weights_stacked", _ptr(grad_weight), _ptr(grad_output), _ptr(input),
              input.shape[1], in_features, out_features, count, grad_output.stride(0), input.stride(0),
              _code(grad_output), _stream(stream))


def embedding_forward(output, device_token_ids, token_count, weight, stream=None):
    """include/ops/embedding.h."""
    name = "embedding_forward"
    _require_device(name, output, weight)
    _same_dtype(name, weight, output)
    _ids(name, device_token_ids, token_count)
    if weight.dim() != 2 or output.numel() != token_count * weight.shape[1]:
        raise ValueError(f"{name}: incompatible tensors or token count")
    capi.call("cgptx_embedding_forward", _ptr(output), _ptr(device_token_ids), token_count, _ptr(weight),
              weight.shape[0], weight.shape[1], _code(weight), _stream(stream))


def flash_gqa_attention_forward_with_lse(output, logsumexp, query, key, value, stream=None,
                                         options: FlashAttentionOptions = FlashAttentionOptions()):
    """include/ops/attention.h:70-78."""
    name = "flash_gqa_attention_forward_with_lse"
    tensors = [output, query, key, value] + ([logsumexp] if logsumexp is not None else [])
    _require_device(name, *tensors)
    _attention_check(name, query, key, value, options, (output,))
    if output.shape != query.shape:
        raise ValueError(f"{name}: output must match query")
    if logsumexp is not None and (logsumexp.dtype != torch.float32 or
                                  tuple(logsumexp.shape) != tuple(query.shape[:3])):
        raise ValueError(f"{name}: invalid logsumexp tensor")
    capi.call("cgptx_flash_gqa_attention_forward", _ptr(output), _ptr(logsumexp), _ptr(query), _ptr(key), _ptr(value),
              query.shape[0], query.shape[1], key.shape[1], options.num_query_heads, options.num_kv_heads,
              options.head_dim, options.attention_scale, int(options.causal), options.query_position_offset,
              _code(query), _stream(stream))


def flash_gqa_attention_forward(output, query, key, value, stream=None,
                                options: FlashAttentionOptions = FlashAttentionOptions()):
    """include/ops/attention.h:47-54."""
    flash_gqa_attention_forward_with_lse(output, None, query, key, value, stream, options)


def add_tensors(output, a, b, stream=None):
    """src/core/transformer_block.cu:242-248."""
    name = "add"
    _require_device(name, output, a, b)
    _same_dtype(name, a, output, b)
    if output.shape != a.shape or b.shape != a.shape:
        raise ValueError(f"{name}: shape mismatch")
    capi.call("cgptx_add", _ptr(output), _ptr(a), _ptr(b), a.numel(), _code(a), _stream(stream))
