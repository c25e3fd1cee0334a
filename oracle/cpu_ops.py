"""ctypes front end of the float32 CPU checker (oracle/cgpt_cpu_ops.c).

TEST INFRASTRUCTURE — only tests/, __graft_entry__.smoke() and the cpu_baseline
leg of bench.py may import this module. Functions take contiguous torch CPU
tensors (float16, bfloat16 or float32) and write their outputs in place, with
the argument order of the reference operators they restate.
"""
from __future__ import annotations

import ctypes
import pathlib

import torch

_HERE = pathlib.Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libcgpt_oracle.so"
_lib = None

_DTYPE = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            from oracle import build as _build

            _build.build()
        _lib = ctypes.CDLL(str(_LIB_PATH))
        _lib.cg_adamw_cpu.restype = ctypes.c_int
        _lib.cg_adamw_cpu_parallel.restype = ctypes.c_int
        _lib.cg_max_threads.restype = ctypes.c_int
    return _lib


def _p(t):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.device.type == "cpu" and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _code(t: torch.Tensor) -> int:
    return _DTYPE[t.dtype]


_sz = ctypes.c_size_t
_f = ctypes.c_float
_i = ctypes.c_int


def max_threads() -> int:
    return lib().cg_max_threads()


def rmsnorm_backward(grad_input, grad_weight, grad_output, input, weight, epsilon):
    rows, hidden = input.shape
    lib().cg_rmsnorm_backward_cpu(_p(grad_input), _p(grad_weight), _p(grad_output), _p(input), _p(weight),
                                  _sz(rows), _sz(hidden), _f(epsilon), _i(_code(input)))


def rmsnorm_forward(output, input, weight, epsilon):
    rows, hidden = input.shape
    lib().cg_rmsnorm_forward_cpu(_p(output), _p(input), _p(weight), _sz(rows), _sz(hidden), _f(epsilon),
                                 _i(_code(input)))


def rope_backward(grad_query, grad_key, grad_rotated_query, grad_rotated_key, cos_cache, sin_cache, rotary_dim=0,
                  position_offset=0):
    b, s, q, d = grad_query.shape
    k = grad_key.shape[2]
    lib().cg_rope_backward_cpu(_p(grad_query), _p(grad_key), _p(grad_rotated_query), _p(grad_rotated_key),
                               _p(cos_cache), _p(sin_cache), _sz(b), _sz(s), _sz(q), _sz(k), _sz(d), _sz(rotary_dim),
                               _sz(position_offset), _i(_code(grad_query)))


def rope_forward(query, key, cos_cache, sin_cache, rotary_dim=0, position_offset=0):
    b, s, q, d = query.shape
    k = key.shape[2]
    lib().cg_rope_forward_cpu(_p(query), _p(key), _p(cos_cache), _p(sin_cache), _sz(b), _sz(s), _sz(q), _sz(k), _sz(d),
                              _sz(rotary_dim), _sz(position_offset), _i(_code(query)))


def swiglu_backward(grad_gate, grad_up, grad_output, gate, up, accumulate_gate=False, accumulate_up=False):
    lib().cg_swiglu_backward_cpu(_p(grad_gate), _p(grad_up), _p(grad_output), _p(gate), _p(up), _sz(gate.numel()),
                                 _i(int(accumulate_gate)), _i(int(accumulate_up)), _i(_code(gate)))


def swiglu_backward_packed(grad_gate_up, grad_output, gate_up, accumulate=False):
    hidden = grad_output.shape[-1]
    rows = grad_output.numel() // hidden
    lib().cg_swiglu_backward_packed_cpu(_p(grad_gate_up), _p(grad_output), _p(gate_up), _sz(rows), _sz(hidden),
                                        _i(int(accumulate)), _i(_code(gate_up)))


def swiglu_forward(output, gate, up):
    lib().cg_swiglu_forward_cpu(_p(output), _p(gate), _p(up), _sz(gate.numel()), _i(_code(gate)))


def linear_backward(grad_input, grad_weight, grad_bias, grad_output, input, weight, accumulate_input=False,
                    accumulate_weight=False, accumulate_bias=False):
    out_features, in_features = weight.shape
    rows = input.numel() // in_features
    lib().cg_linear_backward_cpu(_p(grad_input), _p(grad_weight), _p(grad_bias), _p(grad_output), _p(input), _p(weight),
                                 _sz(rows), _sz(in_features), _sz(out_features), _i(int(accumulate_input)),
                                 _i(int(accumulate_weight)), _i(int(accumulate_bias)), _i(_code(input)))


def linear_forward(output, input, weight, bias=None):
    out_features, in_features = weight.shape
    rows = input.numel() // in_features
    lib().cg_linear_forward_cpu(_p(output), _p(input), _p(weight), _p(bias), _sz(rows), _sz(in_features),
                                _sz(out_features), _i(_code(input)))


def embedding_backward(grad_weight, grad_output, token_ids, bounds_check=True, accumulate_weight=False):
    vocab, hidden = grad_weight.shape
    assert token_ids.dtype == torch.int32 or token_ids.dtype == torch.uint32
    lib().cg_embedding_backward_cpu(_p(grad_weight), _p(grad_output), _p(token_ids), _sz(token_ids.numel()), _sz(vocab),
                                    _sz(hidden), _i(int(bounds_check)), _i(int(accumulate_weight)),
                                    _i(_code(grad_weight)))


def embedding_forward(output, token_ids, weight):
    vocab, hidden = weight.shape
    lib().cg_embedding_forward_cpu(_p(output), _p(token_ids), _sz(token_ids.numel()), _p(weight), _sz(vocab),
                                   _sz(hidden), _i(_code(weight)))


def cross_entropy_forward_backward(loss, gradient, logits, targets, gradient_scale=1.0):
    rows, vocab = logits.shape
    lib().cg_cross_entropy_forward_backward_cpu(_p(loss), _p(gradient), _p(logits), _p(targets), _sz(rows), _sz(vocab),
                                                _f(gradient_scale), _i(_code(logits)))


def cross_entropy_forward(loss, logits, targets):
    rows, vocab = logits.shape
    lib().cg_cross_entropy_forward_cpu(_p(loss), _p(logits), _p(targets), _sz(rows), _sz(vocab), _i(_code(logits)))


def attention_forward(output, logsumexp, query, key, value, num_query_heads, num_kv_heads, head_dim,
                      attention_scale=0.0, causal=True, query_position_offset=0):
    b, qs = query.shape[0], query.shape[1]
    ks = key.shape[1]
    lib().cg_attention_forward_cpu(_p(output), _p(logsumexp), _p(query), _p(key), _p(value), _sz(b), _sz(qs), _sz(ks),
                                   _sz(num_query_heads), _sz(num_kv_heads), _sz(head_dim), _f(attention_scale),
                                   _i(int(causal)), _sz(query_position_offset), _i(_code(query)))


def attention_backward(grad_query, grad_key, grad_value, grad_output, query, key, value, num_query_heads, num_kv_heads,
                       head_dim, attention_scale=0.0, causal=True, query_position_offset=0, accumulate_grads=False):
    b, qs = query.shape[0], query.shape[1]
    ks = key.shape[1]
    lib().cg_attention_backward_cpu(_p(grad_query), _p(grad_key), _p(grad_value), _p(grad_output), _p(query), _p(key),
                                    _p(value), _sz(b), _sz(qs), _sz(ks), _sz(num_query_heads), _sz(num_kv_heads),
                                    _sz(head_dim), _f(attention_scale), _i(int(causal)), _sz(query_position_offset),
                                    _i(int(accumulate_grads)), _i(_code(query)))


def adamw(parameter, gradient, master, first_moment, second_moment, next_step, learning_rate=1e-3, beta1=0.9,
          beta2=0.999, epsilon=1e-8, weight_decay=1e-2, loss_scale=1.0, max_grad_norm=float("inf"), parallel=False):
    """F32 tensors only. Returns False (and changes nothing) on a non-finite gradient."""
    fn = lib().cg_adamw_cpu_parallel if parallel else lib().cg_adamw_cpu
    return bool(fn(_p(parameter), _p(gradient), _p(master), _p(first_moment), _p(second_moment),
                   _sz(parameter.numel()), _f(learning_rate), _f(beta1), _f(beta2), _f(epsilon), _f(weight_decay),
                   _f(loss_scale), _f(max_grad_norm), ctypes.c_uint64(next_step)))


def add(output, a, b):
    lib().cg_add_cpu(_p(output), _p(a), _p(b), _sz(a.numel()), _i(_code(a)))
