"""ctypes binding of libcgptx.so (the C-ABI declared in include/cgptx.h).

The library must have been built in-tree (python -m cgpt_amd.build); loading
fails loudly otherwise. There is no CPU fallback anywhere in this package.
"""
from __future__ import annotations

import ctypes
import pathlib

LIB_PATH = pathlib.Path(__file__).resolve().parent / "lib" / "libcgptx.so"

OK, INVALID_ARGUMENT, OVERFLOW, RUNTIME, CAPTURE_ALLOC = 0, 1, 2, 3, 4

F16, BF16, F32 = 0, 1, 2

_vp = ctypes.c_void_p
_sz = ctypes.c_size_t
_i = ctypes.c_int
_f = ctypes.c_float
_u64 = ctypes.c_uint64


class AdamWOptions(ctypes.Structure):
    """cgptx_adamw_options; defaults follow AdamWOptions in the reference (include/optim/adamw.h:12-27)."""

    _fields_ = [("learning_rate", _f), ("beta1", _f), ("beta2", _f), ("epsilon", _f), ("weight_decay", _f),
                ("loss_scale", _f), ("max_grad_norm", _f)]

    def __init__(self, learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8, weight_decay=1e-2, loss_scale=1.0,
                 max_grad_norm=float("inf")):
        super().__init__(learning_rate, beta1, beta2, epsilon, weight_decay, loss_scale, max_grad_norm)


class AdamWEntry(ctypes.Structure):
    _fields_ = [("parameter", _vp), ("gradient", _vp), ("master_parameter", _vp), ("first_moment", _vp),
                ("second_moment", _vp), ("count", _sz), ("dtype", _i)]


class ModelConfig(ctypes.Structure):
    """cgptx_model_config (include/cgptx_train.h)."""

    _fields_ = [("vocabulary_size", _sz), ("num_layers", _sz), ("hidden_size", _sz), ("intermediate_size", _sz),
                ("num_query_heads", _sz), ("num_kv_heads", _sz), ("head_dim", _sz), ("rotary_dim", _sz),
                ("rms_epsilon", _f), ("rope_base", _f), ("dtype", _i)]


# name -> argtypes, in the order of include/cgptx.h and include/cgptx_train.h
PROTOTYPES = {
    "cgptx_release_scratch": [],
    "cgptx_rmsnorm_backward": [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _f, _i, _vp],
    "cgptx_rmsnorm_backward_static": [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _f, _i, _vp],
    "cgptx_rope_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _i, _vp],
    "cgptx_swiglu_backward": [_vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _vp],
    "cgptx_swiglu_backward_packed": [_vp, _vp, _vp, _sz, _sz, _i, _i, _vp],
    "cgptx_linear_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _i, _i, _i, _i, _vp],
    "cgptx_embedding_backward": [_vp, _vp, _vp, _sz, _sz, _sz, _i, _i, _i, _vp],
    "cgptx_cross_entropy_forward_backward": [_vp, _vp, _vp, _vp, _sz, _sz, _f, _i, _vp],
    "cgptx_cross_entropy_forward": [_vp, _vp, _vp, _sz, _sz, _i, _vp],
    "cgptx_cut_cross_entropy_forward_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _f, _i, _i, _vp],
    "cgptx_flash_gqa_attention_backward_with_lse": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz,
                                                    _sz, _sz, _f, _i, _sz, _i, _i, _vp],
    "cgptx_flash_gqa_attention_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _f, _i,
                                           _sz, _i, _i, _vp],
    "cgptx_adamw_workspace_create": [ctypes.POINTER(_vp)],
    "cgptx_adamw_workspace_destroy": [_vp],
    "cgptx_adamw_step_many_async": [_vp, ctypes.POINTER(AdamWEntry), _sz, ctypes.POINTER(AdamWOptions), _u64, _vp],
    "cgptx_adamw_check": [_vp, ctypes.POINTER(_i), ctypes.POINTER(_u64), _vp],
    "cgptx_adamw_step": [_vp, _vp, _vp, _vp, _vp, _sz, _i, ctypes.POINTER(AdamWOptions), _u64, ctypes.POINTER(_i),
                         _vp],
    "cgptx_rmsnorm_forward": [_vp, _vp, _vp, _sz, _sz, _f, _i, _vp],
    "cgptx_rope_forward": [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _i, _vp],
    "cgptx_swiglu_forward": [_vp, _vp, _vp, _sz, _i, _vp],
    "cgptx_swiglu_forward_packed": [_vp, _vp, _sz, _sz, _i, _vp],
    "cgptx_linear_forward": [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _i, _vp],
    "cgptx_linear_swiglu_forward": [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _i, _vp],
    "cgptx_linear_swiglu_backward": [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _i, _vp],
    "cgptx_linear_backward_weights_stacked": [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _i, _vp],
    "cgptx_embedding_forward": [_vp, _vp, _sz, _vp, _sz, _sz, _i, _vp],
    "cgptx_flash_gqa_attention_forward": [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _f, _i, _sz, _i, _vp],
    "cgptx_add": [_vp, _vp, _vp, _sz, _i, _vp],
    "cgptx_model_create": [ctypes.POINTER(_vp), ctypes.POINTER(ModelConfig), _sz, _sz, _u64],
    "cgptx_model_destroy": [_vp],
    "cgptx_model_set_tokens": [_vp, _vp, _vp],
    "cgptx_model_forward_backward": [_vp, _f, _i, _i, _vp],
    "cgptx_model_optimizer_step": [_vp, ctypes.POINTER(AdamWOptions), _vp],
    "cgptx_model_train_step": [_vp, ctypes.POINTER(AdamWOptions), _i, _i, _vp],
    "cgptx_model_status": [_vp, ctypes.POINTER(_f), ctypes.POINTER(_i), ctypes.POINTER(_u64), _vp],
    "cgptx_model_parameter": [_vp, _sz, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(_vp), ctypes.POINTER(_vp),
                              ctypes.POINTER(_sz)],
    "cgptx_model_activation": [_vp, ctypes.c_char_p, ctypes.POINTER(_vp), ctypes.POINTER(_sz)],
    "cgptx_model_describe": [_vp, ctypes.POINTER(ModelConfig), ctypes.POINTER(_sz), ctypes.POINTER(_sz)],
    "cgptx_model_optimizer_state": [_vp, _sz, ctypes.POINTER(_vp), ctypes.POINTER(_vp), ctypes.POINTER(_vp)],
    "cgptx_model_set_optimizer_step": [_vp, _u64],
    "cgptx_model_save_checkpoint": [_vp, ctypes.c_char_p, _sz],
    "cgptx_model_load_checkpoint": [_vp, ctypes.c_char_p],
    "cgptx_model_save_optimizer": [_vp, ctypes.c_char_p, _u64],
    "cgptx_model_load_optimizer": [_vp, ctypes.c_char_p, ctypes.POINTER(_u64)],
    "cgptx_token_upload_create": [ctypes.POINTER(_vp), _sz, _sz],
    "cgptx_token_upload_destroy": [_vp],
    "cgptx_token_upload_acquire": [_vp, ctypes.POINTER(_vp), ctypes.POINTER(_vp)],
    "cgptx_token_upload_submit": [_vp, _vp, _vp, _vp],
    "cgptx_model_upload_tokens": [_vp, _vp, _vp],
    "cgptx_pinned_allocate": [ctypes.POINTER(_vp), _sz],
    "cgptx_pinned_release": [_vp],
    "cgptx_device_allocate": [ctypes.POINTER(_vp), _sz],
    "cgptx_device_release": [_vp],
    "cgptx_upload_fence_wait": [_vp],
    "cgptx_upload_fence_destroy": [_vp],
    "cgptx_token_upload_async": [_vp, _vp, _vp, _vp, _sz, ctypes.POINTER(_vp), _vp],
    "cgptx_model_profile": [_vp, _f, _i, _vp],
    "cgptx_model_profile_entry": [_vp, _sz, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(_f)],
    "cgptx_model_record_calls": [_vp, _i],
    "cgptx_model_call": [_vp, _sz, _vp],
}

SIZE_FUNCTIONS = {"cgptx_model_parameter_count": [_vp], "cgptx_model_num_parameters": [_vp],
                  "cgptx_model_profile_count": [_vp], "cgptx_model_call_count": [_vp], "cgptx_scratch_bytes": [_vp]}

STRING_FUNCTIONS = ("cgptx_last_error", "cgptx_version")

_lib = None


class CgptxRuntimeError(RuntimeError):
    """HIP runtime failure reported by the library (the reference exits the process here)."""


class CgptxCaptureError(RuntimeError):
    """Scratch would have to grow while the stream is being captured."""


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m cgpt_amd.build` (there is no CPU fallback)")
        loaded = ctypes.CDLL(str(LIB_PATH))
        for name, argtypes in PROTOTYPES.items():
            fn = getattr(loaded, name)
            fn.argtypes = argtypes
            fn.restype = _i
        for name in STRING_FUNCTIONS:
            getattr(loaded, name).restype = ctypes.c_char_p
        for name, argtypes in SIZE_FUNCTIONS.items():
            getattr(loaded, name).argtypes = argtypes
            getattr(loaded, name).restype = _sz
        _lib = loaded
    return _lib


def check(status: int) -> None:
    """Maps a status code to the exception type the reference throws for it."""
    if status == OK:
        return
    message = lib().cgptx_last_error().decode()
    if status == INVALID_ARGUMENT:
        raise ValueError(message)  # std::invalid_argument
    if status == OVERFLOW:
        raise OverflowError(message)  # std::overflow_error
    if status == CAPTURE_ALLOC:
        raise CgptxCaptureError(message)
    raise CgptxRuntimeError(message)


def call(name: str, *args) -> None:
    check(getattr(lib(), name)(*args))
