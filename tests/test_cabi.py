"""The C-ABI library loads, exports every symbol include/cgptx.h declares, and rejects bad
arguments before touching the GPU (so these run without one)."""
import ctypes
import pathlib
import re

import pytest

from cgpt_amd import capi

ROOT = pathlib.Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "cgptx.h").read_text() + (ROOT / "include" / "cgptx_train.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cgptx_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    lib = capi.lib()
    names = declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/*.h but not exported"


def test_prototype_table_covers_the_header():
    assert set(declared_symbols()) == set(capi.PROTOTYPES) | set(capi.STRING_FUNCTIONS) | set(capi.SIZE_FUNCTIONS)


def test_version_string():
    assert b"gfx950" in capi.lib().cgptx_version()


NULL = ctypes.c_void_p(0)
P = ctypes.c_void_p(0x1000)  # never dereferenced: validation fails first


@pytest.mark.parametrize("name,args", [
    ("cgptx_rmsnorm_backward", (P, P, P, P, P, 4, 8, 0.0, capi.BF16, NULL)),          # epsilon must be > 0
    ("cgptx_rmsnorm_backward", (P, P, P, P, P, 4, 8, float("nan"), capi.BF16, NULL)),
    ("cgptx_rmsnorm_backward", (P, P, P, P, P, 4, 8, 1e-5, 7, NULL)),                 # unknown dtype
    ("cgptx_rmsnorm_backward", (NULL, P, P, P, P, 4, 8, 1e-5, capi.F32, NULL)),
    ("cgptx_rope_backward", (P, P, P, P, P, P, 1, 2, 2, 1, 5, 0, 0, 2, capi.F32, NULL)),   # odd head_dim
    ("cgptx_rope_backward", (P, P, P, P, P, P, 1, 2, 2, 1, 4, 6, 0, 2, capi.F32, NULL)),   # rotary_dim > head_dim
    ("cgptx_rope_backward", (P, P, P, P, P, P, 1, 3, 2, 1, 4, 2, 1, 3, capi.F32, NULL)),   # cache too short
    ("cgptx_swiglu_backward", (P, P, P, P, NULL, 16, 0, 0, capi.F16, NULL)),
    ("cgptx_linear_backward", (P, P, P, P, P, P, 0, 4, 4, 0, 0, 0, capi.F32, NULL)),
    ("cgptx_embedding_backward", (P, P, P, 0, 8, 8, 1, 0, capi.F16, NULL)),
    ("cgptx_cross_entropy_forward_backward", (P, P, P, P, 2, 3, -1.0, capi.F32, NULL)),    # scale must be > 0
    ("cgptx_cross_entropy_forward_backward", (P, P, P, NULL, 2, 3, 1.0, capi.F32, NULL)),
])
def test_invalid_arguments_raise_value_error(name, args):
    with pytest.raises(ValueError):
        capi.call(name, *args)


def test_rope_dimension_overflow_raises_overflow_error():
    with pytest.raises(OverflowError):
        capi.call("cgptx_rope_backward", P, P, P, P, P, P, 1, 2**33, 2, 1, 4, 0, 0, 2**34, capi.F32, NULL)


def test_adamw_option_validation():
    opts = capi.AdamWOptions(beta1=1.0)
    updated = ctypes.c_int(0)
    with pytest.raises(ValueError):
        capi.call("cgptx_adamw_step", P, P, P, P, P, 2, capi.F32, ctypes.byref(opts), 1, ctypes.byref(updated), NULL)
