"""The engine library (csrc/engine, one shared library) loaded with ctypes, its C functions typed.

Everything between a request's tokens and its next token lives in that library: configurations and
architectures, the loader, the parts, the cache storage, the step function, the scheduler's loop and
the sampler. The Python modules beside this one are faces over it and hold no second copy of any of
that. The library is built at first use (build.py) and a library that cannot be built or loaded
raises: there is no other path.
"""
from __future__ import annotations

import ctypes
from typing import Callable

from .build import load_library

_lib = None
_vp, _i, _ll, _ull, _f, _d = (ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_ulonglong, ctypes.c_float,
                              ctypes.c_double)
_cp, _sz = ctypes.c_char_p, ctypes.c_size_t


class EngineError(RuntimeError):
    """An error that the native engine reports (its message is the native one)."""


def lib():
    """The engine library with the types of its functions declared (the ops' types: kernels/ops.py)."""
    global _lib
    if _lib is not None:
        return _lib
    lb = load_library("engine")
    sigs = {
        "mllm_last_error": (_cp, []),
        # configurations, architectures, model folders
        "mllm_load_plugin": (_i, [_cp]),
        "mllm_registered_architectures": (_i, [_cp, _i]),
        "mllm_describe_config": (_i, [_cp, _cp, _i]),
        "mllm_check_model_dir": (_i, [_cp, _cp, _i]),
        "mllm_write_random_model": (_i, [_cp, _ull, _cp, _cp]),
        "mllm_normal_values": (_i, [_ull, _cp, _ll, _ll, _d, _d, _vp]),
        # single parts
        "mllm_params_create": (_vp, []),
        "mllm_params_destroy": (None, [_vp]),
        "mllm_params_set_number": (None, [_vp, _cp, _d]),
        "mllm_params_set_string": (None, [_vp, _cp, _cp]),
        "mllm_params_set_tensor": (None, [_vp, _cp, _vp]),
        "mllm_has_part": (_i, [_cp, _cp]),
        "mllm_norm_create": (_vp, [_cp, _vp]),
        "mllm_norm_destroy": (None, [_vp]),
        "mllm_norm_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _vp]),
        "mllm_feed_forward_create": (_vp, [_cp, _vp]),
        "mllm_feed_forward_destroy": (None, [_vp]),
        "mllm_feed_forward_forward": (_i, [_vp, _vp, _vp, _vp, _sz, _vp]),
        "mllm_embedding_create": (_vp, [_cp, _vp]),
        "mllm_embedding_destroy": (None, [_vp]),
        "mllm_embedding_forward": (_i, [_vp, _cp, _vp, _vp, _vp, _vp, _vp]),
        "mllm_head_create": (_vp, [_cp, _vp]),
        "mllm_head_destroy": (None, [_vp]),
        "mllm_head_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
        # runner
        "mllm_runner_create": (_vp, [_cp, _cp, _ull, _i, _i, _i, _i]),
        "mllm_runner_destroy": (None, [_vp]),
        "mllm_runner_of_box": (_vp, [_vp]),
        "mllm_runner_step": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _ll]),
        "mllm_runner_end_request": (_i, [_vp, _ll]),
        "mllm_runner_poison": (_i, [_vp]),
        "mllm_runner_check": (_i, [_vp, _cp, _i]),
        "mllm_runner_info": (_i, [_vp, _cp, _i]),
        "mllm_runner_synchronize": (None, [_vp]),
        # engine
        "mllm_engine_from_pretrained": (_vp, [_cp, _i, _vp]),
        "mllm_engine_from_random": (_vp, [_cp, _ull, _i, _vp]),
        "mllm_engine_destroy": (None, [_vp]),
        "mllm_engine_runner": (_vp, [_vp]),
        "mllm_engine_add_request": (_ll, [_vp, _vp, _i, _f, _ull, _i, _i, _ll]),
        "mllm_engine_has_unfinished": (_i, [_vp]),
        "mllm_engine_step": (_i, [_vp, _vp, _vp, _vp, _i]),
        "mllm_engine_output_error": (_cp, [_i]),
        "mllm_engine_abort": (_i, [_vp, _ll]),
        "mllm_engine_stats": (_i, [_vp, _vp]),
        "mllm_engine_synchronize": (None, [_vp]),
        # tuning and scratch (tests)
        "mllm_set_tuning": (_i, [_cp, _i, _i]),
        "mllm_get_seen": (_ll, [_cp]),
        "mllm_scratch_address": (_vp, [_cp, _vp]),
        "mllm_scratch_bytes": (_ull, []),
        "mllm_release_scratch": (_i, [_vp]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lb, name)
        fn.restype, fn.argtypes = res, args
    _lib = lb
    return lb


def last_error() -> str:
    return lib().mllm_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise EngineError(last_error())


def text_of(call: Callable[[ctypes.Array, int], int], cap: int = 1 << 16) -> str:
    """Runs ``call(buffer, capacity)``, which writes a text and returns its full length; asks again with
    a larger buffer if the text was cut. A negative length is an error."""
    while True:
        buf = ctypes.create_string_buffer(cap)
        n = call(buf, cap)
        if n < 0:
            raise EngineError(last_error())
        if n < cap:
            return buf.value.decode("utf-8", "replace")
        cap = n + 1


DTYPES = {"bfloat16": 1, "bf16": 1, "float32": 0, "fp32": 0}


def dtype_code(name: str) -> int:
    if name not in DTYPES:
        raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}")
    return DTYPES[name]
